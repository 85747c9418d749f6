"""Convenience layer over the builder: context + builder + module in one object.

Same surface as the reference's python/frisk/common/utils.py:18-163
(create_context, create_session, FriskHelper with memref_type, new_kernel,
alloc_buffer, create_gemm, ensure_insertion_block, dump), plus `tiled_gemm`,
which writes the whole tiled GEMM program of the reference's design sketch
(tmp/ir.mlir:1-17) in one call.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence, Tuple, Union

from ..frisk_ffi import ir

DTypeLike = Union[str, ir.type]
ShapeLike = Sequence[int]

__all__ = ["create_context", "create_session", "FriskHelper"]


def create_context(*, load_dialects: bool = True, disable_multithreading: bool = True) -> ir.context:
    ctx = ir.context()
    if disable_multithreading:
        ctx.disable_multithreading()
    if load_dialects:
        ir.frisk.load_dialects(ctx)
    return ctx


def create_session(*, load_dialects: bool = True, disable_multithreading: bool = True) -> "FriskHelper":
    return FriskHelper.create(load_dialects=load_dialects, disable_multithreading=disable_multithreading)


_DTYPES = {"fp16": "get_f16_ty", "bf16": "get_bf16_ty", "fp32": "get_f32_ty", "fp64": "get_f64_ty", "int64": "get_int64_ty",
           "int32": "get_int32_ty", "int8": "get_int8_ty", "e4m3fn": "get_f8e4m3fn_ty"}
_ACCUMULATOR = {"fp16": "fp32", "bf16": "fp32", "fp32": "fp32", "e4m3fn": "fp32", "int8": "int32"}


@dataclass
class FriskHelper:
    context: ir.context
    builder: ir.builder
    module: ir.module

    @classmethod
    def create(cls, *, load_dialects: bool = True, disable_multithreading: bool = True) -> "FriskHelper":
        ctx = create_context(load_dialects=load_dialects, disable_multithreading=disable_multithreading)
        builder = ir.builder(ctx)
        module = builder.create_module()
        module.context = ctx  # the context owns every IR object: keep it alive with the module
        return cls(ctx, builder, module)

    # ------------------------------------------------------------------ types
    def memref_type(self, shape: ShapeLike, dtype: DTypeLike = "fp16", *, space: ir.MemorySpace = ir.MemorySpace.GLOBAL,
                    layout: ir.AffineMap | None = None) -> ir.memref_buffer:
        element_type = self._as_type(dtype)
        dims = [int(dim) for dim in shape]
        affine_map = layout if layout is not None else ir.AffineMap()
        return self.builder.get_memref_ty(element_type, dims, affine_map, space)

    # ------------------------------------------------------------------ ops
    def new_kernel(self, name: str, arg_types: Sequence[ir.type]) -> Tuple[ir.KernelOp, ir.block]:
        kernel_type = self.builder.get_kernel_ty(list(arg_types))
        kernel = self.builder.create_kernel_op(self.module, name, kernel_type)
        self.module.push_back(kernel)
        entry = kernel.add_entry_block()
        self.builder.set_insertion_point_to_start(entry)
        return kernel, entry

    def alloc_buffer(self, shape: ShapeLike, dtype: DTypeLike = "fp16", *, space: ir.MemorySpace = ir.MemorySpace.LOCAL,
                     alignment: int = 0) -> ir.value:
        dtype_str = self._as_dtype_str(dtype)
        op = self.builder.create_alloc_buffer_op(list(shape), dtype_str, space, alignment)
        return ir.OpState.get_result(op, 0)

    def create_gemm(self, A: ir.value, B: ir.value, C: ir.value, *, trans_a: bool = False, trans_b: bool = False,
                    clear_accum: bool = False) -> ir.GemmOp:
        return self.builder.create_gemm_op(A, B, C, trans_a, trans_b, clear_accum)

    def tiled_gemm(self, name: str, M: int, N: int, K: int, dtype: str = "fp16", *, out_dtype: str | None = None,
                   tile: Tuple[int, int, int] = (256, 256, 64), threads: int = 512, trans_a: bool = False,
                   trans_b: bool = False) -> ir.KernelOp:
        """kernel(A, B, C) { parallel (by, bx) { sA, sB, acc; fill acc 0; for k { copy A, copy B, gemm }; copy acc -> C } }"""
        b = self.builder
        bm, bn, bk = tile
        if M % bm or N % bn or K % bk:
            raise ValueError("tile %r does not divide the problem %r" % (tile, (M, N, K)))
        acc_dtype = _ACCUMULATOR[dtype]
        out_dtype = out_dtype or dtype
        a_shape = (K, M) if trans_a else (M, K)
        b_shape = (N, K) if trans_b else (K, N)
        tys = [self.memref_type(a_shape, dtype), self.memref_type(b_shape, dtype), self.memref_type((M, N), out_dtype)]
        kernel, entry = self.new_kernel(name, tys)
        gA, gB, gC = (entry.get_argument(i) for i in range(3))
        par = b.create_parallel_op([M // bm, N // bn], threads)
        body = par.add_entry_block()
        b.set_insertion_point_to_start(body)
        by, bx = body.get_argument(0), body.get_argument(1)
        sa_shape = (bk, bm) if trans_a else (bm, bk)
        sb_shape = (bn, bk) if trans_b else (bk, bn)
        sA = self.alloc_buffer(sa_shape, dtype, space=ir.MemorySpace.SHARED, alignment=1024)
        sB = self.alloc_buffer(sb_shape, dtype, space=ir.MemorySpace.SHARED, alignment=1024)
        acc = self.alloc_buffer((bm, bn), acc_dtype, space=ir.MemorySpace.LOCAL)
        b.create_fill_op(acc, 0.0, acc_dtype)
        d0, d1 = b.get_affine_dim_expr(0), b.get_affine_dim_expr(1)
        ident = ir.AffineMap.get_multi_dim_identity_map(2)

        def tile_map(e0, e1):
            return ir.AffineMap.get(2, 0, [e0, e1])

        def k_body(bb, k):
            a_map = tile_map(d0 * bk, d1 * bm) if trans_a else tile_map(d0 * bm, d1 * bk)
            b_map = tile_map(d0 * bn, d1 * bk) if trans_b else tile_map(d0 * bk, d1 * bn)
            bb.create_copy_op(gA, sA, [k, by] if trans_a else [by, k], [], a_map, ir.AffineMap.get(0, 0, [bb.get_affine_constant_expr(0)] * 2),
                              list(sa_shape), list(sa_shape))
            bb.create_copy_op(gB, sB, [bx, k] if trans_b else [k, bx], [], b_map, ir.AffineMap.get(0, 0, [bb.get_affine_constant_expr(0)] * 2),
                              list(sb_shape), list(sb_shape))
            bb.create_gemm_op(sA, sB, acc, trans_a, trans_b, False)

        b.create_for_op(0, K // bk, 1, k_body)
        b.create_copy_op(acc, gC, [], [by, bx], ir.AffineMap.get(0, 0, [b.get_affine_constant_expr(0)] * 2), tile_map(d0 * bm, d1 * bn),
                         [bm, bn], [bm, bn])
        del ident
        return kernel

    # ------------------------------------------------------------------ utilities
    def ensure_insertion_block(self) -> ir.block:
        block = self.builder.get_insertion_block()
        if block is not None:
            return block
        new_block = self.builder.new_block()
        self.module.get_region(0).push_back(new_block)
        self.builder.set_insertion_point_to_start(new_block)
        return new_block

    def dump(self, msg: str | None = None) -> None:
        if msg:
            print(msg)
        print(self.module)

    # ------------------------------------------------------------------ internal
    def _as_type(self, dtype: DTypeLike) -> ir.type:
        if isinstance(dtype, ir.type):
            return dtype
        key = dtype.lower()
        if key in _DTYPES:
            return getattr(self.builder, _DTYPES[key])()
        raise ValueError(f"Unsupported dtype '{dtype}'.")

    def _as_dtype_str(self, dtype: DTypeLike) -> str:
        if isinstance(dtype, str):
            return dtype
        if dtype.is_f16():
            return "fp16"
        if dtype.is_bf16():
            return "bf16"
        if dtype.is_f32():
            return "fp32"
        if dtype.is_f64():
            return "fp64"
        raise ValueError("Unsupported type for allocation helper.")
