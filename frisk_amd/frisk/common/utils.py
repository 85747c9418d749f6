"""Session helper of the `frisk` package: one object that owns a context, a builder and a module.

The public names and keyword arguments are those the reference's scripts use
(test/python/helper_test.py:4-24: `create_session`, `.builder`, `.module`, `memref_type(shape, type, space=)`,
`new_kernel(name, types) -> (kernel, entry block)`, `create_gemm(A, B, C)`, `alloc_buffer(shape, "fp16", space=, alignment=)`;
`create_context`, `ensure_insertion_block` and `dump` complete the surface of python/frisk/common/utils.py).  Everything
behind those names is this build's own: element types live in one table, and `tiled_gemm` writes the whole tiled GEMM
program of the reference's design sketch (tmp/ir.mlir:1-17) that `frisk.runtime` lowers to the gfx950 kernels.
"""
from ..frisk_ffi import ir

__all__ = ["create_context", "create_session", "FriskHelper"]


class _Element:
    """one row of the element-type table: how the builder makes the type, how a type object is recognised, and the type a
    GEMM on such operands accumulates in"""

    def __init__(self, name, getter, probe=None, accumulator=None):
        self.name, self.getter, self.probe, self.accumulator = name, getter, probe, accumulator

    def make(self, builder):
        return getattr(builder, self.getter)()

    def matches(self, ty):
        return self.probe is not None and getattr(ty, self.probe)()


_ELEMENTS = [
    _Element("fp16", "get_f16_ty", "is_f16", "fp32"),
    _Element("bf16", "get_bf16_ty", "is_bf16", "fp32"),
    _Element("fp32", "get_f32_ty", "is_f32", "fp32"),
    _Element("fp64", "get_f64_ty", "is_f64"),
    _Element("e4m3fn", "get_f8e4m3fn_ty", None, "fp32"),
    _Element("int8", "get_int8_ty", None, "int32"),
    _Element("int32", "get_int32_ty"),
    _Element("int64", "get_int64_ty"),
]
_BY_NAME = {e.name: e for e in _ELEMENTS}


def _element_named(name):
    try:
        return _BY_NAME[str(name).strip().lower()]
    except KeyError:
        raise ValueError("element type %r is not one of %s" % (name, ", ".join(sorted(_BY_NAME)))) from None


def _name_of_type(ty):
    for e in _ELEMENTS:
        if e.matches(ty):
            return e.name
    raise ValueError("alloc_buffer takes the element type as a string or as an f16 / bf16 / f32 / f64 type object, got %s" % (ty,))


def create_context(*, load_dialects=True, disable_multithreading=True):
    """a fresh IR context, single-threaded and with the Frisk dialect registered unless told otherwise"""
    ctx = ir.context()
    if disable_multithreading:
        ctx.disable_multithreading()
    if load_dialects:
        ir.frisk.load_dialects(ctx)
    return ctx


def create_session(*, load_dialects=True, disable_multithreading=True):
    return FriskHelper.create(load_dialects=load_dialects, disable_multithreading=disable_multithreading)


class FriskHelper:
    """context + builder + module.  The module keeps a reference to the context (`module.context`), which owns every IR
    object, so handing the module around is enough to keep the IR alive."""

    def __init__(self, context, builder, module):
        self.context, self.builder, self.module = context, builder, module

    @classmethod
    def create(cls, *, load_dialects=True, disable_multithreading=True):
        context = create_context(load_dialects=load_dialects, disable_multithreading=disable_multithreading)
        builder = ir.builder(context)
        module = builder.create_module()
        module.context = context
        return cls(context, builder, module)

    def __repr__(self):
        return "FriskHelper(%d top-level ops)" % str(self.module).count("frisk.kernel")

    # ---------------------------------------------------------------- types
    def element_type(self, dtype):
        """`dtype` as a type object: a name from the element table or a type that is passed through"""
        return dtype if isinstance(dtype, ir.type) else _element_named(dtype).make(self.builder)

    def memref_type(self, shape, dtype="fp16", *, space=ir.MemorySpace.GLOBAL, layout=None):
        return self.builder.get_memref_ty(self.element_type(dtype), [int(extent) for extent in shape],
                                          ir.AffineMap() if layout is None else layout, space)

    # ---------------------------------------------------------------- ops
    def new_kernel(self, name, arg_types):
        """appends `frisk.kernel @name(arg_types...)` to the module and leaves the builder at the start of its body"""
        kernel = self.builder.create_kernel_op(self.module, name, self.builder.get_kernel_ty(list(arg_types)))
        self.module.push_back(kernel)
        entry = kernel.add_entry_block()
        self.builder.set_insertion_point_to_start(entry)
        return kernel, entry

    def alloc_buffer(self, shape, dtype="fp16", *, space=ir.MemorySpace.LOCAL, alignment=0):
        """the value of a `frisk.alloc_buffer`"""
        name = dtype if isinstance(dtype, str) else _name_of_type(dtype)
        return ir.OpState.get_result(self.builder.create_alloc_buffer_op([int(extent) for extent in shape], name, space, alignment), 0)

    def create_gemm(self, A, B, C, *, trans_a=False, trans_b=False, clear_accum=False):
        return self.builder.create_gemm_op(A, B, C, trans_a, trans_b, clear_accum)

    def tiled_gemm(self, name, M, N, K, dtype="fp16", *, out_dtype=None, tile=(256, 256, 64), threads=512, trans_a=False, trans_b=False):
        """kernel(A, B, C) { parallel (by, bx) { sA, sB, acc; fill acc 0; for k { copy A, copy B, gemm }; copy acc -> C } }"""
        b = self.builder
        bm, bn, bk = tile
        if M % bm or N % bn or K % bk:
            raise ValueError("tile %r does not divide the problem %r" % (tile, (M, N, K)))
        acc_dtype = _element_named(dtype).accumulator
        if acc_dtype is None:
            raise ValueError("no GEMM on operands of type %r" % (dtype,))
        a_shape = (K, M) if trans_a else (M, K)
        b_shape = (N, K) if trans_b else (K, N)
        kernel, entry = self.new_kernel(name, [self.memref_type(a_shape, dtype), self.memref_type(b_shape, dtype),
                                               self.memref_type((M, N), out_dtype or dtype)])
        gA, gB, gC = (entry.get_argument(i) for i in range(3))
        body = b.create_parallel_op([M // bm, N // bn], threads).add_entry_block()
        b.set_insertion_point_to_start(body)
        by, bx = body.get_argument(0), body.get_argument(1)
        sa_shape = [bk, bm] if trans_a else [bm, bk]
        sb_shape = [bn, bk] if trans_b else [bk, bn]
        sA = self.alloc_buffer(sa_shape, dtype, space=ir.MemorySpace.SHARED, alignment=1024)
        sB = self.alloc_buffer(sb_shape, dtype, space=ir.MemorySpace.SHARED, alignment=1024)
        acc = self.alloc_buffer((bm, bn), acc_dtype, space=ir.MemorySpace.LOCAL)
        b.create_fill_op(acc, 0.0, acc_dtype)
        d0, d1 = b.get_affine_dim_expr(0), b.get_affine_dim_expr(1)

        def scaled(s0, s1):  # (i, j) -> (i * s0, j * s1): tile indices to element offsets
            return ir.AffineMap.get(2, 0, [d0 * s0, d1 * s1])

        def origin(bb):  # () -> (0, 0)
            return ir.AffineMap.get(0, 0, [bb.get_affine_constant_expr(0)] * 2)

        def k_body(bb, k):
            bb.create_copy_op(gA, sA, [k, by] if trans_a else [by, k], [], scaled(*sa_shape), origin(bb), sa_shape, sa_shape)
            bb.create_copy_op(gB, sB, [bx, k] if trans_b else [k, bx], [], scaled(*sb_shape), origin(bb), sb_shape, sb_shape)
            bb.create_gemm_op(sA, sB, acc, trans_a, trans_b, False)

        b.create_for_op(0, K // bk, 1, k_body)
        b.create_copy_op(acc, gC, [], [by, bx], origin(b), scaled(bm, bn), [bm, bn], [bm, bn])
        return kernel

    def online_softmax(self, name, rows, cols, dtype="fp16", **kw):
        """the row softmax with a running log-sum of the reference's sketch (tmp/ir.mlir:21-75); see common/programs.py"""
        from . import programs
        return programs.online_softmax(self, name, rows, cols, dtype, **kw)

    def attention(self, name, batch, heads, seq_q, seq_k, head_dim=128, dtype="fp16", **kw):
        """the fused attention of the reference's sketch (tmp/ir.mlir:88-158); see common/programs.py"""
        from . import programs
        return programs.attention(self, name, batch, heads, seq_q, seq_k, head_dim, dtype, **kw)

    # ---------------------------------------------------------------- utilities
    def ensure_insertion_block(self):
        """the block the builder inserts into; when it has none yet, a new block at the end of the module's body"""
        block = self.builder.get_insertion_block()
        if block is None:
            block = self.builder.new_block()
            self.module.get_region(0).push_back(block)
            self.builder.set_insertion_point_to_start(block)
        return block

    def dump(self, msg=None):
        if msg:
            print(msg)
        print(self.module)
