"""End to end through the drop-in surface: build the tiled GEMM with the IR builder, let
frisk_ffi.runtime lower it to the C ABI, run it on the GPU, compare with the CPU oracle."""
import numpy as np
import pytest

import frisk_amd  # noqa: F401
import frisk as F
import oracle as O
from helpers import from_dev, make_operand, to_dev

pytestmark = pytest.mark.gpu


def _run(kernel, A, B, M, N, out_np, **kw):
    import torch
    dA, dB = to_dev(A), to_dev(B)
    dC = torch.full((M * N * np.dtype(out_np).itemsize,), 0xFF, dtype=torch.uint8, device="cuda")
    F.runtime.launch(kernel, [dA.data_ptr(), dB.data_ptr(), dC.data_ptr()], torch.cuda.current_stream().cuda_stream, **kw)
    torch.cuda.synchronize()
    return from_dev(dC, out_np, (M, N))


def test_config1_fp32_1024_built_through_the_builder(hip):
    """fp32 C = A.B, M = N = K = 1024, uniform[-1, 1] seed 0: the matmul of the reference's design sketch"""
    M = N = K = 1024
    h = F.create_session()
    kernel = h.tiled_gemm("matmul", M, N, K, "fp32", tile=(128, 128, 32), threads=256)
    assert h.module.verify()
    A = make_operand(O.F32, M, K, seed=0, tensor=0, kind="uniform")
    B = make_operand(O.F32, K, N, seed=0, tensor=1, kind="uniform")
    ref = O.gemm_f64(O.F32, A, B)
    for retile in (True, False):     # the planner's kernel for the whole problem, and the 128 x 128 x 32 tile the program is written with
        got = _run(kernel, A, B, M, N, np.float32, retile=retile)
        r = O.compare(O.F32, got, ref)
        assert r["nonfinite"] == 0 and r["max_rel"] <= 1e-4 and r["fro_rel"] <= 1e-4, (retile, r)
    # the naive definition agrees on a window of rows
    ref_naive = O.gemm_naive(O.F32, np.ascontiguousarray(A[:16]), B)
    assert O.compare(O.F32, np.ascontiguousarray(got[:16]), ref_naive)["max_rel"] <= 1e-4


@pytest.mark.parametrize("dtype,odt,np_out,trans_b", [("fp16", O.F16, np.uint16, False), ("bf16", O.BF16, np.uint16, True)])
def test_sixteen_bit_gemm_through_the_builder(hip, dtype, odt, np_out, trans_b):
    M, N, K = 512, 768, 256
    h = F.create_session()
    kernel = h.tiled_gemm("g", M, N, K, dtype, tile=(256, 256, 64), trans_b=trans_b)
    A = make_operand(odt, M, K, seed=21, tensor=0, scale=0.25)
    B = make_operand(odt, *((N, K) if trans_b else (K, N)), seed=21, tensor=1, scale=0.25)
    got = _run(kernel, A, B, M, N, np_out)
    r = O.compare(odt, got, O.gemm_f64(odt, A, B, False, trans_b))
    assert r["nonfinite"] == 0 and r["max_rel"] <= 1e-2 and r["fro_rel"] <= 1e-2, r


def test_int8_with_dequant_epilogue_through_the_builder(hip):
    import torch
    M, N, K = 512, 512, 512
    h = F.create_session()
    kernel = h.tiled_gemm("w8a8", M, N, K, "int8", out_dtype="fp16", tile=(256, 256, 128))
    A = make_operand(O.I8, M, K, seed=3, tensor=0)
    B = make_operand(O.I8, K, N, seed=3, tensor=1)
    sA, sB = O.uniform(M, 3, 2, 0.001, 0.02), O.uniform(N, 3, 3, 0.001, 0.02)
    dsA, dsB = to_dev(sA), to_dev(sB)
    got = _run(kernel, A, B, M, N, np.uint16, epilogue="row_col_scale", scale_a=dsA.data_ptr(), scale_b=dsB.data_ptr())
    assert np.array_equal(got, O.epilogue_rowcol_f16(O.gemm_i32(A, B), sA, sB))
    del torch


def test_data_movement_kernel_through_the_builder(hip):
    """fill, converting window copy and row-wise max built with the IR builder, run op by op on the device, against the oracle"""
    import torch
    from oracle import tile_ops as T
    from test_builder_gemm import _data_movement_kernel
    h = F.create_session()
    kernel = _data_movement_kernel(h)
    x = O.encode(O.F32, O.normal(64 * 96, 51, 0, 2.0)).reshape(64, 96)
    dx = to_dev(x)
    dy = torch.full((64 * 96 * 2,), 0xEE, dtype=torch.uint8, device="cuda")
    dv = torch.full((64 * 2,), 0xEE, dtype=torch.uint8, device="cuda")
    ws_bytes = F.runtime.ops_workspace_bytes(kernel)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
    F.runtime.launch_ops(kernel, [dx.data_ptr(), dy.data_ptr(), dv.data_ptr()], torch.cuda.current_stream().cuda_stream, ws.data_ptr(), ws_bytes)
    torch.cuda.synchronize()
    want_y = T.fill(O.F16, 64, 96, 0.5)
    want_y[8:40, 16:80] = T.copy(O.F32, np.ascontiguousarray(x[0:32, 32:96]), O.F16)
    assert np.array_equal(from_dev(dy, np.uint16, (64, 96)), want_y)
    assert np.array_equal(from_dev(dv, np.uint16, (64,)), T.reduce(O.F16, want_y, 1, "max"))


def test_tiled_copy_through_the_builder(hip):
    """a converting copy written tile by tile (grid over row bands, loop over column tiles, every tile through a shared buffer) runs
    as one window copy on the device; elements outside the destination window keep their bytes"""
    import torch
    from oracle import tile_ops as T
    from test_builder_gemm import _tiled_copy_kernel
    for staged in (True, False):
        h = F.create_session()
        kernel = _tiled_copy_kernel(h, staged=staged)
        x = O.encode(O.F32, O.normal(128 * 256, 77, 0, 3.0)).reshape(128, 256)
        dx = to_dev(x)
        dy = torch.full((160 * 320 * 2,), 0xEE, dtype=torch.uint8, device="cuda")
        F.runtime.launch_ops(kernel, [dx.data_ptr(), dy.data_ptr()], torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want = np.full((160, 320), 0xEEEE, dtype=np.uint16)
        want[16:144, 64:320] = T.copy(O.F32, x, O.F16)
        assert np.array_equal(from_dev(dy, np.uint16, (160, 320)), want)


def test_tiles_placed_transposed_through_the_builder(hip):
    """frisk.copy under a grid whose destination map swaps the grid indices: block (by, bx) of the source becomes block (bx, by)
    of the destination, every tile keeping the order of its elements; one tile-by-tile launch, converting f32 -> f16 on the way"""
    import torch
    from oracle import tile_ops as T
    from test_builder_gemm import _transposed_tiles_kernel
    for n, tile, dt, out_dt in ((64, 32, "fp16", None), (256, 64, "fp32", "fp16"), (96, 24, "bf16", None)):
        h = F.create_session()
        kernel = _transposed_tiles_kernel(h, n, tile, dt, out_dt)
        code, out_code = {"fp16": O.F16, "fp32": O.F32, "bf16": O.BF16}[dt], {"fp16": O.F16, "fp32": O.F32, "bf16": O.BF16}[out_dt or dt]
        x = O.encode(code, O.normal(n * n, 78, 0, 2.0)).reshape(n, n)
        dx = to_dev(x)
        dy = torch.full((n * n * O.NP_STORAGE[out_code]().itemsize,), 0xEE, dtype=torch.uint8, device="cuda")
        F.runtime.launch_ops(kernel, [dx.data_ptr(), dy.data_ptr()], torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        conv = T.copy(code, x, out_code)
        nb = n // tile
        want = conv.reshape(nb, tile, nb, tile).transpose(2, 1, 0, 3).reshape(n, n)   # block indices swapped, tiles as they were
        assert np.array_equal(from_dev(dy, O.NP_STORAGE[out_code], (n, n)), want), (n, tile, dt)


def test_reduction_tiled_over_a_grid_through_the_builder(hip):
    """bands of rows (or columns) staged through a shared tile, reduced into a shared vector and stored to their place: one reduce
    launch on the device, against the oracle's reduction of the whole view"""
    import torch
    from oracle import tile_ops as T
    from test_builder_gemm import _tiled_reduce_kernel
    for dim, kind, dt, code in ((1, "max", "fp16", O.F16), (0, "sum", "fp32", O.F32), (1, "sum", "bf16", O.BF16)):
        h = F.create_session()
        kernel = _tiled_reduce_kernel(h, rows=128, cols=256, dim=dim, kind=kind, dtype=dt)
        x = O.encode(code, O.normal(128 * 256, 79, 0, 1.0)).reshape(128, 256)
        kept = 128 if dim == 1 else 256
        dx = to_dev(x)
        dv = torch.full((kept * O.NP_STORAGE[code]().itemsize,), 0xEE, dtype=torch.uint8, device="cuda")
        F.runtime.launch_ops(kernel, [dx.data_ptr(), dv.data_ptr()], torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        got = O.decode(code, from_dev(dv, O.NP_STORAGE[code], (kept,))).astype(np.float64)
        want = T.reduce_f64(code, x, dim, "add" if kind == "sum" else kind)
        if kind == "max":
            assert np.array_equal(got, want)
        else:
            tol = {O.F32: 1e-5, O.F16: 1e-3, O.BF16: 8e-3}[code]
            assert (np.abs(got - want) / np.maximum(np.abs(want), np.sqrt(np.mean(want ** 2)))).max() <= tol
