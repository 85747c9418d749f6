"""frisk_hip_gemm_static_ws: the GEMM entry point that allocates nothing.  Its split-K and tail-split partial sums live in
a fixed array inside the library instead of a caller workspace; everything else is frisk_hip_gemm.  The results must be
the bits frisk_hip_gemm produces with a caller workspace, on consecutive calls that reuse the array (the second smaller
than the first, so stale partial sums of the first call lie beyond and between what the second one writes)."""
import numpy as np
import pytest

import oracle as O
from helpers import make_operand, to_dev, run_gemm

pytestmark = pytest.mark.gpu


def note(msg):
    print(msg, flush=True)


def _static(hip, dtype, A, B, transB, dtype_out, M, N, K, split_k=0, epilogue=0, sA=None, sB=None):
    import torch
    out_np = O.NP_STORAGE[dtype_out]
    dA, dB = to_dev(A), to_dev(B)
    dC = torch.full((M * N * np.dtype(out_np).itemsize,), 0xFF, dtype=torch.uint8, device="cuda")
    dsA = to_dev(np.asarray(sA, dtype=np.float32)) if sA is not None else None
    dsB = to_dev(np.asarray(sB, dtype=np.float32)) if sB is not None else None
    desc = hip.make_desc(dtype, M, N, K, dtype_out=dtype_out, transB=transB, epilogue=epilogue, split_k=split_k)
    # the property the entry point exists for: with inputs and outputs on the device, the call leaves the device's free
    # memory as it found it (hipMemGetInfo through torch; a hipMalloc anywhere below the call would show here)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    hip.gemm_static_ws(desc, dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), dsA.data_ptr() if dsA is not None else None,
                       dsB.data_ptr() if dsB is not None else None, torch.cuda.current_stream().cuda_stream)
    free_during = torch.cuda.mem_get_info()[0]
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_before == free_during == free_after, "frisk_hip_gemm_static_ws changed the device's free memory"
    return dC.cpu().numpy().view(out_np).reshape(M, N)


def test_static_workspace_matches_caller_workspace_on_two_calls_in_a_row(hip):
    hip.init()  # the set-up call: places the library's device image (the array is part of it) on the GPU, once
    assert hip.static_workspace_bytes() == 32 << 20
    # first call: int8 64 x 2048 x 8192 NN, the planner splits K (skinny problem); dequantising epilogue
    # second call: a smaller problem of the same kind, then an fp16 one with an explicit split on the 256 x 256 tile
    cases = [(O.I8, 64, 2048, 8192, 0, O.F16, 0, hip.EPI_ROW_COL_SCALE), (O.I8, 32, 512, 8192, 0, O.I32, 0, hip.EPI_NONE),
             (O.F16, 512, 512, 2048, 1, O.F16, 4, hip.EPI_NONE)]
    for n, (dt, M, N, K, tB, out_dt, split, epi) in enumerate(cases):
        A = make_operand(dt, M, K, 40 + n, 0, scale=0.05)
        B = make_operand(dt, N if tB else K, K if tB else N, 40 + n, 1, scale=0.05)
        sA = O.uniform(M, 40 + n, 2, 0.001, 0.02) if epi else None
        sB = O.uniform(N, 40 + n, 3, 0.001, 0.02) if epi else None
        d = hip.make_desc(dt, M, N, K, dtype_out=out_dt, transB=tB, epilogue=epi, split_k=split)
        p = hip.plan(d)
        note(f"case static workspace {n}: dtype {dt} {M}x{N}x{K} tB={tB} split_k={p.split_k} workspace={p.workspace_bytes}")
        assert p.split_k > 1 and 0 < p.workspace_bytes <= hip.static_workspace_bytes()
        want = run_gemm(hip, dt, A, B, 0, tB, out_dt, M, N, K, epilogue=epi, sA=sA, sB=sB, split_k=split)
        got = _static(hip, dt, A, B, tB, out_dt, M, N, K, split_k=split, epilogue=epi, sA=sA, sB=sB)
        assert np.array_equal(got, want), f"case {n}: static-workspace result differs from the caller-workspace result"
        if dt == O.I8 and out_dt == O.I32:
            assert np.array_equal(got, O.gemm_i32(A, B)), "int8 accumulators are not exact"


def test_static_workspace_tail_split_and_unsplit_plans(hip):
    hip.init()
    # a tail split that fits the array: 4352 x 4096 x 4096 fp16 NT has 272 tiles, the last 16 split 8 ways = 32 MiB
    M, N, K = 4352, 4096, 4096
    d = hip.make_desc(O.F16, M, N, K, transB=True)
    p = hip.plan(d)
    note(f"case static workspace tail split {M}x{N}x{K}: tail {p.tail_tiles} x {p.tail_split}, workspace {p.workspace_bytes}")
    assert p.tail_split > 1 and p.workspace_bytes <= hip.static_workspace_bytes()
    A = make_operand(O.F16, M, K, 50, 0, scale=0.02)
    B = make_operand(O.F16, N, K, 50, 1, scale=0.02)
    want = run_gemm(hip, O.F16, A, B, 0, 1, O.F16, M, N, K)
    got = _static(hip, O.F16, A, B, 1, O.F16, M, N, K)
    assert np.array_equal(got, want)
    # a plan without partial sums runs exactly as frisk_hip_gemm does
    A = make_operand(O.F16, 256, 128, 51, 0)
    B = make_operand(O.F16, 128, 256, 51, 1)
    assert np.array_equal(_static(hip, O.F16, A, B, 0, O.F16, 256, 256, 128), run_gemm(hip, O.F16, A, B, 0, 0, O.F16, 256, 256, 128))


def test_planner_chosen_split_beyond_the_array_runs_as_one_pass(hip):
    # 4608 x 4096 x 4096 fp16 NT: 288 tiles, the planner splits the last 32 eight ways = 64 MiB of partial sums, twice the
    # array.  Nobody asked for that split: the call runs the single pass frisk_hip_gemm runs without a workspace.
    M, N, K = 4608, 4096, 4096
    d = hip.make_desc(O.F16, M, N, K, transB=True)
    p = hip.plan(d)
    note(f"case static workspace, planner split too large {M}x{N}x{K}: tail {p.tail_tiles} x {p.tail_split}, workspace {p.workspace_bytes}")
    assert p.tail_split > 1 and p.workspace_bytes > hip.static_workspace_bytes()
    A = make_operand(O.F16, M, K, 52, 0, scale=0.02)
    B = make_operand(O.F16, N, K, 52, 1, scale=0.02)
    want = run_gemm(hip, O.F16, A, B, 0, 1, O.F16, M, N, K, workspace=False)
    got = _static(hip, O.F16, A, B, 1, O.F16, M, N, K)
    assert np.array_equal(got, want)
    r = O.compare(O.F16, got[:256].view(np.uint16), O.gemm_f64(O.F16, A[:256], B, transB=1))
    assert r["nonfinite"] == 0 and r["max_rel"] <= 1e-2 and r["fro_rel"] <= 1e-2, r


def test_static_workspace_refuses_what_does_not_fit(hip):
    d = hip.make_desc(O.F16, 4096, 4096, 4096, split_k=8)  # 8 slices x 64 MiB of partial sums
    assert hip.plan(d).workspace_bytes > hip.static_workspace_bytes()
    with pytest.raises(hip.FriskHipError) as e:
        hip.gemm_static_ws(d, 256, 256, 256, None, None, None)  # refused before any pointer is looked at
    assert e.value.status == hip.ERR_WORKSPACE and "static workspace" in str(e.value)
