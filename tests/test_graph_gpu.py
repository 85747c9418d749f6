"""Launches through the C ABI recorded into a HIP graph (stream capture) and replayed: every replay must give the bits
of the same launches made eagerly.  The entry points allocate nothing and synchronise nothing, and frisk_hip_init does
the one piece of non-stream set-up (the kernels' LDS limits) ahead of the capture."""
import numpy as np
import pytest

import oracle as O
from helpers import make_operand, to_dev

pytestmark = pytest.mark.gpu


def test_gemm_split_k_and_reduce_replay_from_a_graph(hip):
    import torch
    hip.init()
    M, N, K = 512, 512, 256
    Ms = 32
    dA = to_dev(make_operand(O.F16, M, K, seed=61, tensor=0, scale=0.25))
    dB = to_dev(make_operand(O.F16, K, N, seed=61, tensor=1, scale=0.25))
    dAs = to_dev(make_operand(O.F16, Ms, 2048, seed=61, tensor=2, scale=0.25))
    dBs = to_dev(make_operand(O.F16, 2048, N, seed=61, tensor=3, scale=0.25))
    dC = torch.zeros(M * N * 2, dtype=torch.uint8, device="cuda")
    dCs = torch.zeros(Ms * N * 2, dtype=torch.uint8, device="cuda")
    dV = torch.zeros(M * 2, dtype=torch.uint8, device="cuda")
    d1 = hip.make_desc(O.F16, M, N, K)
    d2 = hip.make_desc(O.F16, Ms, N, 2048, split_k=4)
    p2 = hip.plan(d2)
    assert p2.split_k == 4 and p2.workspace_bytes > 0
    ws = torch.empty(p2.workspace_bytes, dtype=torch.uint8, device="cuda")

    def launches(stream):
        hip.gemm(d1, dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), None, None, None, 0, stream)
        hip.gemm(d2, dAs.data_ptr(), dBs.data_ptr(), dCs.data_ptr(), None, None, ws.data_ptr(), ws.numel(), stream)
        hip.reduce(O.F16, dC.data_ptr(), M, N, N, 1, "max", True, dV.data_ptr(), None, 0, stream)

    def snapshot():
        torch.cuda.synchronize()
        return dC.cpu().numpy().copy(), dCs.cpu().numpy().copy(), dV.cpu().numpy().copy()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream, as captures want
        launches(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launches(torch.cuda.current_stream().cuda_stream)

    for rep in range(3):
        # new operand contents in the same buffers, then the eager result, then scrub the outputs and replay
        dA.copy_(to_dev(make_operand(O.F16, M, K, seed=70 + rep, tensor=0, scale=0.25)))
        dAs.copy_(to_dev(make_operand(O.F16, Ms, 2048, seed=70 + rep, tensor=2, scale=0.25)))
        launches(torch.cuda.current_stream().cuda_stream)
        want = snapshot()
        for t in (dC, dCs, dV, ws):
            t.fill_(0xA5)
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        for g, w in zip(got, want):
            assert np.array_equal(g, w), "replay %d differs from the eager launches" % rep
    # and the eager result is the oracle's
    A = dA.cpu().numpy().view(np.uint16).reshape(M, K)
    B = dB.cpu().numpy().view(np.uint16).reshape(K, N)
    r = O.compare(O.F16, want[0].view(np.uint16).reshape(M, N), O.gemm_f64(O.F16, A, B))
    assert r["max_rel"] <= 1e-2 and r["fro_rel"] <= 1e-2, r


def test_tail_split_softmax_split_and_attention_replay_from_a_graph(hip):
    """the two-launch paths added later (GEMM tail split + its reduction, softmax of a few long rows split over work-groups)
    and the attention kernel, captured and replayed: same bits as eager"""
    import torch
    hip.init()
    M = N = 17 * 256
    K = 2048
    dA = to_dev(make_operand(O.F16, M, K, seed=81, tensor=0, scale=0.25))
    dB = to_dev(make_operand(O.F16, K, N, seed=81, tensor=1, scale=0.25))
    dC = torch.zeros(M * N * 2, dtype=torch.uint8, device="cuda")
    dg = hip.make_desc(O.F16, M, N, K)
    pg = hip.plan(dg)
    assert pg.tail_split == 4 and pg.workspace_bytes > 0
    wsg = torch.empty(pg.workspace_bytes, dtype=torch.uint8, device="cuda")
    rows, cols = 4, 1 << 17
    dX = to_dev(make_operand(O.F16, rows, cols, seed=82, tensor=0, scale=2.0))
    dY = torch.zeros(rows * cols * 2, dtype=torch.uint8, device="cuda")
    wss_bytes = hip.softmax_workspace_bytes(O.F16, rows, cols)
    assert wss_bytes > 0
    wss = torch.empty(wss_bytes, dtype=torch.uint8, device="cuda")
    heads, seq = 2, 512
    dQ = to_dev(make_operand(O.F16, heads * seq, 128, seed=83, tensor=0, scale=1.0))
    dK = to_dev(make_operand(O.F16, heads * seq, 128, seed=83, tensor=1, scale=1.0))
    dV = to_dev(make_operand(O.F16, heads * seq, 128, seed=83, tensor=2, scale=1.0))
    dO = torch.zeros(heads * seq * 128 * 2, dtype=torch.uint8, device="cuda")
    da = hip.make_attention_desc(O.F16, 1, heads, seq, seq)

    def launches(stream):
        hip.gemm(dg, dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), None, None, wsg.data_ptr(), wsg.numel(), stream)
        hip.softmax(O.F16, dX.data_ptr(), cols, dY.data_ptr(), cols, rows, cols, 1.25, None, stream, wss.data_ptr(), wss.numel())
        hip.attention(da, dQ.data_ptr(), dK.data_ptr(), dV.data_ptr(), dO.data_ptr(), None, stream)

    def snapshot():
        torch.cuda.synchronize()
        return dC.cpu().numpy().copy(), dY.cpu().numpy().copy(), dO.cpu().numpy().copy()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launches(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launches(torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        dA.copy_(to_dev(make_operand(O.F16, M, K, seed=90 + rep, tensor=0, scale=0.25)))
        dX.copy_(to_dev(make_operand(O.F16, rows, cols, seed=90 + rep, tensor=1, scale=2.0)))
        dQ.copy_(to_dev(make_operand(O.F16, heads * seq, 128, seed=90 + rep, tensor=2, scale=1.0)))
        launches(torch.cuda.current_stream().cuda_stream)
        want = snapshot()
        for t in (dC, dY, dO, wsg, wss):
            t.fill_(0xA5)
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        for g, w in zip(got, want):
            assert np.array_equal(g, w), "replay %d differs from the eager launches" % rep


def test_fp8_whole_tile_atom_block_body_and_tile_placement_replay_from_a_graph(hip):
    """the entry points and the kernel added last -- 8-bit floats on the 16x16x128 atom with its split-K store path, a frisk.block body
    through the interpreter, tiles placed transposed -- captured and replayed: same bits as eager"""
    import torch
    hip.init()
    M, N, K = 512, 512, 2048
    dA = to_dev(make_operand(O.E4M3, M, K, seed=101, tensor=0, scale=0.5))
    dB = to_dev(make_operand(O.E4M3, N, K, seed=101, tensor=1, scale=0.5))
    dC = torch.zeros(M * N * 2, dtype=torch.uint8, device="cuda")
    dC2 = torch.zeros(M * N * 4, dtype=torch.uint8, device="cuda")
    scale = torch.full((1,), 0.25, dtype=torch.float32, device="cuda")
    d1 = hip.make_desc(O.E4M3, M, N, K, dtype_out=O.BF16, transB=1, epilogue=hip.EPI_TENSOR_SCALE, tile=(256, 256, 128), atom=16)
    d2 = hip.make_desc(O.E4M3, M, N, K, dtype_out=O.F32, transB=1, tile=(256, 256, 128), atom=16, split_k=4)
    names = hip.kernel_names()
    p2 = hip.plan(d2)
    assert names[hip.plan(d1).kernel_id].endswith("_a16") and names[p2.kernel_id].endswith("_a16_splitk") and p2.workspace_bytes > 0
    ws = torch.empty(p2.workspace_bytes, dtype=torch.uint8, device="cuda")
    rows, cols = 256, 1024
    dX = to_dev(make_operand(O.F16, rows, cols, seed=102, tensor=0, scale=1.0))
    dY = torch.zeros(rows * cols * 2, dtype=torch.uint8, device="cuda")
    dT = torch.zeros(rows * cols * 2, dtype=torch.uint8, device="cuda")
    prog = [("input", 0), ("const", 0.5), "mul", "exp2", ("input", 0), "add"]
    de = hip.make_elementwise_desc(prog, [(O.F16, cols, 1)], O.F16, rows, cols)
    tr, tc = 64, 128  # 4 x 8 tiles of 64 x 128 of the 256 x 1024 view; tile (a, b) goes to block (b, a) of a 512 x 512 view

    def launches(stream):
        hip.gemm(d1, dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), scale.data_ptr(), scale.data_ptr(), None, 0, stream)
        hip.gemm(d2, dA.data_ptr(), dB.data_ptr(), dC2.data_ptr(), None, None, ws.data_ptr(), ws.numel(), stream)
        hip.elementwise(de, [dX.data_ptr()], dY.data_ptr(), stream)
        hip.copy_tiles(O.F16, dY.data_ptr(), cols, O.F16, dT.data_ptr(), 512, tr, tc, 4, tr * cols, tc, 8, tc, tr * 512, stream)

    def snapshot():
        torch.cuda.synchronize()
        return dC.cpu().numpy().copy(), dC2.cpu().numpy().copy(), dY.cpu().numpy().copy(), dT.cpu().numpy().copy()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launches(side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launches(torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        dA.copy_(to_dev(make_operand(O.E4M3, M, K, seed=110 + rep, tensor=0, scale=0.5)))
        dX.copy_(to_dev(make_operand(O.F16, rows, cols, seed=110 + rep, tensor=1, scale=1.0)))
        launches(torch.cuda.current_stream().cuda_stream)
        want = snapshot()
        for t in (dC, dC2, dY, dT, ws):
            t.fill_(0xA5)
        torch.cuda.synchronize()
        graph.replay()
        got = snapshot()
        for g, w in zip(got, want):
            assert np.array_equal(g, w), "replay %d differs from the eager launches" % rep
    # the eager results are the oracles': the split product against float64, the placement against numpy
    A = dA.cpu().numpy().reshape(M, K)
    B = dB.cpu().numpy().reshape(N, K)
    r = O.compare(O.F32, want[1].view(np.float32).reshape(M, N), O.gemm_f64(O.E4M3, A, B, False, True))
    assert r["max_rel"] <= 1e-2 and r["fro_rel"] <= 1e-2, r
    y = want[2].view(np.uint16).reshape(rows, cols)
    t = want[3].view(np.uint16).reshape(512, 512)
    for a in range(4):
        for b in range(8):
            assert np.array_equal(t[b * tr:(b + 1) * tr, a * tc:(a + 1) * tc], y[a * tr:(a + 1) * tr, b * tc:(b + 1) * tc])
