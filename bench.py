#!/usr/bin/env python3
"""Benchmark of the GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one launch of the fp16 4096^3 NN GEMM (fp32 accumulate, fp16 out,
inputs N(0,1)/sqrt(K), seed 1) through the C ABI, inputs resident in HBM.
Prints ONE JSON line: whole-job TFLOP/s, the MFMA roofline of the kernel and
the CPU oracle timed on the host cores beside it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f16": 2516.6, "bf16": 2516.6, "i8": 5033.2, "e4m3": 5033.2, "f32": 157.3}
# L2-miss bytes of one fp16 4096^3 launch from rocprofv3 counters: FETCH_SIZE 98 458.0 KiB x 2.00 (the factor a 1 GiB
# copy shows for this counter) + WRITE_SIZE 36 371.4 KiB x 1.00; see profiles/bench_kernels_f16_4096_i8_4096_fp8_skinny.md
TRAFFIC_BYTES_F16_4096 = int((98458.0 * 2.0 + 36371.4) * 1024)


SETTLE_MS = 100.0


def settle(torch, launch, stream):
    """Untimed launches until SETTLE_MS of GPU time have passed.  After an idle period the part's power management
    first overshoots and then takes about 50 ms of continuous load to reach its steady clocks (launch time goes
    122 -> 145 -> 116 us over the first 400 launches of the fp16 4096^3 kernel; the vendor library shows the same
    curve), so a short warm-up would time the transient, not the kernel."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    spent = 0.0
    while spent < SETTLE_MS:
        e0.record(stream)
        for _ in range(50):
            launch()
        e1.record(stream)
        e1.synchronize()
        spent += e0.elapsed_time(e1)


def gpu_time_gemm(R, torch, desc, ptrs, steps, warmup):
    """returns (wall seconds for `steps` launches, mean kernel ms from HIP events on the launch stream)"""
    stream = torch.cuda.current_stream()
    s = stream.cuda_stream
    settle(torch, lambda: R.gemm(desc, *ptrs, None, 0, s), stream)
    for _ in range(warmup):
        R.gemm(desc, *ptrs, None, 0, s)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(steps):
        R.gemm(desc, *ptrs, None, 0, s)
    e1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) / steps


def cpu_baseline(M, N, K):
    """the CPU oracle (fp32 arithmetic, OpenMP over all host cores) on the same workload"""
    import numpy as np
    import oracle as O
    A = O.encode(O.F16, O.normal(M * K, 1, 0, 1.0 / np.sqrt(K))).reshape(M, K)
    B = O.encode(O.F16, O.normal(K * N, 1, 1, 1.0 / np.sqrt(K))).reshape(K, N)
    O.gemm_f32(O.F16, A, B, nrows=256)  # warm-up: thread pool, first touch
    runs = []
    for _ in range(3):
        t0 = time.perf_counter()
        O.gemm_f32(O.F16, A, B)
        runs.append(time.perf_counter() - t0)
    best = min(runs)
    return {"value": round(2.0 * M * N * K / best / 1e12, 4), "unit": "TFLOP/s", "cores": O.num_threads(), "kind": "port",
            "sample": "full fp16 4096^3 NN GEMM, fp32 arithmetic, best of 3 runs (%.2f s each)" % best}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-mib", type=int, default=0,
                    help="also run 3 plain device copies of this many MiB first: a kernel of known traffic to scale profiler byte counters by")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: the GEMM path has no multi-GPU leg (run with --gpus 1)")

    import torch
    from frisk_amd import runtime as R

    R.lib()
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda:0")
    if a.copy_mib:
        src = torch.empty(a.copy_mib << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    M = N = K = 4096
    g = torch.Generator(device=dev)
    g.manual_seed(1)
    A = (torch.randn(M, K, device=dev, generator=g) / K ** 0.5).half()
    B = (torch.randn(K, N, device=dev, generator=g) / K ** 0.5).half()
    C = torch.empty(M, N, device=dev, dtype=torch.float16)
    desc = R.make_desc(R.F16, M, N, K, dtype_out=R.F16)
    plan = R.plan(desc)
    ptrs = (A.data_ptr(), B.data_ptr(), C.data_ptr(), None, None)
    wall, kern_ms = gpu_time_gemm(R, torch, desc, ptrs, a.steps, a.warmup)
    flops = 2.0 * M * N * K
    value = flops * a.steps / wall / 1e12
    achieved = flops / (kern_ms * 1e-3) / 1e12

    # the same launch with operands rotating over 4 buffer sets (4 x 96 MiB > the 256 MiB last-level cache): every
    # launch streams A and B from HBM instead of finding them cached
    sets = [(A, B, C)] + [((torch.randn(M, K, device=dev, generator=g) / K ** 0.5).half(), (torch.randn(K, N, device=dev, generator=g) / K ** 0.5).half(),
                           torch.empty(M, N, device=dev, dtype=torch.float16)) for _ in range(3)]
    stream0 = torch.cuda.current_stream()

    def cold(n):
        for i in range(n):
            a_, b_, c_ = sets[i % 4]
            R.gemm(desc, a_.data_ptr(), b_.data_ptr(), c_.data_ptr(), None, None, None, 0, stream0.cuda_stream)
    settle(torch, lambda: cold(4), stream0)
    ce0, ce1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ce0.record(stream0)
    cold(a.steps)
    ce1.record(stream0)
    torch.cuda.synchronize()
    cold_ms = ce0.elapsed_time(ce1) / a.steps
    del sets

    # second headline shape of the metric: W8A8 int8 4096^3 with the dequant epilogue (reported, not the timed value)
    A8 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev, generator=g)
    B8 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=dev, generator=g)
    sA = torch.rand(M, device=dev, generator=g) * 0.019 + 0.001
    sB = torch.rand(N, device=dev, generator=g) * 0.019 + 0.001
    C8 = torch.empty(M, N, device=dev, dtype=torch.float16)
    d8 = R.make_desc(R.I8, M, N, K, dtype_out=R.F16, epilogue=R.EPI_ROW_COL_SCALE)
    _, i8_ms = gpu_time_gemm(R, torch, d8, (A8.data_ptr(), B8.data_ptr(), C8.data_ptr(), sA.data_ptr(), sB.data_ptr()),
                             a.steps, a.warmup)
    i8_tops = flops / (i8_ms * 1e-3) / 1e12

    # HBM-bound shape of the configuration list: fp8 e4m3 M=32, N=K=8192 (B stored [N][K]), per-tensor scales, bf16 out.
    # B rotates over 6 buffers (384 MiB > the 256 MiB last-level cache) so every launch streams it from HBM.
    Ms, Ns, Ks = 32, 8192, 8192
    Af = torch.randn(Ms, Ks, device=dev, generator=g).to(torch.float8_e4m3fn)
    Bf = [torch.randn(Ns, Ks, device=dev, generator=g).to(torch.float8_e4m3fn) for _ in range(6)]
    Cf = torch.empty(Ms, Ns, device=dev, dtype=torch.bfloat16)
    one = torch.ones(1, device=dev)
    df = R.make_desc(R.E4M3, Ms, Ns, Ks, dtype_out=R.BF16, transB=True, epilogue=R.EPI_TENSOR_SCALE)
    pf = R.plan(df)
    ws_bytes = R.workspace_bytes(df)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream()

    def skinny(n):
        for i in range(n):
            R.gemm(df, Af.data_ptr(), Bf[i % len(Bf)].data_ptr(), Cf.data_ptr(), one.data_ptr(), one.data_ptr(),
                   ws.data_ptr() if ws_bytes else None, ws_bytes, stream.cuda_stream)
    settle(torch, lambda: skinny(1), stream)
    skinny(a.warmup)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    skinny(a.steps)
    e1.record(stream)
    torch.cuda.synchronize()
    sk_ms = e0.elapsed_time(e1) / a.steps
    sk_bytes = Ms * Ks + Ns * Ks + 2 * Ms * Ns + 8
    sk_gbs = sk_bytes / (sk_ms * 1e-3) / 1e9
    del Bf

    # the dialect's data-movement ops on a 32768 x 8192 f16 view (512 MiB per array: twice the last-level cache)
    def time_op(fn):
        settle(torch, fn, stream)
        e0.record(stream)
        for _ in range(20):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / 20

    orows, ocols = 32768, 8192
    src16 = torch.randn(orows, ocols, device=dev, generator=g).half()
    dst16 = torch.empty_like(src16)
    red = torch.empty(orows, device=dev, dtype=torch.float16)
    rws_bytes = R.reduce_workspace_bytes(R.F16, orows, ocols, 0)
    rws = torch.empty(max(rws_bytes, 16), dtype=torch.uint8, device=dev)
    cs = stream.cuda_stream
    nbytes = orows * ocols * 2
    ops = {}
    for name, moved, fn in (
            ("fill", nbytes, lambda: R.fill(R.F16, dst16.data_ptr(), orows, ocols, ocols, 1.5, cs)),
            ("copy", 2 * nbytes, lambda: R.copy(R.F16, src16.data_ptr(), ocols, R.F16, dst16.data_ptr(), ocols, orows, ocols, cs)),
            ("reduce_dim1_add", nbytes, lambda: R.reduce(R.F16, src16.data_ptr(), orows, ocols, ocols, 1, "add", True, red.data_ptr(), None, 0, cs)),
            ("reduce_dim0_max", nbytes, lambda: R.reduce(R.F16, src16.data_ptr(), orows, ocols, ocols, 0, "max", True, red.data_ptr(), rws.data_ptr(),
                                                         rws_bytes, cs))):
        ms = time_op(fn)
        ops[name] = {"GB/s": round(moved / (ms * 1e-3) / 1e9, 1), "frac_of_8TB/s": round(moved / (ms * 1e-3) / 8e12, 4), "kernel_ms": round(ms, 5)}
    # the reference's @online_softmax sketch at the same size class: one read and one write of every element
    ms = time_op(lambda: R.softmax(R.F16, src16.data_ptr(), ocols, dst16.data_ptr(), ocols, orows, ocols, 1.25, None, cs))
    ops["softmax_rows"] = {"GB/s": round(2 * nbytes / (ms * 1e-3) / 1e9, 1), "frac_of_8TB/s": round(2 * nbytes / (ms * 1e-3) / 8e12, 4), "kernel_ms": round(ms, 5)}
    del src16, dst16

    # fused attention forward at the shape of the reference's sketch: 1 x 32 heads x 4096 x 128, fp16
    ab, ah, aseq, ad = 1, 32, 4096, 128
    aq, ak, av = (torch.randn(ab * ah, aseq, ad, device=dev, generator=g).half() for _ in range(3))
    ao = torch.empty_like(aq)
    adesc = R.make_attention_desc(R.F16, ab, ah, aseq, aseq, ad)
    attn_ms = time_op(lambda: R.attention(adesc, aq.data_ptr(), ak.data_ptr(), av.data_ptr(), ao.data_ptr(), None, cs))
    attn_tflops = 4.0 * ab * ah * aseq * aseq * ad / (attn_ms * 1e-3) / 1e12
    del aq, ak, av, ao

    line = {
        "metric": "GEMM TFLOP/s at 4096^3 fp16 (fp32 accumulate), 1 GPU",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(wall / a.steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic", "settle_ms": SETTLE_MS,
        "config": {"workload": "fp16 GEMM M=N=K=4096 NN row-major, N(0,1)/sqrt(K) seed 1, fp32 accumulate, fp16 out",
                   "kernel": R.kernel_names()[plan.kernel_id], "grid": [plan.grid_x, plan.grid_y],
                   "lds_bytes": plan.lds_bytes},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS["f16"], "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_TFLOPS["f16"], 4), "traffic": TRAFFIC_BYTES_F16_4096, "traffic_unit": "bytes per launch",
                     "kernel_ms": round(kern_ms, 5), "kernel_ms_rotating_4_buffer_sets": round(cold_ms, 5)},
        "int8_4096": {"value": round(i8_tops, 2), "unit": "TOPS", "peak": PEAK_TFLOPS["i8"],
                      "frac": round(i8_tops / PEAK_TFLOPS["i8"], 4), "kernel_ms": round(i8_ms, 5),
                      "workload": "W8A8 int8 4096^3 NN, int32 accumulate, per-row/per-column fp32 scales, fp16 out"},
        "fp8_skinny_32x8192x8192": {"bound": "hbm", "achieved": round(sk_gbs, 1), "peak": 8000.0, "unit": "GB/s",
                                    "frac": round(sk_gbs / 8000.0, 4), "kernel_ms": round(sk_ms, 5),
                                    "kernel": R.kernel_names()[pf.kernel_id], "split_k": pf.split_k,
                                    "workload": "fp8 e4m3 M=32 N=K=8192 NT, per-tensor scales, bf16 out; algorithmic bytes "
                                                "|A|+|B|+|C|+scales per launch, B rotating over 6 buffers"},
        "tile_ops_32768x8192_f16": ops,
        "attention_1x32x4096x128_f16": {"bound": "mfma", "achieved": round(attn_tflops, 2), "peak": PEAK_TFLOPS["f16"], "unit": "TFLOP/s",
                                        "frac": round(attn_tflops / PEAK_TFLOPS["f16"], 4), "kernel_ms": round(attn_ms, 5),
                                        "workload": "softmax(Q K^T / sqrt(128)) V, 32 heads, 4096 queries x 4096 keys, head_dim 128, "
                                                    "fp16 in / out, fp32 accumulate; 4 * heads * seq^2 * head_dim flops per launch"},
    }
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(M, N, K)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
