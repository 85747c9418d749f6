#!/usr/bin/env python3
"""Benchmark of the GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one launch of the fp16 4096^3 NN GEMM (fp32 accumulate, fp16 out, inputs N(0,1)/sqrt(K)) through the C ABI,
inputs resident in HBM.  Prints ONE JSON line: whole-job TFLOP/s, the MFMA roofline of the kernel (against the nominal
peak and against the rate an MFMA-only loop sustains on this box in the same run), the other configurations of the
metric timed the same way, and the CPU oracle timed on the host cores beside them.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published dense peaks (TFLOP/s or TOP/s) and what one CU does per clock for each type (256 CUs x 2.4 GHz)
PEAK_TFLOPS = {"f16": 2516.6, "bf16": 2516.6, "i8": 5033.2, "e4m3": 5033.2, "f32": 157.3}
FLOPS_PER_CU_CLK = {"f16": 4096, "bf16": 4096, "i8": 8192, "e4m3": 8192, "f32": 256}
# L2-miss bytes of one fp16 4096^3 launch, a constant taken from rocprofv3 counters (not measured by this run):
# FETCH_SIZE 98 426.0 KiB x 2.00 (the factor a 1 GiB copy shows for this counter) + WRITE_SIZE 32 774.8 KiB x 1.00
TRAFFIC_BYTES_F16_4096 = int((98508.0 * 2.0 + 32771.0) * 1024)
TRAFFIC_SOURCE = "constant from profiles/bench_gemm_legs_f16_i8_bf16_fp8_f32.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE), not measured by this run"

# duration of the register-only kernel (256 work-groups, 64 MFMAs, no memory) in a rocprofv3 kernel trace; event-timed back to
# back the same launch takes longer by the gap between two launches
REGISTER_ONLY_KERNEL_TRACE_MS = 0.00350

SETTLE_MS = 100.0


def settle(torch, launch, stream, ms=SETTLE_MS):
    """Untimed launches until `ms` of GPU time have passed.  After an idle period the part's power management first
    overshoots and then takes about 50 ms of continuous load to reach its steady clocks (launch time goes
    122 -> 145 -> 116 us over the first 400 launches of the fp16 4096^3 kernel; the vendor library shows the same
    curve), so a short warm-up would time the transient, not the kernel."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    spent = 0.0
    while spent < ms:
        e0.record(stream)
        for _ in range(20):
            launch()
        e1.record(stream)
        e1.synchronize()
        spent += e0.elapsed_time(e1)


def time_launches(torch, launch, steps, warmup, stream):
    """`launch` is timed three ways on `stream` (the stream the kernels are launched on), after the settle period:
    wall clock around `steps` back-to-back launches (bracketed by synchronize), one HIP event pair around the same
    launches (mean kernel time), and one HIP event pair per launch in a second pass (median and min)."""
    settle(torch, launch, stream)
    for _ in range(warmup):
        launch()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(steps):
        launch()
    e1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    mean_ms = e0.elapsed_time(e1) / steps
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in pairs:
        a.record(stream)
        launch()
        b.record(stream)
    torch.cuda.synchronize()
    each = [a.elapsed_time(b) for a, b in pairs]
    return {"wall_s": wall, "mean_ms": mean_ms, "median_ms": statistics.median(each), "min_ms": min(each)}


def mfma_leg(name, dtype_key, flops, t, extra=None):
    """one MFMA-bound configuration: achieved rate from the mean kernel time, fraction of the nominal peak"""
    achieved = flops / (t["mean_ms"] * 1e-3) / 1e12
    out = {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS[dtype_key], "unit": "TOP/s" if dtype_key == "i8" else "TFLOP/s",
           "frac": round(achieved / PEAK_TFLOPS[dtype_key], 4), "kernel_ms": round(t["mean_ms"], 5),
           "kernel_ms_median": round(t["median_ms"], 5), "kernel_ms_min": round(t["min_ms"], 5), "workload": name}
    if extra:
        out.update(extra)
    return out


def mfma_ceiling(torch, HW, stream, cus):
    """The rate a loop of nothing but MFMAs sustains on this box, per instruction kind, with pseudo-random operand
    registers (the values matter: the part is power-limited and constant operands draw less).  One wave per SIMD,
    accumulators of a 128 x 128 wave tile.  Also the shader clock that rate implies: the loop needs a known number of
    matrix-pipe cycles."""
    out = {}
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for kind, (name, dtype_key) in HW.LOOP_KINDS.items():
        iters = 4000
        run = lambda: HW.mfma_loop(kind, iters, True, cus, stream.cuda_stream)
        settle(torch, run, stream, 60.0)
        times = []
        for _ in range(5):
            e0.record(stream)
            run()
            e1.record(stream)
            e1.synchronize()
            times.append(e0.elapsed_time(e1))
        ms = statistics.median(times)
        rate = HW.mfma_loop_flops(kind, iters, cus) / (ms * 1e-3) / 1e12
        out[name] = {"dtype": dtype_key, "rate": round(rate, 1), "frac_of_nominal": round(rate / PEAK_TFLOPS[dtype_key], 4),
                     "implied_clock_mhz": round(HW.mfma_loop_cycles(kind, iters) / (ms * 1e3), 1), "ms": round(ms, 4)}
    e0.record(stream)
    HW.mfma_loop(0, 4000, False, cus, stream.cuda_stream)
    e1.record(stream)
    e1.synchronize()
    ms = e0.elapsed_time(e1)
    out["f16 32x32x16, constant operands"] = {"dtype": "f16", "rate": round(HW.mfma_loop_flops(0, 4000, cus) / (ms * 1e-3) / 1e12, 1),
                                              "implied_clock_mhz": round(HW.mfma_loop_cycles(0, 4000) / (ms * 1e3), 1), "ms": round(ms, 4)}
    return out


def data_fed_ceiling(torch, HW, stream, cus, kind, dtype_key, A, B):
    """the same MFMA-only loop with its operand registers loaded once from the benchmark's own A and B (row-major device
    tensors): the matrix pipe then switches on the bits of the workload, not on a synthetic pattern"""
    iters = 4000
    lda, ldb = A.stride(0) * A.element_size(), B.stride(0) * B.element_size()
    run = lambda: HW.mfma_loop_data(kind, iters, cus, A.data_ptr(), lda, A.shape[0], B.data_ptr(), ldb, B.shape[0], stream.cuda_stream)
    settle(torch, run, stream, 60.0)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    times = []
    for _ in range(5):
        e0.record(stream)
        run()
        e1.record(stream)
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    ms = statistics.median(times)
    rate = HW.mfma_loop_flops(kind, iters, cus) / (ms * 1e-3) / 1e12
    return {"dtype": dtype_key, "rate": round(rate, 1), "frac_of_nominal": round(rate / PEAK_TFLOPS[dtype_key], 4),
            "implied_clock_mhz": round(HW.mfma_loop_cycles(kind, iters) / (ms * 1e3), 1), "ms": round(ms, 4)}


def vendor_leg(torch, name, call, flops_or_bytes, steps, warmup, stream, ours_ms, note=""):
    """One launch of the vendor library (torch -> hipBLASLt / rocBLAS) on the same device tensors, timed with the same
    settle and event protocol as the product's legs.  An external comparator: never the product path.  A call that this
    torch build does not offer is recorded with its error text."""
    try:
        call()
        torch.cuda.synchronize()
        t = time_launches(torch, call, steps, warmup, stream)
    except Exception as exc:  # noqa: BLE001  (whatever the library raises is the record)
        return {"error": "%s: %s" % (type(exc).__name__, str(exc).split("\n")[0][:300]), "call": name}
    out = {"call": name, "kernel_ms": round(t["mean_ms"], 5), "kernel_ms_median": round(t["median_ms"], 5), "kernel_ms_min": round(t["min_ms"], 5),
           "rate": round(flops_or_bytes / (t["mean_ms"] * 1e-3) / 1e12, 2), "ours_ms": round(ours_ms, 5),
           "vs_vendor": round(t["mean_ms"] / ours_ms, 4)}
    if note:
        out["note"] = note
    return out


def sustained_peak(ceiling, dtype_key):
    """best MFMA-only rate any atom of this element type sustained in this run"""
    return max(v["rate"] for k, v in ceiling.items() if v["dtype"] == dtype_key and "constant" not in k and "operands of" not in k)


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


def cpu_baseline_int8(M, N, K):
    """the CPU oracle's exact int8 x int8 -> int32 GEMM (OpenMP over all host cores) on the second headline shape"""
    import oracle as O
    A = O.int8_uniform(M * K, 3, 0).reshape(M, K)
    B = O.int8_uniform(K * N, 3, 1).reshape(K, N)
    O.gemm_i32(A, B, nrows=256)
    runs = []
    for _ in range(3):
        t0 = time.perf_counter()
        O.gemm_i32(A, B)
        runs.append(time.perf_counter() - t0)
    best = min(runs)
    return {"value": round(2.0 * M * N * K / best / 1e12, 4), "unit": "TOP/s", "cores": O.num_threads(), "kind": "port",
            "sample": "full int8 4096^3 NN GEMM, int32 accumulate, best of 3 runs (%.2f s each)" % best}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-headline", action="store_true", help="time the fp16 and int8 4096^3 kernels only (for profiler runs)")
    ap.add_argument("--copy-mib", type=int, default=0,
                    help="also run 3 plain device copies of this many MiB first: a kernel of known traffic to scale profiler byte counters by")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: the GEMM path has no multi-GPU leg (run with --gpus 1)")

    import torch
    from frisk_amd import runtime as R
    from frisk_amd import hwcheck as HW

    R.lib()
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    dev = torch.device("cuda:0")
    prop = torch.cuda.get_device_properties(0)
    info = HW.device_info()  # hipDeviceGetAttribute: torch's properties carry no clock on this build
    cus, clock_khz = info["compute_units"], info["clock_khz"]
    stream = torch.cuda.current_stream()
    cs = stream.cuda_stream
    if a.copy_mib:
        src = torch.empty(a.copy_mib << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    g = torch.Generator(device=dev)
    g.manual_seed(1)

    def gemm_launcher(desc, ptrs, ws=None, ws_bytes=0):
        return lambda: R.gemm(desc, *ptrs, ws, ws_bytes, cs)

    # ---------------------------------------------------------------- headline: fp16 4096^3 NN (the configuration the metric is quoted on)
    M = N = K = 4096
    flops = 2.0 * M * N * K
    A = (torch.randn(M, K, device=dev, generator=g) / K ** 0.5).half()
    B = (torch.randn(K, N, device=dev, generator=g) / K ** 0.5).half()
    C = torch.empty(M, N, device=dev, dtype=torch.float16)
    desc = R.make_desc(R.F16, M, N, K, dtype_out=R.F16)
    plan = R.plan(desc)
    t16 = time_launches(torch, gemm_launcher(desc, (A.data_ptr(), B.data_ptr(), C.data_ptr(), None, None)), a.steps, a.warmup, stream)
    value = flops * a.steps / t16["wall_s"] / 1e12
    achieved = flops / (t16["mean_ms"] * 1e-3) / 1e12

    # second headline shape of the metric: W8A8 int8 4096^3 with the dequant epilogue
    A8 = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev, generator=g)
    B8 = torch.randint(-127, 128, (K, N), dtype=torch.int8, device=dev, generator=g)
    sA = torch.rand(M, device=dev, generator=g) * 0.019 + 0.001
    sB = torch.rand(N, device=dev, generator=g) * 0.019 + 0.001
    C8 = torch.empty(M, N, device=dev, dtype=torch.float16)
    d8 = R.make_desc(R.I8, M, N, K, dtype_out=R.F16, epilogue=R.EPI_ROW_COL_SCALE)
    t8 = time_launches(torch, gemm_launcher(d8, (A8.data_ptr(), B8.data_ptr(), C8.data_ptr(), sA.data_ptr(), sB.data_ptr())), a.steps, a.warmup, stream)
    legs = {"int8_4096": mfma_leg("W8A8 int8 4096^3 NN, int32 accumulate, per-row/per-column fp32 scales, fp16 out (configs[3])", "i8", flops, t8,
                                  {"kernel": R.kernel_names()[R.plan(d8).kernel_id]})}
    vendor = {}

    line = {
        "metric": "GEMM TFLOP/s at 4096^3 fp16 (fp32 accumulate), 1 GPU",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(t16["wall_s"] / a.steps * 1e3, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic", "settle_ms": SETTLE_MS,
        "config": {"workload": "fp16 GEMM M=N=K=4096 NN row-major, N(0,1)/sqrt(K), fp32 accumulate, fp16 out; values drawn on the device by "
                               "torch's generator (seed 1), not by the parity tests' counter-based generator",
                   "kernel": R.kernel_names()[plan.kernel_id], "grid": [plan.grid_x, plan.grid_y], "lds_bytes": plan.lds_bytes,
                   "library": R.LIB_PATH},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS["f16"], "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_TFLOPS["f16"], 4), "traffic": TRAFFIC_BYTES_F16_4096, "traffic_unit": "bytes per launch",
                     "traffic_source": TRAFFIC_SOURCE, "kernel_ms": round(t16["mean_ms"], 5), "kernel_ms_median": round(t16["median_ms"], 5),
                     "kernel_ms_min": round(t16["min_ms"], 5)},
        "device": {"name": prop.name, "compute_units": cus, "clock_mhz_reported": round(clock_khz / 1e3, 1),
                   "peak_from_device_properties": {k: round(cus * clock_khz * 1e3 * v / 1e12, 1) for k, v in FLOPS_PER_CU_CLK.items()},
                   "peak_nominal": PEAK_TFLOPS, "note": "CUs x reported clock x flops per CU and clock (4096 16-bit, 8192 8-bit, 256 fp32)",
                   "memory_clock_mhz_reported": round(info["memory_clock_khz"] / 1e3, 1), "memory_bus_bits": info["memory_bus_bits"],
                   "hbm_peak_from_device_properties_GBps": round(4.0 * info["memory_clock_khz"] * 1e3 * info["memory_bus_bits"] / 8 / 1e9, 1),
                   "hbm_note": "bus bits x reported memory clock x 4 transfers per clock (HBM3E at 8 Gb/s per pin on a 2 GHz reported clock) / 8"},
    }

    if not a.only_headline:
        # the same launch with operands rotating over 4 buffer sets (4 x 96 MiB > the 256 MiB last-level cache): every
        # launch streams A and B from HBM instead of finding them cached
        sets = [(A, B, C)] + [((torch.randn(M, K, device=dev, generator=g) / K ** 0.5).half(), (torch.randn(K, N, device=dev, generator=g) / K ** 0.5).half(),
                               torch.empty(M, N, device=dev, dtype=torch.float16)) for _ in range(3)]
        turn = [0]

        def cold():
            a_, b_, c_ = sets[turn[0] % 4]
            turn[0] += 1
            R.gemm(desc, a_.data_ptr(), b_.data_ptr(), c_.data_ptr(), None, None, None, 0, cs)
        line["roofline"]["kernel_ms_rotating_4_buffer_sets"] = round(time_launches(torch, cold, a.steps, a.warmup, stream)["mean_ms"], 5)
        del sets
        Cv = torch.empty(M, N, device=dev, dtype=torch.float16)
        vendor["fp16_4096_nn"] = vendor_leg(torch, "torch.matmul(A, B, out=C), fp16 4096^3 NN", lambda: torch.matmul(A, B, out=Cv), flops, a.steps, a.warmup,
                                            stream, t16["mean_ms"])
        C32 = torch.empty(M, N, device=dev, dtype=torch.int32)
        vendor["int8_4096"] = vendor_leg(torch, "torch._int_mm(A, B, out=C), int8 4096^3 NN", lambda: torch._int_mm(A8, B8, out=C32), flops, a.steps, a.warmup,
                                         stream, t8["mean_ms"], "the vendor call writes raw int32 accumulators (64 MiB), the product leg dequantises to fp16 (32 MiB)")
        del C32

        # the same problem with B stored [N][K]: both operands K-contiguous in LDS, no transpose reads
        Bt = B.t().contiguous()
        dnt = R.make_desc(R.F16, M, N, K, dtype_out=R.F16, transB=True)
        tnt = time_launches(torch, gemm_launcher(dnt, (A.data_ptr(), Bt.data_ptr(), C.data_ptr(), None, None)), a.steps, a.warmup, stream)
        legs["fp16_4096_nt"] = mfma_leg("fp16 4096^3 NT (B stored [N][K])", "f16", flops, tnt, {"kernel": R.kernel_names()[R.plan(dnt).kernel_id]})
        vendor["fp16_4096_nt"] = vendor_leg(torch, "torch.matmul(A, Bt.t(), out=C), fp16 4096^3 NT", lambda: torch.matmul(A, Bt.t(), out=Cv), flops, a.steps, a.warmup,
                                            stream, tnt["mean_ms"])
        del Cv

        # what the matrix pipe sustains on this box when nothing else runs
        ceiling = mfma_ceiling(torch, HW, stream, cus)
        # the atoms the headline kernels run on, fed from the workloads' own operands
        ceiling["f16 16x16x32, operands of the fp16 4096^3 workload"] = data_fed_ceiling(torch, HW, stream, cus, 1, "f16", A, Bt)
        ceiling["i8 16x16x64, operands of the int8 4096^3 workload"] = data_fed_ceiling(torch, HW, stream, cus, 5, "i8", A8, B8)
        del Bt, A8, B8, C8
        line["mfma_ceiling"] = ceiling
        sp = sustained_peak(ceiling, "f16")
        line["roofline"]["sustained_peak"] = sp
        line["roofline"]["frac_of_sustained"] = round(achieved / sp, 4)
        for key, dk in (("int8_4096", "i8"), ("fp16_4096_nt", "f16")):
            legs[key]["sustained_peak"] = sustained_peak(ceiling, dk)
            legs[key]["frac_of_sustained"] = round(legs[key]["achieved"] / legs[key]["sustained_peak"], 4)

        # configs[0]: fp32 1024^3 built through the IR builder, lowered by frisk_ffi.runtime, launched through the C ABI
        import frisk_amd  # noqa: F401  (puts the builder package on the path)
        import frisk as F
        M1 = 1024
        h = F.create_session()
        kern = h.tiled_gemm("matmul", M1, M1, M1, "fp32", tile=(128, 128, 32), threads=256)
        A1 = torch.rand(M1, M1, device=dev, generator=g) * 2 - 1
        B1 = torch.rand(M1, M1, device=dev, generator=g) * 2 - 1
        C1 = torch.empty(M1, M1, device=dev)
        p1 = [A1.data_ptr(), B1.data_ptr(), C1.data_ptr()]
        t1 = time_launches(torch, lambda: F.runtime.launch(kern, p1, cs), a.steps, a.warmup, stream)
        legs["fp32_1024_builder"] = mfma_leg("fp32 1024^3 NN, U[-1,1], built with the IR builder (128x128x32 tiles as in the design sketch) and launched by "
                                             "frisk_ffi.runtime, which matches the program and lets the planner pick the kernel (configs[0]); the time "
                                             "includes that host work per launch", "f32", 2.0 * M1 ** 3, t1)
        d1 = R.make_desc(R.F32, M1, M1, M1)
        t1c = time_launches(torch, gemm_launcher(d1, (A1.data_ptr(), B1.data_ptr(), C1.data_ptr(), None, None)), a.steps, a.warmup, stream)
        legs["fp32_1024"] = mfma_leg("fp32 1024^3 NN through the C ABI, planner's choice of tile", "f32", 2.0 * M1 ** 3, t1c,
                                     {"kernel": R.kernel_names()[R.plan(d1).kernel_id]})
        C1v = torch.empty(M1, M1, device=dev)
        vendor["fp32_1024"] = vendor_leg(torch, "torch.matmul(A, B, out=C), fp32 1024^3 NN (allow_tf32 = %s)" % torch.backends.cuda.matmul.allow_tf32,
                                         lambda: torch.matmul(A1, B1, out=C1v), 2.0 * M1 ** 3, a.steps, a.warmup, stream, t1c["mean_ms"])

        # configs[2]: bf16 8192^3 NT; configs[4], square part: fp8 e4m3 8192^3 NT with per-tensor scales, bf16 out
        Mb = 8192
        big_steps = max(5, min(a.steps, 40))
        Ab = (torch.randn(Mb, Mb, device=dev, generator=g) * 0.02).bfloat16()
        Bb = (torch.randn(Mb, Mb, device=dev, generator=g) * 0.02).bfloat16()
        Cb = torch.empty(Mb, Mb, device=dev, dtype=torch.bfloat16)
        db = R.make_desc(R.BF16, Mb, Mb, Mb, dtype_out=R.BF16, transB=True)
        tb = time_launches(torch, gemm_launcher(db, (Ab.data_ptr(), Bb.data_ptr(), Cb.data_ptr(), None, None)), big_steps, 3, stream)
        legs["bf16_8192_nt"] = mfma_leg("bf16 8192^3 NT, N(0,1)*0.02, fp32 accumulate, bf16 out (configs[2])", "bf16", 2.0 * Mb ** 3, tb,
                                        {"kernel": R.kernel_names()[R.plan(db).kernel_id], "steps": big_steps,
                                         "sustained_peak": sustained_peak(ceiling, "bf16")})
        legs["bf16_8192_nt"]["frac_of_sustained"] = round(legs["bf16_8192_nt"]["achieved"] / legs["bf16_8192_nt"]["sustained_peak"], 4)
        Cbv = torch.empty(Mb, Mb, device=dev, dtype=torch.bfloat16)
        vendor["bf16_8192_nt"] = vendor_leg(torch, "torch.matmul(A, Bt.t(), out=C), bf16 8192^3 NT", lambda: torch.matmul(Ab, Bb.t(), out=Cbv), 2.0 * Mb ** 3, big_steps, 3,
                                            stream, tb["mean_ms"])
        ceiling["bf16 16x16x32, operands of the bf16 8192^3 workload"] = data_fed_ceiling(torch, HW, stream, cus, 3, "bf16", Ab, Bb)
        A8f = (torch.randn(Mb, Mb, device=dev, generator=g) * 100).clamp(-448, 448).to(torch.float8_e4m3fn)
        B8f = (torch.randn(Mb, Mb, device=dev, generator=g) * 100).clamp(-448, 448).to(torch.float8_e4m3fn)
        one = torch.full((1,), 0.01, device=dev)
        d8f = R.make_desc(R.E4M3, Mb, Mb, Mb, dtype_out=R.BF16, transB=True, epilogue=R.EPI_TENSOR_SCALE)
        t8f = time_launches(torch, gemm_launcher(d8f, (A8f.data_ptr(), B8f.data_ptr(), Cb.data_ptr(), one.data_ptr(), one.data_ptr())), big_steps, 3, stream)
        legs["fp8_8192_nt"] = mfma_leg("fp8 e4m3 8192^3 NT, N(0,1) scaled to the e4m3 range, per-tensor fp32 scales, bf16 out (configs[4], square part)",
                                       "e4m3", 2.0 * Mb ** 3, t8f, {"kernel": R.kernel_names()[R.plan(d8f).kernel_id], "steps": big_steps,
                                                                    "sustained_peak": sustained_peak(ceiling, "e4m3")})
        legs["fp8_8192_nt"]["frac_of_sustained"] = round(legs["fp8_8192_nt"]["achieved"] / legs["fp8_8192_nt"]["sustained_peak"], 4)
        vendor["fp8_8192_nt"] = vendor_leg(torch, "torch._scaled_mm(A, Bt.t(), scale_a, scale_b, out_dtype=bfloat16), e4m3 8192^3 NT",
                                           lambda: torch._scaled_mm(A8f, B8f.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16), 2.0 * Mb ** 3, big_steps, 3,
                                           stream, t8f["mean_ms"], "the vendor call allocates its output in every call (torch's caching allocator)")
        ceiling["f8f6f4 32x32x64, operands of the fp8 8192^3 workload"] = data_fed_ceiling(torch, HW, stream, cus, 6, "e4m3", A8f, B8f)
        ceiling["f8f6f4 16x16x128, operands of the fp8 8192^3 workload"] = data_fed_ceiling(torch, HW, stream, cus, 7, "e4m3", A8f, B8f)
        del Ab, Bb, Cb, Cbv, A8f, B8f

        # HBM-bound shape of the configuration list: fp8 e4m3 M=32, N=K=8192 (B stored [N][K]), per-tensor scales, bf16 out.
        # B rotates over 6 buffers (384 MiB > the 256 MiB last-level cache) so every launch streams it from HBM.
        Ms, Ns, Ks = 32, 8192, 8192
        Af = torch.randn(Ms, Ks, device=dev, generator=g).to(torch.float8_e4m3fn)
        Bf = [torch.randn(Ns, Ks, device=dev, generator=g).to(torch.float8_e4m3fn) for _ in range(6)]
        Cf = torch.empty(Ms, Ns, device=dev, dtype=torch.bfloat16)
        df = R.make_desc(R.E4M3, Ms, Ns, Ks, dtype_out=R.BF16, transB=True, epilogue=R.EPI_TENSOR_SCALE)
        pf = R.plan(df)
        ws_bytes = R.workspace_bytes(df)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        sk_turn = [0]

        def skinny():
            b_ = Bf[sk_turn[0] % len(Bf)]
            sk_turn[0] += 1
            R.gemm(df, Af.data_ptr(), b_.data_ptr(), Cf.data_ptr(), one.data_ptr(), one.data_ptr(), ws.data_ptr() if ws_bytes else None, ws_bytes, cs)
        tsk = time_launches(torch, skinny, a.steps, a.warmup, stream)
        sk_bytes = Ms * Ks + Ns * Ks + 2 * Ms * Ns + 8
        sk_gbs = sk_bytes / (tsk["mean_ms"] * 1e-3) / 1e9
        legs["fp8_skinny_32x8192x8192"] = {"bound": "hbm", "achieved": round(sk_gbs, 1), "peak": 8000.0, "unit": "GB/s", "frac": round(sk_gbs / 8000.0, 4),
                                           "kernel_ms": round(tsk["mean_ms"], 5), "kernel_ms_median": round(tsk["median_ms"], 5),
                                           "kernel_ms_min": round(tsk["min_ms"], 5), "kernel": R.kernel_names()[pf.kernel_id], "split_k": pf.split_k,
                                           "workload": "fp8 e4m3 M=32 N=K=8192 NT, per-tensor scales, bf16 out (configs[4], decode part); algorithmic bytes "
                                                       "|A|+|B|+|C|+scales per launch, B rotating over 6 buffers"}
        vk_turn = [0]

        def vendor_skinny():
            b_ = Bf[vk_turn[0] % len(Bf)]
            vk_turn[0] += 1
            return torch._scaled_mm(Af, b_.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
        vendor["fp8_skinny_32x8192x8192"] = vendor_leg(torch, "torch._scaled_mm(A, Bt.t(), ...), e4m3 32x8192x8192 NT, B rotating over the same 6 buffers", vendor_skinny,
                                                       float(sk_bytes) , a.steps, a.warmup, stream, tsk["mean_ms"], "rate in TB/s of algorithmic bytes")
        # what bounds this shape: the same kernel and grid with K shrunk to one K tile (the fixed cost of a launch: dispatch,
        # the first tile's trip from HBM, the epilogue) and with K doubled; the slope between K and 2K is the rate at which the
        # kernel streams B once it runs
        kernel_bk = pf.tile_k

        def skinny_at(k):
            a_ = torch.randn(Ms, k, device=dev, generator=g).to(torch.float8_e4m3fn)
            bs = [torch.randn(Ns, k, device=dev, generator=g).to(torch.float8_e4m3fn) for _ in range(max(2, (384 << 20) // (Ns * k)) if k >= Ks else 2)]
            dk = R.make_desc(R.E4M3, Ms, Ns, k, dtype_out=R.BF16, transB=True, epilogue=R.EPI_TENSOR_SCALE, tile=(pf.tile_m, pf.tile_n, kernel_bk),
                             stages=pf.stages_b, split_k=1)
            wk = R.workspace_bytes(dk)
            wsk = torch.empty(max(wk, 16), dtype=torch.uint8, device=dev)
            turn_k = [0]

            def fn():
                b_ = bs[turn_k[0] % len(bs)]
                turn_k[0] += 1
                R.gemm(dk, a_.data_ptr(), b_.data_ptr(), Cf.data_ptr(), one.data_ptr(), one.data_ptr(), wsk.data_ptr() if wk else None, wk, cs)
            return time_launches(torch, fn, a.steps, a.warmup, stream)["mean_ms"]
        floor_ms, double_ms = skinny_at(kernel_bk), skinny_at(2 * Ks)
        # what the platform charges for any launch: a kernel of the same grid (256 work-groups of 256 lanes) that issues 64 MFMAs on
        # registers and touches no memory
        empty_ms = time_launches(torch, lambda: HW.mfma_loop(0, 1, False, cus, cs), a.steps, a.warmup, stream)["mean_ms"]
        stream_gbs = (Ms + Ns) * Ks / ((double_ms - tsk["mean_ms"]) * 1e-3) / 1e9
        legs["fp8_skinny_32x8192x8192"].update({
            "launch_floor_ms": round(floor_ms, 5), "register_only_kernel_ms": round(empty_ms, 5), "kernel_ms_at_2K": round(double_ms, 5),
            "streaming_GBps": round(stream_gbs, 1),
            "frac_at_2K": round((Ms * 2 * Ks + Ns * 2 * Ks + 2 * Ms * Ns + 8) / (double_ms * 1e-3) / 8e12, 4),
            "kernel_ms_without_launch_gap": round(tsk["mean_ms"] - max(0.0, empty_ms - REGISTER_ONLY_KERNEL_TRACE_MS), 5),
            "frac_without_launch_gap": round(sk_bytes / ((tsk["mean_ms"] - max(0.0, empty_ms - REGISTER_ONLY_KERNEL_TRACE_MS)) * 1e-3) / 8e12, 4),
            "launch_gap_note": "kernel_ms is an event pair around back-to-back launches and so holds the gap between two launches; the gap is taken as "
                               "register_only_kernel_ms minus that kernel's own duration in a kernel trace (%.5f ms, a constant of the committed profile): "
                               "kernel_ms_without_launch_gap is the figure to hold against a rocprofv3 kernel duration" % REGISTER_ONLY_KERNEL_TRACE_MS,
            "bound_note": "launch_floor_ms is this kernel and grid with K of one K tile; register_only_kernel_ms a launch of the same grid that "
                          "touches no memory; streaming_GBps the slope between K=8192 and K=16384; kernel_ms is close to "
                          "launch_floor_ms + bytes / streaming rate"})
        del Bf

        # grids far below one round of tiles (a few hundred rows against an 8192 x 8192 fp16 B stored [N][K], rotating over 3 buffers of
        # 128 MiB): the planner's small-grid choice of a (variant, split-K) pair, beside the vendor library on the same tensors
        small = {}
        Bs = [(torch.randn(8192, 8192, device=dev, generator=g) / 64).half() for _ in range(3)]
        for Msm in (64, 256):
            Asm = (torch.randn(Msm, 8192, device=dev, generator=g) / 64).half()
            Csm = torch.empty(Msm, 8192, device=dev, dtype=torch.float16)
            Cvm = torch.empty_like(Csm)
            dsm = R.make_desc(R.F16, Msm, 8192, 8192, dtype_out=R.F16, transB=True)
            psm = R.plan(dsm)
            wsm_bytes = R.workspace_bytes(dsm)
            wsm = torch.empty(max(wsm_bytes, 16), dtype=torch.uint8, device=dev)
            turn = [0, 0]

            def ours_small():
                b_ = Bs[turn[0] % len(Bs)]
                turn[0] += 1
                R.gemm(dsm, Asm.data_ptr(), b_.data_ptr(), Csm.data_ptr(), None, None, wsm.data_ptr() if wsm_bytes else None, wsm_bytes, cs)

            def vendor_small():
                b_ = Bs[turn[1] % len(Bs)]
                turn[1] += 1
                return torch.matmul(Asm, b_.t(), out=Cvm)
            tsm = time_launches(torch, ours_small, a.steps, a.warmup, stream)
            sm_bytes = 2 * (Msm * 8192 + 8192 * 8192 + Msm * 8192)
            key = "%dx8192x8192" % Msm
            small[key] = {"kernel": R.kernel_names()[psm.kernel_id], "split_k": psm.split_k, "workspace_bytes": wsm_bytes,
                          "kernel_ms": round(tsm["mean_ms"], 5), "kernel_ms_median": round(tsm["median_ms"], 5), "kernel_ms_min": round(tsm["min_ms"], 5),
                          "algorithmic_GBps": round(sm_bytes / (tsm["mean_ms"] * 1e-3) / 1e9, 1),
                          "TFLOPs": round(2.0 * Msm * 8192 * 8192 / (tsm["mean_ms"] * 1e-3) / 1e12, 1)}
            vendor["fp16_small_grid_" + key + "_nt"] = vendor_leg(torch, "torch.matmul(A, Bt.t(), out=C), fp16 %s NT, B rotating over the same 3 buffers" % key,
                                                                  vendor_small, 2.0 * Msm * 8192 * 8192, a.steps, a.warmup, stream, tsm["mean_ms"])
            del Asm, Csm, Cvm, wsm
        legs["fp16_small_grid_nt"] = small
        del Bs

        # fp32 on grids that leave CUs idle (one 64x64 work-group keeps a CU's matrix pipe busy, so the planner splits K over the idle
        # CUs): 32 rows against a 4096 x 4096 B stored [K][N] rotating over 8 buffers of 64 MiB, and a 256 x 256 result with K = 8192
        # and B stored [N][K] (a kernel of its own in a trace: the [K][N] one is the 1024^3 leg's)
        small32 = {}
        for Msm, Nsm, Ksm, tBsm, nbuf in ((32, 4096, 4096, False, 8), (256, 256, 8192, True, 4)):
            Bs = [torch.randn((Nsm, Ksm) if tBsm else (Ksm, Nsm), device=dev, generator=g) / 64 for _ in range(nbuf)]
            Asm = torch.randn(Msm, Ksm, device=dev, generator=g) / 64
            Csm = torch.empty(Msm, Nsm, device=dev)
            Cvm = torch.empty_like(Csm)
            dsm = R.make_desc(R.F32, Msm, Nsm, Ksm, dtype_out=R.F32, transB=tBsm)
            psm = R.plan(dsm)
            wsm_bytes = R.workspace_bytes(dsm)
            wsm = torch.empty(max(wsm_bytes, 16), dtype=torch.uint8, device=dev)
            turn = [0, 0]

            def ours_small32():
                b_ = Bs[turn[0] % len(Bs)]
                turn[0] += 1
                R.gemm(dsm, Asm.data_ptr(), b_.data_ptr(), Csm.data_ptr(), None, None, wsm.data_ptr() if wsm_bytes else None, wsm_bytes, cs)

            def vendor_small32():
                b_ = Bs[turn[1] % len(Bs)]
                turn[1] += 1
                return torch.matmul(Asm, b_.t() if tBsm else b_, out=Cvm)
            tsm = time_launches(torch, ours_small32, a.steps, a.warmup, stream)
            key = "%dx%dx%d_%s" % (Msm, Nsm, Ksm, "nt" if tBsm else "nn")
            small32[key] = {"kernel": R.kernel_names()[psm.kernel_id], "split_k": psm.split_k, "workspace_bytes": wsm_bytes,
                            "kernel_ms": round(tsm["mean_ms"], 5), "kernel_ms_median": round(tsm["median_ms"], 5), "kernel_ms_min": round(tsm["min_ms"], 5),
                            "algorithmic_GBps": round(4 * (Msm * Ksm + Ksm * Nsm + Msm * Nsm) / (tsm["mean_ms"] * 1e-3) / 1e9, 1),
                            "TFLOPs": round(2.0 * Msm * Nsm * Ksm / (tsm["mean_ms"] * 1e-3) / 1e12, 1)}
            vendor["fp32_small_grid_" + key] = vendor_leg(torch, "torch.matmul, fp32 %s, B rotating over the same %d buffers" % (key, nbuf),
                                                          vendor_small32, 2.0 * Msm * Nsm * Ksm, a.steps, a.warmup, stream, tsm["mean_ms"])
            del Asm, Csm, Cvm, wsm, Bs
        legs["fp32_small_grid"] = small32

        # shapes off the tiles, fp16 NN: M off every tile (edge variant of the 256x256 kernel), 48 rows against a large B rotating over
        # 3 buffers (edge variant of a skinny split-K kernel), K off the K tile (the guarded kernel that stages whole 16-byte chunks)
        ragged = {}
        for Mr, Nr, Kr, nbuf in ((4000, 4096, 4096, 1), (48, 8192, 8192, 3), (4096, 4096, 4000, 1)):
            Bs = [(torch.randn(Kr, Nr, device=dev, generator=g) / 64).half() for _ in range(nbuf)]
            Ar = (torch.randn(Mr, Kr, device=dev, generator=g) / 64).half()
            Cr = torch.empty(Mr, Nr, device=dev, dtype=torch.float16)
            Cvr = torch.empty_like(Cr)
            dr = R.make_desc(R.F16, Mr, Nr, Kr, dtype_out=R.F16)
            pr = R.plan(dr)
            wr_bytes = R.workspace_bytes(dr)
            wr = torch.empty(max(wr_bytes, 16), dtype=torch.uint8, device=dev)
            turn = [0, 0]

            def ours_ragged():
                b_ = Bs[turn[0] % len(Bs)]
                turn[0] += 1
                R.gemm(dr, Ar.data_ptr(), b_.data_ptr(), Cr.data_ptr(), None, None, wr.data_ptr() if wr_bytes else None, wr_bytes, cs)

            def vendor_ragged():
                b_ = Bs[turn[1] % len(Bs)]
                turn[1] += 1
                return torch.matmul(Ar, b_, out=Cvr)
            trg = time_launches(torch, ours_ragged, a.steps, a.warmup, stream)
            key = "%dx%dx%d" % (Mr, Nr, Kr)
            ragged[key] = {"kernel": R.kernel_names()[pr.kernel_id], "split_k": pr.split_k, "kernel_ms": round(trg["mean_ms"], 5),
                           "kernel_ms_median": round(trg["median_ms"], 5), "kernel_ms_min": round(trg["min_ms"], 5),
                           "TFLOPs": round(2.0 * Mr * Nr * Kr / (trg["mean_ms"] * 1e-3) / 1e12, 1)}
            vendor["fp16_ragged_" + key + "_nn"] = vendor_leg(torch, "torch.matmul(A, B, out=C), fp16 %s NN" % key, vendor_ragged, 2.0 * Mr * Nr * Kr,
                                                              a.steps, a.warmup, stream, trg["mean_ms"])
            del Ar, Cr, Cvr, wr, Bs
        legs["fp16_ragged_nn"] = ragged

        # the dialect's data-movement ops on a 32768 x 8192 f16 view (512 MiB per array: twice the last-level cache)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

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
        # a free-standing frisk.block body through the interpreter: y = log2(max(x, c) / (x + c)), one read and one write per element
        prog = [("input", 0), ("const", 0.5), "max", ("input", 0), ("const", 0.5), "add", "div", "log2"]
        ew = R.make_elementwise_desc(prog, [(R.F16, ocols, 1)], R.F16, orows, ocols)
        src16.abs_().add_(0.01)
        ms = time_op(lambda: R.elementwise(ew, [src16.data_ptr()], dst16.data_ptr(), cs))
        ops["block_body_log2_max_div"] = {"GB/s": round(2 * nbytes / (ms * 1e-3) / 1e9, 1), "frac_of_8TB/s": round(2 * nbytes / (ms * 1e-3) / 8e12, 4), "kernel_ms": round(ms, 5),
                                          "program": "x0 c0.5 max x0 c0.5 add div log2 (8 steps, interpreted per 8 elements)"}
        # tiles placed transposed: 64 x 64 tiles of the 8192 x 8192 head of the view, block (a, b) -> block (b, a)
        tb = 8192 // 64
        ms = time_op(lambda: R.copy_tiles(R.F16, src16.data_ptr(), ocols, R.F16, dst16.data_ptr(), ocols, 64, 64, tb, 64 * ocols, 64, tb, 64, 64 * ocols, cs))
        moved = 2 * 8192 * 8192 * 2
        ops["copy_tiles_transposed_8192x8192"] = {"GB/s": round(moved / (ms * 1e-3) / 1e9, 1), "frac_of_8TB/s": round(moved / (ms * 1e-3) / 8e12, 4), "kernel_ms": round(ms, 5)}
        del src16, dst16
        line["tile_ops_32768x8192_f16"] = ops

        # fused attention forward at the shape of the reference's sketch: 1 x 32 heads x 4096 x 128, fp16
        ab, ah, aseq, ad = 1, 32, 4096, 128
        aq, ak, av = (torch.randn(ab * ah, aseq, ad, device=dev, generator=g).half() for _ in range(3))
        ao = torch.empty_like(aq)
        adesc = R.make_attention_desc(R.F16, ab, ah, aseq, aseq, ad)
        attn_ms = time_op(lambda: R.attention(adesc, aq.data_ptr(), ak.data_ptr(), av.data_ptr(), ao.data_ptr(), None, cs))
        attn_tflops = 4.0 * ab * ah * aseq * aseq * ad / (attn_ms * 1e-3) / 1e12
        del aq, ak, av, ao
        line["attention_1x32x4096x128_f16"] = {"bound": "mfma", "achieved": round(attn_tflops, 2), "peak": PEAK_TFLOPS["f16"], "unit": "TFLOP/s",
                                               "frac": round(attn_tflops / PEAK_TFLOPS["f16"], 4), "frac_of_sustained": round(attn_tflops / sp, 4),
                                               "kernel_ms": round(attn_ms, 5),
                                               "workload": "softmax(Q K^T / sqrt(128)) V, 32 heads, 4096 queries x 4096 keys, head_dim 128, "
                                                           "fp16 in / out, fp32 accumulate; 4 * heads * seq^2 * head_dim flops per launch"}

    for key, v in vendor.items():
        leg = line["roofline"] if key == "fp16_4096_nn" else legs.get(key)
        if leg is not None and "vs_vendor" in v:
            leg["vs_vendor"] = v["vs_vendor"]
            leg["vendor_kernel_ms"] = v["kernel_ms"]
    if vendor:
        line["vendor_same_run"] = {"what": "torch %s -> hipBLASLt / rocBLAS on the same device tensors, same settle and HIP-event protocol; vs_vendor = vendor "
                                           "time / this build's time (above 1: this build is faster); an external comparator, never the product path" % torch.__version__,
                                   **vendor}
    line.update(legs)
    if not a.no_cpu and not a.only_headline:
        line["cpu_baseline"] = cpu_baseline(M, N, K)
        line["cpu_baseline_int8"] = cpu_baseline_int8(M, N, K)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
