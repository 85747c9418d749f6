#!/usr/bin/env python3
"""GEMM tile layouts for gfx950 as JSON: the counterpart of the reference's `frisk_layout_tool`
(exp/layout/gemm_layout_tool.cpp: flags :330-372, JSON schema :272-326, 453-497) and of the summary printed by
exp/layout/analyze_bank_conflicts.py:59-109, with the gfx950 LDS model in place of the 32-bank histogram.

    python -m frisk_amd.layout_tool --block-m 256 --block-n 256 --block-k 64 --dtype fp16 [--trans-b] [--summary]

Same keys as the reference's output.  `bank_stats` of a shared operand holds the conflict degree of the kernel's own
fragment reads under the chosen swizzle (modelled LDS cycles of a wave-wide read / cycles of a conflict-free read;
1.0 = conflict free) and `baseline_row_major` the same without a swizzle; `cycles_per_access` and `read_instruction`
say what was modelled.  Pure host code: needs libfrisk_hip.so and the frisk_ffi extension, no GPU.
"""
import argparse
import json
import math
import sys

DTYPES = {"fp16": (2, 16), "bf16": (2, 16), "fp32": (4, 4), "int8": (1, 16), "fp8": (1, 32)}   # element bytes, bytes per lane per MFMA
READ_INSTR = {0: ("ds_read_b128", 4.0), 1: ("ds_read_b64_tr_b16", 3.0), 2: ("ds_read_b64_tr_b8", 3.0), 3: ("ds_read_b32", 2.0)}   # name, measured cycles of a conflict-free wave-wide read


def operand_entry(R, ffi_runtime, label, rows, cols, k_contiguous, es, frag, tile_mn, tile_k, waves):
    best, unswizzled = R.lds_search(rows, cols * es, int(k_contiguous), es, frag, tile_mn, tile_k, waves)
    name, ideal = READ_INSTR[best.read_instr]

    def stats(cycles):
        degree = max(1.0, cycles / ideal)
        return {"avg_max_conflict": round(degree, 3), "max_conflict": int(math.ceil(degree - 1e-9)), "samples": 64,
                "cycles_per_access": round(cycles, 3), "read_instruction": name}
    text = ffi_runtime.lds_layout_string(rows, cols * es, es, best.row_shift, best.row_mask, best.chunk_shift,
                                         best.row_shift2, best.row_mask2, best.chunk_shift2)
    return {"operand": label, "shape": [rows, cols], "element_bits": es * 8, "memory_space": "Shared",
            "forward_index": text[text.index("index=") + 6:-1], "swizzle": {"row_shift": best.row_shift, "row_mask": best.row_mask, "chunk_shift": best.chunk_shift,
                        "row_shift2": best.row_shift2, "row_mask2": best.row_mask2, "chunk_shift2": best.chunk_shift2},
            "bank_stats": stats(best.read_cycles), "baseline_row_major": stats(unswizzled)}


def report(args):
    import frisk_amd  # noqa: F401
    import frisk as F
    from frisk_amd import runtime as R
    if not args.target.startswith("gfx950"):
        raise SystemExit("layout inference here supports gfx950 only (the reference's supports sm_80 ... sm_90)")
    if args.dtype not in DTYPES:
        raise SystemExit("unsupported dtype %r (%s)" % (args.dtype, ", ".join(DTYPES)))
    for label, space, want in (("A", args.a_space, "shared"), ("B", args.b_space, "shared"), ("C", args.c_space, "local")):
        if space.lower() != want:
            raise SystemExit("operand %s must reside in %s memory on gfx950 (MFMA operands are staged through LDS, accumulators live in registers)" % (label, want))
    es, frag = DTYPES[args.dtype]
    bm, bn, bk = args.block_m, args.block_n, args.block_k
    waves = max(1, args.threads // 64)
    wm, wn = R.wave_partition(R.POLICY_SQUARE, bm, bn, waves)
    a_shape = (bk, bm) if args.trans_a else (bm, bk)        # as stored: [K][M] when transposed
    b_shape = (bn, bk) if args.trans_b else (bk, bn)        # as stored: [N][K] when transposed
    lane_vector = max(4 if args.ldmatrix else 1, args.lane_vector)
    acc = F.runtime.accumulator_layout_string(bm, bn, wm, wn)
    idx = acc[acc.index("index=") + 6:acc.index(", thread=")]
    thr = acc[acc.index("thread=") + 7:acc.index(", replicate=")]
    return {
        "config": {"target": args.target, "dtype": args.dtype, "threads": args.threads, "block_shape": {"M": bm, "N": bn, "K": bk},
                   "grid": list(args.grid) if args.grid else [1, 1], "memory_spaces": {"A": "Shared", "B": "Shared", "C": "Local"},
                   "lane_vector": lane_vector, "ldmatrix_like": bool(args.ldmatrix), "wave_partition": [wm, wn]},
        "layouts": [
            operand_entry(R, F.runtime, "A", a_shape[0], a_shape[1], not args.trans_a, es, frag, bm, bk, waves),
            operand_entry(R, F.runtime, "B", b_shape[0], b_shape[1], args.trans_b, es, frag, bn, bk, waves),
            {"operand": "C", "shape": [bm, bn], "element_bits": 32, "memory_space": "Local", "forward_index": idx, "forward_thread": thr, "replicate": 1},
        ],
    }


def print_summary(result, out=sys.stdout):
    """the text form of exp/layout/analyze_bank_conflicts.py:59-109"""
    c = result["config"]
    b = c["block_shape"]
    print("== Config ==", file=out)
    print("target      : %s" % c["target"], file=out)
    print("shape       : M=%d N=%d K=%d" % (b["M"], b["N"], b["K"]), file=out)
    print("dtype       : %s" % c["dtype"], file=out)
    print("threads     : %d" % c["threads"], file=out)
    print("lane vector : %d%s" % (c["lane_vector"], " (ldmatrix)" if c["ldmatrix_like"] else ""), file=out)
    print("grid        : %s" % list(c["grid"]), file=out)
    print("spaces      : " + ", ".join("%s=%s" % kv for kv in c["memory_spaces"].items()), file=out)
    print(file=out)
    for e in result["layouts"]:
        print("Operand %s (%s):" % (e["operand"], e["memory_space"]), file=out)
        print("  layout index     : %s" % e.get("forward_index", "<none>"), file=out)
        if "bank_stats" in e:
            print("  bank stats       : avg_max=%.2f  max=%d" % (e["bank_stats"]["avg_max_conflict"], e["bank_stats"]["max_conflict"]), file=out)
            print("  baseline (torch) : avg_max=%.2f  max=%d" % (e["baseline_row_major"]["avg_max_conflict"], e["baseline_row_major"]["max_conflict"]), file=out)
        print(file=out)


def parser():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--target", default="gfx950")
    ap.add_argument("--block-m", type=int, default=256)
    ap.add_argument("--block-n", type=int, default=256)
    ap.add_argument("--block-k", type=int, default=64)
    ap.add_argument("--dtype", default="fp16")
    ap.add_argument("--a-space", default="shared")
    ap.add_argument("--b-space", default="shared")
    ap.add_argument("--c-space", default="local")
    ap.add_argument("--threads", type=int, default=256)
    ap.add_argument("--grid", type=lambda s: [int(x) for x in s.split(",")], default=None, help="comma separated")
    ap.add_argument("--trans-a", action="store_true")
    ap.add_argument("--trans-b", action="store_true")
    ap.add_argument("--lane-vector", type=int, default=1)
    ap.add_argument("--ldmatrix", action="store_true")
    ap.add_argument("--summary", action="store_true", help="print the text summary instead of JSON")
    return ap


def main(argv=None):
    args = parser().parse_args(argv)
    result = report(args)
    if args.summary:
        print_summary(result)
    else:
        print(json.dumps(result, indent=2, sort_keys=True))
    return 0


if __name__ == "__main__":
    sys.exit(main())
