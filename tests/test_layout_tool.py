"""`python -m frisk_amd.layout_tool`: the gfx950 counterpart of the reference's frisk_layout_tool.  The JSON carries every key of
the reference's schema (exp/layout/gemm_layout_tool.cpp:272-326, 453-497; sample exp/layout/result/log_12_23); the printed maps
are checked by evaluating them: LDS index maps against frisk_hip_lds_offset, the accumulator fragment as a bijection."""
import io
import json
import subprocess
import sys

import numpy as np
import pytest

from frisk_amd import layout_tool as T
from frisk_amd import runtime as R
from oracle import layouts as L

CONFIG_KEYS = {"block_shape", "dtype", "grid", "lane_vector", "ldmatrix_like", "memory_spaces", "target", "threads"}
SHARED_KEYS = {"bank_stats", "baseline_row_major", "element_bits", "forward_index", "memory_space", "operand", "shape"}
STAT_KEYS = {"avg_max_conflict", "max_conflict", "samples"}


def run(*argv):
    return T.report(T.parser().parse_args(list(argv)))


@pytest.mark.parametrize("argv", [(), ("--trans-b",), ("--dtype", "bf16", "--trans-a"), ("--dtype", "int8", "--block-k", "128"),
                                  ("--dtype", "fp8", "--block-k", "128", "--trans-b"), ("--dtype", "fp32", "--block-m", "128", "--block-n", "128", "--block-k", "32"),
                                  ("--block-m", "128", "--block-n", "128", "--threads", "512")])
def test_report_has_the_reference_schema_and_consistent_maps(argv):
    r = run(*argv)
    assert CONFIG_KEYS <= set(r["config"]) and set(r["config"]["block_shape"]) == {"M", "N", "K"} and set(r["config"]["memory_spaces"]) == {"A", "B", "C"}
    a, b, c = r["layouts"]
    assert [e["operand"] for e in (a, b, c)] == ["A", "B", "C"]
    es = a["element_bits"] // 8
    for e in (a, b):
        assert SHARED_KEYS <= set(e) and STAT_KEYS <= set(e["bank_stats"]) and STAT_KEYS <= set(e["baseline_row_major"]) and e["memory_space"] == "Shared"
        assert e["bank_stats"]["avg_max_conflict"] <= e["baseline_row_major"]["avg_max_conflict"]   # the chosen swizzle never loses to none
        rows, cols = e["shape"]
        i, j = L.grid(rows, cols)
        (idx,) = L.eval_affine_map(e["forward_index"], i, j)
        sw = e["swizzle"]
        lay = R.LdsLayout(rows=rows, row_bytes=cols * es, k_contiguous=1, row_shift=sw["row_shift"], row_mask=sw["row_mask"], chunk_shift=sw["chunk_shift"],
                          row_shift2=sw["row_shift2"], row_mask2=sw["row_mask2"], chunk_shift2=sw["chunk_shift2"])
        for rr, cc in zip(np.random.default_rng(2).integers(0, rows, 200), np.random.default_rng(3).integers(0, cols, 200)):
            assert R.lds_offset(lay, int(rr), int(cc) * es) == int(idx[rr, cc]) * es
        assert len(np.unique(idx)) == rows * cols
    # accumulators: (thread, register) is a bijection onto threads x registers
    assert {"forward_index", "forward_thread", "replicate", "shape"} <= set(c) and c["replicate"] == 1 and c["memory_space"] == "Local"
    bm, bn = c["shape"]
    i, j = L.grid(bm, bn)
    (reg,) = L.eval_affine_map(c["forward_index"], i, j)
    (thr,) = L.eval_affine_map(c["forward_thread"], i, j)
    threads = r["config"]["threads"]
    assert thr.min() == 0 and thr.max() == threads - 1 and reg.min() == 0 and reg.max() == bm * bn // threads - 1
    assert len(np.unique(thr * (reg.max() + 1) + reg)) == bm * bn


def test_fp16_default_tile_is_conflict_free_and_row_major_is_not():
    a, b, _ = run()["layouts"]
    assert a["bank_stats"]["avg_max_conflict"] == 1.0 and a["baseline_row_major"]["avg_max_conflict"] == 8.0
    assert a["bank_stats"]["read_instruction"] == "ds_read_b128" and b["bank_stats"]["read_instruction"] == "ds_read_b64_tr_b16"


def test_summary_and_command_line():
    out = io.StringIO()
    T.print_summary(run("--trans-b"), out)
    text = out.getvalue()
    assert text.startswith("== Config ==\ntarget      : gfx950\nshape       : M=256 N=256 K=64\n") and "Operand A (Shared):" in text and "bank stats       : avg_max=1.00  max=1" in text
    p = subprocess.run([sys.executable, "-m", "frisk_amd.layout_tool", "--dtype", "int8", "--block-k", "128"], capture_output=True, text=True, check=True)
    assert json.loads(p.stdout)["config"]["dtype"] == "int8"
    p = subprocess.run([sys.executable, "-m", "frisk_amd.layout_tool", "--target", "sm_80"], capture_output=True, text=True)
    assert p.returncode != 0 and "gfx950 only" in p.stderr
