#!/usr/bin/env python3
"""Collects the layout strings and bank statistics the reference holds for its GEMM layout inference into one JSON
fixture (tests/golden/nvidia_gemm_layouts.json).

Sources (text logs checked into the reference, read as data):
  tmp/log_12_18                 output of frisk_attr_test: 6 cases sm80/sm90 x {shared,local} operands, 128x128x64 f16
  exp/layout/result/log_12_23   JSON of frisk_layout_tool: sm_80, 128x128x64 f16, lane_vector 8, with bank statistics
  exp/layout/result/log         text of analyze_bank_conflicts.py: sm_80, 256x128x64 f16, lane vector 4

Run once where the reference tree is present:  python tests/golden/make_nvidia_layout_fixture.py /root/reference
"""
import json
import os
import re
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
out = {"cases": [], "bank_stats": []}

# ---- tmp/log_12_18
text = open(os.path.join(ref, "tmp/log_12_18")).read()
case_re = re.compile(r"Case '(\w+)' \(target=(\w+), A=(\w+), B=(\w+)\)(.*?)(?=\n-{20,}|\n={20,})", re.S)
for name, target, a_space, b_space, body in case_re.findall(text):
    g = re.search(r"frisk\.gemm.*?\{K = (\d+) : i64, M = (\d+) : i64, N = (\d+) : i64, clear_accum = \w+, frisk\.threads = (\d+) : i64, "
                  r"policy = #frisk<gemm_warp_policy (\w+)>, transA = (\w+), transB = (\w+)\}", body)
    K, M, N, threads = (int(g.group(i)) for i in (1, 2, 3, 4))
    case = {"name": name, "source": "tmp/log_12_18", "target": target, "M": M, "N": N, "K": K, "threads": threads, "policy": g.group(5),
            "transA": g.group(6) == "true", "transB": g.group(7) == "true", "element_bits": 16,
            "spaces": {"A": a_space, "B": b_space, "C": "local"}, "layouts": {}}
    for op, kind, shape, rest in re.findall(r"^([ABC]) layout: (Layout|Fragment)\(shape=\[([\d, ]+)\], (.*)\)$", body, re.M):
        lay = {"kind": kind, "shape": [int(x) for x in shape.split(",")]}
        lay["index"] = re.search(r"index=(affine_map<.*?>)(?:, thread=|$)", rest).group(1)
        t = re.search(r"thread=(affine_map<.*?>), replicate=(\d+)", rest)
        if t:
            lay["thread"], lay["replicate"] = t.group(1), int(t.group(2))
        case["layouts"][op] = lay
    out["cases"].append(case)

# ---- exp/layout/result/log_12_23 (JSON)
j = json.load(open(os.path.join(ref, "exp/layout/result/log_12_23")))
cfg = j["config"]
case = {"name": "layout_tool_sm80_128", "source": "exp/layout/result/log_12_23", "target": cfg["target"], "M": cfg["block_shape"]["M"],
        "N": cfg["block_shape"]["N"], "K": cfg["block_shape"]["K"], "threads": cfg["threads"], "policy": "Square", "transA": False,
        "transB": False, "element_bits": 16, "spaces": {k: v.lower() for k, v in cfg["memory_spaces"].items()}, "layouts": {}}
for lay in j["layouts"]:
    op = lay.get("operand")
    if not op or "forward_index" not in lay:
        continue
    e = {"kind": "Fragment" if "forward_thread" in lay else "Layout", "shape": lay["shape"], "index": lay["forward_index"]}
    if "forward_thread" in lay:
        e["thread"], e["replicate"] = lay["forward_thread"], lay["replicate"]
    case["layouts"][op] = e
    if "bank_stats" in lay:
        out["bank_stats"].append({"source": "exp/layout/result/log_12_23", "operand": op, "shape": lay["shape"], "element_bits": lay["element_bits"],
                                  "lane_vector": cfg["lane_vector"], "index": lay["forward_index"],
                                  "layout": {"avg_max": lay["bank_stats"]["avg_max_conflict"], "max": lay["bank_stats"]["max_conflict"],
                                             "samples": lay["bank_stats"]["samples"]},
                                  "row_major": {"avg_max": lay["baseline_row_major"]["avg_max_conflict"],
                                                "max": lay["baseline_row_major"]["max_conflict"], "samples": lay["baseline_row_major"]["samples"]}})
out["cases"].append(case)

# ---- exp/layout/result/log (text)
text = open(os.path.join(ref, "exp/layout/result/log")).read()
m = re.search(r"shape\s*: M=(\d+) N=(\d+) K=(\d+)", text)
M, N, K = (int(x) for x in m.groups())
lane_vector = int(re.search(r"lane vector : (\d+)", text).group(1))
case = {"name": "bank_script_sm80_256", "source": "exp/layout/result/log", "target": re.search(r"target\s*: (\w+)", text).group(1), "M": M, "N": N, "K": K,
        "threads": int(re.search(r"threads\s*: (\d+)", text).group(1)), "policy": "Square", "transA": False, "transB": False, "element_bits": 16,
        "spaces": {"A": "shared", "B": "shared", "C": "local"}, "layouts": {}}
for block in text.split("Operand ")[1:]:
    op = block[0]
    idx = re.search(r"layout index\s+: (affine_map<.*?>)\n", block).group(1)
    shape = {"A": [M, K], "B": [K, N], "C": [M, N]}[op]
    case["layouts"][op] = {"kind": "Layout", "shape": shape, "index": idx}
    b = re.search(r"bank stats\s+: avg_max=([\d.]+)\s+max=(\d+)", block)
    r = re.search(r"baseline \(torch\) : avg_max=([\d.]+)\s+max=(\d+)", block)
    if b:
        out["bank_stats"].append({"source": "exp/layout/result/log", "operand": op, "shape": shape, "element_bits": 16, "lane_vector": lane_vector,
                                  "index": idx, "layout": {"avg_max": float(b.group(1)), "max": int(b.group(2))},
                                  "row_major": {"avg_max": float(r.group(1)), "max": int(r.group(2))}})
out["cases"].append(case)

dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "nvidia_gemm_layouts.json")
json.dump(out, open(dst, "w"), indent=1)
print("wrote", dst, ":", len(out["cases"]), "cases,", len(out["bank_stats"]), "bank statistics")
