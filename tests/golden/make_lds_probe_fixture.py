#!/usr/bin/env python3
"""Writes tests/golden/lds_probe_gfx950.json: lane-address patterns and the LDS cycles per
wave-wide instruction measured for them on an MI355X (16 waves of one work-group issuing the
same access in a loop, time per instruction converted to cycles with the all-conflict case as the
clock reference).  The measured numbers are copied from the output of a stand-alone micro-benchmark run on the
device (not kept in the tree); the patterns are regenerated here from their definitions.
"""
import json
import os

B128, B64, B32 = 0, 1, 3
cases = []


def add(name, instr, addrs, measured):
    assert len(addrs) == 64
    cases.append({"name": name, "instr": instr, "addr": [int(a) for a in addrs], "measured_cycles": measured})


lin = lambda s: [l * s for l in range(64)]
# ds_read_b128
add("b128 linear", B128, lin(16), 4.13)
add("b128 broadcast", B128, [0] * 64, 4.12)
add("b128 stride 32", B128, lin(32), 8.06)
add("b128 stride 64", B128, lin(64), 16.07)
add("b128 stride 128", B128, lin(128), 32.1)
add("b128 stride 256", B128, lin(256), 64.2)
for D, cyc in ((1, 7.98), (2, 8.02), (4, 4.12), (8, 4.11), (16, 4.10), (32, 4.10)):
    a = []
    for l in range(64):
        lo, hi = l & (D - 1), (l >> 1) & ~(D - 1)
        slot, bit = hi | lo, (l // D) & 1
        a.append((slot % 16) * 16 + (slot // 16) * 256 + bit * 512)
    add("b128 pair D=%d" % D, B128, a, cyc)
for sw, cyc in ((0, 32.12), (1, 8.04), (2, 4.10), (3, 8.05)):
    a = []
    for l in range(64):
        row, c = l % 32, l // 32
        f = [0, row & 7, (row >> 1) & 7, (row >> 2) & 7][sw]
        a.append(row * 128 + ((c ^ f) * 16))
    add("b128 fragment rows of 128 B, swizzle %d" % sw, B128, a, cyc)
add("b128 fragment rows padded to 144 B", B128, [(l % 32) * 144 + (l // 32) * 16 for l in range(64)], 4.12)
# ds_read_b64_tr_b16: B operand of a 32x32x16 MFMA from a tile with 512-byte rows
for sw, cyc in ((0, 8.09), (1, 3.11), (2, 4.11), (3, 4.11), (4, 2.90)):
    a = []
    for l in range(64):
        b, L = l // 16, l % 16
        row, colb = 8 * (b // 2) + L // 4, 32 * (b % 2) + 8 * (L % 4)
        c, w = colb // 16, colb % 16
        x = [0, (row & 3) << 2, (row & 7) << 1, (row & 3) << 1, (row & 7) << 2][sw]
        a.append(row * 512 + ((c ^ x) * 16) + w)
    add("tr16 fragment rows of 512 B, swizzle %d" % sw, B64, a, cyc)
# ds_read_b64_tr_b8: rows of 256 bytes
for sw, cyc in ((0, 16.06), (1, 3.11), (2, 4.11), (3, 4.11)):
    a = []
    for l in range(64):
        b, L = l // 16, l % 16
        row, colb = 16 * (b // 2) + L // 2, 16 * (b % 2) + 8 * (L % 2)
        c, w = colb // 16, colb % 16
        x = [0, (row & 7) << 1, row & 15, (row & 3) << 2][sw]
        a.append(row * 256 + ((c ^ x) * 16) + w)
    add("tr8 fragment rows of 256 B, swizzle %d" % sw, B64, a, cyc)
# ds_read_b64 / ds_read_b32 strides
for s, cyc in ((8, 2.92), (16, 4.12), (32, 8.10), (64, 16.04), (128, 32.1), (256, 64.1)):
    add("b64 stride %d" % s, B64, lin(s), cyc)
for s, cyc in ((4, 3.03), (8, 4.05), (16, 7.98), (32, 15.8), (64, 31.6), (128, 63.7)):
    add("b32 stride %d" % s, B32, lin(s), cyc)

out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lds_probe_gfx950.json")
with open(out, "w") as f:
    json.dump({"device": "MI355X gfx950", "clock_reference": "stride-256 ds_read_b32 = 64 cycles", "cases": cases}, f, indent=0)
print("wrote", out, len(cases), "cases")
