#!/usr/bin/env python3
"""Writes the per-dtype kernel translation units (kernels_<dtype>.hip).

Each unit explicitly instantiates the GEMM kernel template for a list of
(transA, transB, BM, BN, BK, WM, WN, stages, guard, split-K) variants and exports a table of them.
Run from this directory after editing VARIANTS; the generated files are
committed so a build needs only hipcc.
"""
import os

def full(v):
    """(…, WK) -> (…, WK, stages of B, atom, edge): B has as many stages as A, the atom is 32x32 and the kernel wants whole tiles
    unless the variant says otherwise"""
    v = tuple(v)
    if len(v) == 11:
        v += (v[7],)
    if len(v) == 12:
        v += (32,)
    return v if len(v) == 14 else v + (0,)


def edge(v):
    """the variant once more for M and N that are not multiples of the tile"""
    return full(v)[:13] + (1,)


# a variant: (transA, transB, BM, BN, BK, WM, WN, stages of A, guard, split-K, WK, stages of B[, MFMA atom])
# atom16: the default 256x256 variant (and its split-K copy) exists once more built from 16x16 atoms of twice the K depth: the
# part holds a higher clock on them (fp16 4096^3 NT 100 against 112 us, NN 104 against 108; int8 gains nothing).  Listed first;
# the planner prefers the 32x32 atoms where the clock is not the limit (grids below one round with a transpose-read operand)
def square(bk, atom16=False, skinny_ta=(0,)):
    out = []
    # The first variant of a tile size is the planner's default.  256x256: 4 waves of 128x128 (fewest LDS reads per MFMA)
    # with 2 LDS tiles of A and 3 of B (160 KiB), B fetched two tiles ahead and spread over the K tile; then the same
    # with 2 + 2 tiles, then 8 waves of 128x64.
    # 256x128 / 128x256 (3 + 3 tiles, 144 KiB) for problems with one short side; 128x128 with 2 + 2 tiles (two work-groups
    # per CU) for many tiles and 3 + 3 (96 KiB) when the grid is a single wave.
    for bm, bn, k, wm, wn, st, sb in ((256, 256, bk, 2, 2, 2, 3), (256, 256, bk, 2, 2, 2, 2), (256, 256, bk, 2, 4, 2, 2), (256, 128, bk, 2, 2, 3, 3),
                                      (128, 256, bk, 2, 2, 3, 3), (128, 128, bk, 2, 2, 2, 2), (128, 128, bk, 2, 2, 3, 3)):
        for ta in (0, 1):
            for tb in (0, 1):
                if atom16 and (bm, bn, wm, wn, st, sb) == (256, 256, 2, 2, 2, 3):
                    out.append((ta, tb, bm, bn, k, wm, wn, st, 0, 0, 1, sb, 16))
                out.append((ta, tb, bm, bn, k, wm, wn, st, 0, 0, 1, sb))
    # the default 256x256 variant once more with the split-K store path: for grids a little over a whole number of rounds
    # of 256 tiles, whose last tiles are then split along K over several work-groups (a tail split)
    for ta in (0, 1):
        for tb in (0, 1):
            if atom16:
                out.append((ta, tb, 256, 256, bk, 2, 2, 2, 0, 1, 1, 3, 16))
            out.append((ta, tb, 256, 256, bk, 2, 2, 2, 0, 1, 1, 3))
    # the 128x128 variant with 3 + 3 tiles once more with the split-K store path: grids of well under 256 tiles with a long K
    # (M of a few hundred rows), where K is split over the idle CUs
    for ta in (0, 1):
        for tb in (0, 1):
            out.append((ta, tb, 128, 128, bk, 2, 2, 3, 0, 1, 1, 3))
    # skinny variants (M a multiple of 32), bound by streaming B: K may be split over the grid's y dimension.
    #   B stored [N][K]: 32x32 tile, 512-byte K rows, the 4 waves split the K steps of a tile
    #   B stored [K][N]: 32x128 tile, 4 waves side by side
    out.append((0, 1, 32, 32, 4 * bk, 1, 1, 4, 0, 1, 4))
    # the same with a ring of 2 tiles (64 KiB): two work-groups share a CU, for grids of more than 256 tiles, where the
    # start of one work-group then overlaps the steady state of another
    out.append((0, 1, 32, 32, 4 * bk, 1, 1, 2, 0, 1, 4))
    # (16-bit types: A stored [K][M] too, or a 32- or 64-row problem with A transposed falls to the guarded kernel, 10x slower; the
    # 8-bit types' transposed rows of 32 and 64 bytes are shorter than their LDS swizzle needs)
    for ta in skinny_ta:
        for tb in (0, 1):
            out.append((ta, tb, 32, 128, bk, 1, 4, 3, 0, 1, 1))
    # 64 rows: from M = 64 to a few hundred rows a 32-row tile streams B once per 32 rows of A (fp16 64x8192x8192 NT 34.2 us, the
    # vendor library 26.6); with 64-row tiles 26.6, 128x8192x8192 28.6 against 47.4, 256x4096x4096 18.3 against 23.6
    for ta in skinny_ta:
        for tb in (0, 1):
            out.append((ta, tb, 64, 128, bk, 2, 2, 3, 0, 1, 1))
    # B stored [N][K] streamed from HBM against 64 and 128 rows (fp16, B rotating over 400 MiB, us): the 32x32 kernel's shape with 64
    # rows, the 4 waves splitting the K steps, 64x8192x8192 31.6 against 36.2 for 64x128 tiles (the vendor library 34.1); a
    # 128x64 tile with K tiles twice as deep, 128x16384x4096 35.2 against 39.6 (vendor 36.0), 128x4096x16384 40.5 against 42.8
    out.append((0, 1, 64, 32, 4 * bk, 1, 1, 3, 0, 1, 4))
    out.append((0, 1, 128, 64, 2 * bk, 2, 2, 3, 0, 1, 1))
    # M and N that are not multiples of the tile (K a multiple of the K tile, rows and pointers on 16-byte boundaries): the default
    # 256x256 variant and the 128x128 one with 2 + 2 tiles once more with clamped lane offsets and checked stores.  (fp16
    # 4000x4096x4096 ran 539 us on 32-row tiles and 4096x4000x4096 933 us on the guarded kernel, the vendor library 110 and 125.)
    for ta in (0, 1):
        for tb in (0, 1):
            out.append(edge((ta, tb, 256, 256, bk, 2, 2, 2, 0, 0, 1, 3) + ((16,) if atom16 else ())))
            out.append(edge((ta, tb, 128, 128, bk, 2, 2, 2, 0, 0, 1, 2)))
    # ... and the 32x128 and 64x128 tiles with the split-K store path likewise: a number of rows that is no multiple of 32 against
    # a large B (fp16 48x8192x8192: 68 us on 128x128 edge tiles, the vendor library 27-35)
    for tb in (0, 1):
        out.append(edge((0, tb, 32, 128, bk, 1, 4, 3, 0, 1, 1)))
        out.append(edge((0, tb, 64, 128, bk, 2, 2, 3, 0, 1, 1)))
    # guarded variants: any shape, any leading dimension, element-aligned pointers; listed first, the same with whole 16-byte chunks
    # for rows and pointers on 16-byte boundaries and a K of whole chunks (K off the K tile, everything else in order)
    for ta in (0, 1):
        for tb in (0, 1):
            out.append(edge((ta, tb, 128, 128, bk, 2, 2, 2, 1, 0, 1)))
    for ta in (0, 1):
        for tb in (0, 1):
            out.append((ta, tb, 128, 128, bk, 2, 2, 2, 1, 0, 1))
    return out

VARIANTS = {
    "f16": ("FRISK_F16", "F16", square(64, atom16=True, skinny_ta=(0, 1))),
    "bf16": ("FRISK_BF16", "BF16", square(64, atom16=True, skinny_ta=(0, 1))),
    "i8": ("FRISK_I8", "I8", square(128, atom16=True)),
    # 8-bit floats: the 256x256 NT variant once more on the 16x16x128 atom, whose K is the whole K tile (listed first: the planner's
    # choice for B stored [N][K] from four K tiles on), and its copy with the split-K store path
    "e4m3": ("FRISK_E4M3", "E4M3", [(0, 1, 256, 256, 128, 2, 2, 2, 0, 0, 1, 3, 16), (0, 1, 256, 256, 128, 2, 2, 2, 0, 1, 1, 3, 16)] + square(128)),
    # fp32: 128x128 for large problems; 64x64 (one atom per wave) fills the chip at 1024^3, K tiles of 64 measured 5 % faster than 32;
    # the same tile with K tiles of 128 shared by two sets of four waves (8 waves, two per SIMD) another 9 % at 1024^3 (21.6 against
    # 23.9 us), where a CU holds a single work-group and nothing else hides its waits
    # 128x128 with K tiles of 16 in a ring of 4 (64 KiB, two work-groups per CU): 944 us at 4096^3 against 1000 for K tiles of 32 in a
    # ring of 2, 124 against 145 at 2048^3 (rings of 3, 6, 8 and K tiles of 8 measured no better)
    "f32": ("FRISK_F32", "F32", [(ta, tb, 128, 128, 16, 2, 2, 4, 0, 0, 1) for ta in (0, 1) for tb in (0, 1)]
            + [(ta, tb, bm, bn, bk, 2, 2, 2, 0, 0, 1) for bm, bn, bk in ((128, 128, 32), (64, 64, 64), (64, 64, 32)) for ta in (0, 1) for tb in (0, 1)]
            + [(ta, tb, 64, 64, 128, 2, 2, 2, 0, 0, 2) for ta in (0, 1) for tb in (0, 1)]
            # grids that leave CUs idle, or a few rows against a large B streamed from HBM: K split over the idle CUs (one 64x64 work-group of
            # four waves keeps a CU's matrix pipe busy, so 64 tiles on 256 CUs run at a quarter of the rate).  64x64x32 in a ring of 3
            # (256x4096x4096, B from HBM: 70 against 82 us for the ring of 2); 32x128x32 for 32 rows; for B stored [N][K] 32x32x128 and
            # 64x32x128 with the four waves splitting the K tile (512-byte rows of B: 32x16384x4096 47.5 against 61.4 us)
            + [(ta, tb, 64, 64, 32, 2, 2, 3, 0, 1, 1) for ta in (0, 1) for tb in (0, 1)]
            + [(ta, tb, 32, 128, 32, 1, 4, 3, 0, 1, 1) for ta in (0, 1) for tb in (0, 1)]
            + [(0, 1, 32, 32, 128, 1, 1, 4, 0, 1, 4), (0, 1, 32, 32, 128, 1, 1, 2, 0, 1, 4), (0, 1, 64, 32, 128, 1, 1, 3, 0, 1, 4)]
            + [edge((ta, tb, bm, bm, 32, 2, 2, 2, 0, 0, 1)) for bm in (128, 64) for ta in (0, 1) for tb in (0, 1)]
            + [edge((0, tb, 32, 128, 32, 1, 4, 3, 0, 1, 1)) for tb in (0, 1)] + [edge((0, tb, 64, 64, 32, 2, 2, 3, 0, 1, 1)) for tb in (0, 1)]
            + [edge((ta, tb, 64, 64, 32, 2, 2, 2, 1, 0, 1)) for ta in (0, 1) for tb in (0, 1)]
            + [(ta, tb, 64, 64, 32, 2, 2, 2, 1, 0, 1) for ta in (0, 1) for tb in (0, 1)]),
}

def cfg_of(enum, v):
    ta, tb, bm, bn, bk, wm, wn, st, gd, sk, wk, sb, at, eg = full(v)
    return f"GemmCfg<{enum}, {ta}, {tb}, {bm}, {bn}, {bk}, {wm}, {wn}, {st}, {'true' if gd else 'false'}, {'true' if sk else 'false'}, {wk}, {sb}" + (f", {at}, true>" if eg else (f", {at}>" if at != 32 else ">"))

HERE = os.path.dirname(os.path.abspath(__file__))
# A type's variants go into two translation units of about equal size (kernels_<type>.hip, kernels_<type>_2.hip), each with a
# table of its own: the units compile in parallel, and the longest of them sets the time of a build.  The planner walks the
# first table, then the second, so the order of the list above is the order it sees.
written = []
for tag, (enum, suffix, variants) in VARIANTS.items():
    half = (len(variants) + 1) // 2
    for part, chunk in ((1, variants[:half]), (2, variants[half:])):
        ext = "" if part == 1 else "_2"
        lines = [f"// {enum} kernel instantiations, part {part} of 2.  Generated by gen_kernels.py; do not edit by hand.",
                 '#include "gemm_kernel.hip.inc"', "namespace frisk {"]
        for v in chunk:
            lines.append(f"template __global__ void gemm_kernel<{cfg_of(enum, v)}>(GemmParams);")
        lines.append("#ifndef __HIP_DEVICE_COMPILE__")
        lines.append(f"const KernelEntry kKernels{suffix}{ext}[] = {{")
        for v in chunk:
            ta, tb, bm, bn, bk, wm, wn, st, gd, sk, wk, sb, at, eg = full(v)
            cfg = cfg_of(enum, v)
            waves = f"w{wm}x{wn}" + (f"x{wk}" if wk > 1 else "")
            name = f"{tag}_{'t' if ta else 'n'}{'t' if tb else 'n'}_{bm}x{bn}x{bk}_{waves}_s{st}" + (f"x{sb}" if sb != st else "") + (f"_a{at}" if at != 32 else "") + ("_guard_chunks" if gd and eg else "_guard" if gd else "") + ("_splitk" if sk else "") + ("_edge" if eg and not gd else "")
            lines.append(f'    {{"{name}", {enum}, {ta}, {tb}, {bm}, {bn}, {bk}, {wm}, {wn}, {st}, {sb}, {wk}, {gd}, {sk}, {at}, {eg}, {cfg}::LDS_BYTES, {cfg}::MIN_K_TILES, &launch_gemm<{cfg}>, &prepare_gemm<{cfg}>}},')
        lines.append("};")
        lines.append(f"const int kNumKernels{suffix}{ext} = sizeof(kKernels{suffix}{ext}) / sizeof(kKernels{suffix}{ext}[0]);")
        lines.append("#endif")
        lines.append("}  // namespace frisk")
        fn = f"kernels_{tag}{ext}.hip"
        with open(os.path.join(HERE, fn), "w") as f:
            f.write("\n".join(lines) + "\n")
        written.append(fn)
print("wrote", ", ".join(written))
