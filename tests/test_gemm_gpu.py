"""Parity of the HIP GEMM path against the CPU oracle, through the C ABI.

Bars: int8 -> int32 bit-exact; the dequant epilogue bit-exact (fixed fp32
operation order); fp16 / bf16 / fp8 within 1e-2 and fp32 within 1e-4, both as
max |d-r| / max(|r|, rms(R)) over all elements and as ||D-R||_F / ||R||_F.
"""
import sys

import numpy as np
import pytest

import oracle as O
from helpers import DEFAULT_OUT, NAMES, TOL, make_operand, run_gemm, stored_shapes

pytestmark = pytest.mark.gpu

BK = {O.F32: 32, O.F16: 64, O.BF16: 64, O.I8: 128, O.E4M3: 128}
BIG = {O.F32: 128, O.F16: 256, O.BF16: 256, O.I8: 256, O.E4M3: 256}
SMALL = {O.F32: 64, O.F16: 128, O.BF16: 128, O.I8: 128, O.E4M3: 128}


def note(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def check(dtype, dtype_out, got, ref64):
    r = O.compare(dtype_out, got, ref64)
    tol = TOL[dtype]
    assert r["nonfinite"] == 0, r
    assert r["max_rel"] <= tol and r["fro_rel"] <= tol, (r, tol)
    return r


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.I8, O.E4M3, O.F32])
@pytest.mark.parametrize("transA,transB", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("which", ["big", "small"])
def test_layouts_small_shapes(hip, dtype, transA, transB, which):
    t = BIG[dtype] if which == "big" else SMALL[dtype]
    M, N, K = 2 * t, 3 * t, 3 * BK[dtype]
    note(f"case layouts {NAMES[dtype]} tA={transA} tB={transB} tile={t} M={M} N={N} K={K}")
    sa, sb = stored_shapes(M, N, K, transA, transB)
    A = make_operand(dtype, *sa, seed=11, tensor=0, scale=0.5)
    B = make_operand(dtype, *sb, seed=11, tensor=1, scale=0.5)
    out_dt = DEFAULT_OUT[dtype]
    got = run_gemm(hip, dtype, A, B, transA, transB, out_dt, M, N, K, tile=(t, t, BK[dtype]))
    if dtype == O.I8:
        ref = O.gemm_i32(A, B, transA, transB)
        assert np.array_equal(got, ref)
    else:
        check(dtype, out_dt, got, O.gemm_f64(dtype, A, B, transA, transB))


@pytest.mark.parametrize("dtype", [O.F16, O.BF16])
@pytest.mark.parametrize("transA,transB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_deeper_ring_for_b(hip, dtype, transA, transB):
    """the variant with 2 LDS tiles of A and 3 of B: K of 1, 2, 3, 4 and 7 tiles walks every phase of its pipeline
    (fewer tiles than stages, A-only tail, steady state) and must give the bits of the 2 + 2 variant"""
    for ktiles in (1, 2, 3, 4, 7):
        M, N, K = 256, 512, ktiles * 64
        note(f"case deep-B {NAMES[dtype]} tA={transA} tB={transB} K={K}")
        sa, sb = stored_shapes(M, N, K, transA, transB)
        A = make_operand(dtype, *sa, seed=12, tensor=0, scale=0.5)
        B = make_operand(dtype, *sb, seed=12, tensor=1, scale=0.5)
        d = hip.make_desc(dtype, M, N, K, transA=bool(transA), transB=bool(transB), tile=(256, 256, 64), stages=3)
        p = hip.plan(d)
        assert (p.stages, p.stages_b, p.lds_bytes) == (2, 3, 160 * 1024)
        got = run_gemm(hip, dtype, A, B, transA, transB, dtype, M, N, K, tile=(256, 256, 64), stages=3)
        check(dtype, dtype, got, O.gemm_f64(dtype, A, B, transA, transB))
        same = run_gemm(hip, dtype, A, B, transA, transB, dtype, M, N, K, tile=(256, 256, 64), stages=2)
        assert np.array_equal(got, same)


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.E4M3, O.F32])
def test_identity_is_exact(hip, dtype):
    """A = I  =>  C == B bit for bit (every product is exact, every sum has one non-zero term)"""
    n = 2 * BIG[dtype]
    K = n
    eye = O.encode(dtype, np.eye(n, dtype=np.float32))
    B = make_operand(dtype, K, n, seed=5, tensor=1, scale=1.0)
    out_dt = dtype if dtype != O.E4M3 else O.F32
    got = run_gemm(hip, dtype, eye, B, 0, 0, out_dt, n, n, K)
    if dtype == O.E4M3:
        assert np.array_equal(got, O.decode(dtype, B))
    else:
        assert np.array_equal(got.view(np.uint8), B.view(np.uint8))


def test_all_ones_gives_k(hip):
    M = N = 256
    K = 64 * 7
    ones = O.encode(O.F16, np.ones((M, K), dtype=np.float32))
    onesB = O.encode(O.F16, np.ones((K, N), dtype=np.float32))
    got = run_gemm(hip, O.F16, ones, onesB, 0, 0, O.F32, M, N, K)
    assert np.all(got == float(K))


def test_accumulate_into_c(hip):
    """clear_accum = 0: C = C + A.B  (frisk.gemm clear_accum attribute)"""
    M = N = 256
    K = 128
    A = make_operand(O.F16, M, K, seed=7, tensor=0, scale=0.25)
    B = make_operand(O.F16, K, N, seed=7, tensor=1, scale=0.25)
    C0 = O.uniform(M * N, 7, 2, -1.0, 1.0).reshape(M, N).astype(np.float32)
    got = run_gemm(hip, O.F16, A, B, 0, 0, O.F32, M, N, K, C_init=C0, clear_accum=False)
    ref = O.gemm_f64(O.F16, A, B) + C0.astype(np.float64)
    check(O.F16, O.F32, got, ref)
    A8 = make_operand(O.I8, M, K, seed=8, tensor=0)
    B8 = make_operand(O.I8, K, N, seed=8, tensor=1)
    Ci = (np.arange(M * N, dtype=np.int64).reshape(M, N) % 1000 - 500).astype(np.int32)
    goti = run_gemm(hip, O.I8, A8, B8, 0, 0, O.I32, M, N, K, C_init=Ci, clear_accum=False)
    assert np.array_equal(goti, O.gemm_i32(A8, B8) + Ci)


OUT_TYPES = {O.F16: [O.F16, O.F32], O.BF16: [O.BF16, O.F32], O.I8: [O.I32, O.F16, O.F32], O.E4M3: [O.BF16, O.F16, O.F32], O.F32: [O.F32]}


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.I8, O.E4M3, O.F32])
def test_every_output_type_epilogue_and_accumulation(hip, dtype):
    """all valid (output type, epilogue kind, clear_accum) combinations of a type on the unguarded kernels (the large tile with
    both atom sizes where compiled, and a small one): out = convert(old C + (acc * sA) * sB), against the oracle's float64
    accumulators with the same fp32 scale products; int32 outputs exact"""
    M, N, K = 512, 512, 3 * BK[dtype]
    tB = 1 if dtype == O.E4M3 else 0
    A = make_operand(dtype, M, K, seed=21, tensor=0, scale=0.5)
    B = make_operand(dtype, *((N, K) if tB else (K, N)), seed=21, tensor=1, scale=0.5)
    acc = O.gemm_i32(A, B, 0, tB).astype(np.float64) if dtype == O.I8 else O.gemm_f64(dtype, A, B, 0, tB)
    rowA, colB = O.uniform(M, 21, 2, 0.25, 2.0), O.uniform(N, 21, 3, 0.25, 2.0)
    if dtype == O.I8:
        rowA, colB = rowA * np.float32(2.0 ** -9), colB * np.float32(2.0 ** -9)
    tiles = [((0, 0, 0), 0)] if dtype == O.F32 else [((BIG[dtype], BIG[dtype], BK[dtype]), 32), ((SMALL[dtype], SMALL[dtype], BK[dtype]), 0)]
    if dtype in (O.F16, O.BF16, O.I8):
        tiles.insert(0, ((256, 256, BK[dtype]), 16))
    for out_dt in OUT_TYPES[dtype]:
        for epi in (hip.EPI_NONE, hip.EPI_ROW_COL_SCALE, hip.EPI_TENSOR_SCALE):
            if out_dt == O.I32 and epi != hip.EPI_NONE:
                continue
            if dtype == O.I8 and out_dt == O.F16 and epi == hip.EPI_NONE:
                continue  # raw int8 accumulators of this size overflow fp16
            sA = None if epi == hip.EPI_NONE else (rowA if epi == hip.EPI_ROW_COL_SCALE else rowA[:1])
            sB = None if epi == hip.EPI_NONE else (colB if epi == hip.EPI_ROW_COL_SCALE else colB[:1])
            scaled = acc if epi == hip.EPI_NONE else ((acc * (sA.astype(np.float64)[:, None] if len(sA) > 1 else float(sA[0]))) * (sB.astype(np.float64)[None, :] if len(sB) > 1 else float(sB[0])))
            for accumulate in (False, True):
                if out_dt == O.I32:
                    C0 = (np.arange(M * N, dtype=np.int64).reshape(M, N) % 2001 - 1000).astype(np.int32)
                    old = C0.astype(np.float64)
                else:
                    old = O.decode(out_dt, O.encode(out_dt, O.uniform(M * N, 22, 4, -2.0, 2.0))).reshape(M, N).astype(np.float64)
                    C0 = O.encode(out_dt, old.astype(np.float32)).reshape(M, N)
                ref = scaled + (old if accumulate else 0.0)
                for tile, atom in tiles:
                    note(f"case epilogue {NAMES[dtype]}->{out_dt} epi={epi} accumulate={accumulate} tile={tile} atom={atom}")
                    got = run_gemm(hip, dtype, A, B, 0, tB, out_dt, M, N, K, epilogue=epi, sA=sA, sB=sB, C_init=C0 if accumulate else None,
                                   clear_accum=not accumulate, tile=tile, atom=atom)
                    if out_dt == O.I32:
                        assert np.array_equal(got, ref.astype(np.int64).astype(np.int32))
                    else:
                        check(dtype, out_dt, got, ref)


def test_int8_dequant_epilogue_bit_exact(hip):
    """out = f16((float(acc) * sA[m]) * sB[n]) with the multiplication order fixed: bit-exact against the oracle"""
    M, N, K = 512, 512, 1024
    A = make_operand(O.I8, M, K, seed=3, tensor=0)
    B = make_operand(O.I8, K, N, seed=3, tensor=1)
    sA = O.uniform(M, 3, 2, 0.001, 0.02)
    sB = O.uniform(N, 3, 3, 0.001, 0.02)
    got = run_gemm(hip, O.I8, A, B, 0, 0, O.F16, M, N, K, epilogue=hip.EPI_ROW_COL_SCALE, sA=sA, sB=sB)
    acc = O.gemm_i32(A, B)
    assert np.array_equal(got, O.epilogue_rowcol_f16(acc, sA, sB))
    # power-of-two scales: closed form, exact
    sA2 = np.full(M, 2.0 ** -10, dtype=np.float32)
    sB2 = np.full(N, 2.0 ** -6, dtype=np.float32)
    got2 = run_gemm(hip, O.I8, A, B, 0, 0, O.F32, M, N, K, epilogue=hip.EPI_ROW_COL_SCALE, sA=sA2, sB=sB2)
    assert np.array_equal(got2, acc.astype(np.float32) * np.float32(2.0 ** -16))


def test_fp8_tensor_scale_epilogue(hip):
    M, N, K = 256, 512, 512
    xa, xb = O.normal(M * K, 4, 0, 1.0), O.normal(N * K, 4, 1, 1.0)
    sA, sB = np.float32(np.abs(xa).max() / 448.0), np.float32(np.abs(xb).max() / 448.0)
    A = O.encode(O.E4M3, xa / sA).reshape(M, K)
    B = O.encode(O.E4M3, xb / sB).reshape(N, K)  # stored [N][K]
    got = run_gemm(hip, O.E4M3, A, B, 0, 1, O.BF16, M, N, K, epilogue=hip.EPI_TENSOR_SCALE, sA=[sA], sB=[sB])
    ref = O.epilogue_tensor(O.gemm_f64(O.E4M3, A, B, False, True), sA, sB)
    check(O.E4M3, O.BF16, got, ref)


@pytest.mark.parametrize("k_tiles", [4, 5, 6, 7, 8, 9, 16])
def test_fp8_whole_tile_atom_every_loop_path(hip, k_tiles):
    """8-bit floats on the 16x16x128 atom (its K is the whole K tile).  The loop peels its first tile and its last three and
    walks the tiles between them two at a time, with one more single tile or a move of the B fragments between the two
    register buffers depending on the parity of the count: 4 .. 9 K tiles take every combination, 16 several rounds of the pair loop.
    Exact check: integers up to 4 in magnitude (sums stay below 2^24), raw fp32 output."""
    M, N, K = 512, 768, 128 * k_tiles
    note(f"case fp8 16x16x128 atom, {k_tiles} K tiles, {M}x{N}x{K}")
    rng = np.random.default_rng(900 + k_tiles)
    Ai, Bi = rng.integers(-4, 5, size=(M, K)), rng.integers(-4, 5, size=(N, K))
    A = O.encode(O.E4M3, Ai.astype(np.float32).reshape(-1)).reshape(M, K)
    B = O.encode(O.E4M3, Bi.astype(np.float32).reshape(-1)).reshape(N, K)
    got = run_gemm(hip, O.E4M3, A, B, 0, 1, O.F32, M, N, K, tile=(256, 256, 128), atom=16)
    assert np.array_equal(got.astype(np.int64), Ai.astype(np.int64) @ Bi.astype(np.int64).T)
    # random values, tensor scales, bf16 output, accumulation into C
    xa, xb = O.normal(M * K, 40 + k_tiles, 0, 1.0), O.normal(N * K, 40 + k_tiles, 1, 1.0)
    sA, sB = np.float32(np.abs(xa).max() / 448.0), np.float32(np.abs(xb).max() / 448.0)
    A, B = O.encode(O.E4M3, xa / sA).reshape(M, K), O.encode(O.E4M3, xb / sB).reshape(N, K)
    old = O.decode(O.BF16, O.encode(O.BF16, O.uniform(M * N, 41, 4, -2.0, 2.0))).reshape(M, N).astype(np.float64)
    C0 = O.encode(O.BF16, old.astype(np.float32)).reshape(M, N)
    ref = O.epilogue_tensor(O.gemm_f64(O.E4M3, A, B, False, True), sA, sB)
    got = run_gemm(hip, O.E4M3, A, B, 0, 1, O.BF16, M, N, K, epilogue=hip.EPI_TENSOR_SCALE, sA=[sA], sB=[sB], tile=(256, 256, 128), atom=16)
    check(O.E4M3, O.BF16, got, ref)
    got = run_gemm(hip, O.E4M3, A, B, 0, 1, O.BF16, M, N, K, epilogue=hip.EPI_TENSOR_SCALE, sA=[sA], sB=[sB], C_init=C0, clear_accum=False,
                   tile=(256, 256, 128), atom=16)
    check(O.E4M3, O.BF16, got, ref + old)


def test_fp8_whole_tile_atom_needs_four_k_tiles(hip):
    """its loop is written for four or more K tiles: the planner offers it for none fewer, and a descriptor that names it is refused"""
    for k_tiles, ok in ((3, False), (4, True)):
        d = hip.make_desc(O.E4M3, 512, 512, 128 * k_tiles, dtype_out=O.BF16, transB=1, tile=(256, 256, 128), atom=16)
        if ok:
            assert hip.kernel_names()[hip.plan(d).kernel_id].endswith("_a16")
        else:
            with pytest.raises(hip.FriskHipError) as e:
                hip.plan(d)
            assert e.value.status == hip.ERR_TILE
    p = hip.plan(hip.make_desc(O.E4M3, 512, 512, 384, dtype_out=O.BF16, transB=1))
    assert not hip.kernel_names()[p.kernel_id].endswith("_a16")
    # an explicit split counts per slice (a full round of tiles, where the planner prefers the atom): 16 K tiles in 2 slices stay on it,
    # in 8 slices they go to the 32-row atoms
    names = hip.kernel_names()
    assert names[hip.plan(hip.make_desc(O.E4M3, 4096, 4096, 2048, dtype_out=O.BF16, transB=1, tile=(256, 256, 128), split_k=2)).kernel_id].endswith("_a16_splitk")
    assert names[hip.plan(hip.make_desc(O.E4M3, 4096, 4096, 2048, dtype_out=O.BF16, transB=1, tile=(256, 256, 128), split_k=8)).kernel_id].endswith("s2x3_splitk")


def test_fp8_whole_tile_atom_split_k(hip):
    """the 16x16x128 kernel with the split-K store path: 16 K tiles in 2 and 4 slices (8 and 4 tiles each) against the oracle, exact"""
    M, N, K = 512, 512, 2048
    rng = np.random.default_rng(77)
    Ai, Bi = rng.integers(-4, 5, size=(M, K)), rng.integers(-4, 5, size=(N, K))
    A = O.encode(O.E4M3, Ai.astype(np.float32).reshape(-1)).reshape(M, K)
    B = O.encode(O.E4M3, Bi.astype(np.float32).reshape(-1)).reshape(N, K)
    want = Ai.astype(np.int64) @ Bi.astype(np.int64).T
    for split in (2, 4):
        note(f"case fp8 16x16x128 atom, split_k={split}")
        got = run_gemm(hip, O.E4M3, A, B, 0, 1, O.F32, M, N, K, tile=(256, 256, 128), atom=16, split_k=split)
        assert np.array_equal(got.astype(np.int64), want)


# ------------------------------------------------------------------ full-size configurations
def test_config_fp32_1024(hip):
    M = N = K = 1024
    A = make_operand(O.F32, M, K, seed=0, tensor=0, kind="uniform")
    B = make_operand(O.F32, K, N, seed=0, tensor=1, kind="uniform")
    got = run_gemm(hip, O.F32, A, B, 0, 0, O.F32, M, N, K)
    r = check(O.F32, O.F32, got, O.gemm_f64(O.F32, A, B))
    note(f"fp32 1024^3: {r}")


def test_config_fp16_4096(hip):
    M = N = K = 4096
    A = make_operand(O.F16, M, K, seed=1, tensor=0, scale=1.0 / 64.0)
    B = make_operand(O.F16, K, N, seed=1, tensor=1, scale=1.0 / 64.0)
    got = run_gemm(hip, O.F16, A, B, 0, 0, O.F16, M, N, K)
    r = check(O.F16, O.F16, got, O.gemm_f64(O.F16, A, B))
    note(f"fp16 4096^3: {r}")


def test_config_int8_4096(hip):
    M = N = K = 4096
    A = make_operand(O.I8, M, K, seed=3, tensor=0)
    B = make_operand(O.I8, K, N, seed=3, tensor=1)
    sA = O.uniform(M, 3, 2, 0.001, 0.02)
    sB = O.uniform(N, 3, 3, 0.001, 0.02)
    acc = O.gemm_i32(A, B)
    got_i32 = run_gemm(hip, O.I8, A, B, 0, 0, O.I32, M, N, K)
    assert np.array_equal(got_i32, acc)
    got = run_gemm(hip, O.I8, A, B, 0, 0, O.F16, M, N, K, epilogue=hip.EPI_ROW_COL_SCALE, sA=sA, sB=sB)
    assert np.array_equal(got, O.epilogue_rowcol_f16(acc, sA, sB))
    # and within tolerance of the un-narrowed value
    check(O.I8, O.F16, got, O.epilogue_rowcol_f32(acc, sA, sB).astype(np.float64))


def _sampled_rows(M, tile, count=64):
    rows = set(range(0, M, max(1, M // count)))
    for t in range(0, M, tile):
        rows.add(t)
        rows.add(t + tile - 1)
    return sorted(rows)


def check_marginal_sums(dtype, dtype_out, got, A, B, scale=1.0):
    """Every element of C = A B^T (A [M][K], B [N][K]) through two linear properties that cost O(MK + NK + MN): the column sums
    1^T C = (1^T A) B^T and the row sums C 1 = A (B^T 1), in float64.  The rounding of the M (or N) summed outputs is independent
    from element to element, so a sum is off by about sqrt(count) * eps/3 * rms(C), at most 6e-3 * sqrt(count) * rms(C) over 8192
    sums of bf16 outputs; one 256 x 256 tile of an 8192^2 result that is wrong by 2 % moves its sums by 4.5e-2 of that unit.
    Bar: 2e-2 of sqrt(count) * rms(C)."""
    C = O.decode(dtype_out, got).astype(np.float64)
    Af, Bf = O.decode(dtype, A).astype(np.float64), O.decode(dtype, B).astype(np.float64)
    M, N = C.shape
    rms = float(np.sqrt(np.mean(C * C)))
    col_ref = (Af.sum(axis=0) @ Bf.T) * scale
    row_ref = (Af @ Bf.sum(axis=0)) * scale
    col_err = float(np.abs(C.sum(axis=0) - col_ref).max() / (np.sqrt(M) * rms))
    row_err = float(np.abs(C.sum(axis=1) - row_ref).max() / (np.sqrt(N) * rms))
    assert np.isfinite(C).all()
    assert col_err <= 2e-2 and row_err <= 2e-2, (col_err, row_err)
    return {"col_sum_err": col_err, "row_sum_err": row_err}


def test_config_bf16_8192_nt(hip):
    """8192^3: the oracle checks 64 evenly spaced rows plus the first and last row of every tile band"""
    M = N = K = 8192
    A = make_operand(O.BF16, M, K, seed=2, tensor=0, scale=0.02)
    B = make_operand(O.BF16, N, K, seed=2, tensor=1, scale=0.02)
    got = run_gemm(hip, O.BF16, A, B, 0, 1, O.BF16, M, N, K)
    rows = _sampled_rows(M, 256)
    ref = O.gemm_f64(O.BF16, np.ascontiguousarray(A[rows]), B, False, True)
    r = check(O.BF16, O.BF16, np.ascontiguousarray(got[rows]), ref)
    note(f"bf16 8192^3 NT ({len(rows)} rows): {r}")
    note(f"bf16 8192^3 NT, all elements through row and column sums: {check_marginal_sums(O.BF16, O.BF16, got, A, B)}")


def test_config_fp8_8192(hip):
    M = N = K = 8192
    xa, xb = O.normal(M * K, 4, 0, 1.0), O.normal(N * K, 4, 1, 1.0)
    sA, sB = np.float32(np.abs(xa).max() / 448.0), np.float32(np.abs(xb).max() / 448.0)
    A = O.encode(O.E4M3, xa / sA).reshape(M, K)
    B = O.encode(O.E4M3, xb / sB).reshape(N, K)
    del xa, xb
    got = run_gemm(hip, O.E4M3, A, B, 0, 1, O.BF16, M, N, K, epilogue=hip.EPI_TENSOR_SCALE, sA=[sA], sB=[sB])
    rows = _sampled_rows(M, 256)
    ref = O.gemm_f64(O.E4M3, np.ascontiguousarray(A[rows]), B, False, True)
    r = check(O.E4M3, O.BF16, np.ascontiguousarray(got[rows]), O.epilogue_tensor(ref, sA, sB))
    note(f"fp8 8192^3 NT ({len(rows)} rows): {r}")
    sums = check_marginal_sums(O.E4M3, O.BF16, got, A, B, scale=float(sA) * float(sB))
    note(f"fp8 8192^3 NT, all elements through row and column sums: {sums}")


# ------------------------------------------------------------------ ragged shapes, odd leading dimensions, K = 0
RAGGED = [(1, 1, 1), (100, 75, 40), (257, 129, 65), (33, 500, 130), (128, 128, 1)]


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.I8, O.E4M3, O.F32])
@pytest.mark.parametrize("transA,transB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_ragged_shapes_run_the_guarded_kernel(hip, dtype, transA, transB):
    for (M, N, K) in RAGGED:
        note(f"case ragged {NAMES[dtype]} tA={transA} tB={transB} M={M} N={N} K={K}")
        sa, sb = stored_shapes(M, N, K, transA, transB)
        A = make_operand(dtype, *sa, seed=31, tensor=0, scale=0.5)
        B = make_operand(dtype, *sb, seed=31, tensor=1, scale=0.5)
        out_dt = DEFAULT_OUT[dtype]
        got = run_gemm(hip, dtype, A, B, transA, transB, out_dt, M, N, K)
        if dtype == O.I8:
            assert np.array_equal(got, O.gemm_i32(A, B, transA, transB))
        else:
            check(dtype, out_dt, got, O.gemm_f64(dtype, A, B, transA, transB))


def test_odd_leading_dimensions_and_unaligned_pointers(hip):
    """rows padded by 3 elements and buffers entered one element in: no 16-byte alignment anywhere"""
    M, N, K = 256, 256, 128
    A = make_operand(O.F16, M, K, seed=32, tensor=0, scale=0.5)
    B = make_operand(O.F16, K, N, seed=32, tensor=1, scale=0.5)
    ref = O.gemm_f64(O.F16, A, B)
    for pad, shift in ((3, 0), (0, 1), (5, 3)):
        got = run_gemm(hip, O.F16, A, B, 0, 0, O.F16, M, N, K, pad=pad, shift=shift)
        check(O.F16, O.F16, got, ref)
    # the aligned call of the same problem on the fast kernel of the same tile agrees bit for bit with the guarded one (another tile
    # shape may add the K steps in another order)
    fast = run_gemm(hip, O.F16, A, B, 0, 0, O.F16, M, N, K, tile=(128, 128, 64))
    slow = run_gemm(hip, O.F16, A, B, 0, 0, O.F16, M, N, K, pad=8, shift=0, tile=(128, 128, 64))  # rows still 16-byte aligned: fast kernel
    check(O.F16, O.F16, run_gemm(hip, O.F16, A, B, 0, 0, O.F16, M, N, K), ref)  # the planner's own choice
    assert np.array_equal(fast, slow)
    assert np.array_equal(fast, run_gemm(hip, O.F16, A, B, 0, 0, O.F16, M, N, K, pad=3))


def test_ragged_int8_dequant_and_accumulate(hip):
    M, N, K = 70, 90, 200
    A = make_operand(O.I8, M, K, seed=33, tensor=0)
    B = make_operand(O.I8, K, N, seed=33, tensor=1)
    sA, sB = O.uniform(M, 33, 2, 0.001, 0.02), O.uniform(N, 33, 3, 0.001, 0.02)
    got = run_gemm(hip, O.I8, A, B, 0, 0, O.F16, M, N, K, epilogue=hip.EPI_ROW_COL_SCALE, sA=sA, sB=sB)
    assert np.array_equal(got, O.epilogue_rowcol_f16(O.gemm_i32(A, B), sA, sB))
    C0 = (np.arange(M * N, dtype=np.int64).reshape(M, N) % 77 - 30).astype(np.int32)
    goti = run_gemm(hip, O.I8, A, B, 0, 0, O.I32, M, N, K, C_init=C0, clear_accum=False)
    assert np.array_equal(goti, O.gemm_i32(A, B) + C0)


def test_empty_problems(hip):
    """K = 0: C = 0 (or C unchanged when accumulating); M = 0 or N = 0: nothing is launched"""
    M, N = 64, 48
    A = np.zeros((M, 0), dtype=np.uint16)
    B = np.zeros((0, N), dtype=np.uint16)
    got = run_gemm(hip, O.F16, np.zeros((M, 1), np.uint16), np.zeros((1, N), np.uint16), 0, 0, O.F32, M, N, 0)
    assert np.all(got == 0.0)
    C0 = O.uniform(M * N, 5, 0, -1.0, 1.0).reshape(M, N)
    got = run_gemm(hip, O.F16, np.zeros((M, 1), np.uint16), np.zeros((1, N), np.uint16), 0, 0, O.F32, M, N, 0, C_init=C0, clear_accum=False)
    assert np.array_equal(got, C0)
    d = hip.make_desc(hip.F16, 0, 128, 64)
    hip.gemm(d, None, None, None)
    del A, B


# ------------------------------------------------------------------ skinny problems: 32-row tiles, K split over work-groups
@pytest.mark.parametrize("dtype,transA", [(O.F16, 0), (O.BF16, 0), (O.I8, 0), (O.E4M3, 0), (O.F16, 1), (O.BF16, 1)])
@pytest.mark.parametrize("transB", [0, 1])
def test_skinny_split_k(hip, dtype, transA, transB):
    """M = 32 and 64: a 32- or 64-row kernel runs (32 rows, B stored [N][K]: 32x32 tile whose 4 waves split the K steps; B stored
    [K][N]: 32x128 tile; 64 rows: 64x128); every split factor gives the oracle's result (int8: the same bits).  K is deep enough for the planner to
    split it by itself (slices of at least 16 K tiles).  The 16-bit types have the 32x128 and 64x128 tiles for A stored [K][M] too."""
    for M in (32, 64):
        N, K = 384, 128 * BK[dtype]
        sa, sb = stored_shapes(M, N, K, transA, transB)
        A = make_operand(dtype, *sa, seed=41, tensor=0, scale=0.5)
        B = make_operand(dtype, *sb, seed=41, tensor=1, scale=0.5)
        out_dt = DEFAULT_OUT[dtype]
        ref = O.gemm_i32(A, B, transA, transB) if dtype == O.I8 else O.gemm_f64(dtype, A, B, transA, transB)
        d = hip.make_desc(dtype, M, N, K, dtype_out=out_dt, transA=bool(transA), transB=bool(transB))
        p = hip.plan(d)
        assert p.tile_m in (32, 64) and p.tile_m <= M and p.split_k > 1 and p.workspace_bytes == p.split_k * M * N * 4, (p.tile_m, p.split_k, p.workspace_bytes)
        # the planner's variant at every split, then the 32-row kernels by name (at M = 64 the planner prefers 64-row tiles)
        for split, rows in ((0, 0), (1, 0), (2, 0), (4, 0), (8, 0), (0, 32), (2, 32)):
            note(f"case skinny {NAMES[dtype]} tA={transA} tB={transB} M={M} N={N} K={K} split_k={split} tile_m={rows}")
            got = run_gemm(hip, dtype, A, B, transA, transB, out_dt, M, N, K, split_k=split, tile=(rows, 0, 0))
            if dtype == O.I8:
                assert np.array_equal(got, ref)
            else:
                check(dtype, out_dt, got, ref)
        # the planner's own split needs no workspace to be correct: without one the launch runs unsplit
        got = run_gemm(hip, dtype, A, B, transA, transB, out_dt, M, N, K, workspace=False)
        if dtype == O.I8:
            assert np.array_equal(got, ref)
        else:
            check(dtype, out_dt, got, ref)


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.I8, O.E4M3])
@pytest.mark.parametrize("transB", [0, 1])
def test_small_grid_gets_a_split_of_its_own(hip, dtype, transB):
    """a few hundred rows and a long K: the planner's small-grid model picks a variant with the split-K store path and a split of
    its own; same result as the oracle with the planner's pair, without a workspace (one pass), and with the small-grid variants
    (128x128, 64x128, 64x32 with waves splitting K, 128x64) named by the descriptor at several splits"""
    M, N, K = 512, 512, 128 * BK[dtype]
    sa, sb = stored_shapes(M, N, K, 0, transB)
    A = make_operand(dtype, *sa, seed=47, tensor=0, scale=0.5)
    B = make_operand(dtype, *sb, seed=47, tensor=1, scale=0.5)
    out_dt = DEFAULT_OUT[dtype]
    ref = O.gemm_i32(A, B, 0, transB) if dtype == O.I8 else O.gemm_f64(dtype, A, B, 0, transB)
    p = hip.plan(hip.make_desc(dtype, M, N, K, dtype_out=out_dt, transB=bool(transB)))
    name = hip.kernel_names()[p.kernel_id]
    assert p.tile_m in (64, 128) and p.split_k > 1 and name.endswith("_s3_splitk") and p.workspace_bytes == p.split_k * M * N * 4, (name, p.split_k)
    cases = [dict(workspace=True), dict(workspace=False)]
    cases += [dict(tile=(bm, 128, BK[dtype]), split_k=sk) for bm in (64, 128) for sk in (2, 4)]
    if transB:  # the two variants that stream a B stored [N][K]: 64x32 with the waves splitting K, 128x64 with K tiles twice as deep
        cases += [dict(tile=(64, 32, 4 * BK[dtype]), split_k=sk) for sk in (1, 2)] + [dict(tile=(128, 64, 2 * BK[dtype]), split_k=sk) for sk in (1, 4)]
    for kw in cases:
        note(f"case small grid {NAMES[dtype]} tB={transB} M={M} N={N} K={K} {kw}")
        got = run_gemm(hip, dtype, A, B, 0, transB, out_dt, M, N, K, **kw)
        if dtype == O.I8:
            assert np.array_equal(got, ref)
        else:
            check(dtype, out_dt, got, ref)


@pytest.mark.parametrize("transA,transB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_fp32_small_grids_split_k(hip, transA, transB):
    """fp32 on grids that leave CUs idle: one 64x64 work-group already keeps a CU's matrix pipe busy, so the planner splits K over
    the idle CUs (32-row tiles for 32 rows).  The planner's own pair, the same without a workspace (one pass), and every fp32
    variant with the split-K store path named by the descriptor at several splits, all against the oracle at 1e-4; accumulation
    into C through the split path"""
    K = 128 * BK[O.F32]
    for M, N in ((32, 384), (64, 256), (256, 384)):
        sa, sb = stored_shapes(M, N, K, transA, transB)
        A = make_operand(O.F32, *sa, seed=53, tensor=0, scale=0.5)
        B = make_operand(O.F32, *sb, seed=53, tensor=1, scale=0.5)
        ref = O.gemm_f64(O.F32, A, B, transA, transB)
        p = hip.plan(hip.make_desc(O.F32, M, N, K, dtype_out=O.F32, transA=bool(transA), transB=bool(transB)))
        name = hip.kernel_names()[p.kernel_id]
        assert p.split_k > 1 and name.endswith("_splitk") and p.tile_m <= M and p.workspace_bytes == p.split_k * M * N * 4, (name, p.split_k)
        cases = [dict(workspace=True), dict(workspace=False)]
        if M % 64 == 0:
            cases += [dict(tile=(64, 64, 32), stages=3, split_k=sk) for sk in (2, 4, 16)]
        cases += [dict(tile=(32, 128, 32), split_k=sk) for sk in (1, 2, 8)]
        if not transA and transB:  # A stored [M][K], B stored [N][K]: the four waves split the K tile
            cases += [dict(tile=(32, 32, 128), stages=st, split_k=sk) for st in (2, 4) for sk in (1, 2, 4)]
            if M % 64 == 0:
                cases += [dict(tile=(64, 32, 128), split_k=sk) for sk in (1, 4)]
        for kw in cases:
            note(f"case fp32 small grid tA={transA} tB={transB} M={M} N={N} K={K} {kw}")
            check(O.F32, O.F32, run_gemm(hip, O.F32, A, B, transA, transB, O.F32, M, N, K, **kw), ref)
        C0 = O.uniform(M * N, 53, 2, -1.0, 1.0).reshape(M, N).astype(np.float32)
        note(f"case fp32 small grid accumulate tA={transA} tB={transB} M={M} N={N}")
        check(O.F32, O.F32, run_gemm(hip, O.F32, A, B, transA, transB, O.F32, M, N, K, C_init=C0, clear_accum=False), ref + C0)


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.I8, O.E4M3, O.F32])
@pytest.mark.parametrize("transA,transB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_edge_kernels_take_any_m_and_n(hip, dtype, transA, transB):
    """M and N that are not multiples of any tile, K a multiple of the K tile, rows on 16-byte boundaries: the edge variants of the
    256x256 and 128x128 kernels (fp32: 128x128 and 64x64) run, whose lanes fetch the last valid row or chunk instead of one beyond
    the operand and whose stores are checked against M and N.  Planner's choice and both tiles by name, against the oracle; the
    rows and columns of C beyond M and N (inside padded rows) stay untouched."""
    M, N, K = 304, 400, 3 * BK[dtype]  # 304 = 2 * 128 + 48 = 256 + 48, 400 = 3 * 128 + 16 = 256 + 144; all rows multiples of 16 bytes
    sa, sb = stored_shapes(M, N, K, transA, transB)
    A = make_operand(dtype, *sa, seed=61, tensor=0, scale=0.5)
    B = make_operand(dtype, *sb, seed=61, tensor=1, scale=0.5)
    out_dt = DEFAULT_OUT[dtype]
    ref = O.gemm_i32(A, B, transA, transB) if dtype == O.I8 else O.gemm_f64(dtype, A, B, transA, transB)
    name = hip.kernel_names()[hip.plan(hip.make_desc(dtype, M, N, K, dtype_out=out_dt, transA=bool(transA), transB=bool(transB))).kernel_id]
    assert name.endswith("_edge"), name
    big = 128 if dtype == O.F32 else 256
    for tile in ((0, 0, 0), (big, big, 0), (big // 2, big // 2, 0)):
        note(f"case edge {NAMES[dtype]} tA={transA} tB={transB} M={M} N={N} K={K} tile={tile}")
        got = run_gemm(hip, dtype, A, B, transA, transB, out_dt, M, N, K, tile=tile, pad_c=16)
        if dtype == O.I8:
            assert np.array_equal(got, ref)
        else:
            check(dtype, out_dt, got, ref)


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.I8, O.E4M3, O.F32])
@pytest.mark.parametrize("transB", [0, 1])
def test_edge_kernels_with_split_k(hip, dtype, transB):
    """a number of rows that is no multiple of 32 against a deep K: the 32- and 64-row tiles with the split-K store path exist as
    edge kernels too, so the planner still splits K over the idle CUs; its own pair and both tiles by name at several splits
    against the oracle (int8: the same bits)"""
    N, K = 384, 128 * BK[dtype]
    for M in (48, 100):
        sa, sb = stored_shapes(M, N, K, 0, transB)
        A = make_operand(dtype, *sa, seed=67, tensor=0, scale=0.5)
        B = make_operand(dtype, *sb, seed=67, tensor=1, scale=0.5)
        out_dt = DEFAULT_OUT[dtype]
        ref = O.gemm_i32(A, B, 0, transB) if dtype == O.I8 else O.gemm_f64(dtype, A, B, 0, transB)
        p = hip.plan(hip.make_desc(dtype, M, N, K, dtype_out=out_dt, transB=bool(transB)))
        name = hip.kernel_names()[p.kernel_id]
        assert name.endswith("_splitk_edge") and p.split_k > 1 and p.workspace_bytes == p.split_k * M * N * 4, (name, p.split_k)
        tiles = ((32, 128, 0), (64, 64, 0)) if dtype == O.F32 else ((32, 128, 0), (64, 128, 0))
        cases = [dict(), dict(workspace=False)] + [dict(tile=t, split_k=sk, stages=3) for t in tiles for sk in (1, 2, 8)]
        for kw in cases:
            note(f"case edge split-K {NAMES[dtype]} tB={transB} M={M} N={N} K={K} {kw}")
            got = run_gemm(hip, dtype, A, B, 0, transB, out_dt, M, N, K, **kw)
            if dtype == O.I8:
                assert np.array_equal(got, ref)
            else:
                check(dtype, out_dt, got, ref)


@pytest.mark.parametrize("dtype", [O.F16, O.BF16, O.I8, O.E4M3, O.F32])
@pytest.mark.parametrize("transA,transB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_guarded_kernel_moves_whole_chunks_when_only_k_is_off_the_tile(hip, dtype, transA, transB):
    """K a whole number of 16-byte chunks but no multiple of the K tile, rows on 16-byte boundaries, M and N arbitrary: the
    guarded kernel that stages 16-byte chunks (zero beyond K, whole or not at all) runs instead of the element-wise one"""
    es = {O.F32: 4, O.F16: 2, O.BF16: 2}.get(dtype, 1)
    M, N, K = 208, 400, 2 * BK[dtype] + 3 * (16 // es)
    sa, sb = stored_shapes(M, N, K, transA, transB)
    A = make_operand(dtype, *sa, seed=71, tensor=0, scale=0.5)
    B = make_operand(dtype, *sb, seed=71, tensor=1, scale=0.5)
    out_dt = DEFAULT_OUT[dtype]
    name = hip.kernel_names()[hip.plan(hip.make_desc(dtype, M, N, K, dtype_out=out_dt, transA=bool(transA), transB=bool(transB))).kernel_id]
    assert name.endswith("_guard_chunks"), name
    note(f"case guarded chunks {NAMES[dtype]} tA={transA} tB={transB} M={M} N={N} K={K}")
    got = run_gemm(hip, dtype, A, B, transA, transB, out_dt, M, N, K)
    if dtype == O.I8:
        assert np.array_equal(got, O.gemm_i32(A, B, transA, transB))
        sA, sB = O.uniform(M, 71, 2, 0.001, 0.02), O.uniform(N, 71, 3, 0.001, 0.02)
        got = run_gemm(hip, dtype, A, B, transA, transB, O.F16, M, N, K, epilogue=hip.EPI_ROW_COL_SCALE, sA=sA, sB=sB)
        assert np.array_equal(got, O.epilogue_rowcol_f16(O.gemm_i32(A, B, transA, transB), sA, sB))
    else:
        check(dtype, out_dt, got, O.gemm_f64(dtype, A, B, transA, transB))


def test_edge_kernels_epilogues_accumulation_and_partial_chunks(hip):
    """the edge kernels with scales, accumulation into C and an N that ends inside a lane's 16 bytes of output (the row length of
    C padded to the boundary): int8 with row and column scales to f16 and exact to int32, fp8 with tensor scales to bf16, fp16 with
    fp32 output accumulated into C"""
    M, K = 200, 512
    for N in (392, 396, 397):  # 397: B stored [N][K] only (its rows of C are padded, a B stored [K][N] would have rows of 397 elements)
        Ai = make_operand(O.I8, M, K, seed=62, tensor=0)
        Bi = make_operand(O.I8, N, K, seed=62, tensor=1)
        sA, sB = O.uniform(M, 62, 2, 0.001, 0.02), O.uniform(N, 62, 3, 0.001, 0.02)
        acc = O.gemm_i32(Ai, Bi, 0, 1)
        pad_c = 400 - N
        note(f"case edge epilogue i8 row/col scales N={N}")
        got = run_gemm(hip, O.I8, Ai, Bi, 0, 1, O.F16, M, N, K, epilogue=hip.EPI_ROW_COL_SCALE, sA=sA, sB=sB, pad_c=pad_c)
        assert np.array_equal(got, O.epilogue_rowcol_f16(acc, sA, sB))
        C0 = (np.arange(M * N, dtype=np.int64).reshape(M, N) % 91 - 45).astype(np.int32)
        note(f"case edge epilogue i8 -> i32 accumulate N={N}")
        goti = run_gemm(hip, O.I8, Ai, Bi, 0, 1, O.I32, M, N, K, C_init=C0, clear_accum=False, pad_c=pad_c)
        assert np.array_equal(goti, acc + C0)
        Ae = make_operand(O.E4M3, M, K, seed=63, tensor=0, scale=0.5)
        Be = make_operand(O.E4M3, N, K, seed=63, tensor=1, scale=0.5)
        note(f"case edge epilogue e4m3 tensor scale N={N}")
        gote = run_gemm(hip, O.E4M3, Ae, Be, 0, 1, O.BF16, M, N, K, epilogue=hip.EPI_TENSOR_SCALE, sA=np.array([0.5], np.float32), sB=np.array([0.25], np.float32), pad_c=pad_c)
        check(O.E4M3, O.BF16, gote, O.gemm_f64(O.E4M3, Ae, Be, 0, 1) * 0.125)
        Ah = make_operand(O.F16, M, K, seed=64, tensor=0, scale=0.5)
        Bh = make_operand(O.F16, N, K, seed=64, tensor=1, scale=0.5)
        C0f = O.uniform(M * N, 64, 2, -1.0, 1.0).reshape(M, N).astype(np.float32)
        note(f"case edge epilogue f16 -> f32 accumulate N={N}")
        goth = run_gemm(hip, O.F16, Ah, Bh, 0, 1, O.F32, M, N, K, C_init=C0f, clear_accum=False, pad_c=pad_c)
        check(O.F16, O.F32, goth, O.gemm_f64(O.F16, Ah, Bh, 0, 1) + C0f)


def test_split_k_epilogues_and_accumulate(hip):
    M, N, K = 32, 256, 2048
    A = make_operand(O.I8, M, K, seed=42, tensor=0)
    B = make_operand(O.I8, K, N, seed=42, tensor=1)
    sA, sB = O.uniform(M, 42, 2, 0.001, 0.02), O.uniform(N, 42, 3, 0.001, 0.02)
    acc = O.gemm_i32(A, B)
    got = run_gemm(hip, O.I8, A, B, 0, 0, O.F16, M, N, K, epilogue=hip.EPI_ROW_COL_SCALE, sA=sA, sB=sB, split_k=4)
    assert np.array_equal(got, O.epilogue_rowcol_f16(acc, sA, sB))
    C0 = (np.arange(M * N, dtype=np.int64).reshape(M, N) % 91 - 45).astype(np.int32)
    goti = run_gemm(hip, O.I8, A, B, 0, 0, O.I32, M, N, K, C_init=C0, clear_accum=False, split_k=8)
    assert np.array_equal(goti, acc + C0)
    # fp16 with fp32 output, accumulating into C, ldc padded
    Ah = make_operand(O.F16, M, K, seed=43, tensor=0, scale=0.5)
    Bh = make_operand(O.F16, N, K, seed=43, tensor=1, scale=0.5)
    C0f = O.uniform(M * N, 43, 2, -1.0, 1.0).reshape(M, N).astype(np.float32)
    gotf = run_gemm(hip, O.F16, Ah, Bh, 0, 1, O.F32, M, N, K, C_init=C0f, clear_accum=False, split_k=4, pad=8)
    check(O.F16, O.F32, gotf, O.gemm_f64(O.F16, Ah, Bh, False, True) + C0f.astype(np.float64))


def test_split_k_status_codes(hip):
    import torch
    M, N, K = 32, 256, 2048
    d = hip.make_desc(O.F16, M, N, K, split_k=3)
    with pytest.raises(hip.FriskHipError) as e:
        hip.plan(d)
    assert e.value.status == hip.ERR_TILE
    d = hip.make_desc(O.F16, M, N, K, split_k=4)
    buf = torch.zeros(M * K + K * N + M * N, dtype=torch.float16, device="cuda")
    with pytest.raises(hip.FriskHipError) as e:
        hip.gemm(d, buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), None, None, None, 0, None)
    assert e.value.status == hip.ERR_WORKSPACE
    # a tile named by the descriptor whose variants have no split path: an explicit split is refused
    d = hip.make_desc(O.F32, 256, 256, 2048, tile=(128, 128, 32), split_k=4)
    with pytest.raises(hip.FriskHipError) as e:
        hip.plan(d)
    assert e.value.status == hip.ERR_TILE
    p = hip.plan(hip.make_desc(O.F32, 256, 256, 2048, split_k=4))
    assert p.split_k == 4 and hip.kernel_names()[p.kernel_id].endswith("_splitk")
    # an explicit split looks for a variant that can split: the 256 x 256 tile has one in every layout
    p = hip.plan(hip.make_desc(O.F16, 256, 256, 2048, transA=True, split_k=4))
    assert p.split_k == 4 and hip.kernel_names()[p.kernel_id].endswith("_splitk")


# ------------------------------------------------------------------ grids a little over a whole number of rounds: tail split
@pytest.mark.parametrize("dtype,transA,transB", [(O.F16, 0, 0), (O.BF16, 0, 1), (O.F16, 1, 0), (O.BF16, 1, 1), (O.I8, 0, 0), (O.E4M3, 0, 1)])
def test_tail_split(hip, dtype, transA, transB):
    """17 x 17 = 289 tiles of 256 x 256: one round of 256 and 33 left over, which run as 4 work-groups each (a quarter of the
    32 K tiles apiece; the 8-bit types as 2 each, their slices hold at least 16 K tiles) and are summed through the workspace;
    without a workspace the same launch runs unsplit.  Both give the oracle's result (int8: the same bits)"""
    M = N = 17 * 256
    K = 32 * BK[dtype]
    sa, sb = stored_shapes(M, N, K, transA, transB)
    A = make_operand(dtype, *sa, seed=61, tensor=0, scale=0.5)
    B = make_operand(dtype, *sb, seed=61, tensor=1, scale=0.5)
    out_dt = DEFAULT_OUT[dtype]
    ref = O.gemm_i32(A, B, transA, transB) if dtype == O.I8 else O.gemm_f64(dtype, A, B, transA, transB)
    p = hip.plan(hip.make_desc(dtype, M, N, K, dtype_out=out_dt, transA=bool(transA), transB=bool(transB)))
    ts = 2 if dtype in (O.I8, O.E4M3) else 4
    assert (p.tile_m, p.tile_n, p.tail_tiles, p.tail_split) == (256, 256, 33, ts) and p.workspace_bytes == ts * 33 * 256 * 256 * 4
    for workspace in (True, False):
        note(f"case tail split {NAMES[dtype]} tA={transA} tB={transB} {M}x{N}x{K} workspace={workspace}")
        got = run_gemm(hip, dtype, A, B, transA, transB, out_dt, M, N, K, workspace=workspace)
        if dtype == O.I8:
            assert np.array_equal(got, ref)
        else:
            check(dtype, out_dt, got, ref)


def test_explicit_split_k_on_the_large_tile(hip):
    """512 x 512 x 4096 on 256 x 256 tiles with split_k = 8: 4 tiles x 8 slices, summed by the reduction kernel"""
    M, N, K = 512, 512, 4096
    A = make_operand(O.F16, K, M, seed=65, tensor=0, scale=0.5)   # stored transposed
    B = make_operand(O.F16, K, N, seed=65, tensor=1, scale=0.5)
    note("case explicit split_k=8 on 256x256 tiles, TN")
    got = run_gemm(hip, O.F16, A, B, 1, 0, O.F16, M, N, K, tile=(256, 256, 64), split_k=8)
    check(O.F16, O.F16, got, O.gemm_f64(O.F16, A, B, True, False))
    Ai = make_operand(O.I8, M, K, seed=66, tensor=0)
    Bi = make_operand(O.I8, K, N, seed=66, tensor=1)
    note("case explicit split_k=4 on 256x256 tiles, int8")
    goti = run_gemm(hip, O.I8, Ai, Bi, 0, 0, O.I32, M, N, K, tile=(256, 256, 128), split_k=4)
    assert np.array_equal(goti, O.gemm_i32(Ai, Bi))


def test_tail_split_with_the_xcd_tile_map(hip):
    """11 x 24 = 264 tiles, a multiple of 8, so work-group ids are regrouped per XCD; the 8 tiles left over after one round run as
    8 work-groups each, 8 of the 64 K tiles apiece"""
    M, N, K = 11 * 256, 24 * 256, 64 * 64
    A = make_operand(O.F16, M, K, seed=64, tensor=0, scale=0.5)
    B = make_operand(O.F16, N, K, seed=64, tensor=1, scale=0.5)
    p = hip.plan(hip.make_desc(O.F16, M, N, K, transB=True))
    assert (p.tail_tiles, p.tail_split, p.xcd_remap) == (8, 8, 1)
    note(f"case tail split with xcd map {M}x{N}x{K}")
    got = run_gemm(hip, O.F16, A, B, 0, 1, O.F16, M, N, K)
    check(O.F16, O.F16, got, O.gemm_f64(O.F16, A, B, False, True))


def test_tail_split_epilogues_and_accumulate(hip):
    M = N = 17 * 256
    K = 32 * 128
    A = make_operand(O.I8, M, K, seed=62, tensor=0)
    B = make_operand(O.I8, K, N, seed=62, tensor=1)
    sA, sB = O.uniform(M, 62, 2, 0.001, 0.02), O.uniform(N, 62, 3, 0.001, 0.02)
    acc = O.gemm_i32(A, B)
    note("case tail split int8 dequant epilogue")
    got = run_gemm(hip, O.I8, A, B, 0, 0, O.F16, M, N, K, epilogue=hip.EPI_ROW_COL_SCALE, sA=sA, sB=sB)
    assert np.array_equal(got, O.epilogue_rowcol_f16(acc, sA, sB))
    C0 = (np.arange(M * N, dtype=np.int64).reshape(M, N) % 91 - 45).astype(np.int32)
    note("case tail split int8 accumulate into int32")
    goti = run_gemm(hip, O.I8, A, B, 0, 0, O.I32, M, N, K, C_init=C0, clear_accum=False)
    assert np.array_equal(goti, acc + C0)
    K = 32 * 64
    Ah = make_operand(O.F16, M, K, seed=63, tensor=0, scale=0.5)
    Bh = make_operand(O.F16, N, K, seed=63, tensor=1, scale=0.5)
    C0f = O.uniform(M * N, 63, 2, -1.0, 1.0).reshape(M, N).astype(np.float32)
    note("case tail split fp16 -> fp32 accumulate, padded ldc")
    gotf = run_gemm(hip, O.F16, Ah, Bh, 0, 1, O.F32, M, N, K, C_init=C0f, clear_accum=False, pad=8)
    check(O.F16, O.F32, gotf, O.gemm_f64(O.F16, Ah, Bh, False, True) + C0f.astype(np.float64))


def test_config_fp8_skinny_decode(hip):
    """M = 32, N = K = 8192, e4m3 with per-tensor scales, bf16 output: every row checked"""
    M, N, K = 32, 8192, 8192
    xa, xb = O.normal(M * K, 4, 0, 1.0), O.normal(N * K, 4, 1, 1.0)
    sA, sB = np.float32(np.abs(xa).max() / 448.0), np.float32(np.abs(xb).max() / 448.0)
    A = O.encode(O.E4M3, xa / sA).reshape(M, K)
    B = O.encode(O.E4M3, xb / sB).reshape(N, K)
    del xa, xb
    d = hip.make_desc(O.E4M3, M, N, K, dtype_out=O.BF16, transB=True, epilogue=hip.EPI_TENSOR_SCALE)
    p = hip.plan(d)
    assert p.tile_m == 32 and p.grid_x * p.grid_y * p.split_k >= 256
    got = run_gemm(hip, O.E4M3, A, B, 0, 1, O.BF16, M, N, K, epilogue=hip.EPI_TENSOR_SCALE, sA=[sA], sB=[sB])
    ref = O.epilogue_tensor(O.gemm_f64(O.E4M3, A, B, False, True), sA, sB)
    r = check(O.E4M3, O.BF16, got, ref)
    note(f"fp8 skinny 32x8192x8192 NT split_k={p.split_k}: {r}")
