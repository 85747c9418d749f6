"""Pins the CPU oracle (oracle/frisk_oracle.c) without the reference.

The reference holds no arithmetic and no numerical vectors for the GEMM path
(its tests only print IR), so each oracle routine is pinned by mathematics:
exhaustive codec tables against numpy / torch, closed forms (identity, all-ones,
rank-1 products), integer exactness against numpy int64, and numpy's own
float64 matmul of the decoded operands.  A dropped term, a swapped index or a
transposed operand fails at least one of these.
"""
import numpy as np
import pytest
import torch

import oracle as O


# ------------------------------------------------------------------ codecs
def test_f16_decode_all_codes_matches_numpy():
    codes = np.arange(65536, dtype=np.uint16)
    mine = O.decode(O.F16, codes)
    ref = codes.view(np.float16).astype(np.float32)
    assert np.array_equal(mine.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    assert np.all(np.isnan(mine[np.isnan(ref)]))


def test_f16_encode_round_to_nearest_even_matches_numpy():
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 3.0,
        (rng.standard_normal(100000) * 1e-6).astype(np.float32),      # half subnormals and underflow
        (rng.standard_normal(50000) * 4e4).astype(np.float32),        # around the overflow threshold 65504/65520
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, np.inf, -np.inf],
                 dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.encode(O.F16, x), ref)
    # every finite code survives decode -> encode, and every tie (midpoint of neighbours) goes to the even code
    codes = np.arange(0x7C00, dtype=np.uint16)
    vals = O.decode(O.F16, codes)
    assert np.array_equal(O.encode(O.F16, vals), codes)
    mid = ((vals[:-1].astype(np.float64) + vals[1:].astype(np.float64)) / 2).astype(np.float32)  # exact in fp32
    enc = O.encode(O.F16, mid)
    assert np.all(enc % 2 == 0) and np.all((enc == codes[:-1]) | (enc == codes[1:]))


def test_bf16_codec_matches_torch():
    codes = np.arange(65536, dtype=np.uint16)
    mine = O.decode(O.BF16, codes)
    ref = (codes.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(mine.view(np.uint32), ref.view(np.uint32))
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.standard_normal(300000).astype(np.float32) * 10, (rng.standard_normal(1000) * 1e-38).astype(np.float32),
                        np.array([0.0, -0.0, 3.3895314e38, np.inf, -np.inf, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8], dtype=np.float32)])
    ref_enc = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.encode(O.BF16, x), ref_enc)


def _e4m3_table():
    """the 256 values of OCP e4m3fn from the format definition (bias 7, no inf, S.1111.111 = NaN)"""
    t = np.empty(256, dtype=np.float64)
    for c in range(256):
        e, m, s = (c >> 3) & 0xF, c & 7, -1.0 if c & 0x80 else 1.0
        if e == 0xF and m == 7:
            t[c] = np.nan
        elif e == 0:
            t[c] = s * m * 2.0 ** -9
        else:
            t[c] = s * (1 + m / 8.0) * 2.0 ** (e - 7)
    return t


def test_e4m3_decode_table():
    table = _e4m3_table()
    mine = O.decode(O.E4M3, np.arange(256, dtype=np.uint8)).astype(np.float64)
    ok = ~np.isnan(table)
    assert np.array_equal(mine[ok], table[ok]) and np.all(np.isnan(mine[~ok]))
    assert np.nanmax(table) == 448.0 and table[1] == 2.0 ** -9 and np.isnan(table[0x7F]) and np.isnan(table[0xFF])
    tref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy().astype(np.float64)
    assert np.array_equal(tref[ok], table[ok])


def test_e4m3_encode_is_nearest_even_with_saturation():
    table = _e4m3_table()
    pos = table[:0x7F]                                   # 0 .. 448 ascending
    rng = np.random.default_rng(3)
    x = np.concatenate([rng.standard_normal(100000) * 100, rng.standard_normal(100000), rng.standard_normal(50000) * 0.01,
                        (pos[:-1] + pos[1:]) / 2, -(pos[:-1] + pos[1:]) / 2, pos, [448.0, 464.0, 465.0, 1e6, -1e6, 0.0]]).astype(np.float32)
    enc = O.encode(O.E4M3, x)
    a = np.abs(x.astype(np.float64))
    # brute force: nearest table entry, ties to the even code, beyond 448 saturates
    d = np.abs(a[:, None] - pos[None, :])
    best = d.min(axis=1)
    cand = d == best[:, None]
    lo = cand.argmax(axis=1)
    hi = 0x7E - cand[:, ::-1].argmax(axis=1)
    want = np.where(lo == hi, lo, np.where(lo % 2 == 0, lo, hi))
    want = np.where(a >= 448.0, 0x7E, want).astype(np.uint8)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    assert np.array_equal(enc, want | sign)
    # torch agrees wherever it does not overflow to NaN
    inr = a <= 448.0
    tenc = torch.from_numpy(x[inr]).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(enc[inr] & 0x7F, tenc & 0x7F)
    assert O.encode(O.E4M3, np.array([np.nan], dtype=np.float32))[0] & 0x7F == 0x7F


# ------------------------------------------------------------------ RNG
def test_rng_is_counter_based_and_in_range():
    a = O.uniform(1000, 0, 0, -1.0, 1.0)
    b = O.uniform(5000, 0, 0, -1.0, 1.0)
    assert np.array_equal(a, b[:1000])                   # value i does not depend on how many are drawn
    assert not np.array_equal(a, O.uniform(1000, 1, 0, -1.0, 1.0)) and not np.array_equal(a, O.uniform(1000, 0, 1, -1.0, 1.0))
    assert a.min() >= -1.0 and a.max() <= 1.0
    u = O.uniform(400000, 7, 3, 0.001, 0.02)
    assert u.min() >= 0.001 and u.max() <= 0.02 and abs(u.mean() - 0.0105) < 1e-4
    z = O.normal(400000, 1, 0, 1.0)
    assert abs(z.mean()) < 0.01 and abs(z.std() - 1.0) < 0.01 and abs((z ** 3).mean()) < 0.03
    i8 = O.int8_uniform(510000, 3, 0)
    assert i8.min() == -127 and i8.max() == 127
    counts = np.bincount(i8.astype(np.int32) + 127, minlength=255)
    assert counts.min() > 1700 and counts.max() < 2300  # 2000 expected per value


# ------------------------------------------------------------------ GEMM
SHAPES = [(1, 1, 1), (3, 5, 7), (37, 29, 53), (130, 70, 300), (5, 2049, 257), (64, 64, 512)]


@pytest.mark.parametrize("dtype", [O.F32, O.F16, O.BF16, O.E4M3, O.I8])
@pytest.mark.parametrize("transA,transB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_blocked_gemm_matches_numpy_and_naive(dtype, transA, transB):
    rng = np.random.default_rng(10 * dtype + 2 * transA + transB)
    for (m, n, k) in SHAPES:
        sa, sb = ((k, m) if transA else (m, k)), ((n, k) if transB else (k, n))
        if dtype == O.I8:
            A = rng.integers(-127, 128, sa).astype(np.int8)
            B = rng.integers(-127, 128, sb).astype(np.int8)
        else:
            A = O.encode(dtype, rng.standard_normal(sa).astype(np.float32))
            B = O.encode(dtype, rng.standard_normal(sb).astype(np.float32))
        Af, Bf = O.decode(dtype, A).astype(np.float64), O.decode(dtype, B).astype(np.float64)
        ref = (Af.T if transA else Af) @ (Bf.T if transB else Bf)   # numpy's own matmul: an independent implementation
        got = O.gemm_f64(dtype, A, B, transA, transB)
        assert np.allclose(got, ref, rtol=1e-12, atol=1e-12)
        assert np.allclose(O.gemm_naive(dtype, A, B, transA, transB), ref, rtol=1e-12, atol=1e-12)
        assert np.allclose(O.gemm_f32(dtype, A, B, transA, transB), ref, rtol=2e-5, atol=2e-5 * max(1.0, np.abs(ref).max()))
        if dtype == O.I8:
            exact = (A.astype(np.int64).T if transA else A.astype(np.int64)) @ (B.astype(np.int64).T if transB else B.astype(np.int64))
            assert np.array_equal(O.gemm_i32(A, B, transA, transB), exact.astype(np.int32))


def test_gemm_closed_forms():
    n, k = 96, 160
    eye = O.encode(O.F16, np.eye(n, dtype=np.float32))
    B = O.encode(O.F16, O.normal(n * n, 5, 1).reshape(n, n))
    assert np.array_equal(O.gemm_f64(O.F16, eye, B), O.decode(O.F16, B).astype(np.float64))      # I.B = B
    assert np.array_equal(O.gemm_f64(O.F16, B, eye, True, False), O.decode(O.F16, B).T.astype(np.float64))  # B^T.I = B^T
    ones_a = O.encode(O.BF16, np.ones((n, k), dtype=np.float32))
    ones_b = O.encode(O.BF16, np.ones((k, n), dtype=np.float32))
    assert np.all(O.gemm_f64(O.BF16, ones_a, ones_b) == float(k))                                  # all ones -> K
    # rank-1: (u 1^T)(1 v^T) = K u v^T with small integers, exactly representable
    u = (np.arange(n) % 7 - 3).astype(np.float32)
    v = (np.arange(n) % 5 - 2).astype(np.float32)
    A1 = O.encode(O.F16, np.outer(u, np.ones(k, dtype=np.float32)))
    B1 = O.encode(O.F16, np.outer(np.ones(k, dtype=np.float32), v))
    assert np.array_equal(O.gemm_f64(O.F16, A1, B1), k * np.outer(u, v).astype(np.float64))
    # a non-symmetric case that a transposed operand or swapped indices would break
    A2 = np.zeros((4, 3), dtype=np.float32); A2[1, 2] = 2.0
    B2 = np.zeros((3, 5), dtype=np.float32); B2[2, 4] = 3.0
    want = np.zeros((4, 5)); want[1, 4] = 6.0
    assert np.array_equal(O.gemm_f64(O.F32, A2, B2), want)
    assert np.array_equal(O.gemm_f64(O.F32, np.ascontiguousarray(A2.T), B2, True, False), want)
    assert np.array_equal(O.gemm_f64(O.F32, A2, np.ascontiguousarray(B2.T), False, True), want)


def test_row_window_equals_slice_of_full_result():
    A = O.encode(O.F16, O.normal(200 * 96, 9, 0).reshape(200, 96))
    B = O.encode(O.F16, O.normal(96 * 80, 9, 1).reshape(96, 80))
    full = O.gemm_f64(O.F16, A, B)
    assert np.array_equal(O.gemm_f64(O.F16, A, B, row0=57, nrows=31), full[57:88])
    assert O.gemm_f64(O.F16, A, B, row0=10, nrows=0).shape == (0, 80)


def test_int8_accumulator_bound_of_the_benchmark_shape():
    # K = 4096 of extreme values stays inside int32: 4096 * 127^2 = 66 064 384 < 2^31
    A = np.full((4, 4096), -127, dtype=np.int8)
    B = np.full((4096, 4), 127, dtype=np.int8)
    assert np.all(O.gemm_i32(A, B) == -4096 * 127 * 127)


# ------------------------------------------------------------------ epilogues and norms
def test_dequant_epilogue_order_and_rounding():
    rng = np.random.default_rng(4)
    acc = rng.integers(-60_000_000, 60_000_000, (33, 47)).astype(np.int32)
    sA = rng.uniform(0.001, 0.02, 33).astype(np.float32)
    sB = rng.uniform(0.001, 0.02, 47).astype(np.float32)
    want32 = (acc.astype(np.float32) * sA[:, None]) * sB[None, :]          # numpy float32: each multiply rounds once
    assert np.array_equal(O.epilogue_rowcol_f32(acc, sA, sB), want32)
    with np.errstate(over="ignore"):
        assert np.array_equal(O.epilogue_rowcol_f16(acc, sA, sB), want32.astype(np.float16).view(np.uint16))
    # power-of-two scales: exact closed form
    small = rng.integers(-2 ** 20, 2 ** 20, (8, 8)).astype(np.int32)
    out = O.epilogue_rowcol_f32(small, np.full(8, 2.0 ** -10, np.float32), np.full(8, 2.0 ** -6, np.float32))
    assert np.array_equal(out, small.astype(np.float32) * np.float32(2.0 ** -16))
    t = O.epilogue_tensor(np.array([[1.5, -2.0]]), 0.5, 4.0)
    assert np.array_equal(t, np.array([[3.0, -4.0]]))


def test_compare_norms():
    ref = np.array([1.0, -2.0, 0.0, 4.0])
    got = np.array([1.0, -2.0, 0.5, 4.0], dtype=np.float32)
    r = O.compare(O.F32, got, ref)
    rms = np.sqrt((1 + 4 + 0 + 16) / 4)
    assert abs(r["rms"] - rms) < 1e-12 and abs(r["max_rel"] - 0.5 / rms) < 1e-12
    assert abs(r["fro_rel"] - 0.5 / np.sqrt(21.0)) < 1e-12 and r["nonfinite"] == 0
    assert O.compare(O.F32, np.array([np.inf, 1.0], dtype=np.float32), np.array([1.0, 1.0]))["nonfinite"] == 1
