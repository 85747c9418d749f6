"""Fused attention forward: the oracle against closed forms and scipy (CPU), the C ABI's argument checks (CPU), and the
HIP kernel against the oracle through the C ABI (GPU).

Bar (16-bit operands, fp32 accumulation), against the float64 softmax(scale * Q K^T) V: ||D - R||_F / ||R||_F <= 1e-2,
and for every element |d - r| <= tol * max(|r|, rms(R)) with tol = 1e-2 for f16 and 2e-2 for bf16 (the probabilities
enter the second product rounded to the element type: bf16 leaves each with up to 2^-8 relative error, which over a
few hundred keys reaches 1e-2 of the output's rms in the worst of 10^5 elements); log-sum-exp within 1e-3 (f16) or
4e-3 (bf16) absolute: the denominator is the sum of the rounded probabilities, the one the output is normalised
by, so a row dominated by one key carries that key's rounding, 2^-11 or 2^-8 relative."""
import numpy as np
import pytest

import oracle as O
from oracle import attention as A

NAMES = {O.F16: "f16", O.BF16: "bf16"}
ELEMENT_TOL = {O.F16: 1e-2, O.BF16: 2e-2}
LSE_TOL = {O.F16: 1e-3, O.BF16: 4e-3}


def make_qkv(dtype, bh, sq, sk, d, seed, k_transposed=False, q_scale=1.0):
    q = O.encode(dtype, O.normal(bh * sq * d, seed, 0, q_scale)).reshape(bh, sq, d)
    k = O.encode(dtype, O.normal(bh * sk * d, seed, 1, 1.0)).reshape(bh, sk, d)
    v = O.encode(dtype, O.normal(bh * sk * d, seed, 2, 1.0)).reshape(bh, sk, d)
    if k_transposed:
        k = np.ascontiguousarray(np.swapaxes(k, 1, 2))
    return q, k, v


# ------------------------------------------------------------------ oracle (CPU)
def test_oracle_tiled_recurrence_equals_plain_softmax():
    q, k, v = make_qkv(O.F16, 2, 40, 192, 16, seed=3)
    ref, lse = A.attention_f64(O.F16, q, k, v, 0.25)
    for tile in (64, 32, 192):
        out, l2 = A.attention_tiled(O.F16, q, k, v, 0.25, key_tile=tile, round_p=False)
        assert np.allclose(out, ref, rtol=1e-12, atol=1e-12) and np.allclose(l2, lse, rtol=1e-12, atol=1e-12)
    # rounding the probabilities to f16 moves the result by about one f16 ulp of a probability, not more
    out, _ = A.attention_tiled(O.F16, q, k, v, 0.25, round_p=True)
    assert np.abs(out - ref).max() < 2e-3 and np.abs(out - ref).max() > 0
    # transposed storage of K is the same function
    kt = np.ascontiguousarray(np.swapaxes(k, 1, 2))
    out_t, lse_t = A.attention_f64(O.F16, q, kt, v, 0.25, k_transposed=True)
    assert np.array_equal(out_t, ref) and np.array_equal(lse_t, lse)


def test_oracle_against_scipy_and_closed_forms():
    from scipy.special import logsumexp, softmax
    q, k, v = make_qkv(O.BF16, 1, 24, 128, 32, seed=5)
    scale = 0.3
    ref, lse = A.attention_f64(O.BF16, q, k, v, scale)
    dec = lambda x: O.decode(O.BF16, x.reshape(-1)).astype(np.float64).reshape(x.shape)
    s = scale * dec(q)[0] @ dec(k)[0].T
    assert np.allclose(ref[0], softmax(s, axis=1) @ dec(v)[0], rtol=1e-12, atol=1e-13)
    assert np.allclose(lse[0], logsumexp(s, axis=1), rtol=1e-12)
    # K = 0: every score is equal, the output is the mean of V and lse = log(number of keys)
    zero_k = np.zeros_like(k)
    out, l0 = A.attention_tiled(O.BF16, q, zero_k, v, scale, round_p=False)
    assert np.allclose(out[0], np.broadcast_to(dec(v)[0].mean(axis=0), out[0].shape), atol=1e-12) and np.allclose(l0, np.log(128))
    # one key dominating by 200 nats: the output is that key's row of V
    qq = O.encode(O.F16, np.full(16, 4.0, dtype=np.float32)).reshape(1, 1, 16)
    kk = O.encode(O.F16, np.zeros(64 * 16, dtype=np.float32)).reshape(1, 64, 16)
    kk[0, 37] = O.encode(O.F16, np.full(16, 4.0, dtype=np.float32))
    vv = O.encode(O.F16, O.normal(64 * 16, 6, 0, 1.0)).reshape(1, 64, 16)
    out, l1 = A.attention_tiled(O.F16, qq, kk, vv, 1.0)
    assert np.allclose(out[0, 0], O.decode(O.F16, vv[0, 37]), atol=1e-12) and np.allclose(l1, 256.0)


# ------------------------------------------------------------------ C ABI argument checks (no device needed)
def test_attention_status_codes_before_any_launch():
    from frisk_amd import runtime as R

    def status(desc, *ptrs):
        with pytest.raises(R.FriskHipError) as e:
            R.attention(desc, *ptrs)
        return e.value.status

    ok = dict(batch=1, heads=2, seq_q=256, seq_k=128)
    p = 1 << 20
    assert status(R.make_attention_desc(R.F32, **ok), p, p, p, p) == R.ERR_DTYPE
    assert status(R.make_attention_desc(R.F16, head_dim=64, **ok), p, p, p, p) == R.ERR_SHAPE
    assert status(R.make_attention_desc(R.F16, 1, 2, 200, 128), p, p, p, p) == R.ERR_SHAPE
    assert status(R.make_attention_desc(R.F16, 1, 2, 256, 100), p, p, p, p) == R.ERR_SHAPE
    assert status(R.make_attention_desc(R.F16, 1, 2, 256, 0), p, p, p, p) == R.ERR_SHAPE
    assert status(R.make_attention_desc(R.F16, scale=0.0, **ok), p, p, p, p) == R.ERR_ARGUMENT
    assert status(R.make_attention_desc(R.F16, scale=float("nan"), **ok), p, p, p, p) == R.ERR_ARGUMENT
    assert status(R.make_attention_desc(R.F16, **ok), None, p, p, p) == R.ERR_NULL
    assert status(R.make_attention_desc(R.F16, **ok), p, p + 8, p, p) == R.ERR_ALIGNMENT
    d = R.make_attention_desc(R.F16, **ok)
    d.abi_version = 99
    assert status(d, p, p, p, p) == R.ERR_ABI
    # nothing to do: no launch, no device needed
    R.attention(R.make_attention_desc(R.F16, 0, 2, 256, 128), None, None, None, None)


# ------------------------------------------------------------------ HIP kernel vs oracle (GPU)
def run_attention(dtype, q, k, v, scale, k_transposed=False, want_lse=True):
    import torch
    from frisk_amd import runtime as R
    from helpers import to_dev, from_dev
    bh, sq, d = q.shape
    sk = v.shape[1]
    dq, dk, dv = to_dev(q), to_dev(k), to_dev(v)
    do = torch.full((bh * sq * d * 2,), 0xFF, dtype=torch.uint8, device="cuda")
    dl = torch.full((bh * sq,), float("nan"), dtype=torch.float32, device="cuda") if want_lse else None
    desc = R.make_attention_desc(dtype, 1, bh, sq, sk, d, scale, k_transposed)
    R.attention(desc, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr(), dl.data_ptr() if want_lse else None,
                torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return from_dev(do, np.uint16, (bh, sq, d)), (dl.cpu().numpy().reshape(bh, sq) if want_lse else None)


def check(dtype, got, lse, ref, ref_lse):
    r = O.compare(dtype, got, ref)
    assert r["nonfinite"] == 0 and r["max_rel"] <= ELEMENT_TOL[dtype] and r["fro_rel"] <= 1e-2, r
    if lse is not None:
        assert np.abs(lse - ref_lse).max() <= LSE_TOL[dtype], np.abs(lse - ref_lse).max()
    return r


CASES = [
    # (batch*heads, seq_q, seq_k, scale)           what it exercises
    (2, 256, 64, None),        # one key tile
    (1, 256, 128, None),       # two tiles: the ring never wraps
    (3, 512, 448, None),       # ring wraps; 6 work-groups: no XCD remap
    (8, 256, 1024, 0.5),       # 8 work-groups: XCD remap; sharp softmax, the running maximum moves often
    (16, 512, 256, 0.02),      # nearly uniform probabilities
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [O.F16, O.BF16], ids=lambda d: NAMES[d])
@pytest.mark.parametrize("k_transposed", [False, True], ids=["k_rows", "k_transposed"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "bh%d_q%d_k%d" % c[:3])
def test_attention_matches_oracle(dtype, k_transposed, case):
    bh, sq, sk, scale = case
    scale = 128 ** -0.5 if scale is None else scale
    q, k, v = make_qkv(dtype, bh, sq, sk, 128, seed=11 + bh, k_transposed=k_transposed)
    got, lse = run_attention(dtype, q, k, v, scale, k_transposed)
    ref, ref_lse = A.attention_f64(dtype, q, k, v, scale, k_transposed)
    check(dtype, got, lse, ref, ref_lse)
    # the tile-by-tile restatement rounds its probabilities against each tile's running maximum, the kernel against
    # a reference it raises less often: the roundings differ element by element, the aggregate error does not
    tiled, _ = A.attention_tiled(dtype, q, k, v, scale, k_transposed)
    r = O.compare(dtype, got, tiled)
    assert r["fro_rel"] <= 5e-3, r


@pytest.mark.gpu
def test_attention_closed_forms_on_device():
    dtype, bh, sq, sk, d = O.F16, 2, 256, 320, 128
    q, k, v = make_qkv(dtype, bh, sq, sk, d, seed=21)
    # K = 0: the output is the mean of V over the keys, lse = log(seq_k)
    got, lse = run_attention(dtype, q, np.zeros_like(k), v, 0.1)
    mean = O.decode(dtype, v.reshape(-1)).astype(np.float64).reshape(bh, sk, d).mean(axis=1)
    r = O.compare(dtype, got, np.broadcast_to(mean[:, None, :], (bh, sq, d)))
    assert r["max_rel"] <= 1e-2 and np.abs(lse - np.log(sk)).max() <= 1e-4
    # V with equal rows: the output is that row whatever the probabilities are (rows sum to one)
    row = O.encode(dtype, O.normal(d, 22, 0, 1.0))
    vc = np.broadcast_to(row, (bh, sk, d)).copy()
    got, _ = run_attention(dtype, q, k, vc, 0.2, want_lse=False)
    want = np.broadcast_to(O.decode(dtype, row).astype(np.float64), (bh, sq, d))
    assert O.compare(dtype, got, want)["max_rel"] <= 2e-3
    # one key far above the rest: its row of V comes back exactly
    qq = O.encode(dtype, np.full(bh * sq * d, 1.0, dtype=np.float32)).reshape(bh, sq, d)
    kk = np.zeros_like(k)
    kk[:, 133] = O.encode(dtype, np.full(d, 1.0, dtype=np.float32))
    got, lse = run_attention(dtype, qq, kk, v, 1.0)
    assert np.array_equal(got, np.broadcast_to(v[:, 133:134], (bh, sq, d))) and np.abs(lse - 128.0).max() <= 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("k_transposed", [False, True], ids=["k_rows", "k_transposed"])
def test_attention_sketch_shape_32_heads_4096(k_transposed):
    """the shape of the reference sketch (tmp/ir.mlir:88: 1 x 32 x 4096 x 128); the oracle checks three heads, the
    rest through the property that a head's output does not depend on which head slot it occupies"""
    dtype, bh, s, d = O.F16, 32, 4096, 128
    q1, k1, v1 = make_qkv(dtype, 3, s, s, d, seed=31, k_transposed=k_transposed)
    pick = [0, 1, 2] * 10 + [2, 0]
    q, k, v = q1[pick], k1[pick], v1[pick]
    got, lse = run_attention(dtype, q, k, v, d ** -0.5, k_transposed)
    ref, ref_lse = A.attention_f64(dtype, q1, k1, v1, d ** -0.5, k_transposed)
    for slot in (0, 1, 31):
        check(dtype, got[slot], lse[slot], ref[pick[slot]], ref_lse[pick[slot]])
    for slot in range(3, bh):
        assert np.array_equal(got[slot], got[pick[slot]]) and np.array_equal(lse[slot], lse[pick[slot]])
