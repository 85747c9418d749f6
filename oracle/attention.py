"""CPU restatement of the reference's fused-attention sketch -- TEST INFRASTRUCTURE ONLY.

tmp/ir.mlir:87-157 writes the kernel as dialect ops: copy a Q tile; for every tile of 64 keys { copy K; gemm
(scores); copy the old running maximum (:111); reduce max (:113); block: scale = exp2(cst * (old max - new max))
(:114-122); block: scores = exp2(cst * scores - cst * max) (:123-131); reduce sum (:132); block: logsum = logsum *
scale + sum (:133-140); copy scores -> 16-bit (:141); block: acc_o *= scale (:142-147); copy V; gemm (acc_o +=
P V) }; copy acc_o out (:151-152).  The sketch is not executable (the builder has no arith / math ops and nothing
lowers the dialect), it never divides by logsum, and it holds no numbers: numerical parity against the reference is
unpinned.  What is restated and what pins it:
  attention_tiled  the sketch's loop, tile by tile, with the final division by the denominator added; `cst` is
                   scale * log2(e), probabilities are rounded to the element type before the second product
  attention_f64    the same function without tiles: softmax(scale * Q K^T) V in float64
Pins (tests/test_attention.py): the two agree (the running-maximum recurrence is an identity); constant scores give
the mean of V; one dominant key returns its V row; a single key tile reduces to a plain softmax; scipy's softmax and
logsumexp on the same scores.
Arrays are in the storage types of oracle.NP_STORAGE (uint16 for f16 / bf16), shapes [batch*heads, seq, head_dim]
(K as [batch*heads, head_dim, seq_k] when k_transposed).
"""
import numpy as np

import oracle as O

LOG2E = 1.4426950408889634


def _decode(dtype, x):
    return O.decode(dtype, np.ascontiguousarray(x).reshape(-1)).astype(np.float64).reshape(x.shape)


def _operands(dtype, Q, K, V, k_transposed):
    q, k, v = _decode(dtype, Q), _decode(dtype, K), _decode(dtype, V)
    if k_transposed:
        k = np.swapaxes(k, 1, 2)
    return q, k, v


def attention_f64(dtype, Q, K, V, scale, k_transposed=False):
    """(O, lse) in float64: O = softmax(scale * Q K^T) V, lse = log sum_k exp(scale * s_k)"""
    q, k, v = _operands(dtype, Q, K, V, k_transposed)
    out = np.empty(q.shape[:2] + (v.shape[2],), dtype=np.float64)
    lse = np.empty(q.shape[:2], dtype=np.float64)
    for h in range(q.shape[0]):
        s = scale * (q[h] @ k[h].T)
        m = s.max(axis=1, keepdims=True)
        e = np.exp(s - m)
        den = e.sum(axis=1, keepdims=True)
        out[h] = (e @ v[h]) / den
        lse[h] = (m + np.log(den))[:, 0]
    return out, lse


def attention_tiled(dtype, Q, K, V, scale, k_transposed=False, key_tile=64, round_p=True):
    """the sketch's loop (tmp/ir.mlir:107-150) in float64 arithmetic, probabilities rounded to `dtype` when round_p"""
    q, k, v = _operands(dtype, Q, K, V, k_transposed)
    cst = scale * LOG2E
    out = np.empty(q.shape[:2] + (v.shape[2],), dtype=np.float64)
    lse = np.empty(q.shape[:2], dtype=np.float64)
    for h in range(q.shape[0]):
        nq = q.shape[1]
        acc_o = np.zeros((nq, v.shape[2]))                 # fill(acc_o, 0)      :104
        logsum = np.zeros(nq)                              # fill(logsum, 0)     :105
        scores_max = np.full(nq, -np.inf)                  # fill(scores_max, -inf) :106
        for k0 in range(0, k.shape[1], key_tile):
            acc_s = q[h] @ k[h, k0:k0 + key_tile].T        # gemm                :110
            prev = scores_max.copy()                       # copy                :111
            scores_max = np.maximum(prev, acc_s.max(axis=1))   # reduce max (accumulating)
            scores_scale = np.exp2(prev * cst - scores_max * cst)          # :114-122
            acc_s = np.exp2(acc_s * cst - scores_max[:, None] * cst)       # :123-131
            logsum = logsum * scores_scale + acc_s.sum(axis=1)             # :132-140
            if round_p:                                                    # copy f32 -> 16-bit :141
                acc_s = _decode(dtype, O.encode(dtype, acc_s.astype(np.float32).reshape(-1)).reshape(acc_s.shape))
            acc_o = acc_o * scores_scale[:, None] + acc_s @ v[h, k0:k0 + key_tile]   # :142-149
        out[h] = acc_o / logsum[:, None]
        lse[h] = (scores_max * cst + np.log2(logsum)) / LOG2E
    return out, lse
