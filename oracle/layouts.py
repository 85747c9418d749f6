"""CPU restatement of the reference's GEMM layout inference (NVIDIA targets), numerically: every layout is a function
from logical (i, j) to integers, evaluated with numpy over a whole tile.  TEST INFRASTRUCTURE ONLY: nothing in the
product imports this; it exists so that the pieces of the reference's algorithm that the gfx950 planner re-targets
(wave partition, XOR swizzles of 16-byte chunks, fragment composition by repeat/replicate, the bank-conflict count) are
pinned against the layout strings and statistics the reference itself holds (tests/golden/nvidia_gemm_layouts.json).

Follows lib/Dialect/Frisk/IR/FriskOps.cpp of the reference:
  xor2x2/4x4/8x8 :123-143, FragmentExpr.repeat/replicate :155-231, atoms :233-287, accumulator fragments :304-347,
  operand fragments :349-451, linear/padded layouts :453-470, bank swizzles :500-558, selectors :560-618,
  inferGemmInst :620-625, computeWarpPartition :825-888, GemmOp::inferLayout :1285-1407
and exp/layout/gemm_layout_tool.cpp: analyzeLayout :135-208, analyzeRowMajorBaseline :210-263.
Also holds a small evaluator for the textual affine_map form those strings are written in.
"""
import re

import numpy as np


# ------------------------------------------------------------------ affine_map text evaluator
_TOKEN = re.compile(r"\s*(floordiv|ceildiv|mod|d\d+|s\d+|\d+|[()+\-*,])")


class _Parser:
    def __init__(self, text, dims, symbols=()):
        self.symbols = symbols
        self.toks = _TOKEN.findall(text)
        if "".join(self.toks) != re.sub(r"\s+", "", text):
            raise ValueError("cannot tokenize affine expression: %r" % text)
        self.pos = 0
        self.dims = dims

    def peek(self):
        return self.toks[self.pos] if self.pos < len(self.toks) else None

    def take(self):
        t = self.peek()
        self.pos += 1
        return t

    def expr(self):  # sums bind weakest
        v = self.term()
        while self.peek() in ("+", "-"):
            op = self.take()
            r = self.term()
            v = v + r if op == "+" else v - r
        return v

    def term(self):  # *, floordiv, ceildiv, mod: one level, left to right
        v = self.factor()
        while self.peek() in ("*", "floordiv", "ceildiv", "mod"):
            op = self.take()
            r = self.factor()
            if op == "*":
                v = v * r
            elif op == "floordiv":
                v = np.floor_divide(v, r)
            elif op == "ceildiv":
                v = -np.floor_divide(-v, r)
            else:
                v = np.mod(v, r)
        return v

    def factor(self):
        t = self.take()
        if t == "(":
            v = self.expr()
            if self.take() != ")":
                raise ValueError("unbalanced parentheses")
            return v
        if t == "-":
            return -self.factor()
        if t[0] == "d":
            return self.dims[int(t[1:])]
        if t[0] == "s":
            return self.symbols[int(t[1:])]
        return np.int64(int(t))


def eval_affine_map(text, *dims, symbols=()):
    """`affine_map<(d0, d1)[s0] -> (e0, e1, ...)>` (the `affine_map<>` wrapper and the symbol list are optional) evaluated at
    integer (arrays of) d0, d1, ... and symbol values; returns the list of results"""
    m = re.fullmatch(r"\s*(?:affine_map<)?\(([^)]*)\)\s*(?:\[([^\]]*)\])?\s*->\s*\((.*)\)>?\s*", text, re.S)
    if not m:
        raise ValueError("not an affine_map: %r" % text)
    names = [x.strip() for x in m.group(1).split(",") if x.strip()]
    if len(names) != len(dims):
        raise ValueError("map has %d dims, %d values given" % (len(names), len(dims)))
    nsym = len([x for x in (m.group(2) or "").split(",") if x.strip()])
    if nsym != len(symbols):
        raise ValueError("map has %d symbols, %d values given" % (nsym, len(symbols)))
    dims = [np.asarray(d, dtype=np.int64) for d in dims]
    p = _Parser(m.group(3), dims, [np.asarray(v, dtype=np.int64) for v in symbols])
    out = [p.expr()]
    while p.peek() == ",":
        p.take()
        out.append(p.expr())
    if p.peek() is not None:
        raise ValueError("trailing tokens in %r" % text)
    shape = np.broadcast(*dims, *[np.asarray(v) for v in symbols]).shape if (dims or symbols) else ()
    return [np.broadcast_to(np.asarray(o, dtype=np.int64), shape) for o in out]


def grid(rows, cols):
    i, j = np.meshgrid(np.arange(rows, dtype=np.int64), np.arange(cols, dtype=np.int64), indexing="ij")
    return i, j


# ------------------------------------------------------------------ XOR written with + and floordiv (FriskOps.cpp:123-143)
def xor2x2(a, b):
    s = a + b
    return s - 2 * (s // 2)


def xor4x4(a, b):
    return 2 * xor2x2(a // 2, b // 2) + xor2x2(a % 2, b % 2)


def xor8x8(a, b):
    return 2 * xor4x4(a // 2, b // 2) + xor2x2(a % 2, b % 2)


# ------------------------------------------------------------------ shared-memory layouts: (i, j) -> (tc, ts, index) or (index,)
def linear_layout(rows, cols, stride=None):  # :453-462
    stride = cols if stride is None or stride < 0 else stride
    return lambda i, j: (i * stride + j,)


def padded_layout(rows, cols, bits):  # :464-470
    padded = cols + (128 // bits if bits > 0 and (bits * cols) % 256 == 0 else 0)
    return linear_layout(rows, cols, padded)


def _bank_swizzle(bits, chunks, xor, row_div):
    vec = 128 // bits

    def f(i, j):
        ts, s = i // 8, i % 8
        block = j // vec
        tc, c = block // chunks, block % chunks
        return tc, ts, j % vec + (xor(c, s // row_div) + s * chunks) * vec
    return f


def quarter_bank_swizzle(rows, cols, bits):  # :500-518
    return _bank_swizzle(bits, 2, xor2x2, 4)


def half_bank_swizzle(rows, cols, bits):  # :520-538
    return _bank_swizzle(bits, 4, xor4x4, 2)


def full_bank_swizzle(rows, cols, bits):  # :540-558
    return _bank_swizzle(bits, 8, xor8x8, 1)


def ampere_shared_layout(rows, cols, bits, k_inner):  # :560-587 (64-bit element branches not restated: no golden)
    vec = 128 // bits
    if not k_inner and bits == 8:
        return "padded", padded_layout(rows, cols, bits)
    if cols % (vec * 8) == 0:
        return "full", full_bank_swizzle(rows, cols, bits)
    if cols % (vec * 4) == 0:
        return "half", half_bank_swizzle(rows, cols, bits)
    return "padded", padded_layout(rows, cols, bits)


def hopper_shared_layout(rows, cols, bits, k_inner):  # :589-618
    vec = 128 // bits
    if cols % (vec * 8) == 0:
        return "full", full_bank_swizzle(rows, cols, bits)
    if cols % (vec * 4) == 0:
        return "half", half_bank_swizzle(rows, cols, bits)
    if cols % (vec * 2) == 0:
        return "quarter", quarter_bank_swizzle(rows, cols, bits)
    if cols % vec == 0:
        return "linear", linear_layout(rows, cols)
    return None, None


# ------------------------------------------------------------------ register fragments (:155-287)
class Fragment:
    """index(i, j) = register slot inside a thread, thread(i, j) = owning thread; composed by repeat / replicate"""

    def __init__(self, shape, index, index_extent, thread, thread_extent, replicate=1):
        self.shape, self.index, self.index_extent = tuple(shape), index, index_extent
        self.thread, self.thread_extent, self.replicate_size = thread, thread_extent, replicate

    def repeat(self, repeats, on_thread, lower_dim_first):
        old = self.shape
        shape = tuple(o * r for o, r in zip(old, repeats))
        base_index, base_thread = self.index, self.thread
        order = range(len(old) - 1, -1, -1) if lower_dim_first else range(len(old))

        def rep_index(i, j):
            d = (i, j)
            v, stride = 0, 1
            for k in order:
                v = v + (d[k] // old[k]) * stride
                stride *= repeats[k]
            return v

        local_i = lambda i, j: base_index(i % old[0], j % old[1])
        local_t = lambda i, j: base_thread(i % old[0], j % old[1])
        prod = int(np.prod(repeats))
        if on_thread:
            te = self.thread_extent
            return Fragment(shape, local_i, self.index_extent, lambda i, j: local_t(i, j) + te * rep_index(i, j), te * prod, self.replicate_size)
        ie = self.index_extent
        return Fragment(shape, lambda i, j: local_i(i, j) + ie * rep_index(i, j), ie * prod, local_t, self.thread_extent, self.replicate_size)

    def replicate(self, n):
        assert n >= 1
        return Fragment(self.shape, self.index, self.index_extent, self.thread, self.thread_extent, self.replicate_size * n)


def fragment_8x4():
    return Fragment((8, 4), lambda i, j: j % 1, 1, lambda i, j: j // 1 + 4 * i, 32)


def fragment_8x8():
    return Fragment((8, 8), lambda i, j: j % 2, 2, lambda i, j: j // 2 + 4 * i, 32)


def fragment_8x16():
    return Fragment((8, 16), lambda i, j: j % 4, 4, lambda i, j: j // 4 + 4 * i, 32)


def fragment_8x8_transposed():
    return Fragment((8, 8), lambda i, j: i % 2, 2, lambda i, j: i // 2 + 4 * j, 32)


def ampere_fragment_c(bm, bn, wtm, wtn):  # :304-325
    if wtm % 16 or wtn % 8 or bm % wtm or bn % wtn:
        return None
    base = fragment_8x8().repeat((2, 1), False, True)
    warp = base.repeat((max(1, bm // wtm), max(1, bn // wtn)), True, False)
    return warp.repeat((max(1, wtm // 16), max(1, wtn // 8)), False, False)


def hopper_fragment_c(bm, bn, wtm, wtn):  # :327-347
    if wtm % 16 or wtn % 8 or bm % wtm or bn % wtn:
        return None
    warp = fragment_8x8().repeat((2, max(1, wtn // 8)), False, False)
    block = warp.repeat((max(1, bm // wtm), max(1, bn // wtn)), True, False)
    return block.repeat((max(1, wtm // 16), 1), False, False)


def gemm_fragment_a(bm, bn, bk, wtm, wtn, bits, transposed):  # :349-413
    if min(bm, bn, bk, wtm, wtn) <= 0 or bm % wtm or bn % wtn or wtm % 16 or bk % 16 or bits not in (8, 16, 32):
        return None
    rm, rn = bm // wtm, bn // wtn
    if transposed:
        base = fragment_8x8_transposed().repeat((2, 2), False, True)
        return base.repeat((1, rm), True, False).replicate(rn).repeat((bk // 16, wtm // 16), False, True)
    if bits == 8:
        if bk % 32:
            return None
        base = fragment_8x16().repeat((2, 2), False, False)
        return base.repeat((rm, 1), True, True).replicate(rn).repeat((wtm // 16, bk // 32), False, False)
    if bits == 16:
        base = fragment_8x8().repeat((2, 2), False, False)
        return base.repeat((rm, 1), True, True).replicate(rn).repeat((wtm // 16, bk // 16), False, False)
    if bk % 8:
        return None
    base = fragment_8x4().repeat((2, 2), False, False)
    return base.repeat((rm, 1), True, True).replicate(rn).repeat((wtm // 16, bk // 8), False, False)


def gemm_fragment_b(bm, bn, bk, wtm, wtn, transposed):  # :415-451
    if min(bm, bn, bk, wtm, wtn) <= 0 or bm % wtm or bn % wtn or wtn % 8 or bk % 16:
        return None
    rm, rn = bm // wtm, bn // wtn
    if transposed:
        base = fragment_8x8().repeat((1, 2), False, False)
        return base.replicate(rm).repeat((rn, 1), True, False).repeat((wtn // 8, bk // 16), False, False)
    base = fragment_8x8_transposed().repeat((2, 1), False, False)
    return base.replicate(rm).repeat((1, rn), True, True).repeat((bk // 16, wtn // 8), False, True)


# ------------------------------------------------------------------ warp partition (:825-888), generic in the per-warp atom
SQUARE, FULL_ROW, FULL_COL = 0, 1, 2


def warp_partition(policy, M, N, block_size, warp_size=32, k_m=16, k_n=8):
    """the reference fixes k_m = 16 and k_n = 8 (CUDA sm >= 70) or 16; the gfx950 planner calls the same rule with 64-wide
    waves and 32 x 32 atoms"""
    num = block_size // warp_size if warp_size else 1
    if M == 0 or N == 0 or num == 0:
        return 1, 1
    m_w, n_w = 1, num
    if policy == FULL_ROW:
        m_w = num
        if M % (m_w * k_m) != 0:
            m_w = max(1, min(num, max(1, M // k_m)))
        n_w = max(1, num // m_w)
    elif policy == FULL_COL:
        n_w = num
        if N % (n_w * k_n) != 0:
            n_w = max(1, min(num, max(1, N // k_n)))
        m_w = max(1, num // n_w)
    else:
        ideal = np.float32(M) / np.float32(N) if N > 0 else np.float32(1)
        best = np.float32(np.finfo(np.float32).max)
        for m in range(1, num + 1):
            if num % m:
                continue
            n = num // m
            mp = np.float32(M) / np.float32(m * k_m)
            npw = np.float32(N) / np.float32(n * k_n)
            if mp < 1 or npw < 1:
                continue
            score = np.abs(np.float32(mp / npw) - ideal)
            if score < best:
                best, m_w, n_w = score, m, n
    return max(1, m_w), max(1, n_w)


# ------------------------------------------------------------------ GemmOp::inferLayout (:1285-1407) for sm_80 / sm_90
def infer_gemm_layouts(target, threads, M, N, K, spaces, bits=16, transA=False, transB=False, policy=SQUARE):
    """returns {"A": ..., "B": ..., "C": ...}; a shared operand maps to ("shared", kind, fn), a local one to ("fragment", Fragment)"""
    sm = int(target[3:])
    hopper, ampere = sm >= 90, 80 <= sm < 90
    if not (hopper or ampere):
        raise ValueError("layout inference currently supports only Ampere or Hopper targets")
    wm, wn = warp_partition(policy, M, N, threads, 32, 16, 8 if sm >= 70 else 16)
    if M % wm or N % wn:
        raise ValueError("block shape must be divisible by warp partition")
    wtm, wtn = M // wm, N // wn
    wgmma = hopper and threads % 128 == 0 and M >= 64 and N >= 64  # inferGemmInst :620-625
    shared = hopper_shared_layout if hopper else ampere_shared_layout
    out = {}
    a_shape = (K, M) if transA else (M, K)
    b_shape = (N, K) if transB else (K, N)
    if spaces["A"] == "shared":
        out["A"] = ("shared",) + shared(a_shape[0], a_shape[1], bits, not transA)
    else:
        out["A"] = ("fragment", gemm_fragment_a(M, N, K, wtm, wtn, bits, transA))
    if spaces["B"] == "shared":
        out["B"] = ("shared",) + shared(b_shape[0], b_shape[1], bits, transB)
    else:
        out["B"] = ("fragment", gemm_fragment_b(M, N, K, wtm, wtn, transB))
    out["C"] = ("fragment", hopper_fragment_c(M, N, wtm, wtn) if wgmma else ampere_fragment_c(M, N, wtm, wtn))
    return out


# ------------------------------------------------------------------ the reference's bank-conflict count (gemm_layout_tool.cpp:135-263)
def bank_stats(index_fn, rows, cols, element_bytes, lane_vector, bank_count=32, bank_width=4, warp_size=32):
    """windows of warp_size * lane_vector row-major-consecutive elements; lane l touches lane_vector consecutive ones;
    every element access is counted in its bank (index_fn = the LAST result of the layout map, None = row-major baseline)"""
    lane_vector = max(1, lane_vector)
    window = warp_size * lane_vector
    total = rows * cols
    samples, worst, acc = 0, 0, 0.0
    for chunk in range(0, total, window):
        lin = chunk + np.arange(window, dtype=np.int64)
        lin = lin[lin < total]
        if lin.size == 0:
            continue
        idx = lin if index_fn is None else np.asarray(index_fn(lin // cols, lin % cols), dtype=np.int64)
        bank = ((idx * element_bytes) // bank_width) % bank_count
        local = int(np.bincount(bank, minlength=bank_count).max())
        samples += 1
        worst = max(worst, local)
        acc += local
    return {"avg_max": acc / samples if samples else 0.0, "max": worst, "samples": samples}


# ------------------------------------------------------------------ brute-force statements of what the generic inference computes
def used_extent_brute(map_text, shape, pos):
    """the largest number of distinct result tuples the map takes along dim `pos` (extent shape[pos]) with the other
    dims held fixed, over every setting of the others: what computeUsedExtentForDim (LayoutUtils.cpp:181-218) computes
    structurally for maps that use the pieces of a dim as independent digits"""
    import itertools
    best = 0
    others = [range(n) if k != pos else [0] for k, n in enumerate(shape)]
    for fixed in itertools.product(*others):
        dims = [np.arange(shape[pos]) if k == pos else np.int64(v) for k, v in enumerate(fixed)]
        res = eval_affine_map(map_text, *dims)
        best = max(best, len({tuple(int(r[t]) for r in res) for t in range(shape[pos])}))
    return best


def reduce_thread_sets(thread_map_text, shape, dim):
    """for every coordinate of the reduction's destination (the source's with `dim` removed): the set of threads that
    hold a source element reduced into it -- the threads that own a partial result, hence must hold the result"""
    import itertools
    out = {}
    rest = [n for k, n in enumerate(shape) if k != dim]
    for x in itertools.product(*[range(n) for n in rest]):
        dims = list(x[:dim]) + [np.arange(shape[dim])] + list(x[dim:])
        out[x] = frozenset(int(v) for v in eval_affine_map(thread_map_text, *dims)[0])
    return out
