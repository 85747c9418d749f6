"""CPU restatement of frisk.fill, frisk.copy, frisk.reduce and elementwise frisk.block bodies on rank-2 views -- TEST INFRASTRUCTURE ONLY.

The reference declares these ops and verifies their shapes (include/Dialect/Frisk/IR/FriskOps.td:348-441,
lib/Dialect/Frisk/IR/FriskOps.cpp:1551-1767) but defines no arithmetic for them and holds no numerical
vectors: numerical parity against the reference is unpinned.  What this file fixes, and what pins it:
  fill    every element := value rounded to the element type                    (closed form; codecs pinned in test_oracle.py)
  copy    window -> window, conversion through fp32, round to nearest even      (identity on equal types, round trips)
  reduce  kind in add | mul | min | max along dim of a rank-2 view, in float64, result rounded to the element
          type; clear = False combines the old destination value with the reduction (the accumulating form the
          online-softmax sketch of tmp/ir.mlir:33-57 relies on); shape rule of ReduceOp::verify (:1733-1767):
          destination rank = source rank - 1, the other extent is kept            (numpy's own reductions, closed forms)
  elementwise  a frisk.block body (FriskOps.td:143-190; arith / math ops created by ffi/ir.cpp:383-394) as a postfix program
          over operands read with a row stride and a column stride of 0 or 1, evaluated in float64 by numpy's own
          add / subtract / multiply / divide / maximum / minimum / negative / exp2 / log2, rounded once to the output type
          (the reference defines no arithmetic for block bodies either: parity unpinned; pinned here by closed forms --
          identities such as log2(exp2(x)) = x, x / x = 1, max(x, x) = x -- and by numpy expressions written independently
          in the tests)
Arrays are in the storage types of oracle.NP_STORAGE (uint16 for f16 / bf16).
"""
import numpy as np

import oracle as O

KINDS = ("add", "mul", "min", "max")


def fill(dtype, rows, cols, value):
    one = O.encode(dtype, np.array([value], dtype=np.float32))
    return np.full((rows, cols), one[0], dtype=O.NP_STORAGE[dtype])


def copy(src_dtype, src, dst_dtype):
    if src_dtype == dst_dtype:
        return src.copy()
    return O.encode(dst_dtype, O.decode(src_dtype, src).astype(np.float32).reshape(-1)).reshape(src.shape)


def reduce_f64(dtype, src, dim, kind, old=None):
    """exact-as-possible value of the reduction (float64), before rounding to the element type; `old` (storage type)
    is combined in when given (clear = False)"""
    if kind not in KINDS:
        raise ValueError("unsupported reduce kind: %s. Supported: add, mul, min, max" % kind)
    if dim not in (0, 1):
        raise ValueError("dimension %d is out of range for source of rank 2" % dim)
    x = O.decode(dtype, src).astype(np.float64).reshape(src.shape)
    f = {"add": np.sum, "mul": np.prod, "min": np.min, "max": np.max}[kind]
    ident = {"add": 0.0, "mul": 1.0, "min": np.inf, "max": -np.inf}[kind]
    r = f(x, axis=dim) if x.shape[dim] else np.full(x.shape[1 - dim], ident)
    if old is not None:
        o = O.decode(dtype, old).astype(np.float64).reshape(-1)
        r = {"add": np.add, "mul": np.multiply, "min": np.minimum, "max": np.maximum}[kind](o, r)
    return r


def reduce(dtype, src, dim, kind, old=None):
    return O.encode(dtype, reduce_f64(dtype, src, dim, kind, old).astype(np.float32))


def softmax_f64(dtype, src, scale_log2):
    """(y, lse2) in float64: y = 2^(c x) / sum_j 2^(c x) along dim 1, lse2 = log2 of the denominator"""
    x = O.decode(dtype, np.ascontiguousarray(src).reshape(-1)).astype(np.float64).reshape(src.shape) * scale_log2
    m = x.max(axis=1, keepdims=True)
    e = np.exp2(x - m)
    den = e.sum(axis=1, keepdims=True)
    return e / den, (m + np.log2(den))[:, 0]


def online_softmax_sketch(dtype, src, cst, chunk=1024):
    """the reference's @online_softmax, op by op (tmp/ir.mlir:33-68), in float64: a running log-sum over chunks of the row
    (copy; reduce max :37-38; block exp2(x * cst - max * cst) :39-47; reduce sum :48; lse update :49-60), then a second
    sweep y = exp2(x * cst - lse) (:62-72)"""
    x = O.decode(dtype, np.ascontiguousarray(src).reshape(-1)).astype(np.float64).reshape(src.shape)
    rows, cols = x.shape
    lse = np.full(rows, -np.inf)                                   # fill(lse, -inf)        :32
    for c0 in range(0, cols, chunk):
        xs = x[:, c0:c0 + chunk]
        max_x = xs.max(axis=1)                                     # reduce max, clear = 1
        exp_x = np.exp2(xs * cst - max_x[:, None] * cst)
        sum_exp_x = exp_x.sum(axis=1)                              # reduce sum, clear = 1
        with np.errstate(invalid="ignore"):
            lse = max_x * cst + np.log2(np.where(np.isneginf(lse), 0.0, np.exp2(lse - max_x * cst)) + sum_exp_x)
    return np.exp2(x * cst - lse[:, None]), lse


def elementwise(program, inputs, rows, cols):
    """frisk.block body (FriskOps.td:143-190) as the postfix program frisk_hip_elementwise takes, in float64.
    program: steps ("input", k) | ("const", v) | "add" | "sub" | "mul" | "div" | "max" | "min" | "neg" | "exp2" | "log2";
    inputs: arrays that broadcast against (rows, cols).  max / min ignore a NaN operand (arith.maxnumf / minnumf)."""
    stack = []
    for step in program:
        name, val = (step, None) if isinstance(step, str) else step
        if name == "input":
            stack.append(np.broadcast_to(np.asarray(inputs[val], dtype=np.float64), (rows, cols)))
        elif name == "const":
            stack.append(np.full((rows, cols), float(val)))
        elif name in ("neg", "exp2", "log2"):
            x = stack.pop()
            with np.errstate(all="ignore"):
                stack.append(-x if name == "neg" else np.exp2(x) if name == "exp2" else np.log2(x))
        else:
            b, a = stack.pop(), stack.pop()
            with np.errstate(all="ignore"):
                stack.append({"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide, "max": np.fmax, "min": np.fmin}[name](a, b))
    assert len(stack) == 1, "the program must leave one value"
    return stack[0]
