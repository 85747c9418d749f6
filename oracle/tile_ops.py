"""CPU restatement of frisk.fill, frisk.copy and frisk.reduce on rank-2 views -- TEST INFRASTRUCTURE ONLY.

The reference declares these ops and verifies their shapes (include/Dialect/Frisk/IR/FriskOps.td:348-441,
lib/Dialect/Frisk/IR/FriskOps.cpp:1551-1767) but defines no arithmetic for them and holds no numerical
vectors: numerical parity against the reference is unpinned.  What this file fixes, and what pins it:
  fill    every element := value rounded to the element type                    (closed form; codecs pinned in test_oracle.py)
  copy    window -> window, conversion through fp32, round to nearest even      (identity on equal types, round trips)
  reduce  kind in add | mul | min | max along dim of a rank-2 view, in float64, result rounded to the element
          type; clear = False combines the old destination value with the reduction (the accumulating form the
          online-softmax sketch of tmp/ir.mlir:33-57 relies on); shape rule of ReduceOp::verify (:1733-1767):
          destination rank = source rank - 1, the other extent is kept            (numpy's own reductions, closed forms)
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
