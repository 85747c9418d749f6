"""frisk.fill / frisk.copy / frisk.reduce: the oracle against closed forms (CPU), the C ABI's argument checks (CPU),
and the HIP kernels against the oracle through the C ABI (GPU).

Bars: fill and same-type copy bit-exact; converting copies bit-exact (one rounding, the oracle's codec); min / max
bit-exact; add / mul within 1e-3 (f16, bf16: the result's own rounding dominates) or 1e-5 (f32) of the float64 value,
relative to max(|r|, rms(R))."""
import numpy as np
import pytest

import oracle as O
from oracle import tile_ops as T

FLOATS = [O.F32, O.F16, O.BF16]
NAMES = {O.F32: "f32", O.F16: "f16", O.BF16: "bf16"}


# ------------------------------------------------------------------ oracle (CPU)
def test_oracle_fill_and_copy_closed_forms():
    for dt in FLOATS:
        a = T.fill(dt, 3, 5, 1.25)
        assert a.shape == (3, 5) and np.all(O.decode(dt, a) == 1.25)
        assert np.all(O.decode(dt, T.fill(dt, 2, 2, -np.inf)) == -np.inf)
    # 1/3 is not representable: the fill value is the type's nearest
    assert O.decode(O.F16, T.fill(O.F16, 1, 1, 1.0 / 3.0))[0, 0] == np.float32(np.float16(1.0 / 3.0))
    x = O.encode(O.F32, O.normal(77, 9, 0, 3.0)).reshape(7, 11)
    assert np.array_equal(T.copy(O.F32, x, O.F32), x)
    h = T.copy(O.F32, x, O.F16)
    assert np.array_equal(h.view(np.float16), x.astype(np.float16))          # numpy's own RNE conversion
    assert np.array_equal(T.copy(O.F16, h, O.F32), h.view(np.float16).astype(np.float32))   # widening is exact
    assert np.array_equal(T.copy(O.F32, T.copy(O.F16, h, O.F32), O.F16), h)  # so the round trip is the identity


def test_oracle_reduce_closed_forms_and_shape_rule():
    n = 64
    ramp = O.encode(O.F32, np.arange(1, n + 1, dtype=np.float32)).reshape(1, n)
    assert O.decode(O.F32, T.reduce(O.F32, ramp, 1, "add"))[0] == n * (n + 1) / 2
    assert O.decode(O.F32, T.reduce(O.F32, ramp, 1, "max"))[0] == n and O.decode(O.F32, T.reduce(O.F32, ramp, 1, "min"))[0] == 1
    pw = O.encode(O.F32, np.array([[2.0, 0.5, 4.0, 0.25, 8.0]], dtype=np.float32))
    assert O.decode(O.F32, T.reduce(O.F32, pw, 1, "mul"))[0] == 8.0           # powers of two: exact
    x = O.encode(O.F16, O.normal(6 * 9, 10, 0, 1.0)).reshape(6, 9)
    assert T.reduce(O.F16, x, 0, "add").shape == (9,) and T.reduce(O.F16, x, 1, "add").shape == (6,)   # rank - 1, other extent kept
    xf = O.decode(O.F16, x).astype(np.float64).reshape(6, 9)
    assert np.array_equal(T.reduce_f64(O.F16, x, 0, "max"), xf.max(axis=0)) and np.array_equal(T.reduce_f64(O.F16, x, 1, "min"), xf.min(axis=1))
    # clear = False combines with the old destination
    old = O.encode(O.F16, np.full(6, 100.0, dtype=np.float32))
    assert np.all(O.decode(O.F16, T.reduce(O.F16, x, 1, "max", old)) == 100.0)
    assert np.allclose(T.reduce_f64(O.F16, x, 1, "add", old), 100.0 + xf.sum(axis=1))
    with pytest.raises(ValueError):
        T.reduce(O.F16, x, 2, "add")
    with pytest.raises(ValueError):
        T.reduce(O.F16, x, 0, "xor")


# ------------------------------------------------------------------ C ABI argument checks (no device needed)
def test_tile_op_status_codes_before_any_launch():
    from frisk_amd import runtime as R

    def status(fn, *a):
        with pytest.raises(R.FriskHipError) as e:
            fn(*a)
        return e.value.status
    assert status(R.fill, R.I8, 0x1000, 4, 4, 4, 0.0) == R.ERR_DTYPE
    assert status(R.fill, R.F16, 0x1000, -1, 4, 4, 0.0) == R.ERR_SHAPE
    assert status(R.fill, R.F16, 0x1000, 4, 8, 4, 0.0) == R.ERR_SHAPE          # ld < cols
    assert status(R.fill, R.F16, None, 4, 4, 4, 0.0) == R.ERR_NULL
    assert status(R.fill, R.F32, 0x1002, 4, 4, 4, 0.0) == R.ERR_ALIGNMENT
    assert status(R.copy, R.F32, 0x1000, 4, R.E4M3, 0x2000, 4, 4, 4) == R.ERR_DTYPE
    assert status(R.copy, R.F32, 0x1000, 2, R.F16, 0x2000, 4, 4, 4) == R.ERR_SHAPE
    assert status(R.reduce, R.F32, 0x1000, 4, 4, 4, 2, "add", True, 0x2000) == R.ERR_ARGUMENT   # dim out of range for rank 2
    assert status(R.reduce, R.F32, 0x1000, 4, 4, 4, 0, 9, True, 0x2000) == R.ERR_ARGUMENT       # kind
    assert status(R.reduce, R.F32, 0x1000, 4, 4, 4, 0, "add", True, None) == R.ERR_NULL
    # empty views are legal and touch nothing
    R.fill(R.F16, None, 0, 4, 4, 1.0)
    R.copy(R.F16, None, 8, R.F32, None, 8, 4, 0)
    R.reduce(R.F16, None, 0, 0, 0, 1, "add", True, None)
    # the workspace request: nothing for short reductions, slices x kept extent x 4 bytes for long ones
    assert R.reduce_workspace_bytes(R.F16, 8192, 8192, 1) == 0
    w = R.reduce_workspace_bytes(R.F16, 8192, 8192, 0)
    assert w > 0 and w % (8192 * 4) == 0
    assert R.reduce_workspace_bytes(R.F16, 4, 1 << 22, 1) % (4 * 4) == 0 and R.reduce_workspace_bytes(R.F16, 4, 1 << 22, 1) > 0


# ------------------------------------------------------------------ HIP kernels against the oracle (GPU)
def _dev(arr):
    import torch
    return torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1).copy()).cuda()


def _host(t, np_dtype):
    return t.cpu().numpy().view(np_dtype)


VIEWS = [(1, 1, 0, 0), (1, 1000, 0, 0), (37, 53, 0, 0), (64, 256, 0, 0), (64, 256, 8, 0), (33, 100, 3, 1), (300, 7, 1, 0), (5, 4096, 0, 0)]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", FLOATS, ids=[NAMES[d] for d in FLOATS])
def test_fill_gpu(hip, dt):
    import torch
    st = O.NP_STORAGE[dt]
    es = np.dtype(st).itemsize
    for rows, cols, pad, shift in VIEWS:
        ld = cols + pad
        buf = np.full(shift + rows * ld, 0x5A5A5A5A if es == 4 else 0x5A5A, dtype=st)
        d = _dev(buf)
        hip.fill(dt, d.data_ptr() + shift * es, rows, cols, ld, -2.71828, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        got = _host(d, st)
        view = got[shift:shift + rows * ld].reshape(rows, ld)
        assert np.array_equal(view[:, :cols], T.fill(dt, rows, cols, -2.71828)), (rows, cols, pad, shift)
        assert np.array_equal(view[:, cols:], buf[shift:].reshape(rows, ld)[:, cols:]) and np.array_equal(got[:shift], buf[:shift])   # nothing outside the view


@pytest.mark.gpu
@pytest.mark.parametrize("sdt", FLOATS, ids=[NAMES[d] for d in FLOATS])
@pytest.mark.parametrize("ddt", FLOATS, ids=[NAMES[d] for d in FLOATS])
def test_copy_gpu(hip, sdt, ddt):
    import torch
    sst, dst_t = O.NP_STORAGE[sdt], O.NP_STORAGE[ddt]
    ses, des = np.dtype(sst).itemsize, np.dtype(dst_t).itemsize
    for rows, cols, pad, shift in VIEWS:
        sld, dld = cols + pad, cols + 2 * pad
        src = np.zeros(shift + rows * sld, dtype=sst)
        vals = O.encode(sdt, O.normal(rows * cols, 21, 0, 50.0)).reshape(rows, cols)
        src[shift:].reshape(rows, sld)[:, :cols] = vals
        dst0 = np.full(shift + rows * dld, 0x7B7B7B7B if des == 4 else 0x7B7B, dtype=dst_t)
        dS, dD = _dev(src), _dev(dst0)
        hip.copy(sdt, dS.data_ptr() + shift * ses, sld, ddt, dD.data_ptr() + shift * des, dld, rows, cols, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        got = _host(dD, dst_t)
        view = got[shift:].reshape(rows, dld)
        assert np.array_equal(view[:, :cols], T.copy(sdt, vals, ddt)), (rows, cols, pad, shift)
        assert np.array_equal(view[:, cols:], dst0[shift:].reshape(rows, dld)[:, cols:]) and np.array_equal(got[:shift], dst0[:shift])


def _close(dt, got, ref64):
    g = O.decode(dt, got).astype(np.float64).reshape(-1)
    r = np.asarray(ref64, dtype=np.float64).reshape(-1)
    tol = 1e-5 if dt == O.F32 else (1e-3 if dt == O.F16 else 8e-3)   # bf16 keeps 8 bits: half an ulp is 2^-9
    scale = np.maximum(np.abs(r), np.sqrt(np.mean(r * r)) if r.size else 0.0)
    assert np.all(np.isfinite(g)) and np.all(np.abs(g - r) <= tol * np.maximum(scale, 1e-30)), float(np.max(np.abs(g - r) / np.maximum(scale, 1e-30)))


REDUCE_VIEWS = [(1, 1, 0), (7, 5, 0), (64, 256, 0), (33, 1000, 3), (300, 9, 1), (4, 70000, 0), (70000, 4, 0), (2048, 2048, 0), (16, 1 << 18, 0), (1 << 16, 40, 8),
                # short rows shared by 1 ... 64 lanes with 1, 2 and 4 groups per lane; views narrower than a column strip
                (1000, 24, 0), (999, 100, 4), (130, 600, 0), (77, 1500, 4), (50, 1003, 5), (1 << 17, 16, 0), (5000, 8, 0)]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", FLOATS, ids=[NAMES[d] for d in FLOATS])
@pytest.mark.parametrize("dim", [0, 1])
def test_reduce_gpu(hip, dt, dim):
    import torch
    st = O.NP_STORAGE[dt]
    stream = torch.cuda.current_stream().cuda_stream
    for rows, cols, pad in REDUCE_VIEWS:
        ld = cols + pad
        for kind in T.KINDS:
            # products need factors near 1 and few of them to stay finite
            if kind == "mul":
                if (cols if dim == 1 else rows) > 300:
                    continue
                f = 1.0 + 0.01 * O.normal(rows * cols, 31, 0, 1.0)
            else:
                f = O.normal(rows * cols, 31, 1, 1.0)
            vals = O.encode(dt, f.astype(np.float32)).reshape(rows, cols)
            src = np.zeros(rows * ld, dtype=st)
            src.reshape(rows, ld)[:, :cols] = vals
            kept = rows if dim == 1 else cols
            old = O.encode(dt, O.normal(kept, 32, 2, 0.5))
            ws_bytes = hip.reduce_workspace_bytes(dt, rows, cols, dim)
            ws = torch.full((max(ws_bytes, 4),), 0xFF, dtype=torch.uint8, device="cuda")
            dS = _dev(src)
            for clear, use_ws in ((True, True), (False, True), (True, False)):
                dD = _dev(old)
                hip.reduce(dt, dS.data_ptr(), rows, cols, ld, dim, kind, clear, dD.data_ptr(), ws.data_ptr() if use_ws and ws_bytes else None,
                           ws_bytes if use_ws else 0, stream)
                torch.cuda.synchronize()
                got = _host(dD, st)
                if kind in ("min", "max"):
                    assert np.array_equal(got, T.reduce(dt, vals, dim, kind, None if clear else old)), (rows, cols, pad, kind, clear, use_ws)
                else:
                    _close(dt, got, T.reduce_f64(dt, vals, dim, kind, None if clear else old))


# ------------------------------------------------------------------ row softmax (the @online_softmax sketch)
def test_oracle_softmax_sketch_equals_plain_softmax_and_scipy():
    from scipy.special import logsumexp, softmax
    x = O.encode(O.F16, O.normal(5 * 3000, 41, 0, 3.0)).reshape(5, 3000)
    cst = 1.25
    y, lse = T.softmax_f64(O.F16, x, cst)
    for chunk in (1024, 7, 3000, 5000):      # the running log-sum is an identity, whatever the chunking
        ys, ls = T.online_softmax_sketch(O.F16, x, cst, chunk)
        assert np.allclose(ys, y, rtol=1e-12, atol=1e-300) and np.allclose(ls, lse, rtol=1e-13)
    xf = O.decode(O.F16, x.reshape(-1)).astype(np.float64).reshape(x.shape)
    assert np.allclose(y, softmax(xf * cst * np.log(2.0), axis=1), rtol=1e-12)          # base 2 with cst = base e with cst * ln 2
    assert np.allclose(lse * np.log(2.0), logsumexp(xf * cst * np.log(2.0), axis=1), rtol=1e-13)
    assert np.allclose(y.sum(axis=1), 1.0, rtol=1e-13)
    flat = O.encode(O.F32, np.full(64, 7.0, dtype=np.float32)).reshape(1, 64)
    yc, lc = T.softmax_f64(O.F32, flat, 2.0)
    assert np.allclose(yc, 1.0 / 64) and np.allclose(lc, 14.0 + 6.0)                       # constant row: uniform, lse = c x + log2 n


def test_softmax_status_codes_before_any_launch():
    from frisk_amd import runtime as R

    def status(*a):
        with pytest.raises(R.FriskHipError) as e:
            R.softmax(*a)
        return e.value.status
    p = 1 << 20
    assert status(R.I8, p, 8, p, 8, 4, 8) == R.ERR_DTYPE
    assert status(R.F16, p, 4, p, 8, 4, 8) == R.ERR_SHAPE           # leading dimension below the row length
    assert status(R.F16, None, 8, p, 8, 4, 8) == R.ERR_NULL
    assert status(R.F16, p + 1, 8, p, 8, 4, 8) == R.ERR_ALIGNMENT
    assert status(R.F16, p, 8, p, 8, 4, 8, float("inf")) == R.ERR_ARGUMENT
    R.softmax(R.F16, None, 8, None, 8, 0, 8)                          # nothing to do
    # pure host: only fewer than 1024 rows of at least 32 KiB ask for a workspace, 8 bytes per row and slice
    assert R.softmax_workspace_bytes(R.F16, 8, 1 << 24) == 8 * 128 * 8 and R.softmax_workspace_bytes(R.F16, 128, 1 << 20) == 128 * 8 * 8
    assert R.softmax_workspace_bytes(R.F16, 2000, 1 << 20) == 0 and R.softmax_workspace_bytes(R.F32, 4, 4096) == 0 and R.softmax_workspace_bytes(R.I8, 4, 1 << 20) == 0


SOFTMAX_VIEWS = [(1, 1, 0, 0), (3, 8, 0, 0), (7, 1000, 0, 0), (5, 1003, 3, 1), (64, 2048, 8, 0), (16, 4096, 0, 0), (9, 8192, 0, 0), (4, 16384, 0, 0),
                 (3, 16392, 0, 0), (2, 70000, 0, 0), (300, 40, 0, 0),
                 # rows shared by 1 ... 64 lanes of a wave with 1, 2 and 4 groups per lane, whole and partial last groups
                 (513, 8, 0, 0), (1000, 24, 0, 0), (999, 100, 4, 0), (130, 600, 0, 0), (77, 1500, 4, 0), (50, 1003, 5, 0), (31, 2040, 8, 0),
                 # long rows split over work-groups through the workspace: aligned, odd, padded
                 (3, 300000, 0, 0), (2, 100003, 5, 1), (40, 32768, 8, 0)]


@pytest.mark.gpu
@pytest.mark.parametrize("dt", FLOATS, ids=[NAMES[d] for d in FLOATS])
def test_softmax_gpu(hip, dt):
    """every path: rows shared by the lanes of a wave, a work-group per row with the row in registers (2, 4, 8 groups per
    lane), two sweeps (long rows), long rows split over work-groups (with a workspace), element by element (odd views);
    bar: each element within 2e-3 (f16), 8e-3 (bf16), 2e-5 (f32) of the float64 value relative to max(|r|, rms), rows sum
    to one within that, log-sum within 1e-4"""
    import torch
    st = O.NP_STORAGE[dt]
    es = np.dtype(st).itemsize
    tol = {O.F32: 2e-5, O.F16: 2e-3, O.BF16: 8e-3}[dt]
    floor = 2.0 ** -25 if dt == O.F16 else 0.0      # probabilities of very long rows are f16 subnormals: half a step of 2^-24
    stream = torch.cuda.current_stream().cuda_stream
    for rows, cols, pad, shift in SOFTMAX_VIEWS:
        for cst in (1.25, -0.4):
            ld = cols + pad
            vals = O.encode(dt, O.normal(rows * cols, 43, 0, 4.0)).reshape(rows, cols)
            src = np.zeros(shift + rows * ld, dtype=st)
            src[shift:].reshape(rows, ld)[:, :cols] = vals
            dst0 = np.full(shift + rows * ld, 0x7B7B7B7B if es == 4 else 0x7B7B, dtype=st)
            ref, lse = T.softmax_f64(dt, vals, cst)
            scale = np.maximum(np.abs(ref), np.sqrt(np.mean(ref * ref)))
            ws_bytes = hip.softmax_workspace_bytes(dt, rows, cols)
            assert (ws_bytes > 0) == (cols * es >= 32768), (rows, cols)     # only a few very long rows are split
            ws = torch.full((max(ws_bytes, 4),), 0xFF, dtype=torch.uint8, device="cuda")
            dS = _dev(src)
            for use_ws in ((False, True) if ws_bytes else (False,)):
                dD = _dev(dst0)
                dL = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
                hip.softmax(dt, dS.data_ptr() + shift * es, ld, dD.data_ptr() + shift * es, ld, rows, cols, cst, dL.data_ptr(), stream,
                            ws.data_ptr() if use_ws else None, ws_bytes if use_ws else 0)
                torch.cuda.synchronize()
                got = _host(dD, st)
                view = got[shift:].reshape(rows, ld)
                g = O.decode(dt, np.ascontiguousarray(view[:, :cols]).reshape(-1)).astype(np.float64).reshape(rows, cols)
                assert np.all(np.isfinite(g)) and np.all(np.abs(g - ref) <= tol * scale + floor), (rows, cols, pad, shift, cst, use_ws, float(np.max(np.abs(g - ref) / scale)))
                assert np.abs(dL.cpu().numpy() - lse).max() <= 1e-4 * max(1.0, np.abs(lse).max()), (rows, cols, use_ws)
                assert np.array_equal(view[:, cols:], dst0[shift:].reshape(rows, ld)[:, cols:]) and np.array_equal(got[:shift], dst0[:shift])   # nothing outside the view
    # in place, and a masked column (-inf) gets probability exactly zero
    vals = O.encode(dt, O.normal(4 * 512, 44, 0, 1.0)).reshape(4, 512)
    vals[:, 17] = O.encode(dt, np.array([-np.inf], dtype=np.float32))[0]
    d = _dev(vals)
    hip.softmax(dt, d.data_ptr(), 512, d.data_ptr(), 512, 4, 512, 1.4426950408889634, None, stream)
    torch.cuda.synchronize()
    g = O.decode(dt, _host(d, st)).astype(np.float64).reshape(4, 512)
    assert np.all(g[:, 17] == 0.0) and np.allclose(g.sum(axis=1), 1.0, atol=64 * tol)
    # the same on the streaming paths, whose running (maximum, sum) meets the mask first: masked columns incl. column 0 in a
    # row of two sweeps (over 16384 elements per row), an odd-length long row (element by element) and a row split over work-groups
    for rows, cols, use_ws in ((3, 20480, False), (2, 18001, False), (2, 65536, True)):
        vals = O.encode(dt, O.normal(rows * cols, 45, 0, 1.0)).reshape(rows, cols)
        masked = [0, 1, 7, cols // 2, cols - 1]
        vals[:, masked] = O.encode(dt, np.array([-np.inf], dtype=np.float32))[0]
        ref, lse = T.softmax_f64(dt, vals, 1.25)
        dS = _dev(vals)
        dD = torch.zeros_like(dS)
        dL = torch.full((rows,), float("nan"), dtype=torch.float32, device="cuda")
        ws_bytes = hip.softmax_workspace_bytes(dt, rows, cols) if use_ws else 0
        assert ws_bytes > 0 or not use_ws
        ws = torch.full((max(ws_bytes, 4),), 0xFF, dtype=torch.uint8, device="cuda")
        hip.softmax(dt, dS.data_ptr(), cols, dD.data_ptr(), cols, rows, cols, 1.25, dL.data_ptr(), stream, ws.data_ptr() if ws_bytes else None, ws_bytes)
        torch.cuda.synchronize()
        g = O.decode(dt, _host(dD, st)).astype(np.float64).reshape(rows, cols)
        scale = np.maximum(np.abs(ref), np.sqrt(np.mean(ref * ref)))
        assert np.all(np.isfinite(g)) and np.all(g[:, masked] == 0.0), (rows, cols)
        assert np.all(np.abs(g - ref) <= tol * scale + floor), (rows, cols, float(np.max(np.abs(g - ref) / scale)))
        assert np.abs(dL.cpu().numpy() - lse).max() <= 1e-4 * max(1.0, np.abs(lse).max()), (rows, cols)


# ------------------------------------------------------------------ frisk.block bodies as postfix programs, tiled copies
def test_oracle_elementwise_closed_forms():
    x = np.array([[0.25, 1.0, 4.0, 1024.0]])
    assert np.array_equal(T.elementwise([("input", 0), "log2", "exp2"], [x], 1, 4), x)                       # powers of two: exact both ways
    assert np.array_equal(T.elementwise([("input", 0), ("input", 0), "sub"], [x], 1, 4), np.zeros((1, 4)))
    # the operand pushed first is the left one
    assert np.array_equal(T.elementwise([("input", 0), ("const", 2.0), "div"], [x], 1, 4), x / 2) and np.array_equal(T.elementwise([("const", 2.0), ("input", 0), "sub"], [x], 1, 4), 2 - x)
    # max / min ignore a NaN operand
    n = np.array([[np.nan, 3.0]])
    assert np.array_equal(T.elementwise([("input", 0), ("const", 1.0), "max"], [n], 1, 2), [[1.0, 3.0]]) and np.array_equal(T.elementwise([("input", 0), ("const", 1.0), "min"], [n], 1, 2), [[1.0, 1.0]])
    # operands broadcast: a value per row, a value per column
    r, c = np.arange(3.0).reshape(3, 1), np.arange(4.0).reshape(1, 4)
    assert np.array_equal(T.elementwise([("input", 0), ("input", 1), "mul", "neg"], [r, c], 3, 4), -(r * c))


def test_elementwise_and_tiled_copy_status_codes_before_any_launch():
    from frisk_amd import runtime as R

    def status(program, inputs=((R.F32, 8, 1),), ptrs=(0x1000,), out=0x2000, rows=4, cols=8, out_dtype=R.F32):
        with pytest.raises(R.FriskHipError) as e:
            R.elementwise(R.make_elementwise_desc(program, list(inputs), out_dtype, rows, cols), list(ptrs), out)
        return e.value.status
    x = ("input", 0)
    assert status(["add"]) == R.ERR_ARGUMENT                                              # pops an empty stack
    assert status([x, x]) == R.ERR_ARGUMENT                                               # leaves two values
    assert status([x] * 7 + ["add"] * 6) == R.ERR_ARGUMENT                                # needs a stack of 7
    assert status([("input", 1)]) == R.ERR_ARGUMENT                                       # no such operand
    assert status([x], inputs=((R.F32, 8, 2),)) == R.ERR_SHAPE                            # column stride
    assert status([x], inputs=((R.I8, 8, 1),)) == R.ERR_DTYPE
    assert status([x], ptrs=(None,)) == R.ERR_NULL
    assert status([x], out=None) == R.ERR_NULL
    assert status([x], ptrs=(0x1002,)) == R.ERR_ALIGNMENT
    d = R.make_elementwise_desc([x], [(R.F32, 8, 1)], R.F32, 4, 8)
    d.n_ops = 0
    with pytest.raises(R.FriskHipError) as e:
        R.elementwise(d, [0x1000], 0x2000)
    assert e.value.status == R.ERR_ARGUMENT
    R.elementwise(R.make_elementwise_desc([x], [(R.F32, 8, 1)], R.F32, 0, 8), [0x1000], None)   # an empty space touches nothing
    with pytest.raises(R.FriskHipError) as e:
        R.copy_tiles(R.F16, 0x1000, 64, R.F16, 0x2000, 64, 8, 8, 2, -8, 8)
    assert e.value.status == R.ERR_SHAPE
    with pytest.raises(R.FriskHipError) as e:
        R.copy_tiles(R.F16, 0x1000, 4, R.F16, 0x2000, 64, 8, 8, 2, 8, 8)                  # ld < tile cols
    assert e.value.status == R.ERR_SHAPE
    R.copy_tiles(R.F16, None, 64, R.F16, None, 64, 8, 8, 0, 8, 8)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", FLOATS, ids=[NAMES[d] for d in FLOATS])
def test_elementwise_gpu(hip, dt):
    """every opcode, walked / per-row / per-column / scalar operands, padded rows (vector path), odd extents and an element-
    aligned pointer (scalar path), in place; against numpy float64 through the oracle's evaluator"""
    import torch
    tol = {O.F32: 3e-6, O.F16: 1e-3, O.BF16: 8e-3}[dt]
    prog = [("input", 0), ("input", 1), "mul", ("input", 2), "sub", ("const", 0.75), "max", ("input", 3), "min", "neg", ("const", 3.0), "add", "log2",
            ("input", 0), ("const", 0.125), "mul", "exp2", "div"]
    for rows, cols, pad, shift in ((1, 8, 0, 0), (64, 256, 0, 0), (40, 136, 8, 0), (33, 100, 3, 1), (7, 5000, 0, 0), (1000, 3, 0, 0)):
        ld = cols + pad
        x = O.encode(dt, O.normal(rows * ld + shift, 95, 0, 1.0))
        s = O.uniform(rows, 95, 1, 0.5, 1.5).astype(np.float32)
        m = O.encode(dt, O.uniform(cols, 95, 2, -0.5, 0.5))
        k = np.array([2.5], dtype=np.float32)
        xf = O.decode(dt, x)[shift:].reshape(rows, ld)[:, :cols].astype(np.float64)
        ins = [xf, s.astype(np.float64).reshape(rows, 1), O.decode(dt, m).astype(np.float64).reshape(1, cols), np.array([[2.5]])]
        want = T.elementwise(prog, ins, rows, cols)
        assert np.all(np.isfinite(want))
        dx, ds, dm, dk = _dev(x), _dev(s), _dev(m), _dev(k)
        es = O.NP_STORAGE[dt]().itemsize
        dy = torch.full(((rows * ld + shift) * es,), 0xEE, dtype=torch.uint8, device="cuda")
        desc = hip.make_elementwise_desc(prog, [(dt, ld, 1), (hip.F32, 1, 0), (dt, 0, 1), (hip.F32, 0, 0)], dt, rows, cols, out_ld=ld)
        hip.elementwise(desc, [dx.data_ptr() + shift * es, ds.data_ptr(), dm.data_ptr(), dk.data_ptr()], dy.data_ptr() + shift * es, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        full = _host(dy, O.NP_STORAGE[dt])[shift:].reshape(rows, ld)
        got = O.decode(dt, np.ascontiguousarray(full[:, :cols])).astype(np.float64).reshape(rows, cols)
        err = np.abs(got - want) / np.maximum(np.abs(want), np.sqrt(np.mean(want ** 2)))
        assert err.max() <= tol, (rows, cols, pad, shift, err.max())
        if pad:
            assert np.all(full[:, cols:].view(np.uint8) == 0xEE), "the kernel wrote into the padding"
        # in place: the output over operand 0
        hip.elementwise(desc, [dx.data_ptr() + shift * es, ds.data_ptr(), dm.data_ptr(), dk.data_ptr()], dx.data_ptr() + shift * es, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        again = _host(dx, O.NP_STORAGE[dt])[shift:].reshape(rows, ld)[:, :cols]
        assert np.array_equal(again, full[:, :cols])


@pytest.mark.gpu
def test_copy_tiles_gpu(hip):
    """tiles placed elsewhere than they came from: block-transposed, gathered at another pitch, converting on the way; bytes
    between the destination tiles stay as they were"""
    import torch
    for sdt, ddt, tr, tc, n0, n1, sld, dld in ((O.F16, O.F16, 32, 32, 4, 4, 128, 128), (O.F32, O.BF16, 16, 24, 3, 5, 130, 80), (O.BF16, O.F32, 5, 7, 2, 3, 23, 40),
                                               (O.F16, O.F16, 64, 512, 8, 1, 512, 600)):
        src_rows, dst_rows = n0 * tr, n1 * tr if n1 > 1 else n0 * tr
        x = O.encode(sdt, O.normal(src_rows * sld, 96, 0, 2.0)).reshape(src_rows, sld)
        dx = _dev(x)
        if n1 > 1:   # source tile (a, b) at rows a, columns b -> destination rows b, columns a
            dst_cols_needed = n0 * tc
            dld = max(dld, dst_cols_needed)
            steps = dict(n0=n0, src_step0=tr * sld, dst_step0=tc, n1=n1, src_step1=tc, dst_step1=tr * dld)
        else:        # one column of tiles copied at another row pitch
            steps = dict(n0=n0, src_step0=tr * sld, dst_step0=tr * dld, n1=1, src_step1=0, dst_step1=0)
        des = O.NP_STORAGE[ddt]().itemsize
        dy = torch.full((dst_rows * dld * des,), 0xEE, dtype=torch.uint8, device="cuda")
        hip.copy_tiles(sdt, dx.data_ptr(), sld, ddt, dy.data_ptr(), dld, tr, tc, stream=torch.cuda.current_stream().cuda_stream, **steps)
        torch.cuda.synchronize()
        want = np.frombuffer(bytes([0xEE]) * (dst_rows * dld * des), dtype=O.NP_STORAGE[ddt]).reshape(dst_rows, dld).copy()
        conv = T.copy(sdt, x, ddt)
        for a in range(n0):
            for b in range(n1):
                so, do = a * steps["src_step0"] + b * steps["src_step1"], a * steps["dst_step0"] + b * steps["dst_step1"]
                sr, sc, dr, dc = so // sld, so % sld, do // dld, do % dld
                want[dr:dr + tr, dc:dc + tc] = conv[sr:sr + tr, sc:sc + tc]
        assert np.array_equal(_host(dy, O.NP_STORAGE[ddt]).reshape(dst_rows, dld), want), (sdt, ddt, tr, tc)
