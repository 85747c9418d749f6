"""The two programs of the reference's design sketches beyond the lone GEMM (tmp/ir.mlir:21-75 @online_softmax, :88-158
@attention): built with the IR builder incl. their frisk.block bodies (FriskOps.td:143-190), printed, parsed back,
recognised by frisk.runtime.match, and (GPU) launched through the C ABI against the oracle.

The sketches hold no numbers and are not parseable text (free-form headers, undefined values): parity against the reference
is unpinned.  The oracles restate the sketches op by op (oracle/tile_ops.py: online_softmax_sketch, oracle/attention.py:
attention_tiled) and are pinned against the plain float64 softmax / scipy in tests/test_tile_ops.py and tests/test_attention.py."""
import numpy as np
import pytest

import frisk_amd  # noqa: F401
import frisk as F
import oracle as O
from oracle import attention as A
from oracle import tile_ops as T


def reparse(module, name):
    ctx = F.create_context()
    m = F.parse_module(ctx, str(module))
    m.context = ctx
    return m, m.get_kernel(name)


# ------------------------------------------------------------------ host
def test_block_bodies_build_print_parse_and_verify():
    h = F.create_session()
    b = h.builder
    kernel, entry = h.new_kernel("scale", [h.memref_type((64,), "fp16"), h.memref_type((64,), "fp32")])
    x, y = entry.get_argument(0), entry.get_argument(1)
    c = b.get_f32(0.5)

    def body(bb, ivs):
        v = bb.create_extf(bb.create_load_op(x, [ivs[0]]), bb.get_f32_ty())
        bb.create_store_op(bb.create_log2(bb.create_divf(bb.create_maxnumf(v, c), bb.create_addf(v, c))), y, [ivs[0]])
    blk = b.create_block_op([64], body)
    assert blk.get_block_ranges() == [64] and kernel.verify() and h.module.verify()
    text = str(h.module)
    for line in ("%0 = arith.constant 5.000000e-01 : f32", "%1 = affine.load %arg0[%arg2] : memref<64xf16, 1>", "%2 = arith.extf %1 : f16 to f32",
                 "%3 = arith.maxnumf %2, %0 : f32", "%6 = math.log2 %5 : f32", "affine.store %6, %arg1[%arg2] : memref<64xf32, 1>"):
        assert line in text, line
    m2, k2 = reparse(h.module, "scale")
    assert str(m2) == text and k2.verify()
    # the creators check their operands
    with pytest.raises(ValueError, match="one type"):
        b.create_mulf(c, b.get_f16(1.0))
    with pytest.raises(ValueError, match="widening"):
        b.create_extf(c, b.get_f16_ty())
    with pytest.raises(ValueError, match="element type"):
        b.create_store_op(c, x, [], F.AffineMap.get(0, 0, [b.get_affine_constant_expr(0)]))
    # and the parser reports type errors of the text
    with pytest.raises(ValueError, match="expects different type"):
        F.parse_module(F.create_context(), text.replace("arith.maxnumf %2, %0 : f32", "arith.maxnumf %2, %0 : f16"))


def _scale_kernel(h, n=64, in_dtype="fp16", out_dtype="fp32", c=0.5):
    """y[i] = log2(max(x[i], c) / (x[i] + c)): a free-standing frisk.block body"""
    b = h.builder
    kernel, entry = h.new_kernel("scale", [h.memref_type((n,), in_dtype), h.memref_type((n,), out_dtype)])
    x, y = entry.get_argument(0), entry.get_argument(1)
    cv = b.get_f32(c)

    def body(bb, ivs):
        v = bb.create_load_op(x, [ivs[0]])
        if in_dtype != "fp32":
            v = bb.create_extf(v, bb.get_f32_ty())
        r = bb.create_log2(bb.create_divf(bb.create_maxnumf(v, cv), bb.create_addf(v, cv)))
        if out_dtype != "fp32":
            r = bb.create_truncf(r, bb.get_f16_ty() if out_dtype == "fp16" else bb.get_bf16_ty())
        bb.create_store_op(r, y, [ivs[0]])
    b.create_block_op([n], body)
    return kernel


def _row_scale_kernel(h, rows=48, cols=40, dtype="fp16"):
    """two blocks over a rank-2 space: t[i, j] = x[i, j] * s[i] - m[j];  y[i, j] = exp2(min(t[i, j], t[i, 0])) + k[0]"""
    b = h.builder
    mat, rowv, colv = h.memref_type((rows, cols), dtype), h.memref_type((rows,), "fp32"), h.memref_type((cols,), "fp32")
    kernel, entry = h.new_kernel("row_scale", [mat, rowv, colv, h.memref_type((rows, cols), "fp32"), h.memref_type((rows, cols), dtype), h.memref_type((4,), "fp32")])
    x, s, m, t, y, k = (entry.get_argument(i) for i in range(6))
    zero = b.get_affine_constant_expr(0)

    def first(bb, ivs):
        v = bb.create_extf(bb.create_load_op(x, [ivs[0], ivs[1]]), bb.get_f32_ty())
        bb.create_store_op(bb.create_subf(bb.create_mulf(v, bb.create_load_op(s, [ivs[0]])), bb.create_load_op(m, [ivs[1]])), t, [ivs[0], ivs[1]])

    def second(bb, ivs):
        d0 = bb.get_affine_dim_expr(0)
        head = bb.create_load_op(t, [ivs[0]], F.AffineMap.get(1, 0, [d0, zero]))          # t[i, 0]: one element per row
        k0 = bb.create_load_op(k, [], F.AffineMap.get(0, 0, [zero]))                      # a scalar
        r = bb.create_addf(bb.create_exp2(bb.create_minnumf(bb.create_load_op(t, [ivs[0], ivs[1]]), head)), k0)
        bb.create_store_op(bb.create_truncf(r, bb.get_f16_ty() if dtype == "fp16" else bb.get_bf16_ty()), y, [ivs[0], ivs[1]])
    b.create_block_op([rows, cols], first)
    b.create_block_op([rows, cols], second)
    return kernel


def test_free_standing_block_bodies_become_postfix_programs():
    h = F.create_session()
    k = _scale_kernel(h)
    assert k.verify()
    want = {"program": "elementwise", "kernel": "scale", "target": "gfx950",
            "blocks": [{"rows": 1, "cols": 64, "out": (1, 0, 0, "f32"), "inputs": [(0, 0, 0, 1, "f16")], "postfix": "x0 c0.5 max x0 c0.5 add div log2", "stack": 3}]}
    assert F.runtime.match(k) == want
    assert F.runtime.match(reparse(h.module, "scale")[1]) == want
    # operands that broadcast: a value per row (row stride 1, column stride 0), a value per column (0, 1), a scalar (0, 0); the
    # second block reads what the first one stored
    h = F.create_session()
    p = F.runtime.match(_row_scale_kernel(h))
    b0, b1 = p["blocks"]
    assert (b0["rows"], b0["cols"]) == (48, 40) and b0["out"] == (3, 0, 40, "f32")
    assert b0["inputs"] == [(0, 0, 40, 1, "f16"), (1, 0, 1, 0, "f32"), (2, 0, 0, 1, "f32")] and b0["postfix"] == "x0 x1 mul x2 sub"
    assert b1["inputs"] == [(3, 0, 40, 1, "f32"), (3, 0, 40, 0, "f32"), (5, 0, 0, 0, "f32")] and b1["postfix"] == "x0 x1 min exp2 x2 add" and b1["out"] == (4, 0, 40, "f16")
    assert F.runtime.match(reparse(h.module, "row_scale")[1]) == p


def test_block_bodies_that_are_not_one_value_per_point_are_refused():
    sessions = []   # op handles do not own their module: the sessions stay alive with the test

    def kernel_with(body, ranges=(32,), shapes=((32,), (32,))):
        h = F.create_session()
        sessions.append(h)
        kernel, entry = h.new_kernel("k", [h.memref_type(s, "fp32") for s in shapes])
        h.builder.create_block_op(list(ranges), lambda bb, ivs: body(bb, ivs, [entry.get_argument(i) for i in range(len(shapes))]))
        return kernel

    def strided_store(bb, ivs, a):
        bb.create_store_op(bb.create_load_op(a[0], [ivs[0]]), a[1], [ivs[0]], F.AffineMap.get(1, 0, [bb.get_affine_dim_expr(0) * 2]))
    with pytest.raises(ValueError, match="column stride 2"):
        F.runtime.match(kernel_with(strided_store, (16,), ((32,), (32,))))

    def outside(bb, ivs, a):
        bb.create_store_op(bb.create_load_op(a[0], [ivs[0]], F.AffineMap.get(1, 0, [bb.get_affine_dim_expr(0) + 8])), a[1], [ivs[0]])
    with pytest.raises(ValueError, match="outside its extents"):
        F.runtime.match(kernel_with(outside))

    def shifted_in_place(bb, ivs, a):
        bb.create_store_op(bb.create_load_op(a[0], [ivs[0]], F.AffineMap.get(1, 0, [bb.get_affine_dim_expr(0) + 1])), a[0], [ivs[0]])
    with pytest.raises(ValueError, match="reads its own output"):
        F.runtime.match(kernel_with(shifted_in_place, (31,), ((32,),)))

    def two_stores(bb, ivs, a):
        v = bb.create_load_op(a[0], [ivs[0]])
        bb.create_store_op(v, a[1], [ivs[0]])
        bb.create_store_op(v, a[0], [ivs[0]])
    with pytest.raises(ValueError, match="more than one store"):
        F.runtime.match(kernel_with(two_stores))

    def deep(bb, ivs, a):   # a right-leaning chain of seven additions holds eight values at once
        v = bb.create_load_op(a[0], [ivs[0]])
        leaves = [bb.create_mulf(v, bb.get_f32(float(i + 2))) for i in range(8)]
        acc = leaves[7]
        for i in range(6, -1, -1):
            acc = bb.create_addf(leaves[i], acc)
        bb.create_store_op(acc, a[1], [ivs[0]])
    with pytest.raises(ValueError, match="evaluation stack"):
        F.runtime.match(kernel_with(deep))


def test_online_softmax_program_is_recognised():
    h = F.create_session()
    k = h.online_softmax("online_softmax", 8192, 8192, "fp16", chunk=1024, cst=1.25)     # the sketch's sizes
    assert k.verify() and h.module.verify()
    want = {"program": "online_softmax", "kernel": "online_softmax", "rows": 8192, "cols": 8192, "chunk": 1024, "scale_log2": 1.25, "dtype": "f16",
            "args": (0, 1), "target": "gfx950"}
    assert F.runtime.match(k) == want
    m2, k2 = reparse(h.module, "online_softmax")
    assert str(m2) == str(h.module) and F.runtime.match(k2) == want
    text = str(h.module)
    variants = {
        "other constant in one product": (text.replace("%12 = arith.mulf %11, %0 : f32", "%12 = arith.mulf %11, %11 : f32"), "first block"),
        "sum instead of max": (text.replace('kind = "max"', 'kind = "sum"'), "chunk maximum"),
        "log-sum not cleared to -inf": (text.replace("value = 0xFF800000 : f32", "value = 0.000000e+00 : f32"), "wrong fill value"),
        "second sweep reads other columns": (text.replace("frisk.copy %arg0[%arg2, %arg6 * 1024]", "frisk.copy %arg0[%arg2, %arg6 * 512]"), "chunk t of row bx"),
        "second sweep without the log-sum": (text.replace("%29 = arith.subf %27, %28 : f32", "%29 = arith.addf %27, %28 : f32"), "second sweep"),
        "first sweep short of the row": (text.replace("frisk.for %arg3 = 0 to 8 {", "frisk.for %arg3 = 0 to 7 {"), "does not cover the row"),
    }
    for name, (changed, message) in variants.items():
        assert changed != text, name
        with pytest.raises(ValueError, match=message):
            F.runtime.match(reparse(changed, "online_softmax")[1])


@pytest.mark.parametrize("k_transposed", [True, False])
def test_attention_program_is_recognised(k_transposed):
    h = F.create_session()
    k = h.attention("attention", 1, 32, 4096, 4096, 128, "fp16", cst=1.25, k_transposed=k_transposed)     # the sketch's sizes
    assert k.verify() and h.module.verify()
    p = F.runtime.match(k)
    assert p == {"program": "attention", "kernel": "attention", "batch": 1, "heads": 32, "seq_q": 4096, "seq_k": 4096, "head_dim": 128, "tile": (64, 64),
                 "k_transposed": k_transposed, "scale_log2": 1.25, "scale": 1.25 / 1.4426950408889634, "dtype": "f16", "args": (0, 1, 2, 3), "target": "gfx950"}
    m2, k2 = reparse(h.module, "attention")
    assert str(m2) == str(h.module) and F.runtime.match(k2) == p
    text = str(h.module)
    lines = text.splitlines()
    division = [i for i, l in enumerate(lines) if "arith.divf" in l]
    assert len(division) == 1
    start = max(i for i in range(division[0]) if "frisk.block" in lines[i])
    end = min(i for i in range(division[0], len(lines)) if lines[i].strip() == "}")
    variants = {
        # as the sketch has it: no division by the running sum, i.e. not a softmax
        "no normalisation": ("\n".join(lines[:start] + lines[end + 1:]), "two copies out"),
        "running maximum restarted every tile": (text.replace('{clear = false, dim = 1 : i64, kind = "max"}', '{clear = true, dim = 1 : i64, kind = "max"}'), "running maximum"),
        "value tile of another head": (text.replace("frisk.copy %arg2[%arg4, %arg5,", "frisk.copy %arg2[%arg4, %arg4,"), "value tile"),
        "rescale by the wrong factor": (text.replace("arith.divf", "arith.mulf"), "after the key loop"),
        "output stored to another query tile": (text.replace("%arg3[%arg4, %arg5, %arg6 * 64, 0]", "%arg3[%arg4, %arg5, %arg6 * 64 + 64, 0]"), "output tile"),
    }
    for name, (changed, message) in variants.items():
        assert changed != text, name
        with pytest.raises(ValueError, match=message):
            F.runtime.match(reparse(changed, "attention")[1])


def test_tiled_gemm_is_still_a_program_of_its_own():
    h = F.create_session()
    k = h.tiled_gemm("g", 512, 512, 256, "fp16", tile=(256, 256, 64))
    assert F.runtime.match(k)["program"] == "tiled_gemm"


# ------------------------------------------------------------------ GPU
def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1).copy()).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,odt,tol", [("fp16", O.F16, 2e-3), ("bf16", O.BF16, 8e-3), ("fp32", O.F32, 2e-5)])
def test_parsed_online_softmax_module_runs_to_the_oracles_result(hip, dtype, odt, tol):
    import torch
    rows, cols, cst = 96, 8192, 1.25
    h = F.create_session()
    h.online_softmax("online_softmax", rows, cols, dtype, chunk=1024, cst=cst)
    module, kernel = reparse(h.module, "online_softmax")            # from text, as a saved module would be
    print(f"case parsed online softmax {dtype} {rows}x{cols}", flush=True)
    x = O.encode(odt, O.normal(rows * cols, 61, 0, 3.0)).reshape(rows, cols)
    dx = _dev(x)
    dy = torch.zeros_like(dx)
    F.runtime.launch(kernel, [dx.data_ptr(), dy.data_ptr()], torch.cuda.current_stream().cuda_stream, module)
    torch.cuda.synchronize()
    got = O.decode(odt, dy.cpu().numpy().view(O.NP_STORAGE[odt])).astype(np.float64).reshape(rows, cols)
    sketch, _ = T.online_softmax_sketch(odt, x, cst, chunk=1024)      # the sketch op by op, float64
    ref, _ = T.softmax_f64(odt, x, cst)
    assert np.allclose(sketch, ref, rtol=1e-10, atol=1e-300)
    scale = np.maximum(np.abs(ref), np.sqrt(np.mean(ref * ref)))
    floor = 2.0 ** -25 if odt == O.F16 else 0.0
    assert np.all(np.isfinite(got)) and np.all(np.abs(got - ref) <= tol * scale + floor), float(np.max(np.abs(got - ref) / scale))


@pytest.mark.gpu
@pytest.mark.parametrize("k_transposed", [True, False])
def test_parsed_attention_module_runs_to_the_oracles_result(hip, k_transposed):
    import torch
    batch, heads, seq, dim = 1, 3, 512, 128
    scale = dim ** -0.5
    h = F.create_session()
    h.attention("attention", batch, heads, seq, seq, dim, "fp16", cst=scale * A.LOG2E, k_transposed=k_transposed)
    module, kernel = reparse(h.module, "attention")
    print(f"case parsed attention k_transposed={k_transposed}", flush=True)
    bh = batch * heads
    q = O.encode(O.F16, O.normal(bh * seq * dim, 62, 0, 1.0)).reshape(bh, seq, dim)
    k = O.encode(O.F16, O.normal(bh * seq * dim, 62, 1, 1.0)).reshape(bh, seq, dim)
    v = O.encode(O.F16, O.normal(bh * seq * dim, 62, 2, 1.0)).reshape(bh, seq, dim)
    if k_transposed:
        k = np.ascontiguousarray(np.swapaxes(k, 1, 2))
    dq, dk, dv = _dev(q), _dev(k), _dev(v)
    do = torch.zeros_like(dq)
    F.runtime.launch(kernel, [dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), do.data_ptr()], torch.cuda.current_stream().cuda_stream, module)
    torch.cuda.synchronize()
    got = O.decode(O.F16, do.cpu().numpy().view(np.uint16)).astype(np.float64).reshape(bh, seq, dim)
    ref, _ = A.attention_f64(O.F16, q, k, v, scale, k_transposed=k_transposed)
    tiled, _ = A.attention_tiled(O.F16, q, k, v, scale, k_transposed=k_transposed, key_tile=64)     # the sketch's loop, tile by tile
    assert np.abs(tiled - ref).max() < 2e-3
    rms = np.sqrt(np.mean(ref * ref))
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) <= 1e-2
    assert np.all(np.abs(got - ref) <= 1e-2 * np.maximum(np.abs(ref), rms))


@pytest.mark.gpu
@pytest.mark.parametrize("in_dtype,out_dtype,n,tol", [("fp16", "fp32", 64, 2e-6), ("fp16", "fp16", 4096 * 33, 1e-3), ("bf16", "bf16", 1000, 8e-3), ("fp32", "fp32", 8 * 1031, 2e-6)])
def test_free_standing_block_body_runs_to_numpys_result(hip, in_dtype, out_dtype, n, tol):
    """y[i] = log2(max(x[i], c) / (x[i] + c)) built with the IR builder, matched, lowered to one interpreted kernel and compared
    with numpy's float64 value of the same formula (written out here, not the oracle's postfix evaluator); the oracle's
    evaluator is pinned to the same formula on the way"""
    import torch
    from helpers import to_dev, from_dev
    codes = {"fp16": O.F16, "bf16": O.BF16, "fp32": O.F32}
    h = F.create_session()
    kernel = _scale_kernel(h, n, in_dtype, out_dtype, c=0.5)
    x = O.encode(codes[in_dtype], np.abs(O.normal(n, 91, 0, 2.0)) + 0.01)
    xf = O.decode(codes[in_dtype], x).astype(np.float64)
    want = np.log2(np.fmax(xf, 0.5) / (xf + 0.5))
    prog = [("input", 0), ("const", 0.5), "max", ("input", 0), ("const", 0.5), "add", "div", "log2"]
    assert np.array_equal(T.elementwise(prog, [xf.reshape(1, n)], 1, n).reshape(n), want)
    dx = to_dev(x)
    dy = torch.full((n * O.NP_STORAGE[codes[out_dtype]]().itemsize,), 0xEE, dtype=torch.uint8, device="cuda")
    F.runtime.launch(kernel, [dx.data_ptr(), dy.data_ptr()], torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = O.decode(codes[out_dtype], from_dev(dy, O.NP_STORAGE[codes[out_dtype]], (n,))).astype(np.float64)
    assert np.all(np.isfinite(got))
    err = np.abs(got - want) / np.maximum(np.abs(want), np.sqrt(np.mean(want ** 2)))
    assert err.max() <= tol, err.max()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_two_blocks_with_broadcast_operands_run_in_program_order(hip, dtype):
    import torch
    from helpers import to_dev, from_dev
    code = {"fp16": O.F16, "bf16": O.BF16}[dtype]
    rows, cols = 48, 40
    h = F.create_session()
    kernel = reparse(h.module, "row_scale")[1] if False else _row_scale_kernel(h, rows, cols, dtype)
    x = O.encode(code, O.normal(rows * cols, 92, 0, 1.0)).reshape(rows, cols)
    s = O.uniform(rows, 92, 1, 0.5, 2.0).astype(np.float32)
    m = O.uniform(cols, 92, 2, -1.0, 1.0).astype(np.float32)
    k = np.array([0.25, 9.0, 9.0, 9.0], dtype=np.float32)
    xf = O.decode(code, x).astype(np.float64).reshape(rows, cols)
    t64 = (xf * s[:, None].astype(np.float64)).astype(np.float32).astype(np.float64) - m[None, :]      # the kernel multiplies and subtracts in fp32
    t32 = t64.astype(np.float32)
    want = np.exp2(np.fmin(t32.astype(np.float64), t32[:, :1].astype(np.float64))) + 0.25
    d = [to_dev(a) for a in (x, s, m)] + [torch.zeros(rows * cols, dtype=torch.float32, device="cuda"), torch.zeros(rows * cols, dtype=torch.int16, device="cuda"), to_dev(k)]
    F.runtime.launch(kernel, [t.data_ptr() for t in d], torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got_t = d[3].cpu().numpy().reshape(rows, cols)
    assert np.abs(got_t - t32).max() <= 2e-6 * max(1.0, np.abs(t32).max())
    got = O.decode(code, from_dev(d[4], np.uint16, (rows, cols))).astype(np.float64)
    tol = 1e-3 if dtype == "fp16" else 8e-3
    assert (np.abs(got - want) / np.maximum(np.abs(want), 1.0)).max() <= tol
