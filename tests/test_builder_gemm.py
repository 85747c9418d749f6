"""The builder surface, driven exactly as the reference's own scripts drive it
(test/python/bind_test.py:3-62, test/python/helper_test.py:4-24), and checked against the
output the reference saved for bind_test.py (tmp/log_11_18, kept as tests/golden/bind_test_module.mlir)."""
import os

import pytest

import frisk_amd  # noqa: F401  (puts the `frisk` package on the path)
import frisk as F

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def create_gemmop():
    """call for call the body of bind_test.py:create_gemmop"""
    context = F.context()
    F.frisk.load_dialects(context)
    builder = F.builder(context)
    module = builder.create_module()
    module.context = context

    shape = [4096, 4096]
    shape2 = [4096]
    dtype = builder.get_f16_ty()
    mem_type = builder.get_memref_ty(dtype, shape, F.AffineMap(), F.MemorySpace.GLOBAL)
    mem2_type = builder.get_memref_ty(dtype, shape2, F.AffineMap(), F.MemorySpace.GLOBAL)
    kernel_type = builder.get_kernel_ty([mem_type, mem_type, mem_type, mem2_type])
    kernel = builder.create_kernel_op(module, "test_gemm", kernel_type)
    module.push_back(kernel)
    entry1 = kernel.add_entry_block()
    builder.set_insertion_point_to_start(entry1)
    prarllel = builder.create_parallel_op([8, 8], 128)
    entry2 = prarllel.add_entry_block()
    builder.set_insertion_point_to_start(entry2)

    input_val = [entry1.get_argument(0), entry1.get_argument(1), entry1.get_argument(2), entry1.get_argument(3)]

    builder.create_alloc_buffer_op([128, 32], "fp16", F.MemorySpace.SHARED, 1024)
    builder.create_alloc_buffer_op([32, 128], "fp16", F.MemorySpace.SHARED, 1024)
    builder.create_alloc_buffer_op([128, 128], "fp16", F.MemorySpace.LOCAL)

    def for_body_test(b, iv):
        builder.create_fill_op(input_val[0], 0.0, "fp16")
        builder.create_reduce_op(input_val[0], input_val[3], "max", 1, True)
        builder.create_copy_op(input_val[0], input_val[1], [iv, iv], [iv, iv])

        def block_body_test(b, ivs):
            b.create_gemm_op(input_val[0], input_val[1], input_val[2])

        builder.create_block_op([128, 128], block_body_test)

    builder.create_for_op(0, 128, 1, for_body_test)
    return module


def test_bind_test_module_prints_as_the_reference_saved_it():
    module = create_gemmop()
    want = open(os.path.join(GOLDEN, "bind_test_module.mlir")).read().strip("\n")
    assert str(module) == want
    assert module.verify()


def test_helper_test_sequence():
    """call for call helper_test.py:build_sample_module, with its three asserts"""
    helper = F.create_session()
    f16 = helper.builder.get_f16_ty()
    a_ty = helper.memref_type((128, 64), f16, space=F.MemorySpace.SHARED)
    b_ty = helper.memref_type((64, 128), f16, space=F.MemorySpace.SHARED)
    c_ty = helper.memref_type((128, 128), f16, space=F.MemorySpace.LOCAL)
    kernel, entry = helper.new_kernel("helper_demo", [a_ty, b_ty, c_ty])
    args = [entry.get_argument(i) for i in range(3)]
    gemm = helper.create_gemm(args[0], args[1], args[2])
    scratch = helper.alloc_buffer((32, 32), "fp16", space=F.MemorySpace.SHARED, alignment=64)
    assert "memref" in str(scratch.get_type())
    assert kernel.verify()
    assert helper.module.verify()
    assert (gemm.get_m(), gemm.get_n(), gemm.get_k()) == (128, 128, 64)
    text = str(helper.module)
    assert "frisk.kernel @helper_demo(memref<128x64xf16, 3>, memref<64x128xf16, 3>, memref<128x128xf16>)" in text
    assert '%0 = frisk.alloc_buffer {scope = "shared", alignment = 64} -> memref<32x32xf16, 3>' in text


def test_enum_values_and_type_printing():
    # Local = 0, Global = 1, Shared = 3 (reference output tmp/log_11_25:5-8); the number is what a memref prints
    assert int(F.MemorySpace.LOCAL) == 0 and int(F.MemorySpace.GLOBAL) == 1 and int(F.MemorySpace.SHARED) == 3
    h = F.create_session()
    assert str(h.memref_type((4, 8), "fp32")) == "memref<4x8xf32, 1>"
    assert str(h.memref_type((4, 8), "bf16", space=F.MemorySpace.LOCAL)) == "memref<4x8xbf16>"
    assert not F.AffineMap() and F.AffineMap.get_multi_dim_identity_map(2)
    t = h.memref_type((16, 32), "fp16", space=F.MemorySpace.SHARED)
    assert t.get_shape() == [16, 32] and t.get_rank() == 2 and t.get_elem_width() == 16 and t.get_memory_space() == F.MemorySpace.SHARED


def test_error_conventions():
    h = F.create_session()
    f16, f32 = h.builder.get_f16_ty(), h.builder.get_f32_ty()
    kernel, entry = h.new_kernel("k", [h.memref_type((128, 64), f16), h.memref_type((32, 128), f16), h.memref_type((128, 128), f16),
                                       h.memref_type((64, 128), f32), h.memref_type((128,), f16)])
    a, b_bad, c, b_f32, vec = (entry.get_argument(i) for i in range(5))
    with pytest.raises(ValueError, match="inner dimensions"):
        h.builder.create_gemm_op(a, b_bad, c)
    with pytest.raises(ValueError, match="matching element types"):
        h.builder.create_gemm_op(a, b_f32, c)
    with pytest.raises(ValueError, match="rank-2"):
        h.builder.create_gemm_op(a, vec, c)
    with pytest.raises(ValueError, match="invalid float type"):
        h.builder.create_alloc_buffer_op([8, 8], "fp13")
    with pytest.raises(ValueError, match="non-negative"):
        h.builder.create_alloc_buffer_op([8, 8], "fp16", F.MemorySpace.SHARED, -4)
    with pytest.raises(IndexError):
        entry.get_argument(9)
    with pytest.raises(ValueError, match="copy op map error"):
        h.builder.create_copy_op(a, c, [], [], F.AffineMap.get_multi_dim_identity_map(2))   # only one of the two maps
    # parallel must be the first op of a block that holds only its terminator
    h.builder.create_alloc_buffer_op([8, 8], "fp16")
    with pytest.raises(ValueError, match="invalid parallel create"):
        h.builder.create_parallel_op([2, 2], 64)
    # verifier failures are reported through the return value, not raised
    h2 = F.create_session()
    k2, e2 = h2.new_kernel("k2", [h2.memref_type((8, 8), f16)])
    h2.builder.create_fill_op(e2.get_argument(0), 1.0, "fp32")
    assert not k2.verify() and not h2.module.verify()


def test_body_callbacks_propagate_python_errors_and_restore_the_insertion_point():
    h = F.create_session()
    kernel, entry = h.new_kernel("k", [h.memref_type((8, 8), "fp16")])

    def boom(b, iv):
        raise KeyError("inside the body")

    with pytest.raises(KeyError):
        h.builder.create_for_op(0, 4, 1, boom)
    h.builder.create_fill_op(entry.get_argument(0), 0.0, "fp16")   # lands in the kernel body, not in the abandoned loop
    assert str(h.module).count("frisk.fill") == 1 and "frisk.for" not in str(h.module)


def test_affine_maps_of_a_tiled_copy_print_like_mlir():
    h = F.create_session()
    b = h.builder
    d0, d1 = b.get_affine_dim_expr(0), b.get_affine_dim_expr(1)
    m = F.AffineMap.get(2, 0, [d0 * 128, d1 * 32 + 5])
    assert str(m) == "(d0, d1) -> (d0 * 128, d1 * 32 + 5)"
    assert (d0 * 128).evaluate([3, 0]) == 384 and ((d0 + d1 * 2) % 3).evaluate([4, 1]) == 0
    assert str((d0 + 7).floor_div(4)) == "(d0 + 7) floordiv 4" and str(d0 - d1) == "d0 - d1"


def test_tiled_gemm_program_matches_the_design_sketch():
    """fp32 1024^3, grid 8x8, 128 threads, shared A 128x32, shared B 32x128, fragment C 128x128:
    the matmul program of the reference's tmp/ir.mlir:1-17, built through the builder"""
    h = F.create_session()
    kernel = h.tiled_gemm("matmul", 1024, 1024, 1024, "fp32", tile=(128, 128, 32), threads=128)
    assert kernel.verify() and h.module.verify()
    text = str(h.module)
    assert "frisk.parallel (%arg3, %arg4) = (8, 8), threads = 128 {" in text
    assert "frisk.for %arg5 = 0 to 32 {" in text
    assert "frisk.copy %arg0[%arg3 * 128, %arg5 * 32], %0[0, 0] {src_extents = [128, 32], dst_extents = [128, 32]}" in text
    assert "frisk.copy %arg1[%arg5 * 32, %arg4 * 128], %1[0, 0] {src_extents = [32, 128], dst_extents = [32, 128]}" in text
    assert "frisk.copy %2[0, 0], %arg2[%arg3 * 128, %arg4 * 128]" in text
    p = F.runtime.match(kernel)
    assert (p["M"], p["N"], p["K"]) == (1024, 1024, 1024) and p["tile"] == (128, 128, 32) and p["grid"] == (8, 8)
    assert p["threads"] == 128 and p["clear_accum"] and not p["transA"] and not p["transB"]
    assert (p["dtype_ab"], p["dtype_acc"], p["dtype_out"]) == ("f32", "f32", "f32") and p["args"] == (0, 1, 2)


def test_matcher_rejects_what_is_not_a_tiled_gemm():
    module = create_gemmop()                      # the bind_test module: gemm on global memrefs inside a block op
    with pytest.raises(ValueError, match="not a tiled GEMM"):
        F.runtime.match(module.get_kernel("test_gemm"))
    h = F.create_session()
    kernel = h.tiled_gemm("g", 512, 512, 512, "fp16", tile=(256, 256, 64))
    kernel.set_attr("frisk.target", "sm_80")      # the reference's layout inference only knows sm_80 / sm_90; this path only gfx950
    with pytest.raises(ValueError, match="gfx950"):
        F.runtime.match(kernel)
    kernel.set_attr("frisk.target", "gfx950")
    assert F.runtime.match(kernel)["target"] == "gfx950"


def _reparsed_kernel(text):
    ctx = F.create_context()
    module = F.parse_module(ctx, text)
    module.context = ctx
    return module, module.get_kernel("g")


def test_matcher_checks_what_the_program_computes_not_only_its_shape():
    """A kernel that has the ops of a tiled GEMM but addresses other windows, clears the accumulator with another value or not
    at all, would be silently run as the canonical GEMM: the matcher refuses each of them"""
    h = F.create_session()
    h.tiled_gemm("g", 512, 768, 256, "fp16", tile=(256, 256, 64))
    text = str(h.module)
    assert F.runtime.match(_reparsed_kernel(text)[1])["tile"] == (256, 256, 64)       # the unchanged text is accepted
    # equivalent forms are accepted: the K loop counting elements instead of tiles
    by_elements = text.replace("frisk.for %arg5 = 0 to 4 {", "frisk.for %arg5 = 0 to 256 step = 64 {").replace("%arg5 * 64", "%arg5")
    assert F.runtime.match(_reparsed_kernel(by_elements)[1])["K"] == 256
    variants = {
        "fill value": (text.replace("value = 0.000000e+00", "value = 1.000000e+00"), "filled with 0"),
        "no fill": ("\n".join(l for l in text.splitlines() if "frisk.fill" not in l), "cleared by a frisk.fill"),
        "swapped grid indices in the store": (text.replace("%arg2[%arg3 * 256, %arg4 * 256]", "%arg2[%arg4 * 256, %arg3 * 256]"), "canonical tiling"),
        "offset window of A": (text.replace("%arg0[%arg3 * 256, %arg5 * 64]", "%arg0[%arg3 * 256, %arg5 * 64 + 64]"), "canonical tiling"),
        "A indexed by the wrong grid index": (text.replace("%arg0[%arg3 * 256,", "%arg0[%arg4 * 256,"), "canonical tiling"),
        "wrong K stride of B": (text.replace("%arg1[%arg5 * 64,", "%arg1[%arg5 * 32,"), "canonical tiling"),
        "offset inside the shared tile": (text.replace("%0[0, 0] {src_extents = [256, 64]", "%0[0, 8] {src_extents = [256, 64]"), "canonical tiling"),
        "window smaller than the tile": (text.replace("{src_extents = [256, 64], dst_extents = [256, 64]}", "{src_extents = [128, 64], dst_extents = [128, 64]}"), "whole tile"),
        "K loop short of K": (text.replace("frisk.for %arg5 = 0 to 4 {", "frisk.for %arg5 = 0 to 3 {"), "cover K"),
    }
    for name, (changed, message) in variants.items():
        assert changed != text, name
        module, kernel = _reparsed_kernel(changed)
        with pytest.raises(ValueError, match=message):
            F.runtime.match(kernel)
    # a rank-1 shared buffer is refused before its shape is indexed
    h2 = F.create_session()
    b = h2.builder
    tys = [h2.memref_type((256, 64), "fp16"), h2.memref_type((64, 256), "fp16"), h2.memref_type((256, 256), "fp16")]
    kernel, entry = h2.new_kernel("g", tys)
    body = b.create_parallel_op([1, 1], 256).add_entry_block()
    b.set_insertion_point_to_start(body)
    flat = h2.alloc_buffer((256 * 64,), "fp16", space=F.MemorySpace.SHARED)
    sB = h2.alloc_buffer((64, 256), "fp16", space=F.MemorySpace.SHARED)
    with pytest.raises(ValueError):
        h2.create_gemm(flat, sB, h2.alloc_buffer((256, 256), "fp32", space=F.MemorySpace.LOCAL))      # the builder already refuses rank 1


def test_transpose_flags_stored_transposed_first_then_the_references_reading():
    """ffi/ir.cpp:346-355 reads A as [M][K] and B as [K][N] whatever the flags say; this build reads a flagged operand as stored
    transposed when the shapes allow it, and falls back to the reference's reading (flag = layout hint) when only that fits"""
    h = F.create_session()
    mk = lambda shape, space=F.MemorySpace.SHARED, dt="fp16": h.alloc_buffer(shape, dt, space=space)
    h.new_kernel("k", [])
    acc = mk((128, 256), F.MemorySpace.LOCAL, "fp32")
    stored_t = h.create_gemm(mk((128, 64)), mk((256, 64)), acc, trans_b=True)          # B stored [N][K]
    assert "K = 64 : i64, M = 128 : i64, N = 256 : i64" in str(stored_t) and "transB = true" in str(stored_t)
    hint = h.create_gemm(mk((128, 64)), mk((64, 256)), acc, trans_a=True, trans_b=True)  # the reference's reading: shapes un-transposed
    assert "K = 64 : i64, M = 128 : i64, N = 256 : i64" in str(hint) and hint.verify()
    with pytest.raises(ValueError, match="inner dimensions"):
        h.create_gemm(mk((128, 64)), mk((256, 32)), acc, trans_b=True)                  # fits neither reading
    # in a tiled program the hint form runs as the un-transposed GEMM
    h2 = F.create_session()
    h2.tiled_gemm("g", 512, 768, 256, "fp16", tile=(256, 256, 64))
    text = str(h2.module).replace("transA = false, transB = false", "transA = true, transB = true")
    p = F.runtime.match(_reparsed_kernel(text)[1])
    assert not p["transA"] and not p["transB"] and (p["M"], p["N"], p["K"]) == (512, 768, 256)


def test_plan_goes_through_the_hip_library():
    h = F.create_session()
    kernel = h.tiled_gemm("g", 4096, 4096, 4096, "fp16", tile=(256, 256, 64), trans_b=True)
    p = F.runtime.plan(kernel)
    assert p["hip_tile"] == (256, 256, 64) and p["hip_grid"] == (16, 16) and p["lds_bytes"] <= 160 * 1024
    assert p["hip_kernel"].startswith("f16_nt_256x256x64") and p["flops"] == 2.0 * 4096 ** 3


def test_plan_names_the_kernel_that_launch_runs_for_either_retile():
    """`plan` and `launch` build their descriptor in one place: with retile (the default of both) the planner's tile for the
    whole problem, without it the tile the program is written with"""
    from frisk_amd import runtime as R
    h = F.create_session()
    kernel = h.tiled_gemm("g", 1024, 1024, 1024, "fp32", tile=(128, 128, 32), threads=256)
    own = R.plan(R.make_desc(R.F32, 1024, 1024, 1024))
    kept = R.plan(R.make_desc(R.F32, 1024, 1024, 1024, tile=(128, 128, 32)))
    p = F.runtime.plan(kernel)
    assert p["hip_kernel"] == R.kernel_names()[own.kernel_id] and p["hip_tile"] == (own.tile_m, own.tile_n, own.tile_k) != (128, 128, 32)
    assert p["lds_bytes"] == own.lds_bytes and F.runtime.plan(kernel, retile=True) == p
    q = F.runtime.plan(kernel, retile=False)
    assert q["hip_kernel"] == R.kernel_names()[kept.kernel_id] and q["hip_tile"] == (128, 128, 32) and q["lds_bytes"] == kept.lds_bytes


@pytest.mark.parametrize("dtype,tile,trans_a,trans_b", [("fp16", (256, 256, 64), False, False), ("fp16", (256, 256, 64), False, True),
                                                        ("bf16", (128, 128, 64), True, False),
                                                        ("fp32", (128, 128, 32), False, False)])
def test_plan_prints_lds_layouts_in_the_reference_debug_form(dtype, tile, trans_a, trans_b):
    """Layout(shape=[...], index=affine_map<...>) as printLayoutDebug writes it; evaluating the printed map with the
    oracle's affine evaluator gives, element by element, the offsets frisk_hip_lds_offset computes"""
    import re

    import numpy as np

    from frisk_amd import runtime as R
    from oracle import layouts as L
    es = {"fp16": 2, "bf16": 2, "fp32": 4}[dtype]
    h = F.create_session()
    n = 4 * max(tile)
    kernel = h.tiled_gemm("g", n, n, n, dtype, tile=tile, trans_a=trans_a, trans_b=trans_b)
    p = F.runtime.plan(kernel, retile=False)
    for text, (sh, mk, cs), (sh2, mk2, cs2) in zip((p["lds_a"], p["lds_b"]), p["lds_swizzle"], p["lds_swizzle2"]):
        m = re.fullmatch(r"Layout\(shape=\[(\d+), (\d+)\], index=(affine_map<.*>)\)", text)
        assert m, text
        rows, cols = int(m.group(1)), int(m.group(2))
        i, j = L.grid(rows, cols)
        (idx,) = L.eval_affine_map(m.group(3), i, j)
        lay = R.LdsLayout(rows=rows, row_bytes=cols * es, k_contiguous=1, row_shift=sh, row_mask=mk, chunk_shift=cs, row_shift2=sh2, row_mask2=mk2, chunk_shift2=cs2)
        rr = np.random.default_rng(0).integers(0, rows, 300)
        cc = np.random.default_rng(1).integers(0, cols, 300)
        for r, c in zip(rr, cc):
            assert R.lds_offset(lay, int(r), int(c) * es) == int(idx[r, c]) * es
        assert len(np.unique(idx)) == rows * cols and idx.max() == rows * cols - 1  # a permutation of the tile


def _data_movement_kernel(h):
    """kernel(x: 64x96 f32, y: 64x96 f16, v: 64 f16): y := 0.5; y[8:40, 16:80] := f16(x[0:32, 32:96]); v := max over columns of y"""
    b = h.builder
    x_t, y_t, v_t = h.memref_type((64, 96), "fp32"), h.memref_type((64, 96), "fp16"), h.memref_type((64,), "fp16")
    kernel, entry = h.new_kernel("prep", [x_t, y_t, v_t])
    x, y, v = (entry.get_argument(i) for i in range(3))
    c = b.get_affine_constant_expr
    b.create_fill_op(y, 0.5, "fp16")
    b.create_copy_op(x, y, [], [], srcMap=F.AffineMap.get(0, 0, [c(0), c(32)]), dstMap=F.AffineMap.get(0, 0, [c(8), c(16)]),
                     srcExtents=[32, 64], dstExtents=[32, 64])
    b.create_reduce_op(y, v, "max", 1, True)
    return kernel


def test_data_movement_kernel_is_recognised_op_by_op():
    h = F.create_session()
    kernel = _data_movement_kernel(h)
    assert h.module.verify()
    ops = F.runtime.match_ops(kernel)
    assert [o["op"] for o in ops] == ["fill", "copy", "reduce"]
    assert ops[0] == {"op": "fill", "rows": 64, "cols": 96, "dst": 1, "dst_offset": 0, "dst_dtype": "f16", "dst_ld": 96, "value": 0.5}
    assert ops[1]["src"] == 0 and ops[1]["src_offset"] == 32 and ops[1]["dst_offset"] == 8 * 96 + 16 and (ops[1]["rows"], ops[1]["cols"]) == (32, 64)
    assert (ops[1]["src_ld"], ops[1]["dst_ld"], ops[1]["src_dtype"], ops[1]["dst_dtype"]) == (96, 96, "f32", "f16")
    assert ops[2]["kind"] == "max" and ops[2]["dim"] == 1 and ops[2]["clear"] is True and (ops[2]["src"], ops[2]["dst"]) == (1, 2)
    # a tiled GEMM is not a data-movement kernel, and a window that leaves its memref is refused
    with pytest.raises(ValueError):
        F.runtime.match_ops(h.tiled_gemm("g", 256, 256, 64, "fp16", tile=(128, 128, 32)))
    h2 = F.create_session()
    t = h2.memref_type((8, 8), "fp32")
    k2, e2 = h2.new_kernel("bad", [t, t])
    c = h2.builder.get_affine_constant_expr
    h2.builder.create_copy_op(e2.get_argument(0), e2.get_argument(1), [], [], srcMap=F.AffineMap.get(0, 0, [c(4), c(0)]),
                              dstMap=F.AffineMap.get(0, 0, [c(0), c(0)]), srcExtents=[8, 8], dstExtents=[8, 8])
    with pytest.raises(ValueError) as e:
        F.runtime.match_ops(k2)
    assert "window leaves the memref" in str(e.value)


def _tiled_copy_kernel(h, *, staged=True, dst_origin=(16, 64), src_tile_step=None, dst_scale=(32, 64), rows=128, cols=256, loop=True):
    """kernel(x: rows x cols f32, y: (rows+32) x (cols+64) f16): y[16 + i, 64 + j] := f16(x[i, j]), written tile by tile: a grid over
    32-row bands, a loop over 64-column tiles, every 32 x 64 tile through a shared buffer (or directly)"""
    b = h.builder
    x_t, y_t = h.memref_type((rows, cols), "fp32"), h.memref_type((rows + 32, cols + 64), "fp16")
    kernel, entry = h.new_kernel("tiled_copy", [x_t, y_t])
    x, y = entry.get_argument(0), entry.get_argument(1)
    body = b.create_parallel_op([rows // 32], 256).add_entry_block()
    b.set_insertion_point_to_start(body)
    by = body.get_argument(0)
    tile = h.alloc_buffer((32, 64), "fp32", space=F.MemorySpace.SHARED) if staged else None
    d0, d1 = b.get_affine_dim_expr(0), b.get_affine_dim_expr(1)
    c = b.get_affine_constant_expr
    src_map = F.AffineMap.get(2, 0, [d0 * 32, d1 * (src_tile_step or 1)])
    dst_map = F.AffineMap.get(2, 0, [d0 * dst_scale[0] + dst_origin[0], d1 * (dst_scale[1] // 64) + dst_origin[1]])
    zero = F.AffineMap.get(0, 0, [c(0), c(0)])

    def tile_body(bb, j):  # j walks columns in elements (step 64)
        if staged:
            bb.create_copy_op(x, tile, [by, j], [], src_map, zero, [32, 64], [32, 64])
            bb.create_copy_op(tile, y, [], [by, j], zero, dst_map, [32, 64], [32, 64])
        else:
            bb.create_copy_op(x, y, [by, j], [by, j], src_map, dst_map, [32, 64], [32, 64])

    if loop:
        b.create_for_op(0, cols, 64, tile_body)
    else:
        tile_body(b, by)
    return kernel


def test_tiled_copy_is_lowered_as_one_window_copy():
    """frisk.copy with index operands (FriskOps.cpp:1551-1683): the tiles of a grid and a loop, through a shared buffer or not,
    are recognised as one copy of the rectangle they cover"""
    for staged in (True, False):
        h = F.create_session()
        kernel = _tiled_copy_kernel(h, staged=staged)
        assert h.module.verify()
        ops = F.runtime.match_ops(kernel)
        assert len(ops) == 1 and ops[0]["op"] == "copy"
        o = ops[0]
        assert (o["src"], o["dst"], o["rows"], o["cols"]) == (0, 1, 128, 256)
        assert (o["src_offset"], o["dst_offset"], o["src_ld"], o["dst_ld"]) == (0, 16 * 320 + 64, 256, 320)
        assert (o["src_dtype"], o["dst_dtype"]) == ("f32", "f16")
        # the printed form parses back to the same program
        again = F.parse_module(h.context, str(h.module))
        assert F.runtime.match_ops(again.get_kernel("tiled_copy")) == ops


@pytest.mark.parametrize("kw, message", [
    (dict(src_tile_step=2), "do not tile a rectangle"),            # source tiles 128 columns apart: gaps
    (dict(dst_scale=(16, 64)), "do not tile a rectangle"),         # destination bands overlap
    (dict(dst_scale=(64, 64), rows=64), "do not tile a rectangle"),  # destination bands 64 rows apart: gaps
    (dict(loop=False), "along two dimensions"),                     # one index drives rows and columns
])
def test_tiled_copy_that_is_not_one_rectangle_is_refused(kw, message):
    h = F.create_session()
    kernel = _tiled_copy_kernel(h, **kw)
    with pytest.raises(ValueError) as e:
        F.runtime.match_ops(kernel)
    assert message in str(e.value), str(e.value)


def test_fill_under_a_grid_is_refused():
    h = F.create_session()
    t = h.memref_type((64, 64), "fp16")
    kernel, entry = h.new_kernel("k", [t])
    body = h.builder.create_parallel_op([4], 64).add_entry_block()
    h.builder.set_insertion_point_to_start(body)
    h.builder.create_fill_op(entry.get_argument(0), 1.0, "fp16")
    with pytest.raises(ValueError) as e:
        F.runtime.match_ops(kernel)
    assert "once per iteration" in str(e.value)


def _transposed_tiles_kernel(h, n=64, tile=32, dtype="fp16", out_dtype=None):
    """tile (by, bx) of the n x n source lands at (bx, by) of the destination; the elements of a tile keep their order"""
    b = h.builder
    kernel, entry = h.new_kernel("k", [h.memref_type((n, n), dtype), h.memref_type((n, n), out_dtype or dtype)])
    body = b.create_parallel_op([n // tile, n // tile], 64).add_entry_block()
    b.set_insertion_point_to_start(body)
    by, bx = body.get_argument(0), body.get_argument(1)
    d0, d1 = b.get_affine_dim_expr(0), b.get_affine_dim_expr(1)
    b.create_copy_op(entry.get_argument(0), entry.get_argument(1), [by, bx], [by, bx], F.AffineMap.get(2, 0, [d0 * tile, d1 * tile]),
                     F.AffineMap.get(2, 0, [d1 * tile, d0 * tile]), [tile, tile], [tile, tile])
    return kernel


def test_tiled_copy_that_places_tiles_transposed_is_one_tile_by_tile_copy():
    """both sides tile a square, but tile (by, bx) of the source lands at (bx, by) of the destination: not a window copy; it is
    lowered as one launch that copies tile by tile, each grid index displacing the two sides by its own step"""
    h = F.create_session()
    (op,) = F.runtime.match_ops(_transposed_tiles_kernel(h))
    assert op["op"] == "copy_tiles" and (op["rows"], op["cols"]) == (32, 32) and op["tiles"] == (2, 2)
    assert op["src_steps"] == (32 * 64, 32) and op["dst_steps"] == (32, 32 * 64) and (op["src_ld"], op["dst_ld"]) == (64, 64)
    # a third index that rearranges is more than one launch places
    h = F.create_session()
    b = h.builder
    t = h.memref_type((64, 128), "fp16")
    kernel, entry = h.new_kernel("k", [t, h.memref_type((128, 64), "fp16")])
    body = b.create_parallel_op([2, 2], 64).add_entry_block()
    b.set_insertion_point_to_start(body)
    by, bx = body.get_argument(0), body.get_argument(1)

    def loop(bb, iv):
        d0, d1, d2 = (bb.get_affine_dim_expr(i) for i in range(3))
        bb.create_copy_op(entry.get_argument(0), entry.get_argument(1), [by, bx, iv], [by, bx, iv], F.AffineMap.get(3, 0, [d0 * 32, d1 * 64 + d2 * 32]),
                          F.AffineMap.get(3, 0, [d1 * 64 + d2 * 32, d0 * 32]), [32, 32], [32, 32])
    b.create_for_op(0, 2, 1, loop)
    with pytest.raises(ValueError, match="at most two"):
        F.runtime.match_ops(kernel)


def _tiled_reduce_kernel(h, *, rows=128, cols=256, dim=1, kind="max", dtype="fp16", tile=32, clear=True, tile_reduced_dim=False):
    """kernel(x: rows x cols, v: kept extent): v := reduce(x along dim), written tile by tile: a grid over bands of `tile` kept
    indices, every band through a shared tile, reduced into a shared vector, the vector stored to its place in v"""
    b = h.builder
    kept = rows if dim == 1 else cols
    kernel, entry = h.new_kernel("tiled_reduce", [h.memref_type((rows, cols), dtype), h.memref_type((kept,), dtype)])
    x, v = entry.get_argument(0), entry.get_argument(1)
    grid = [kept // tile] + ([2] if tile_reduced_dim else [])
    body = b.create_parallel_op(grid, 256).add_entry_block()
    b.set_insertion_point_to_start(body)
    band = body.get_argument(0)
    red_extent = (cols if dim == 1 else rows) // (2 if tile_reduced_dim else 1)
    shape = (tile, red_extent) if dim == 1 else (red_extent, tile)
    buf = h.alloc_buffer(shape, dtype, space=F.MemorySpace.SHARED)
    vec = h.alloc_buffer((tile,), dtype, space=F.MemorySpace.SHARED)
    d0, d1 = b.get_affine_dim_expr(0), b.get_affine_dim_expr(1)
    c = b.get_affine_constant_expr
    idx = [band] + ([body.get_argument(1)] if tile_reduced_dim else [])
    other = d1 * red_extent if tile_reduced_dim else c(0)
    src_map = F.AffineMap.get(len(idx), 0, [d0 * tile, other] if dim == 1 else [other, d0 * tile])
    b.create_copy_op(x, buf, idx, [], src_map, F.AffineMap.get(0, 0, [c(0), c(0)]), list(shape), list(shape))
    b.create_reduce_op(buf, vec, kind, dim, clear)
    b.create_copy_op(vec, v, [], [band], F.AffineMap.get(0, 0, [c(0)]), F.AffineMap.get(1, 0, [d0 * tile]), [tile], [tile])
    return kernel


def test_reduction_tiled_over_a_grid_is_one_reduction():
    """copy tile -> buffer; reduce buffer -> vector; copy vector -> global under a grid that walks the kept dimension (FriskOps.td:412-441,
    FriskOps.cpp:1725-1767): recognised as one reduction of the rectangle the tiles cover"""
    for dim, kind in ((1, "max"), (0, "sum")):
        h = F.create_session()
        kernel = _tiled_reduce_kernel(h, dim=dim, kind=kind)
        assert h.module.verify()
        (op,) = F.runtime.match_ops(kernel)
        assert op["op"] == "reduce" and (op["rows"], op["cols"], op["src_ld"]) == (128, 256, 256) and op["dim"] == dim
        assert op["kind"] == ("max" if kind == "max" else "add") and op["clear"] and (op["src"], op["dst"], op["src_offset"], op["dst_offset"]) == (0, 1, 0, 0)
    sessions = []

    def refused(**kw):
        h = F.create_session()
        sessions.append(h)
        with pytest.raises(ValueError) as e:
            F.runtime.match_ops(_tiled_reduce_kernel(h, **kw))
        return str(e.value)
    assert "tiles the reduced dimension" in refused(tile_reduced_dim=True)
    assert "must clear" in refused(clear=False)
