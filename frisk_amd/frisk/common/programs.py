"""The two programs of the reference's design sketches that go beyond a lone GEMM, written with the IR builder: structure
ops of the dialect plus frisk.block bodies of affine.load / arith / math / affine.store.

    online_softmax   tmp/ir.mlir:21-75    row softmax in base 2 with a running log-sum over chunks of the row
    attention        tmp/ir.mlir:88-158   softmax(Q K^T * cst) V with a running maximum and sum over key tiles

The sketches are pseudo-code (no parser reads them and the reference's builder cannot create their block bodies); these
functions emit the same op sequences in well-typed form: 16-bit loads are widened before the arithmetic, the running
maximum of the attention loop accumulates (clear = False), the stray second fill of the scores is left out and the output is
divided by the running sum before it is stored.  `frisk.runtime.match` recognises both and `frisk.runtime.launch` runs them
as one library call each.
"""
from ..frisk_ffi import ir


def _store_block(helper, ranges, buffer, index_of, value_of):
    """frisk.block over `ranges` that stores value_of(builder, ivs) to buffer[index_of(ivs)] (index_of gives (indices, map))"""
    def body(bb, ivs):
        indices, index_map = index_of(ivs)
        bb.create_store_op(value_of(bb, ivs), buffer, indices, index_map)
    return helper.builder.create_block_op(list(ranges), body)


def online_softmax(helper, name, rows, cols, dtype="fp16", *, chunk=1024, cst=1.25, threads=128):
    b = helper.builder
    if cols % chunk:
        raise ValueError("chunk %d does not divide the row length %d" % (chunk, cols))
    kernel, entry = helper.new_kernel(name, [helper.memref_type((rows, cols), dtype), helper.memref_type((rows, cols), dtype)])
    src, dst = entry.get_argument(0), entry.get_argument(1)
    body = b.create_parallel_op([rows], threads).add_entry_block()
    b.set_insertion_point_to_start(body)
    bx = body.get_argument(0)
    f32, elem = b.get_f32_ty(), helper.element_type(dtype)
    c = b.get_f32(cst)
    local = lambda shape, ty: helper.alloc_buffer(shape, ty, space=ir.MemorySpace.LOCAL)
    x, y = local((chunk,), dtype), local((chunk,), dtype)
    lse, max_x, exp_x, sum_exp_x = local((1,), "fp32"), local((1,), dtype), local((chunk,), "fp32"), local((1,), "fp32")
    b.create_fill_op(lse, float("-inf"), "fp32")
    d0, d1 = b.get_affine_dim_expr(0), b.get_affine_dim_expr(1)
    row_chunk = ir.AffineMap.get(2, 0, [d0, d1 * chunk])            # (row, i) -> (row, i * chunk)
    first = ir.AffineMap.get(0, 0, [b.get_affine_constant_expr(0)])  # () -> (0)
    at_j = lambda ivs: ([ivs[0]], ir.AffineMap())
    at_0 = lambda ivs: ([], first)
    wide = lambda q, v: v if v.get_type() == f32 else q.create_extf(v, f32)
    load0 = lambda q, buf: wide(q, q.create_load_op(buf, [], first))

    def first_sweep(bb, i):
        bb.create_copy_op(src, x, [bx, i], [], row_chunk, first, [1, chunk], [chunk])
        bb.create_reduce_op(x, max_x, "max", 0, True)
        _store_block(helper, [chunk], exp_x, at_j, lambda q, ivs: q.create_exp2(q.create_subf(
            q.create_mulf(wide(q, q.create_load_op(x, [ivs[0]])), c), q.create_mulf(load0(q, max_x), c))))
        bb.create_reduce_op(exp_x, sum_exp_x, "sum", 0, True)

        def update(q, ivs):
            scaled_max = q.create_mulf(load0(q, max_x), c)
            old = q.create_exp2(q.create_subf(load0(q, lse), scaled_max))
            return q.create_addf(scaled_max, q.create_log2(q.create_addf(old, load0(q, sum_exp_x))))
        _store_block(helper, [1], lse, at_0, update)

    def second_sweep(bb, i):
        bb.create_copy_op(src, x, [bx, i], [], row_chunk, first, [1, chunk], [chunk])

        def probability(q, ivs):
            v = q.create_exp2(q.create_subf(q.create_mulf(wide(q, q.create_load_op(x, [ivs[0]])), c), load0(q, lse)))
            return v if elem == f32 else q.create_truncf(v, elem)
        _store_block(helper, [chunk], y, at_j, probability)
        bb.create_copy_op(y, dst, [], [bx, i], first, row_chunk, [chunk], [1, chunk])

    b.create_for_op(0, cols // chunk, 1, first_sweep)
    b.create_for_op(0, cols // chunk, 1, second_sweep)
    return kernel


def attention(helper, name, batch, heads, seq_q, seq_k, head_dim=128, dtype="fp16", *, cst=None, tile_q=64, tile_k=64, threads=256, k_transposed=True):
    """cst multiplies the scores before exp2 (softmax scale * log2 e; default 1 / sqrt(head_dim) * log2 e).  k_transposed: K is
    stored [batch, heads, head_dim, seq_k] as in the sketch; otherwise [batch, heads, seq_k, head_dim] and the first product
    carries transB."""
    b = helper.builder
    if seq_q % tile_q or seq_k % tile_k:
        raise ValueError("tiles (%d, %d) do not divide the sequence lengths (%d, %d)" % (tile_q, tile_k, seq_q, seq_k))
    if cst is None:
        cst = head_dim ** -0.5 * 1.4426950408889634
    qo_shape = (batch, heads, seq_q, head_dim)
    k_shape = (batch, heads, head_dim, seq_k) if k_transposed else (batch, heads, seq_k, head_dim)
    kernel, entry = helper.new_kernel(name, [helper.memref_type(qo_shape, dtype), helper.memref_type(k_shape, dtype),
                                             helper.memref_type((batch, heads, seq_k, head_dim), dtype), helper.memref_type(qo_shape, dtype)])
    gq, gk, gv, go = (entry.get_argument(i) for i in range(4))
    body = b.create_parallel_op([batch, heads, seq_q // tile_q], threads).add_entry_block()
    b.set_insertion_point_to_start(body)
    bz, by, bx = (body.get_argument(i) for i in range(3))
    f32, elem = b.get_f32_ty(), helper.element_type(dtype)
    c = b.get_f32(cst)
    shared = lambda shape: helper.alloc_buffer(shape, dtype, space=ir.MemorySpace.SHARED)
    local = lambda shape, ty="fp32": helper.alloc_buffer(shape, ty, space=ir.MemorySpace.LOCAL)
    q = shared((tile_q, head_dim))
    k = shared((head_dim, tile_k) if k_transposed else (tile_k, head_dim))
    v, o = shared((tile_k, head_dim)), shared((tile_q, head_dim))
    acc_s, acc_s_cast, acc_o = local((tile_q, tile_k)), local((tile_q, tile_k), dtype), local((tile_q, head_dim))
    scores_max, scores_max_prev, scores_scale, scores_sum, logsum = (local((tile_q,)) for _ in range(5))
    d = [b.get_affine_dim_expr(i) for i in range(4)]
    zero = b.get_affine_constant_expr(0)
    origin1, origin2 = ir.AffineMap.get(0, 0, [zero]), ir.AffineMap.get(0, 0, [zero, zero])
    rows_of_tile = lambda tile: ir.AffineMap.get(3, 0, [d[0], d[1], d[2] * tile, zero])   # (bz, by, t) -> (bz, by, t * tile, 0)
    cols_of_tile = lambda tile: ir.AffineMap.get(3, 0, [d[0], d[1], zero, d[2] * tile])   # (bz, by, t) -> (bz, by, 0, t * tile)
    at_i = lambda ivs: ([ivs[0]], ir.AffineMap())
    at_ij = lambda ivs: ([ivs[0], ivs[1]], ir.AffineMap())

    b.create_copy_op(gq, q, [bz, by, bx], [], rows_of_tile(tile_q), origin2, [1, 1, tile_q, head_dim], [tile_q, head_dim])
    b.create_fill_op(acc_o, 0.0, "fp32")
    b.create_fill_op(logsum, 0.0, "fp32")
    b.create_fill_op(scores_max, float("-inf"), "fp32")

    def key_tile(bb, t):
        if k_transposed:
            bb.create_copy_op(gk, k, [bz, by, t], [], cols_of_tile(tile_k), origin2, [1, 1, head_dim, tile_k], [head_dim, tile_k])
        else:
            bb.create_copy_op(gk, k, [bz, by, t], [], rows_of_tile(tile_k), origin2, [1, 1, tile_k, head_dim], [tile_k, head_dim])
        bb.create_fill_op(acc_s, 0.0, "fp32")
        bb.create_gemm_op(q, k, acc_s, False, not k_transposed, False)
        bb.create_copy_op(scores_max, scores_max_prev, [], [], origin1, origin1, [tile_q], [tile_q])
        bb.create_reduce_op(acc_s, scores_max, "max", 1, False)
        _store_block(helper, [tile_q], scores_scale, at_i, lambda p, ivs: p.create_exp2(p.create_subf(
            p.create_mulf(p.create_load_op(scores_max_prev, [ivs[0]]), c), p.create_mulf(p.create_load_op(scores_max, [ivs[0]]), c))))
        _store_block(helper, [tile_q, tile_k], acc_s, at_ij, lambda p, ivs: p.create_exp2(p.create_subf(
            p.create_mulf(p.create_load_op(acc_s, [ivs[0], ivs[1]]), c), p.create_mulf(p.create_load_op(scores_max, [ivs[0]]), c))))
        bb.create_reduce_op(acc_s, scores_sum, "sum", 1, True)
        _store_block(helper, [tile_q], logsum, at_i, lambda p, ivs: p.create_addf(
            p.create_mulf(p.create_load_op(logsum, [ivs[0]]), p.create_load_op(scores_scale, [ivs[0]])), p.create_load_op(scores_sum, [ivs[0]])))
        bb.create_copy_op(acc_s, acc_s_cast, [], [], origin2, origin2, [tile_q, tile_k], [tile_q, tile_k])
        _store_block(helper, [tile_q, head_dim], acc_o, at_ij, lambda p, ivs: p.create_mulf(
            p.create_load_op(acc_o, [ivs[0], ivs[1]]), p.create_load_op(scores_scale, [ivs[0]])))
        bb.create_copy_op(gv, v, [bz, by, t], [], rows_of_tile(tile_k), origin2, [1, 1, tile_k, head_dim], [tile_k, head_dim])
        bb.create_gemm_op(acc_s_cast, v, acc_o, False, False, False)

    b.create_for_op(0, seq_k // tile_k, 1, key_tile)
    _store_block(helper, [tile_q, head_dim], acc_o, at_ij, lambda p, ivs: p.create_divf(
        p.create_load_op(acc_o, [ivs[0], ivs[1]]), p.create_load_op(logsum, [ivs[0]])))
    b.create_copy_op(acc_o, o, [], [], origin2, origin2, [tile_q, head_dim], [tile_q, head_dim])
    b.create_copy_op(o, go, [], [bz, by, bx], origin2, rows_of_tile(tile_q), [tile_q, head_dim], [1, 1, tile_q, head_dim])
    del elem, f32
    return kernel
