"""Host-only: whatever the planner picks must be a kernel that may run on the problem.  A fast kernel moves whole tiles with
16-byte transfers, an edge kernel clamps M and N but not K, the chunk-wise guarded kernel needs whole 16-byte chunks along K, and
a split needs whole K tiles per slice: a plan that breaks one of these would send a kernel beyond its operands."""
import random
import re

import pytest

from frisk_amd import runtime as R

ES = {R.F32: 4, R.F16: 2, R.BF16: 2, R.I8: 1, R.E4M3: 1}
OUT = {R.F32: R.F32, R.F16: R.F16, R.BF16: R.BF16, R.I8: R.I32, R.E4M3: R.BF16}
OS = {R.F32: 4, R.F16: 2, R.BF16: 2, R.I32: 4}
NAME = re.compile(r"(\w+?)_(n|t)(n|t)_(\d+)x(\d+)x(\d+)_w(\d+)x(\d+)(?:x(\d+))?_s(\d+)(?:x(\d+))?(_a16)?(_guard_chunks|_guard)?(_splitk)?(_edge)?")


def shapes(rng, n):
    for _ in range(n):
        kind = rng.choice(["whole", "edge", "ragged_k", "any", "skinny", "big"])
        if kind == "whole":
            yield rng.choice([32, 64, 128, 256, 512, 1024, 4096]), rng.choice([32, 128, 256, 1024, 4096, 8192]), rng.choice([128, 512, 1024, 4096, 8192])
        elif kind == "edge":
            yield rng.randint(1, 5000), 16 * rng.randint(1, 700), 128 * rng.randint(1, 64)
        elif kind == "ragged_k":
            yield rng.randint(1, 3000), 16 * rng.randint(1, 300), 16 * rng.randint(1, 500)
        elif kind == "skinny":
            yield rng.randint(1, 300), 128 * rng.randint(1, 128), 128 * rng.randint(8, 128)
        elif kind == "big":
            yield 256 * rng.randint(8, 40), 256 * rng.randint(8, 40), 128 * rng.randint(8, 64)
        else:
            yield rng.randint(1, 2000), rng.randint(1, 2000), rng.randint(1, 2000)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_every_plan_is_a_kernel_that_may_run_on_the_problem(seed):
    rng = random.Random(seed)
    names = R.kernel_names()
    seen = set()
    for M, N, K in shapes(rng, 1500):
        dt = rng.choice([R.F32, R.F16, R.BF16, R.I8, R.E4M3])
        tA, tB = rng.random() < 0.3, rng.random() < 0.5
        split = rng.choice([0, 0, 0, 1, 2, 4])
        d = R.make_desc(dt, M, N, K, dtype_out=OUT[dt], transA=tA, transB=tB, split_k=split)
        try:
            p = R.plan(d)
        except R.FriskHipError as ex:
            assert ex.status in (R.ERR_TILE, R.ERR_SHAPE), (M, N, K, str(ex))
            continue
        name = names[p.kernel_id]
        m = NAME.fullmatch(name)
        assert m, name
        bm, bn, bk = int(m.group(4)), int(m.group(5)), int(m.group(6))
        guard, splitk, edge = m.group(13), bool(m.group(14)), bool(m.group(15))
        es, osz = ES[dt], OS[OUT[dt]]
        what = (name, M, N, K, tA, tB, split)
        seen.add((guard or "") + ("_splitk" if splitk else "") + ("_edge" if edge else ""))
        assert (m.group(2) == "t") == tA and (m.group(3) == "t") == tB and (bm, bn, bk) == (p.tile_m, p.tile_n, p.tile_k), what
        assert p.grid_x == -(-N // bn) and p.grid_y == -(-M // bm), what
        rows_aligned = (d.lda * es) % 16 == 0 and (d.ldb * es) % 16 == 0 and (d.ldc * osz) % 16 == 0
        if guard is None:
            assert rows_aligned and K % bk == 0, what
            if edge:
                assert M % bm or N % bn, what
            else:
                assert M % bm == 0 and N % bn == 0, what
        elif guard == "_guard_chunks":
            assert rows_aligned and K % (16 // es) == 0, what
        assert bool(p.guarded) == (guard is not None), what
        if p.split_k > 1:
            assert splitk and K % bk == 0 and (K // bk) % p.split_k == 0 and p.workspace_bytes == p.split_k * M * N * 4, what
            assert split in (0, p.split_k), what
        else:
            assert p.split_k == 1, what
        if p.tail_split > 1:
            assert splitk and not edge and p.tail_tiles == (p.grid_x * p.grid_y) % 256 and (K // bk) % p.tail_split == 0, what
            assert p.workspace_bytes == p.tail_split * p.tail_tiles * bm * bn * 4, what
        if split == 1:
            assert p.split_k == 1 and p.tail_split == 1 and p.workspace_bytes == 0, what
    # the walk reached every kind of kernel
    assert {"", "_edge", "_splitk", "_splitk_edge", "_guard", "_guard_chunks"} <= seen, seen
