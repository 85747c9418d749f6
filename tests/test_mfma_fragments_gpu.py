"""The register-fragment conventions of the GEMM kernels, checked on the device.

The reference builds its operand and accumulator fragments from NVIDIA atoms (makeFragment8x4/8x8/8x16,
buildGemmFragmentA/B, lib/Dialect/Frisk/IR/FriskOps.cpp:233-451); on gfx950 the atoms are the MFMA instructions, whose lane
and register maps are fixed by the hardware.  Three checks, through libfrisk_hwcheck.so:
  * every MFMA atom on its own: operands packed by the assumed lane map, random integer matrices, host product;
  * the product's own path (LDS tile layout with its swizzle, FragReader addresses incl. the transpose reads, Mma::run,
    the accumulator map the epilogue uses) on one K tile for every element type, atom and operand layout;
  * the lane maps of ds_read_b64_tr_b16 / _tr_b8 at the addresses the fragment reader presents for the planner's LDS layout.
"""
import numpy as np
import pytest

import oracle as O

pytestmark = pytest.mark.gpu


def note(msg):
    print(msg, flush=True)


@pytest.fixture(scope="module")
def hw():
    import torch
    from frisk_amd import hwcheck
    hwcheck.lib()
    assert torch.cuda.is_available()
    return hwcheck


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("atom_id", sorted(range(11)))
def test_single_mfma_atom_against_host_product(hw, atom_id):
    import torch
    name, M, N, K, maxv = hw.ATOMS[atom_id]
    note(f"case atom {atom_id} {name}")
    rng = np.random.default_rng(100 + atom_id)
    A = rng.integers(-maxv, maxv + 1, size=(M, K)).astype(np.float32)
    B = rng.integers(-maxv, maxv + 1, size=(K, N)).astype(np.float32)
    dA, dB = _dev(A), _dev(B)
    dD = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    hw.mfma_atom(atom_id, dA.data_ptr(), dB.data_ptr(), dD.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.array_equal(dD.cpu().numpy().astype(np.float64), want), name


PATHS = [(O.F16, 32), (O.F16, 16), (O.BF16, 32), (O.BF16, 16), (O.I8, 32), (O.I8, 16), (O.E4M3, 32), (O.E4M3, 16), (O.F32, 32)]


@pytest.mark.parametrize("dtype,atom", PATHS)
@pytest.mark.parametrize("transA,transB", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_product_fragment_path_one_k_tile(hw, dtype, atom, transA, transB):
    import torch
    bmn, bk = (128, 32) if dtype == O.F32 else (256, 128 if dtype in (O.I8, O.E4M3) else 64)
    if (dtype, atom) == (O.E4M3, 16) and (transA, transB) != (0, 1):
        pytest.skip("the 16x16x128 atom is compiled for K-contiguous operands only (A [M][K], B [N][K])")
    note(f"case fragment path dtype {dtype} atom {atom} tA={transA} tB={transB} tile {bmn}x{bmn}x{bk}")
    rng = np.random.default_rng(7 * dtype + atom + 2 * transA + transB)
    maxv = {O.F16: 3, O.BF16: 3, O.I8: 127, O.E4M3: 4, O.F32: 100}[dtype]
    A = rng.integers(-maxv, maxv + 1, size=(bmn, bk))  # logical [M][K]
    B = rng.integers(-maxv, maxv + 1, size=(bk, bmn))  # logical [K][N]
    storedA = A.T if transA else A
    storedB = B.T if transB else B
    enc = (lambda x: x.astype(np.int8)) if dtype == O.I8 else (lambda x: O.encode(dtype, x.astype(np.float32).reshape(-1)).reshape(x.shape))
    dA, dB = _dev(enc(np.ascontiguousarray(storedA))), _dev(enc(np.ascontiguousarray(storedB)))
    dD = torch.full((bmn, bmn), 0x7FC00000, dtype=torch.int32, device="cuda")
    hw.fragment_path(dtype, atom, transA, transB, dA.data_ptr(), dB.data_ptr(), dD.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    raw = dD.cpu().numpy()
    got = raw.astype(np.int64) if dtype == O.I8 else raw.view(np.float32).astype(np.float64)
    want = A.astype(np.int64) @ B.astype(np.int64)
    assert np.array_equal(got, want.astype(got.dtype))


def _frag_rows_cols(es, fragb, at, lane, mn0, q):
    """the lane map of the fragment reader for a tile whose rows run along K (transpose reads): which K row and column a
    lane presents; K-groups of fragb / es rows, blocks of 16 lanes side by side along the columns"""
    kpi = 4 if es == 2 else 8
    lpr = 16 // kpi
    blk, l16 = lane >> 4, lane & 15
    col_blocks = at // 16
    col0 = mn0 + 16 * (blk % col_blocks)
    krow0 = (blk // col_blocks) * (fragb // es) + q * kpi
    return krow0, col0, krow0 + l16 // lpr, (col0 + (l16 % lpr) * (8 // es)) * es


@pytest.mark.parametrize("dtype,atom", [(O.F16, 32), (O.F16, 16), (O.I8, 32)])
def test_transpose_read_lane_maps_at_the_planners_addresses(hip, hw, dtype, atom):
    import torch
    es, fragb = (2, 16) if dtype == O.F16 else (1, 16)
    # B stored [K][N]: its LDS tile has rows along K and is read by transpose reads; the descriptor names the atom
    out_dt = O.F16 if dtype == O.F16 else O.I32
    p = hip.plan(hip.make_desc(dtype, 4096, 4096, 4096, dtype_out=out_dt, tile=(256, 256, 0), atom=atom))
    assert p.mfma_m == atom and p.lds_b.k_contiguous == 0 and p.lds_b.read_instr == (1 if es == 2 else 2), (p.mfma_m, p.lds_b.read_instr)
    L = p.lds_b
    kpi = 4 if es == 2 else 8
    for mn0 in (0, atom, 96):
        for q in range(fragb // 8):
            addrs, expect = [], []
            for lane in range(64):
                krow0, col0, krow, colbyte = _frag_rows_cols(es, fragb, atom, lane, mn0, q)
                addrs.append(hip.lds_offset(L, krow, colbyte))
                # the lane receives column (lane % 16) of its block's K rows krow0 .. krow0 + kpi - 1
                expect.append([hip.lds_offset(L, krow0 + e, (col0 + (lane & 15)) * es) // es for e in range(kpi)])
            assert max(addrs) + 8 <= 16384 and all(a % 8 == 0 for a in addrs)
            note(f"case tr read dtype {dtype} atom {atom} mn0 {mn0} q {q}")
            dA = _dev(np.array(addrs, dtype=np.int32))
            stream = torch.cuda.current_stream().cuda_stream
            if es == 2:
                out = torch.zeros(64 * 4, dtype=torch.int16, device="cuda")
                hw.tr_read(16, dA.data_ptr(), out.data_ptr(), 0, stream)
                torch.cuda.synchronize()
                got = out.cpu().numpy().view(np.uint16).reshape(64, 4).astype(np.int64)
            else:
                lo, hi = torch.zeros(64 * 8, dtype=torch.uint8, device="cuda"), torch.zeros(64 * 8, dtype=torch.uint8, device="cuda")
                hw.tr_read(8, dA.data_ptr(), lo.data_ptr(), 0, stream)
                hw.tr_read(8, dA.data_ptr(), hi.data_ptr(), 8, stream)
                torch.cuda.synchronize()
                got = (lo.cpu().numpy().astype(np.int64) + 256 * hi.cpu().numpy().astype(np.int64)).reshape(64, 8)
            assert np.array_equal(got, np.array(expect)), (mn0, q)
