"""Shared helpers of the parity tests: seeded inputs from the oracle's RNG,
device buffers through torch (plumbing only), launches through the C ABI."""
import numpy as np

import oracle as O

TOL = {O.F32: 1e-4, O.F16: 1e-2, O.BF16: 1e-2, O.E4M3: 1e-2, O.I8: 1e-2}
NAMES = {O.F32: "f32", O.F16: "f16", O.BF16: "bf16", O.I8: "i8", O.E4M3: "e4m3"}
DEFAULT_OUT = {O.F32: O.F32, O.F16: O.F16, O.BF16: O.BF16, O.I8: O.I32, O.E4M3: O.BF16}


def make_operand(dtype, rows, cols, seed, tensor, kind="normal", scale=1.0):
    """rows x cols stored operand in the storage type of `dtype`"""
    n = rows * cols
    if dtype == O.I8:
        return O.int8_uniform(n, seed, tensor).reshape(rows, cols)
    if kind == "uniform":
        f = O.uniform(n, seed, tensor, -1.0, 1.0)
    else:
        f = O.normal(n, seed, tensor, scale)
    return O.encode(dtype, f).reshape(rows, cols)


def to_dev(arr):
    import torch
    a = np.ascontiguousarray(arr)
    return torch.from_numpy(a.view(np.uint8).reshape(-1).copy()).cuda()


def from_dev(t, np_dtype, shape):
    return t.cpu().numpy().view(np_dtype).reshape(shape)


def run_gemm(R, dtype, A, B, transA, transB, dtype_out, M, N, K, epilogue=0, sA=None, sB=None, C_init=None,
             clear_accum=True, tile=(0, 0, 0), waves=(0, 0), pad=0, shift=0, split_k=0, workspace=True, stages=0, atom=0, pad_c=None):
    """launch through the C ABI; returns the output as a numpy array in storage type.
    pad: extra elements at the end of every stored row of A, B and C (odd leading dimensions); pad_c: the same for C alone;
    shift: the operands start `shift` elements into their allocations (pointers only element-aligned);
    split_k: descriptor field (0 = planner's choice); workspace=False launches without one."""
    import torch
    out_np = O.NP_STORAGE[dtype_out]

    def padded(x, pad=pad):
        if pad == 0 and shift == 0:
            return np.ascontiguousarray(x), x.shape[1]
        buf = np.zeros(shift + x.shape[0] * (x.shape[1] + pad), dtype=x.dtype)
        buf[shift:].reshape(x.shape[0], x.shape[1] + pad)[:, :x.shape[1]] = x
        return buf, x.shape[1] + pad

    hA, lda = padded(A)
    hB, ldb = padded(B)
    C0 = C_init if C_init is not None else np.full((M, N), 0xFF, dtype=np.uint8).repeat(np.dtype(out_np).itemsize, axis=1).view(out_np)
    hC, ldc = padded(np.ascontiguousarray(C0).view(out_np).reshape(M, N), pad if pad_c is None else pad_c)
    dA, dB, dC = to_dev(hA), to_dev(hB), to_dev(hC)
    es, osz = hA.dtype.itemsize, np.dtype(out_np).itemsize
    dsA = to_dev(np.asarray(sA, dtype=np.float32)) if sA is not None else None
    dsB = to_dev(np.asarray(sB, dtype=np.float32)) if sB is not None else None
    desc = R.make_desc(dtype, M, N, K, dtype_out=dtype_out, transA=transA, transB=transB, clear_accum=clear_accum,
                       epilogue=epilogue, tile=tile, waves=waves, lda=lda, ldb=ldb, ldc=ldc, split_k=split_k, stages=stages, atom=atom)
    stream = torch.cuda.current_stream().cuda_stream
    ws_bytes = R.workspace_bytes(desc) if workspace else 0
    ws = torch.full((ws_bytes,), 0xFF, dtype=torch.uint8, device="cuda") if ws_bytes else None
    R.gemm(desc, dA.data_ptr() + shift * es, dB.data_ptr() + shift * es, dC.data_ptr() + shift * osz,
           dsA.data_ptr() if dsA is not None else None, dsB.data_ptr() if dsB is not None else None,
           ws.data_ptr() if ws is not None else None, ws_bytes, stream)
    torch.cuda.synchronize()
    full = dC.cpu().numpy().view(out_np)
    if M == 0 or N == 0:
        return np.zeros((M, N), dtype=out_np)
    got = full[shift:].reshape(M, ldc)
    if ldc > N:
        assert np.all(got[:, N:] == 0), "the kernel wrote into the padding of C"
    return np.ascontiguousarray(got[:, :N])


def stored_shapes(M, N, K, transA, transB):
    return ((K, M) if transA else (M, K)), ((N, K) if transB else (K, N))
