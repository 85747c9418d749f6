"""ctypes binding of libfrisk_hip.so (include/frisk_hip.h).

This is the thin host layer the builder front end and the benchmarks use to
reach the HIP kernels.  It never falls back to another implementation: if the
library is missing the import fails, and every non-zero status raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfrisk_hip.so")

ABI_VERSION = 1
F32, F16, BF16, I8, E4M3, I32 = 0, 1, 2, 3, 4, 5
EPI_NONE, EPI_ROW_COL_SCALE, EPI_TENSOR_SCALE = 0, 1, 2
POLICY_SQUARE, POLICY_FULL_ROW, POLICY_FULL_COL = 0, 1, 2
DTYPE_BYTES = {F32: 4, F16: 2, BF16: 2, I8: 1, E4M3: 1, I32: 4}
DTYPE_NAMES = {"fp32": F32, "f32": F32, "fp16": F16, "f16": F16, "bf16": BF16, "int8": I8, "i8": I8,
               "e4m3fn": E4M3, "e4m3": E4M3, "fp8": E4M3, "int32": I32, "i32": I32}
ACC_OF = {F32: F32, F16: F32, BF16: F32, I8: I32, E4M3: F32}

STATUS_NAMES = {0: "OK", 1: "ERR_NULL", 2: "ERR_ABI", 3: "ERR_DTYPE", 4: "ERR_SHAPE", 5: "ERR_TILE", 6: "ERR_LDS",
                7: "ERR_EPILOGUE", 8: "ERR_WORKSPACE", 9: "ERR_DEVICE", 10: "ERR_ALIGNMENT", 11: "ERR_ARGUMENT"}


class GemmDesc(ctypes.Structure):
    _fields_ = [("abi_version", ctypes.c_int32), ("dtype_ab", ctypes.c_int32), ("dtype_acc", ctypes.c_int32),
                ("dtype_out", ctypes.c_int32), ("M", ctypes.c_int64), ("N", ctypes.c_int64), ("K", ctypes.c_int64),
                ("lda", ctypes.c_int64), ("ldb", ctypes.c_int64), ("ldc", ctypes.c_int64),
                ("transA", ctypes.c_uint8), ("transB", ctypes.c_uint8), ("clear_accum", ctypes.c_uint8),
                ("split_k", ctypes.c_uint8), ("epilogue", ctypes.c_int32), ("policy", ctypes.c_int32),
                ("tile_m", ctypes.c_int32), ("tile_n", ctypes.c_int32), ("tile_k", ctypes.c_int32),
                ("waves_m", ctypes.c_int32), ("waves_n", ctypes.c_int32), ("stages", ctypes.c_int32), ("atom", ctypes.c_int32)]


class LdsLayout(ctypes.Structure):
    _fields_ = [("rows", ctypes.c_int32), ("row_bytes", ctypes.c_int32), ("k_contiguous", ctypes.c_int32),
                ("row_shift", ctypes.c_int32), ("row_mask", ctypes.c_int32), ("chunk_shift", ctypes.c_int32),
                ("read_instr", ctypes.c_int32), ("read_cycles", ctypes.c_float), ("write_cycles", ctypes.c_float),
                ("row_shift2", ctypes.c_int32), ("row_mask2", ctypes.c_int32), ("chunk_shift2", ctypes.c_int32)]


class GemmPlan(ctypes.Structure):
    _fields_ = [("kernel_id", ctypes.c_int32), ("tile_m", ctypes.c_int32), ("tile_n", ctypes.c_int32),
                ("tile_k", ctypes.c_int32), ("waves_m", ctypes.c_int32), ("waves_n", ctypes.c_int32),
                ("threads", ctypes.c_int32), ("waves_k", ctypes.c_int32), ("mfma_m", ctypes.c_int32), ("mfma_n", ctypes.c_int32),
                ("mfma_k", ctypes.c_int32), ("stages", ctypes.c_int32), ("stages_b", ctypes.c_int32), ("lds_bytes", ctypes.c_int32),
                ("grid_x", ctypes.c_int32), ("grid_y", ctypes.c_int32), ("split_k", ctypes.c_int32),
                ("xcd_remap", ctypes.c_int32), ("guarded", ctypes.c_int32), ("lds_a", LdsLayout), ("lds_b", LdsLayout),
                ("workspace_bytes", ctypes.c_size_t), ("flops", ctypes.c_double), ("bytes", ctypes.c_double),
                ("tail_tiles", ctypes.c_int32), ("tail_split", ctypes.c_int32)]


class AttentionDesc(ctypes.Structure):
    _fields_ = [("abi_version", ctypes.c_int32), ("dtype", ctypes.c_int32), ("batch", ctypes.c_int64), ("heads", ctypes.c_int64),
                ("seq_q", ctypes.c_int64), ("seq_k", ctypes.c_int64), ("head_dim", ctypes.c_int64), ("scale", ctypes.c_float),
                ("k_transposed", ctypes.c_uint8), ("reserved", ctypes.c_uint8 * 3)]


EW_MAX_INPUTS, EW_MAX_OPS, EW_MAX_STACK = 8, 48, 6
EW_OPS = {"input": 0, "const": 1, "add": 2, "sub": 3, "mul": 4, "div": 5, "max": 6, "min": 7, "neg": 8, "exp2": 9, "log2": 10}


class ElementwiseDesc(ctypes.Structure):
    _fields_ = [("abi_version", ctypes.c_int32), ("n_inputs", ctypes.c_int32), ("n_ops", ctypes.c_int32), ("out_dtype", ctypes.c_int32),
                ("rows", ctypes.c_int64), ("cols", ctypes.c_int64), ("out_ld", ctypes.c_int64),
                ("in_dtype", ctypes.c_int32 * EW_MAX_INPUTS), ("in_col_stride", ctypes.c_int32 * EW_MAX_INPUTS),
                ("in_row_stride", ctypes.c_int64 * EW_MAX_INPUTS), ("op", ctypes.c_int32 * EW_MAX_OPS), ("arg", ctypes.c_int32 * EW_MAX_OPS),
                ("imm", ctypes.c_float * EW_MAX_OPS)]


globals().update({name: code for code, name in STATUS_NAMES.items()})  # OK, ERR_NULL, ... as module constants


class FriskHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("frisk_hip status %d (%s): %s" % (status, STATUS_NAMES.get(status, "?"), message))
        self.status = status


_lib = None

EXPORTS = ["frisk_hip_init", "frisk_hip_abi_version", "frisk_hip_last_error", "frisk_hip_plan", "frisk_hip_workspace_bytes",
           "frisk_hip_gemm", "frisk_hip_lds_access_cycles", "frisk_hip_lds_search", "frisk_hip_lds_search_atom", "frisk_hip_lds_offset", "frisk_hip_wave_partition",
           "frisk_hip_kernel_count", "frisk_hip_kernel_name", "frisk_hip_fill", "frisk_hip_copy", "frisk_hip_reduce",
           "frisk_hip_reduce_workspace_bytes", "frisk_hip_attention", "frisk_hip_softmax", "frisk_hip_softmax_workspace_bytes",
           "frisk_hip_gemm_static_ws", "frisk_hip_static_workspace_bytes", "frisk_hip_copy_tiles", "frisk_hip_elementwise"]


def lib():
    """Loads libfrisk_hip.so; raises if it has not been built (python -m frisk_amd.build)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError("libfrisk_hip.so is not built: run `python -m frisk_amd.build` (needs hipcc)")
    L = ctypes.CDLL(LIB_PATH)
    L.frisk_hip_abi_version.restype = ctypes.c_int
    L.frisk_hip_last_error.restype = ctypes.c_char_p
    L.frisk_hip_plan.argtypes = [ctypes.POINTER(GemmDesc), ctypes.POINTER(GemmPlan)]
    L.frisk_hip_workspace_bytes.restype = ctypes.c_size_t
    L.frisk_hip_workspace_bytes.argtypes = [ctypes.POINTER(GemmDesc)]
    L.frisk_hip_gemm.argtypes = [ctypes.POINTER(GemmDesc), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                 ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    L.frisk_hip_gemm_static_ws.argtypes = [ctypes.POINTER(GemmDesc), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    L.frisk_hip_static_workspace_bytes.restype = ctypes.c_size_t
    L.frisk_hip_lds_access_cycles.restype = ctypes.c_float
    L.frisk_hip_lds_access_cycles.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_int32)]
    L.frisk_hip_lds_search.argtypes = [ctypes.POINTER(LdsLayout), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                       ctypes.c_int, ctypes.POINTER(LdsLayout), ctypes.POINTER(ctypes.c_float)]
    L.frisk_hip_lds_search_atom.argtypes = [ctypes.POINTER(LdsLayout), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                            ctypes.c_int, ctypes.c_int, ctypes.POINTER(LdsLayout), ctypes.POINTER(ctypes.c_float)]
    L.frisk_hip_lds_offset.restype = ctypes.c_int32
    L.frisk_hip_lds_offset.argtypes = [ctypes.POINTER(LdsLayout), ctypes.c_int32, ctypes.c_int32]
    L.frisk_hip_wave_partition.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                           ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
    L.frisk_hip_kernel_count.restype = ctypes.c_int
    L.frisk_hip_kernel_name.restype = ctypes.c_char_p
    L.frisk_hip_kernel_name.argtypes = [ctypes.c_int]
    i64, vp = ctypes.c_int64, ctypes.c_void_p
    L.frisk_hip_fill.argtypes = [ctypes.c_int, vp, i64, i64, i64, ctypes.c_double, vp]
    L.frisk_hip_copy.argtypes = [ctypes.c_int, vp, i64, ctypes.c_int, vp, i64, i64, i64, vp]
    L.frisk_hip_copy_tiles.argtypes = [ctypes.c_int, vp, i64, ctypes.c_int, vp, i64, i64, i64, i64, i64, i64, i64, i64, i64, vp]
    L.frisk_hip_elementwise.argtypes = [ctypes.POINTER(ElementwiseDesc), ctypes.POINTER(ctypes.c_void_p), vp, vp]
    L.frisk_hip_reduce_workspace_bytes.restype = ctypes.c_size_t
    L.frisk_hip_reduce_workspace_bytes.argtypes = [ctypes.c_int, i64, i64, ctypes.c_int]
    L.frisk_hip_softmax.argtypes = [ctypes.c_int, vp, i64, vp, i64, i64, i64, ctypes.c_float, vp, vp, ctypes.c_size_t, vp]
    L.frisk_hip_softmax_workspace_bytes.argtypes = [ctypes.c_int, i64, i64]
    L.frisk_hip_softmax_workspace_bytes.restype = ctypes.c_size_t
    L.frisk_hip_attention.argtypes = [ctypes.POINTER(AttentionDesc), vp, vp, vp, vp, vp, vp]
    L.frisk_hip_reduce.argtypes = [ctypes.c_int, vp, i64, i64, i64, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, ctypes.c_size_t, vp]
    if L.frisk_hip_abi_version() != ABI_VERSION:
        raise ImportError("libfrisk_hip.so has ABI %d, binding expects %d" % (L.frisk_hip_abi_version(), ABI_VERSION))
    _lib = L
    return L


def _check(status):
    if status != 0:
        raise FriskHipError(status, lib().frisk_hip_last_error().decode())


def make_desc(dtype_ab, M, N, K, dtype_out=None, transA=False, transB=False, lda=None, ldb=None, ldc=None,
              clear_accum=True, epilogue=EPI_NONE, policy=POLICY_SQUARE, tile=(0, 0, 0), waves=(0, 0), stages=0, split_k=0, atom=0):
    d = GemmDesc()
    d.abi_version = ABI_VERSION
    d.dtype_ab = dtype_ab
    d.dtype_acc = ACC_OF.get(dtype_ab, F32)
    d.dtype_out = dtype_ab if dtype_out is None else dtype_out
    d.M, d.N, d.K = M, N, K
    d.lda = lda if lda is not None else (M if transA else K)
    d.ldb = ldb if ldb is not None else (K if transB else N)
    d.ldc = ldc if ldc is not None else N
    d.transA, d.transB, d.clear_accum = int(transA), int(transB), int(clear_accum)
    d.epilogue, d.policy = epilogue, policy
    d.tile_m, d.tile_n, d.tile_k = tile
    d.waves_m, d.waves_n = waves
    d.stages = stages
    d.atom = atom
    d.split_k = split_k
    return d


def plan(desc):
    p = GemmPlan()
    _check(lib().frisk_hip_plan(ctypes.byref(desc), ctypes.byref(p)))
    return p


def init():
    """one-time set-up on the current device; needed only before launches are captured into a HIP graph"""
    _check(lib().frisk_hip_init())


def workspace_bytes(desc):
    """device workspace a launch of `desc` wants (split-K partial sums); 0 for most shapes"""
    return int(lib().frisk_hip_workspace_bytes(ctypes.byref(desc)))


def gemm(desc, A_ptr, B_ptr, C_ptr, scaleA_ptr=None, scaleB_ptr=None, workspace_ptr=None, workspace_bytes=0, stream=None):
    """Asynchronous launch on `stream` (a raw hipStream_t value or None). Pointers are raw device addresses."""
    _check(lib().frisk_hip_gemm(ctypes.byref(desc), A_ptr, B_ptr, C_ptr, scaleA_ptr, scaleB_ptr, workspace_ptr,
                                workspace_bytes, stream))


def static_workspace_bytes():
    """size of the library's own scratch array, the most a plan run by gemm_static_ws may need"""
    return int(lib().frisk_hip_static_workspace_bytes())


def gemm_static_ws(desc, A_ptr, B_ptr, C_ptr, scaleA_ptr=None, scaleB_ptr=None, stream=None):
    """`gemm` for callers that cannot allocate: split-K / tail-split partial sums go to the library's own scratch array.
    Calls that may overlap on one GPU race on that array."""
    _check(lib().frisk_hip_gemm_static_ws(ctypes.byref(desc), A_ptr, B_ptr, C_ptr, scaleA_ptr, scaleB_ptr, stream))


REDUCE_KINDS = {"add": 0, "sum": 0, "mul": 1, "min": 2, "max": 3}


def fill(dtype, dst_ptr, rows, cols, ld, value, stream=None):
    """frisk.fill on a rank-2 view of device memory (asynchronous on `stream`)"""
    _check(lib().frisk_hip_fill(dtype, dst_ptr, rows, cols, ld, float(value), stream))


def copy(src_dtype, src_ptr, src_ld, dst_dtype, dst_ptr, dst_ld, rows, cols, stream=None):
    """frisk.copy of a rows x cols window, converting between f32 / f16 / bf16 when the types differ"""
    _check(lib().frisk_hip_copy(src_dtype, src_ptr, src_ld, dst_dtype, dst_ptr, dst_ld, rows, cols, stream))


def copy_tiles(src_dtype, src_ptr, src_ld, dst_dtype, dst_ptr, dst_ld, tile_rows, tile_cols, n0, src_step0, dst_step0, n1=1, src_step1=0, dst_step1=0, stream=None):
    """n0 x n1 tiles of tile_rows x tile_cols, tile (a, b) displaced by a * step0 + b * step1 elements on either side"""
    _check(lib().frisk_hip_copy_tiles(src_dtype, src_ptr, src_ld, dst_dtype, dst_ptr, dst_ld, tile_rows, tile_cols, n0, src_step0, dst_step0, n1, src_step1, dst_step1,
                                      stream))


def make_elementwise_desc(program, inputs, out_dtype, rows, cols, out_ld=None):
    """program: postfix steps, each ("input", k) | ("const", value) | "add" | "sub" | "mul" | "div" | "max" | "min" | "neg" | "exp2" | "log2";
    inputs: one (dtype, row_stride, col_stride) per operand"""
    d = ElementwiseDesc()
    d.abi_version = ABI_VERSION
    d.n_inputs, d.n_ops, d.out_dtype = len(inputs), len(program), out_dtype
    d.rows, d.cols, d.out_ld = rows, cols, cols if out_ld is None else out_ld
    if len(inputs) > EW_MAX_INPUTS or len(program) > EW_MAX_OPS:
        raise ValueError("an elementwise program holds at most %d operands and %d steps" % (EW_MAX_INPUTS, EW_MAX_OPS))
    for k, (dt, rs, cs) in enumerate(inputs):
        d.in_dtype[k], d.in_row_stride[k], d.in_col_stride[k] = dt, rs, cs
    for i, step in enumerate(program):
        name, val = (step, None) if isinstance(step, str) else step
        d.op[i] = EW_OPS[name]
        if name == "input":
            d.arg[i] = int(val)
        elif name == "const":
            d.imm[i] = float(val)
    return d


def elementwise(desc, input_ptrs, out_ptr, stream=None):
    """frisk.block body as one interpreted kernel: out = program(inputs) for every point (asynchronous on `stream`)"""
    arr = (ctypes.c_void_p * max(1, len(input_ptrs)))(*input_ptrs)
    _check(lib().frisk_hip_elementwise(ctypes.byref(desc), arr, out_ptr, stream))


def reduce_workspace_bytes(dtype, rows, cols, dim):
    return int(lib().frisk_hip_reduce_workspace_bytes(dtype, rows, cols, dim))


def reduce(dtype, src_ptr, rows, cols, ld, dim, kind, clear, dst_ptr, workspace_ptr=None, workspace_bytes=0, stream=None):
    """frisk.reduce along `dim` with kind "add" | "mul" | "min" | "max" (or its enum value)"""
    k = REDUCE_KINDS[kind] if isinstance(kind, str) else kind
    _check(lib().frisk_hip_reduce(dtype, src_ptr, rows, cols, ld, dim, k, int(bool(clear)), dst_ptr, workspace_ptr, workspace_bytes, stream))


def softmax_workspace_bytes(dtype, rows, cols):
    return int(lib().frisk_hip_softmax_workspace_bytes(dtype, rows, cols))


def softmax(dtype, src_ptr, src_ld, dst_ptr, dst_ld, rows, cols, scale_log2=1.4426950408889634, lse_ptr=None, stream=None, workspace_ptr=None,
            workspace_bytes=0):
    """row softmax in base 2: dst = 2^(scale_log2 * src) / row sum; the default scale makes it the natural softmax.
    A workspace of softmax_workspace_bytes lets a few very long rows be split over several work-groups each."""
    _check(lib().frisk_hip_softmax(dtype, src_ptr, src_ld, dst_ptr, dst_ld, rows, cols, scale_log2, lse_ptr, workspace_ptr, workspace_bytes, stream))


def make_attention_desc(dtype, batch, heads, seq_q, seq_k, head_dim=128, scale=None, k_transposed=False):
    d = AttentionDesc()
    d.abi_version = ABI_VERSION
    d.dtype = dtype
    d.batch, d.heads, d.seq_q, d.seq_k, d.head_dim = batch, heads, seq_q, seq_k, head_dim
    d.scale = head_dim ** -0.5 if scale is None else scale
    d.k_transposed = int(bool(k_transposed))
    return d


def attention(desc, Q_ptr, K_ptr, V_ptr, O_ptr, lse_ptr=None, stream=None):
    """fused softmax(scale * Q K^T) V (asynchronous on `stream`); lse_ptr optionally receives the row log-sum-exp"""
    _check(lib().frisk_hip_attention(ctypes.byref(desc), Q_ptr, K_ptr, V_ptr, O_ptr, lse_ptr, stream))


def wave_partition(policy, tile_m, tile_n, num_waves):
    wm, wn = ctypes.c_int(), ctypes.c_int()
    _check(lib().frisk_hip_wave_partition(policy, tile_m, tile_n, num_waves, ctypes.byref(wm), ctypes.byref(wn)))
    return wm.value, wn.value


def lds_access_cycles(instr, lane_addrs):
    arr = (ctypes.c_int32 * 64)(*lane_addrs)
    return lib().frisk_hip_lds_access_cycles(instr, arr)


def lds_search(rows, row_bytes, k_contiguous, elem_bytes, frag_bytes, tile_mn, tile_k, waves, atom=32):
    """exhaustive swizzle search for one operand tile read by MFMA atoms of `atom` rows; returns (LdsLayout best, unswizzled
    cycles per access)"""
    shape, best, base = LdsLayout(), LdsLayout(), ctypes.c_float()
    shape.rows, shape.row_bytes, shape.k_contiguous = rows, row_bytes, int(k_contiguous)
    _check(lib().frisk_hip_lds_search_atom(ctypes.byref(shape), elem_bytes, frag_bytes, tile_mn, tile_k, waves, atom,
                                           ctypes.byref(best), ctypes.byref(base)))
    return best, base.value


def lds_offset(layout, row, col_byte):
    return lib().frisk_hip_lds_offset(ctypes.byref(layout), row, col_byte)


def kernel_names():
    L = lib()
    return [L.frisk_hip_kernel_name(i).decode() for i in range(L.frisk_hip_kernel_count())]
