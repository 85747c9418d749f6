"""ctypes binding of libfrisk_hwcheck.so (frisk_amd/csrc/hwcheck.hip): device checks of the MFMA fragment conventions
and the MFMA-only loop whose rate bench.py reports as the sustained ceiling.  Used by the GPU tests and the benchmark;
the product library never calls it."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfrisk_hwcheck.so")

# id -> (name, M, N, K, largest |operand value| that keeps the atom exact)
ATOMS = {0: ("f16 32x32x16", 32, 32, 16, 3), 1: ("f16 16x16x32", 16, 16, 32, 3), 2: ("bf16 32x32x16", 32, 32, 16, 3),
         3: ("bf16 16x16x32", 16, 16, 32, 3), 4: ("i8 32x32x32", 32, 32, 32, 127), 5: ("i8 16x16x64", 16, 16, 64, 127),
         6: ("f8f6f4 32x32x64", 32, 32, 64, 4), 7: ("f8f6f4 16x16x128", 16, 16, 128, 4), 8: ("fp8 16x16x32", 16, 16, 32, 4),
         9: ("f32 32x32x2", 32, 32, 2, 100), 10: ("f32 16x16x4", 16, 16, 4, 100)}
# MFMA-only loop kinds: id -> (name, frisk dtype name)
LOOP_KINDS = {0: ("f16 32x32x16", "f16"), 1: ("f16 16x16x32", "f16"), 2: ("bf16 32x32x16", "bf16"), 3: ("bf16 16x16x32", "bf16"),
              4: ("i8 32x32x32", "i8"), 5: ("i8 16x16x64", "i8"), 6: ("f8f6f4 32x32x64", "e4m3"), 7: ("f8f6f4 16x16x128", "e4m3")}

_lib = None
EXPORTS = ["frisk_hwcheck_mfma_atom", "frisk_hwcheck_fragment_path", "frisk_hwcheck_tr_read", "frisk_hwcheck_mfma_loop", "frisk_hwcheck_mfma_loop_data",
           "frisk_hwcheck_mfma_loop_flops", "frisk_hwcheck_mfma_loop_cycles", "frisk_hwcheck_device_info"]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError("libfrisk_hwcheck.so is not built: run `python -m frisk_amd.build` (needs hipcc)")
        L = ctypes.CDLL(LIB_PATH)
        vp, i = ctypes.c_void_p, ctypes.c_int
        L.frisk_hwcheck_mfma_atom.argtypes = [i, vp, vp, vp, vp]
        L.frisk_hwcheck_fragment_path.argtypes = [i, i, i, i, vp, vp, vp, vp]
        L.frisk_hwcheck_tr_read.argtypes = [i, vp, vp, i, vp]
        L.frisk_hwcheck_mfma_loop.argtypes = [i, i, i, i, vp]
        L.frisk_hwcheck_mfma_loop_data.argtypes = [i, i, i, vp, ctypes.c_longlong, i, vp, ctypes.c_longlong, i, vp]
        L.frisk_hwcheck_mfma_loop_flops.argtypes = [i, i, i]
        L.frisk_hwcheck_mfma_loop_flops.restype = ctypes.c_double
        L.frisk_hwcheck_mfma_loop_cycles.argtypes = [i, i]
        L.frisk_hwcheck_mfma_loop_cycles.restype = ctypes.c_double
        L.frisk_hwcheck_device_info.argtypes = [ctypes.POINTER(i)] * 4
        _lib = L
    return _lib


def _check(rc, what):
    if rc != 0:
        raise RuntimeError("%s failed with status %d" % (what, rc))


def mfma_atom(atom_id, A_ptr, B_ptr, D_ptr, stream=None):
    _check(lib().frisk_hwcheck_mfma_atom(atom_id, A_ptr, B_ptr, D_ptr, stream), "frisk_hwcheck_mfma_atom")


def fragment_path(dtype, atom, transA, transB, A_ptr, B_ptr, D_ptr, stream=None):
    _check(lib().frisk_hwcheck_fragment_path(dtype, atom, int(transA), int(transB), A_ptr, B_ptr, D_ptr, stream), "frisk_hwcheck_fragment_path")


def tr_read(bits, lane_addr_ptr, out_ptr, shift=0, stream=None):
    _check(lib().frisk_hwcheck_tr_read(bits, lane_addr_ptr, out_ptr, shift, stream), "frisk_hwcheck_tr_read")


def mfma_loop(kind, iters, random_operands, workgroups, stream=None):
    _check(lib().frisk_hwcheck_mfma_loop(kind, iters, int(bool(random_operands)), workgroups, stream), "frisk_hwcheck_mfma_loop")


def mfma_loop_data(kind, iters, workgroups, A_ptr, lda_bytes, rows_a, B_ptr, ldb_bytes, rows_b, stream=None):
    """the MFMA-only loop with its operand registers loaded once from two row-major device arrays"""
    _check(lib().frisk_hwcheck_mfma_loop_data(kind, iters, workgroups, A_ptr, lda_bytes, rows_a, B_ptr, ldb_bytes, rows_b, stream), "frisk_hwcheck_mfma_loop_data")


def mfma_loop_flops(kind, iters, workgroups):
    return float(lib().frisk_hwcheck_mfma_loop_flops(kind, iters, workgroups))


def mfma_loop_cycles(kind, iters):
    """matrix-pipe cycles one wave of the loop needs at full issue rate"""
    return float(lib().frisk_hwcheck_mfma_loop_cycles(kind, iters))


def device_info():
    """what the driver reports for the current device: {"compute_units", "clock_khz", "memory_clock_khz", "memory_bus_bits"}"""
    vals = [ctypes.c_int(0) for _ in range(4)]
    _check(lib().frisk_hwcheck_device_info(*[ctypes.byref(v) for v in vals]), "device_info")
    return dict(zip(("compute_units", "clock_khz", "memory_clock_khz", "memory_bus_bits"), (v.value for v in vals)))
