"""Builds libfrisk_hip.so (HIP kernels + C ABI) for gfx950, in-tree.

    python -m frisk_amd.build          # rebuild everything (HIP library, the device-check library, frisk_ffi extension)
    python -m frisk_amd.build --if-missing

hipcc cross-compiles without a GPU; the resulting library is loaded from
frisk_amd/lib/ by frisk_amd.runtime.
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(CSRC, "build")
LIB = os.path.join(LIBDIR, "libfrisk_hip.so")
HWCHECK_LIB = os.path.join(LIBDIR, "libfrisk_hwcheck.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-fp32 instructions are kept out of generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    "-Wno-unused-command-line-argument",
]
SOURCES = ["kernels_f16.hip", "kernels_f16_2.hip", "kernels_bf16.hip", "kernels_bf16_2.hip", "kernels_i8.hip", "kernels_i8_2.hip", "kernels_e4m3.hip", "kernels_e4m3_2.hip", "kernels_f32.hip", "kernels_f32_2.hip", "splitk_reduce.hip", "tile_ops.hip", "elementwise.hip", "softmax.hip", "attention.hip", "capi.cpp"]


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + COMMON + (["-x", "hip"] if src.endswith(".cpp") else []) + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(jobs=None, verbose=True):
    os.makedirs(OBJDIR, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    jobs = jobs or min(8, os.cpu_count() or 1)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for obj, err in pool.map(_compile, SOURCES):
            objs.append(obj)
            if verbose and err:
                print(err, file=sys.stderr)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


def build_hwcheck(verbose=True):
    """libfrisk_hwcheck.so: device-side checks of the MFMA fragment conventions and the MFMA-only loop the benchmark times
    (csrc/hwcheck.hip); used by the GPU tests and bench.py, never by the product library"""
    os.makedirs(LIBDIR, exist_ok=True)
    cmd = [HIPCC] + COMMON + ["-shared", os.path.join(CSRC, "hwcheck.hip"), "-o", HWCHECK_LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building libfrisk_hwcheck.so failed:\n" + r.stderr)
    if verbose:
        print("built", HWCHECK_LIB)
    return HWCHECK_LIB


FFI_DIR = os.path.join(HERE, "ffi")
FFI_SOURCES = ["ffi.cpp", "ir.cpp", "runtime.cpp"]


def build_ffi(verbose=True):
    """the `frisk_ffi` CPython extension (IR builder + runtime), host code only"""
    import sysconfig

    import pybind11
    out = os.path.join(HERE, "frisk", "frisk_ffi" + sysconfig.get_config_var("EXT_SUFFIX"))
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
           "-I" + pybind11.get_include(), "-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(ROOT, "include")]
    cmd += [os.path.join(FFI_DIR, f) for f in FFI_SOURCES] + ["-o", out, "-ldl"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building frisk_ffi failed:\n" + r.stderr)
    if verbose:
        print("built", out)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--if-missing", action="store_true")
    ap.add_argument("-j", type=int, default=None)
    a = ap.parse_args()
    if a.if_missing and os.path.exists(LIB):
        print("present", LIB)
        return
    build(a.j)
    build_hwcheck()
    build_ffi()


if __name__ == "__main__":
    main()
