#include "ffi.h"

PYBIND11_MODULE(frisk_ffi, m) {
  m.doc() = "Python bindings of the Frisk IR builder (MLIR-free) and the gfx950 GEMM runtime";
  frisk_ffi::init_ffi_ir(m.def_submodule("ir"));
  frisk_ffi::init_ffi_runtime(m.def_submodule("runtime"));
}
