// Python module `frisk_ffi`: same layout as the reference's (ffi/ffi.h, ffi/ffi.cpp:3-7):
// submodule `ir` with the builder surface, and -- in the slot the reference keeps
// commented out for `init_ffi_passes` (ffi/ffi.h:14) -- submodule `runtime`, which
// lowers a tiled-GEMM kernel to a descriptor and launches it through libfrisk_hip.so.
#ifndef FRISK_AMD_FFI_H_
#define FRISK_AMD_FFI_H_

#include <pybind11/functional.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

namespace py = pybind11;

namespace frisk_ffi {

void init_ffi_ir(py::module_&& m);
void init_ffi_runtime(py::module_&& m);

}  // namespace frisk_ffi

#endif  // FRISK_AMD_FFI_H_
