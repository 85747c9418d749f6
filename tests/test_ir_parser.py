"""Text -> IR (frisk.parse_module): the modules the reference saved (tmp/log_11_18 = tests/golden/bind_test_module.mlir,
tmp/log_11_25:30-39 = tests/golden/attr_test_module.mlir) and everything the builder can build must read back and print
the same text; a parsed kernel must plan and run like the built one."""
import os

import numpy as np
import pytest

import frisk_amd  # noqa: F401  (puts the `frisk` package on the path)
import frisk as F

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def reparse(text):
    return F.parse_module(F.context(), text)


def test_saved_bind_test_module_round_trips():
    text = open(os.path.join(GOLDEN, "bind_test_module.mlir")).read().rstrip("\n")
    m = reparse(text)
    assert str(m) == text
    assert m.verify() and m.get_kernel("test_gemm").verify()
    # and once more from its own output: parsing is idempotent
    assert str(reparse(str(m))) == text


def test_saved_attr_test_module_reads_into_the_canonical_form():
    m = reparse(open(os.path.join(GOLDEN, "attr_test_module.mlir")).read())
    want = ('module attributes {frisk.target = "sm_80"} {\n'
            '  frisk.kernel @test(memref<128x64xf16, 3>, memref<64x128xf16, 3>, memref<128x128xf16>) {\n'
            '    frisk.gemm(%arg0, %arg1, %arg2) {K = 64 : i64, M = 128 : i64, N = 128 : i64, clear_accum = false, frisk.threads = 128 : i64, '
            'policy = #frisk<gemm_warp_policy Square>, transA = false, transB = false} : memref<128x64xf16, 3>, memref<64x128xf16, 3>, memref<128x128xf16>\n'
            '  }\n'
            '}')
    assert str(m) == want and m.verify()


@pytest.mark.parametrize("dtype,tile,ta,tb", [("fp16", (256, 256, 64), False, False), ("bf16", (128, 128, 64), True, True),
                                              ("fp32", (128, 128, 32), False, True), ("int8", (256, 256, 128), False, False),
                                              ("e4m3fn", (256, 256, 128), False, True)])
def test_built_tiled_gemms_round_trip_and_plan_the_same(dtype, tile, ta, tb):
    h = F.create_session()
    out = {"int8": "fp16", "e4m3fn": "bf16"}.get(dtype)
    k = h.tiled_gemm("g", 1024, 512, 768 if tile[2] != 128 else 1024, dtype, out_dtype=out, tile=tile, trans_a=ta, trans_b=tb)
    k.set_attr("frisk.target", "gfx950")
    text = str(h.module)
    m = reparse(text)
    assert str(m) == text and m.verify()
    a, b = F.runtime.plan(k), F.runtime.plan(m.get_kernel("g"))
    assert a == b


def test_every_op_and_expression_form_round_trips():
    text = '''module {
  frisk.kernel @k(memref<64x64xf32, 1>, memref<64xf32, 1>, memref<4x64x64xbf16, affine_map<(d0, d1, d2) -> (d2, d1, d0)>, 1>) -> (f32, index) {
    frisk.parallel (%arg3) = (4), threads = 256 {
      %0 = frisk.alloc_buffer {scope = "shared"} -> memref<16x64xf32, 3>
      %1 = frisk.alloc_buffer {scope = "local", alignment = 16} -> memref<16xf32>
      %2 = frisk.alloc_buffer {scope = "global"} -> memref<?x8xi8, 1>
      frisk.fill %1 {value = -1.500000e+00 : f32} : memref<16xf32>
      frisk.fill %1 {value = 0xFF800000 : f32} : memref<16xf32>
      frisk.for %arg4 = 2 to 64 step = 3 {
        frisk.copy %arg0[%arg3 * 16 + %arg4 floordiv 4 - 1, (%arg4 mod 4) * 16], %0[0, 0] {src_extents = [16, 64], dst_extents = [16, 64]}  : memref<64x64xf32, 1>, memref<16x64xf32, 3>
        frisk.block (%arg5, %arg6) to (16, 64) {
          frisk.reduce %0, %1 {clear = false, dim = 1 : i64, kind = "add"} : memref<16x64xf32, 3>, memref<16xf32>
        }
      }
      frisk.copy %1[0], %arg1[-%arg3 + 3] {src_extents = [16], dst_extents = [16]}  : memref<16xf32>, memref<64xf32, 1>
    }
  } {frisk.target = "gfx950", note = "kept"}
}'''
    m = reparse(text)
    assert str(m) == text
    # names are positional: other spellings of the same program print back in the canonical numbering
    renamed = text.replace("%arg4", "%k").replace("%0", "%tile").replace("%arg5", "%i")
    assert str(reparse(renamed)) == text
    # a module without the wrapper, with comments, and a step of 1 spelled out
    bare = '''// a kernel on its own
frisk.kernel @z(memref<8xf16, 1>) {
  frisk.for %i = 0 to 4 step = 1 {   // step = 1 is what the printer leaves out
    frisk.fill %arg0 {value = 0.000000e+00 : f16} : memref<8xf16, 1>
  }
}'''
    assert str(reparse(bare)) == ('module {\n  frisk.kernel @z(memref<8xf16, 1>) {\n    frisk.for %arg1 = 0 to 4 {\n'
                                  '      frisk.fill %arg0 {value = 0.000000e+00 : f16} : memref<8xf16, 1>\n    }\n  }\n}')


def test_parsed_programs_are_verified_like_built_ones():
    bad_gemm = '''module {
  frisk.kernel @k(memref<128x64xf16, 3>, memref<32x128xf16, 3>, memref<128x128xf32>) {
    frisk.gemm(%arg0, %arg1, %arg2) {K = 64 : i64, M = 128 : i64, N = 128 : i64, clear_accum = false, policy = #frisk<gemm_warp_policy FullRow>, transA = false, transB = false} : memref<128x64xf16, 3>, memref<32x128xf16, 3>, memref<128x128xf32>
  }
}'''
    m = reparse(bad_gemm)
    assert "FullRow" in str(m) and not m.verify()          # B is 32 x 128 where K = 64: the op verifier's business, not the parser's


@pytest.mark.parametrize("text,message", [
    ("module {\n  frisk.kernel @k(memref<8xf16, 1>) {\n    frisk.fill %arg1 {value = 0.000000e+00 : f16} : memref<8xf16, 1>\n  }\n}",
     r"line 3, column \d+: use of undeclared SSA value name '%arg1'"),
    ("module {\n  frisk.kernel @k(memref<8xf16, 1>) {\n    frisk.fill %arg0 {value = 0.000000e+00 : f16} : memref<8xf32, 1>\n  }\n}",
     "expects different type than prior uses"),
    ("module {\n  frisk.kernel @k() {\n    frisk.launch\n  }\n}", "unknown operation 'frisk.launch'"),
    ("module {\n  frisk.kernel @k() {\n    %0 = frisk.alloc_buffer {scope = \"shared\"} -> memref<8xf16>\n  }\n}", "does not match the memory space"),
    ("module {\n  frisk.kernel @k() {\n    %0 = frisk.alloc_buffer {scope = \"local\"} -> f16\n  }\n}", "expected memref type for result"),
    ("module {\n  frisk.kernel @k() {\n    frisk.parallel (%a, %b) = (4), threads = 64 {\n    }\n  }\n}", "number of induction variables"),
    ("module {\n  frisk.kernel @k() {\n    frisk.parallel (%a) = (4) {\n    }\n  }\n}", "expected ','"),
    ("module {\n  frisk.kernel @k(memref<8xf16, 1>) {\n    frisk.for %arg0 = 0 to 4 {\n    }\n  }\n}", "redefinition of SSA value '%arg0'"),
    ("module {\n  frisk.kernel @k(memref<8xq16, 1>) {\n  }\n}", "unknown type 'q16'"),
    ("module {\n  frisk.kernel @k() {\n  }\n} trailing", "unexpected text after the module"),
    ("module {\n  func.func @k() {\n  }\n}", "expected 'frisk.kernel'"),
])
def test_syntax_errors_name_the_place(text, message):
    with pytest.raises(ValueError, match=message):
        reparse(text)


def test_values_do_not_leak_between_kernels():
    text = '''module {
  frisk.kernel @a(memref<8xf16, 1>) {
    frisk.parallel (%arg1) = (1), threads = 64 {
      %0 = frisk.alloc_buffer {scope = "local"} -> memref<8xf16>
    }
  }
  frisk.kernel @b(memref<8xf16, 1>) {
    frisk.fill %0 {value = 0.000000e+00 : f16} : memref<8xf16>
  }
}'''
    with pytest.raises(ValueError, match="undeclared SSA value name '%0'"):
        reparse(text)
    ok = text.replace("frisk.fill %0 {value = 0.000000e+00 : f16} : memref<8xf16>", "frisk.fill %arg0 {value = 0.000000e+00 : f16} : memref<8xf16, 1>")
    m = reparse(ok)
    assert str(m) == ok and m.has_kernel("a") and m.has_kernel("b")


@pytest.mark.gpu
def test_a_parsed_kernel_runs_like_the_built_one():
    import torch
    import oracle as O
    from helpers import to_dev, from_dev
    M, N, K = 512, 384, 256
    h = F.create_session()
    h.tiled_gemm("g", M, N, K, "fp16", tile=(128, 128, 64), threads=256)
    module = reparse(str(h.module))
    kernel = module.get_kernel("g")
    A = O.encode(O.F16, O.normal(M * K, 5, 0, 0.1)).reshape(M, K)
    B = O.encode(O.F16, O.normal(K * N, 5, 1, 0.1)).reshape(K, N)
    dA, dB = to_dev(A), to_dev(B)
    dC = torch.zeros(M * N * 2, dtype=torch.uint8, device="cuda")
    F.runtime.launch(kernel, [dA.data_ptr(), dB.data_ptr(), dC.data_ptr()], torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    r = O.compare(O.F16, from_dev(dC, np.uint16, (M, N)), O.gemm_f64(O.F16, A, B))
    assert r["nonfinite"] == 0 and r["max_rel"] <= 1e-2 and r["fro_rel"] <= 1e-2, r
