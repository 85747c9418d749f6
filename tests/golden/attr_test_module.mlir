module attributes {frisk.target = "sm_80"} {
  frisk.kernel @test(memref<128x64xf16, 3>, memref<64x128xf16, 3>, memref<128x128xf16>) {
    frisk.gemm(%arg0, %arg1, %arg2) {K = 64 : i64, M = 128 : i64, N = 128 : i64, clear_accum = false, 
                                     frisk.threads = 128 : i64, 
                                     policy = #frisk<gemm_warp_policy Square>, 
                                     transA = false, transB = false
                                     } : 
      memref<128x64xf16, 3>, memref<64x128xf16, 3>, memref<128x128xf16>
  }
}
