// The body of a frisk.block (include/Dialect/Frisk/IR/FriskOps.td:143-190; built by ffi/ir.cpp:383-394) run over a
// rank-2 iteration space: for every (row, col) evaluate an expression of loads, constants and arith / math ops and store
// the value.  The reference defines the op and lowers it nowhere.  Here the expression arrives as a postfix program (at
// most FRISK_EW_MAX_OPS steps over FRISK_EW_MAX_INPUTS operands) and ONE kernel interprets it: no run-time compilation.
//
// A lane evaluates 8 consecutive columns at a time through 16-byte accesses; the program counter and every opcode are
// wave-uniform (the program sits in registers, a step is a lane read and a scalar branch), and the evaluation stack lives
// in registers: one switch on (stack depth, opcode) names the slots each snippet touches, so nothing is indexed at run
// time.  All arithmetic is fp32; the result is rounded once to the output type.  A one-step program moves 5.3 TB/s,
// y = log2(max(x, c) / (x + c)) (8 steps, one IEEE division) 2.2 TB/s on a 32768 x 8192 f16 view.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "tile_ops.h"

namespace frisk {
namespace {

typedef unsigned v4u __attribute__((ext_vector_type(4)));
static_assert(FRISK_EW_MAX_STACK == 6, "the interpreter below names six stack slots");

// element (row, col .. col + V - 1) of operand k as floats; cs = 0 broadcasts one element along the row
template <int V, bool VEC>
__device__ __forceinline__ void load_operand(const EwParams& p, int k, int64_t row, int64_t col, int64_t cols, float (&out)[V]) {
  const int dt = p.in_dtype[k];
  const int64_t base = row * p.in_row_stride[k] + (p.in_col_stride[k] ? col : 0);
  const char* ptr = (const char*)p.in[k];
  if (!p.in_col_stride[k]) {
    float x;
    if (dt == FRISK_F32) x = ((const float*)ptr)[base];
    else if (dt == FRISK_F16) x = (float)((const _Float16*)ptr)[base];
    else x = (float)((const __bf16*)ptr)[base];
#pragma unroll
    for (int e = 0; e < V; ++e) out[e] = x;
    return;
  }
  if constexpr (VEC) {
#pragma unroll
    for (int c = 0; c < V / 8; ++c) {  // 8 columns at a time: 32 bytes of a 32-bit operand, 16 of a 16-bit one
      if (dt == FRISK_F32) {
        const v4u* q = (const v4u*)(ptr + (base + 8 * c) * 4);
        const v4u a = __builtin_nontemporal_load(q), b = __builtin_nontemporal_load(q + 1);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const unsigned lo = a[e], hi = b[e];  // copy first: bit_cast applied to a vector element reads element 0
          out[8 * c + e] = __builtin_bit_cast(float, lo);
          out[8 * c + 4 + e] = __builtin_bit_cast(float, hi);
        }
      } else {
        const v4u a = __builtin_nontemporal_load((const v4u*)(ptr + (base + 8 * c) * 2));
        if (dt == FRISK_F16) {
          typedef _Float16 h8 __attribute__((ext_vector_type(8)));
          const h8 h = __builtin_bit_cast(h8, a);
#pragma unroll
          for (int e = 0; e < 8; ++e) out[8 * c + e] = (float)h[e];
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) { out[8 * c + 2 * e] = __builtin_bit_cast(float, a[e] << 16); out[8 * c + 2 * e + 1] = __builtin_bit_cast(float, a[e] & 0xffff0000u); }
        }
      }
    }
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float x = 0.f;
      if (col + e < cols) {
        if (dt == FRISK_F32) x = ((const float*)ptr)[base + e];
        else if (dt == FRISK_F16) x = (float)((const _Float16*)ptr)[base + e];
        else x = (float)((const __bf16*)ptr)[base + e];
      }
      out[e] = x;
    }
  }
}

template <int V> __device__ __forceinline__ void ew_store(const EwParams& p, int64_t at, const float (&r)[V]) {
  char* dst = (char*)p.out;
  if constexpr (V > 1) {
#pragma unroll
    for (int c = 0; c < V / 8; ++c) {
      if (p.out_dtype == FRISK_F32) {
        v4u a, b;
#pragma unroll
        for (int e = 0; e < 4; ++e) { a[e] = __builtin_bit_cast(unsigned, r[8 * c + e]); b[e] = __builtin_bit_cast(unsigned, r[8 * c + 4 + e]); }
        __builtin_nontemporal_store(a, (v4u*)(dst + (at + 8 * c) * 4));
        __builtin_nontemporal_store(b, (v4u*)(dst + (at + 8 * c) * 4) + 1);
      } else if (p.out_dtype == FRISK_F16) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        h8 h;
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = (_Float16)r[8 * c + e];
        __builtin_nontemporal_store(__builtin_bit_cast(v4u, h), (v4u*)(dst + (at + 8 * c) * 2));
      } else {
        typedef __bf16 b8 __attribute__((ext_vector_type(8)));
        b8 h;
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = (__bf16)r[8 * c + e];
        __builtin_nontemporal_store(__builtin_bit_cast(v4u, h), (v4u*)(dst + (at + 8 * c) * 2));
      }
    }
  } else {
    if (p.out_dtype == FRISK_F32) ((float*)dst)[at] = r[0];
    else if (p.out_dtype == FRISK_F16) ((_Float16*)dst)[at] = (_Float16)r[0];
    else ((__bf16*)dst)[at] = (__bf16)r[0];
  }
}

// The interpreter.  The evaluation stack is six plain arrays s0 .. s5 (slot k of the stack is sk); one switch on
// (stack depth, opcode) selects a straight-line snippet in which the slots an opcode touches are named, so nothing is ever
// indexed at run time and the stack stays in registers.  The host has checked that no step underflows or overflows.
template <int V> __global__ void __launch_bounds__(256) elementwise_kernel(EwParams p, int lanes_log2) {
  constexpr bool VEC = V > 1;
  const int64_t groups = (p.cols + V - 1) / V;
  const int lanes = 1 << lanes_log2, row_step = 256 >> lanes_log2;
  const int lane_group = threadIdx.x & (lanes - 1), lane_row = threadIdx.x >> lanes_log2;
  // The program sits in three registers, step i in lane i (FRISK_EW_MAX_OPS <= 64): a step is fetched with a lane read
  // instead of a dependent scalar load from the kernel arguments, whose latency every step of every element group paid.
  static_assert(FRISK_EW_MAX_OPS <= 64, "one program step per lane of a wave");
  const int my_step = (threadIdx.x & 63) < FRISK_EW_MAX_OPS ? (int)(threadIdx.x & 63) : 0;
  int ops_reg = p.op[my_step], args_reg = p.arg[my_step];
  float imms_reg = p.imm[my_step];
  // pinned here, with every lane active: the lane reads below happen inside loops that lanes leave at different times,
  // and a load that the compiler moved down to its use there would fill only the lanes still running
  asm volatile("" : "+v"(ops_reg), "+v"(args_reg), "+v"(imms_reg));
  for (int64_t row = (int64_t)blockIdx.y * row_step + lane_row; row < p.rows; row += (int64_t)gridDim.y * row_step)
    for (int64_t g = (int64_t)blockIdx.x * lanes + lane_group; g < groups; g += (int64_t)gridDim.x * lanes) {
      const int64_t col = g * V;
      float s0[V], s1[V], s2[V], s3[V], s4[V], s5[V];
      int sp = 0;
      for (int pc = 0; pc < p.n_ops; ++pc) {
        const int op = __builtin_amdgcn_readlane(ops_reg, pc), arg = __builtin_amdgcn_readlane(args_reg, pc);
        const float imm = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, imms_reg), pc));
#define FRISK_EW_EACH(STMT) _Pragma("unroll") for (int e = 0; e < V; ++e) { STMT; }
#define FRISK_EW_PUSH(SP, NEXT)                                                                                  \
  case SP * 16 + FRISK_EW_INPUT: load_operand<V, VEC>(p, arg, row, col, p.cols, NEXT); sp = SP + 1; break;     \
  case SP * 16 + FRISK_EW_CONST: FRISK_EW_EACH(NEXT[e] = imm) sp = SP + 1; break;
#define FRISK_EW_UNARY(SP, TOP)                                                                                  \
  case SP * 16 + FRISK_EW_NEG: FRISK_EW_EACH(TOP[e] = -TOP[e]) break;                                            \
  case SP * 16 + FRISK_EW_EXP2: FRISK_EW_EACH(TOP[e] = __builtin_amdgcn_exp2f(TOP[e])) break;                    \
  case SP * 16 + FRISK_EW_LOG2: FRISK_EW_EACH(TOP[e] = __builtin_amdgcn_logf(TOP[e])) break; /* v_log_f32: base 2 */
#define FRISK_EW_BINARY(SP, A, B) /* the operand pushed first (A) is the left one; MAX / MIN ignore a NaN operand */ \
  case SP * 16 + FRISK_EW_ADD: FRISK_EW_EACH(A[e] = A[e] + B[e]) sp = SP - 1; break;                            \
  case SP * 16 + FRISK_EW_SUB: FRISK_EW_EACH(A[e] = A[e] - B[e]) sp = SP - 1; break;                            \
  case SP * 16 + FRISK_EW_MUL: FRISK_EW_EACH(A[e] = A[e] * B[e]) sp = SP - 1; break;                            \
  case SP * 16 + FRISK_EW_DIV: FRISK_EW_EACH(A[e] = A[e] / B[e]) sp = SP - 1; break;                            \
  case SP * 16 + FRISK_EW_MAX: FRISK_EW_EACH(A[e] = __builtin_fmaxf(A[e], B[e])) sp = SP - 1; break;            \
  case SP * 16 + FRISK_EW_MIN: FRISK_EW_EACH(A[e] = __builtin_fminf(A[e], B[e])) sp = SP - 1; break;
        switch (sp * 16 + op) {  // wave-uniform
          FRISK_EW_PUSH(0, s0)
          FRISK_EW_PUSH(1, s1) FRISK_EW_UNARY(1, s0)
          FRISK_EW_PUSH(2, s2) FRISK_EW_UNARY(2, s1) FRISK_EW_BINARY(2, s0, s1)
          FRISK_EW_PUSH(3, s3) FRISK_EW_UNARY(3, s2) FRISK_EW_BINARY(3, s1, s2)
          FRISK_EW_PUSH(4, s4) FRISK_EW_UNARY(4, s3) FRISK_EW_BINARY(4, s2, s3)
          FRISK_EW_PUSH(5, s5) FRISK_EW_UNARY(5, s4) FRISK_EW_BINARY(5, s3, s4)
          FRISK_EW_UNARY(6, s5) FRISK_EW_BINARY(6, s4, s5)
          default: break;
        }
#undef FRISK_EW_EACH
#undef FRISK_EW_PUSH
#undef FRISK_EW_UNARY
#undef FRISK_EW_BINARY
      }
      ew_store<V>(p, row * p.out_ld + col, s0);
    }
}

}  // namespace

hipError_t launch_elementwise(const EwParams& p, int vec_ok, hipStream_t s) {
  // columns per lane and step: 8 through 16-byte accesses, else single elements.  (16 per lane halve the interpreter's cost
  // per element but need 173 registers: two waves per SIMD keep too few bytes in flight, 3.2 against 5.3 TB/s for a copy.)
  const int V = vec_ok ? 8 : 1;
  const int64_t groups = (p.cols + V - 1) / V;
  int lanes_log2 = 0;
  while (lanes_log2 < 8 && ((int64_t)1 << lanes_log2) < groups) ++lanes_log2;
  const int64_t lanes = (int64_t)1 << lanes_log2, row_step = 256 >> lanes_log2;
  // enough work-groups to fill the chip several times over, every lane walking its row / column strides beyond that
  int64_t gx = (groups + lanes - 1) / lanes, gy = (p.rows + row_step - 1) / row_step;
  const int64_t cap = 256 * 16;
  if (gx > cap) gx = cap;
  if (gx * gy > cap) gy = (cap + gx - 1) / gx;
  if (gy > 65535) gy = 65535;
  const dim3 grid((unsigned)gx, (unsigned)gy);
  if (V == 8) hipLaunchKernelGGL(elementwise_kernel<8>, grid, dim3(256), 0, s, p, lanes_log2);
  else hipLaunchKernelGGL(elementwise_kernel<1>, grid, dim3(256), 0, s, p, lanes_log2);
  return hipGetLastError();
}

}  // namespace frisk
