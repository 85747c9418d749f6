// The body of a frisk.block (include/Dialect/Frisk/IR/FriskOps.td:143-190; built by ffi/ir.cpp:383-394) run over a
// rank-2 iteration space: for every (row, col) evaluate an expression of loads, constants and arith / math ops and store
// the value.  The reference defines the op and lowers it nowhere.  Here the expression arrives as a postfix program (at
// most FRISK_EW_MAX_OPS steps over FRISK_EW_MAX_INPUTS operands) and ONE kernel interprets it: no run-time compilation.
//
// A lane evaluates 8 consecutive columns at a time (16 bytes of a 16-bit operand, 32 of a 32-bit one), the program counter
// and every opcode are wave-uniform (scalar loads, scalar branches), and the evaluation stack lives in registers: the
// interpreter is written once per stack depth, so every stack slot an opcode touches is a compile-time register index.
// All arithmetic is fp32; the result is rounded once to the output type.  HBM-bound for short programs.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "tile_ops.h"

namespace frisk {
namespace {

typedef unsigned v4u __attribute__((ext_vector_type(4)));
constexpr int kStack = 6;  // deepest evaluation stack a program may need (checked on the host)

template <int V> struct Vec { float v[V]; };

// element (row, col .. col + V - 1) of operand k as floats; cs = 0 broadcasts one element along the row
template <int V, bool VEC>
__device__ __forceinline__ void load_operand(const EwParams& p, int k, int64_t row, int64_t col, int64_t cols, Vec<V>& out) {
  const int dt = p.in_dtype[k];
  const int64_t base = row * p.in_row_stride[k] + (p.in_col_stride[k] ? col : 0);
  const char* ptr = (const char*)p.in[k];
  if (!p.in_col_stride[k]) {
    float x;
    if (dt == FRISK_F32) x = ((const float*)ptr)[base];
    else if (dt == FRISK_F16) x = (float)((const _Float16*)ptr)[base];
    else x = (float)((const __bf16*)ptr)[base];
#pragma unroll
    for (int e = 0; e < V; ++e) out.v[e] = x;
    return;
  }
  if constexpr (VEC) {
    if (dt == FRISK_F32) {
      const v4u a = __builtin_nontemporal_load((const v4u*)(ptr + base * 4)), b = __builtin_nontemporal_load((const v4u*)(ptr + base * 4) + 1);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const unsigned lo = a[e], hi = b[e];  // copy first: bit_cast applied to a vector element reads element 0
        out.v[e] = __builtin_bit_cast(float, lo);
        out.v[4 + e] = __builtin_bit_cast(float, hi);
      }
    } else {
      const v4u a = __builtin_nontemporal_load((const v4u*)(ptr + base * 2));
      if (dt == FRISK_F16) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 h = __builtin_bit_cast(h8, a);
#pragma unroll
        for (int e = 0; e < 8; ++e) out.v[e] = (float)h[e];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) { out.v[2 * e] = __builtin_bit_cast(float, a[e] << 16); out.v[2 * e + 1] = __builtin_bit_cast(float, a[e] & 0xffff0000u); }
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
      out.v[e] = x;
    }
  }
}

// one step of the program with SP values on the stack; returns the new depth.  The host has checked that no step
// underflows or overflows, so the guards below only keep the compiler from indexing outside the array.
template <int SP, int V, bool VEC>
__device__ __forceinline__ int ew_step(const EwParams& p, int pc, int64_t row, int64_t col, int64_t cols, Vec<V> (&st)[kStack]) {
  const int op = p.op[pc];
  if (op == FRISK_EW_INPUT) {
    if constexpr (SP < kStack) { load_operand<V, VEC>(p, p.arg[pc], row, col, cols, st[SP]); return SP + 1; }
    return SP;
  }
  if (op == FRISK_EW_CONST) {
    if constexpr (SP < kStack) {
      const float c = p.imm[pc];
#pragma unroll
      for (int e = 0; e < V; ++e) st[SP].v[e] = c;
      return SP + 1;
    }
    return SP;
  }
  if (op >= FRISK_EW_NEG) {  // unary
    if constexpr (SP >= 1) {
      Vec<V>& x = st[SP - 1];
#pragma unroll
      for (int e = 0; e < V; ++e) {
        if (op == FRISK_EW_NEG) x.v[e] = -x.v[e];
        else if (op == FRISK_EW_EXP2) x.v[e] = __builtin_amdgcn_exp2f(x.v[e]);
        else x.v[e] = __builtin_amdgcn_logf(x.v[e]);  // v_log_f32: base 2
      }
    }
    return SP;
  }
  if constexpr (SP >= 2) {  // binary: the operand pushed first is the left one
    Vec<V>& a = st[SP - 2];
    const Vec<V>& b = st[SP - 1];
#pragma unroll
    for (int e = 0; e < V; ++e) {
      switch (op) {
        case FRISK_EW_ADD: a.v[e] = a.v[e] + b.v[e]; break;
        case FRISK_EW_SUB: a.v[e] = a.v[e] - b.v[e]; break;
        case FRISK_EW_MUL: a.v[e] = a.v[e] * b.v[e]; break;
        case FRISK_EW_DIV: a.v[e] = a.v[e] / b.v[e]; break;
        case FRISK_EW_MAX: a.v[e] = __builtin_fmaxf(a.v[e], b.v[e]); break;  // maxnumf / minnumf: a NaN operand is ignored
        default: a.v[e] = __builtin_fminf(a.v[e], b.v[e]); break;
      }
    }
    return SP - 1;
  }
  return SP;
}

template <bool VEC> __global__ void __launch_bounds__(256) elementwise_kernel(EwParams p, int lanes_log2) {
  constexpr int V = VEC ? 8 : 1;
  const int64_t groups = (p.cols + V - 1) / V;
  const int lanes = 1 << lanes_log2, row_step = 256 >> lanes_log2;
  const int lane_group = threadIdx.x & (lanes - 1), lane_row = threadIdx.x >> lanes_log2;
  for (int64_t row = (int64_t)blockIdx.y * row_step + lane_row; row < p.rows; row += (int64_t)gridDim.y * row_step)
    for (int64_t g = (int64_t)blockIdx.x * lanes + lane_group; g < groups; g += (int64_t)gridDim.x * lanes) {
      const int64_t col = g * V;
      Vec<V> st[kStack];
      int sp = 0;
      for (int pc = 0; pc < p.n_ops; ++pc) {
        switch (sp) {  // wave-uniform: one copy of the interpreter per stack depth
          case 0: sp = ew_step<0, V, VEC>(p, pc, row, col, p.cols, st); break;
          case 1: sp = ew_step<1, V, VEC>(p, pc, row, col, p.cols, st); break;
          case 2: sp = ew_step<2, V, VEC>(p, pc, row, col, p.cols, st); break;
          case 3: sp = ew_step<3, V, VEC>(p, pc, row, col, p.cols, st); break;
          case 4: sp = ew_step<4, V, VEC>(p, pc, row, col, p.cols, st); break;
          case 5: sp = ew_step<5, V, VEC>(p, pc, row, col, p.cols, st); break;
          default: sp = ew_step<6, V, VEC>(p, pc, row, col, p.cols, st); break;
        }
      }
      const Vec<V>& r = st[0];
      char* dst = (char*)p.out;
      const int64_t at = row * p.out_ld + col;
      if constexpr (VEC) {
        if (p.out_dtype == FRISK_F32) {
          v4u a, b;
#pragma unroll
          for (int e = 0; e < 4; ++e) { a[e] = __builtin_bit_cast(unsigned, r.v[e]); b[e] = __builtin_bit_cast(unsigned, r.v[4 + e]); }
          __builtin_nontemporal_store(a, (v4u*)(dst + at * 4));
          __builtin_nontemporal_store(b, (v4u*)(dst + at * 4) + 1);
        } else if (p.out_dtype == FRISK_F16) {
          typedef _Float16 h8 __attribute__((ext_vector_type(8)));
          h8 h;
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = (_Float16)r.v[e];
          __builtin_nontemporal_store(__builtin_bit_cast(v4u, h), (v4u*)(dst + at * 2));
        } else {
          typedef __bf16 b8 __attribute__((ext_vector_type(8)));
          b8 h;
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = (__bf16)r.v[e];
          __builtin_nontemporal_store(__builtin_bit_cast(v4u, h), (v4u*)(dst + at * 2));
        }
      } else {
        if (p.out_dtype == FRISK_F32) ((float*)dst)[at] = r.v[0];
        else if (p.out_dtype == FRISK_F16) ((_Float16*)dst)[at] = (_Float16)r.v[0];
        else ((__bf16*)dst)[at] = (__bf16)r.v[0];
      }
    }
}

}  // namespace

hipError_t launch_elementwise(const EwParams& p, int vec_ok, hipStream_t s) {
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
  if (vec_ok) hipLaunchKernelGGL(elementwise_kernel<true>, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, p, lanes_log2);
  else hipLaunchKernelGGL(elementwise_kernel<false>, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, p, lanes_log2);
  return hipGetLastError();
}

}  // namespace frisk
