// Register-level helpers shared by the decode-regime kernels (M <= 16).
#pragma once

#include "qmm_common.hpp"

namespace qmm {

constexpr uint32_t kOnesBf16x2 = 0x3F803F80u;

__device__ __forceinline__ bf16x8 as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  u32x4 v = {a, b, c, d};
  return __builtin_bit_cast(bf16x8, v);
}

// 8 eight-bit codes (two words) -> bf16 pairs in natural order.  An integer
// below 256 is exact in the top 16 bits of its float32 form.
__device__ __forceinline__ bf16x8 widen_int8(uint32_t w0, uint32_t w1) {
  const float f0 = (float)(w0 & 0xFFu), f1 = (float)((w0 >> 8) & 0xFFu);
  const float f2 = (float)((w0 >> 16) & 0xFFu), f3 = (float)(w0 >> 24);
  const float f4 = (float)(w1 & 0xFFu), f5 = (float)((w1 >> 8) & 0xFFu);
  const float f6 = (float)((w1 >> 16) & 0xFFu), f7 = (float)(w1 >> 24);
  const uint32_t sel = 0x07060302u;
  return as_bf16x8(byte_perm(__float_as_uint(f1), __float_as_uint(f0), sel),
                   byte_perm(__float_as_uint(f3), __float_as_uint(f2), sel),
                   byte_perm(__float_as_uint(f5), __float_as_uint(f4), sel),
                   byte_perm(__float_as_uint(f7), __float_as_uint(f6), sel));
}

// 8 E2M1 codes times a power-of-two scale -> bf16 pairs in natural order
// (q_2t, q_2t+1), exact: the hardware converter widens the two codes of one
// byte at a time and multiplies by the float32 scale.
__device__ __forceinline__ bf16x8 widen_e2m1(uint32_t w, float scale) {
  bf16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 0);
  bf16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 1);
  bf16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 2);
  bf16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 3);
  return as_bf16x8(__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1),
                   __builtin_bit_cast(uint32_t, p2), __builtin_bit_cast(uint32_t, p3));
}

// Activations x[m, k..k+8) in natural order -> pairs (k+t, k+t+4).
__device__ __forceinline__ bf16x8 pair_stride4(u32x4 x) {
  const uint32_t lo = 0x05040100u, hi = 0x07060302u;
  return as_bf16x8(byte_perm(x[2], x[0], lo), byte_perm(x[2], x[0], hi),
                   byte_perm(x[3], x[1], lo), byte_perm(x[3], x[1], hi));
}

struct GemvArgs {
  const uint16_t* x;   // bf16 [batch, M, K]
  const uint32_t* w;   // [batch, N, K*bits/32]
  const void* s;       // [batch, N, K/gs]
  const void* b;
  void* y;             // [batch, M, N]
  int M, N, K;
  int gshift;          // log2(group_size / CH)
  int y_dtype;
  // gather form: batch entry z multiplies x[lhs_idx[z]] by w[rhs_idx[z]]
  // (rhs_idx set = gather form; then n_experts / n_xrows bound the indices: a
  // pair whose expert is outside [0, n_experts) writes nothing, a row outside
  // [0, n_xrows) reads as zeros)
  const int32_t* lhs_idx;
  const int32_t* rhs_idx;
  int n_experts = 0;
  int n_xrows = 0;
  // grouped decode (loader-wavefront kernel, direct variants): workgroup row
  // blockIdx.y takes segment y of `segments` ([0] = count, then (expert, first
  // sorted position, rows <= 16) triples): it multiplies the rows
  // x[src_row[first + r]] by w[expert] and stores row r at y[out_row[first + r]];
  // x has x_rows rows
  const int32_t* segments = nullptr;
  const int32_t* src_row = nullptr;
  const int32_t* out_row = nullptr;
  int x_rows = 0;
};

// Keeps a loop-invariant constant in a vector register: gfx950's three-operand
// VALU forms take no literals, so without this the and-or pairs are split.
__device__ __forceinline__ uint32_t pin_vgpr(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}

// 8 four-bit codes -> bf16 pairs (128+q_t, 128+q_{t+4}); mask / magic pinned.
__device__ __forceinline__ bf16x8 widen_int4(uint32_t w, uint32_t m, uint32_t magic) {
  return as_bf16x8((w & m) | magic, ((w >> 4) & m) | magic, ((w >> 8) & m) | magic,
                   ((w >> 12) & m) | magic);
}

// Raw buffer descriptor over [p, p + bytes): loads through it take a 32-bit
// lane offset plus a wavefront-uniform offset, and return zero past the end.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  const uint32_t n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}

constexpr uint32_t kOutOfRange = 0x80000000u;     // lane / uniform offset that always misses

// Every argument into scalar registers at the top of a kernel.  Left to
// itself the compiler loads an argument where it is first used, i.e. behind
// each early-exit branch in turn: three or four scalar-load round trips, one
// after the other, before the first useful instruction of a launch that lasts
// ten microseconds.  Naming them all here makes the loads go out together.
__device__ __forceinline__ void load_args_now(const GemvArgs& a) {
  asm volatile("" ::"s"(a.x), "s"(a.w), "s"(a.s), "s"(a.b), "s"(a.y), "s"(a.M), "s"(a.N), "s"(a.K),
               "s"(a.gshift), "s"(a.y_dtype), "s"(a.lhs_idx), "s"(a.rhs_idx), "s"(a.n_experts),
               "s"(a.n_xrows), "s"(a.segments), "s"(a.src_row), "s"(a.out_row), "s"(a.x_rows));
}

}  // namespace qmm
