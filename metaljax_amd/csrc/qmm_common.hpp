// Device-side helpers shared by the gfx950 quantized-matmul kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "../../include/qmm_hip.h"

namespace qmm {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;

constexpr int kWave = 64;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) {
  return __uint_as_float(b << 16);
}

// float32 -> bf16 bits, round to nearest even (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  bf16x2 t;
  t[0] = (__bf16)f;
  t[1] = (__bf16)0.0f;
  return __builtin_bit_cast(uint32_t, t) & 0xFFFFu;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2 t;
  t[0] = (__bf16)lo;
  t[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, t);
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return (uint32_t)__builtin_bit_cast(uint16_t, h);
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}

// One scale / bias table entry as float32 (exact widening).
template <int TAB>
__device__ __forceinline__ float load_table(const void* p, int64_t i) {
  if constexpr (TAB == QMM_F32) {
    return static_cast<const float*>(p)[i];
  } else if constexpr (TAB == QMM_BF16) {
    return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  } else {
    return f16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
  }
}

__device__ __forceinline__ float load_table_rt(const void* p, int64_t i, int tab) {
  if (tab == QMM_F32) return load_table<QMM_F32>(p, i);
  if (tab == QMM_BF16) return load_table<QMM_BF16>(p, i);
  return load_table<QMM_F16>(p, i);
}

__device__ __forceinline__ void store_out(void* y, int64_t i, float v, int yd) {
  if (yd == QMM_BF16) {
    static_cast<uint16_t*>(y)[i] = (uint16_t)f32_to_bf16_bits(v);
  } else if (yd == QMM_F32) {
    static_cast<float*>(y)[i] = v;
  } else {
    static_cast<uint16_t*>(y)[i] = (uint16_t)f32_to_f16_bits(v);
  }
}

// E8M0 byte -> 2^(e-127) as float32.  Byte 0 is the subnormal 2^-127 and byte
// 255 is NaN, as in the OCP MX specification.
__device__ __forceinline__ float e8m0_to_f32(uint32_t e) {
  uint32_t bits = e << 23;
  if (e == 0u) bits = 0x00400000u;
  if (e == 255u) bits = 0x7FC00000u;
  return __uint_as_float(bits);
}

// E2M1 code (4 bits, bit 3 = sign) -> float32, exact.
__device__ __forceinline__ float e2m1_to_f32(uint32_t c) {
  // magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6 as bf16 high bytes+: build f32 bits
  const uint32_t m = c & 7u;
  // normal (m >= 2): exponent (m>>1) with bias 1, mantissa bit (m&1);
  // m == 1 is the subnormal 0.5; m == 0 is zero.
  uint32_t bits;
  if (m >= 2u) bits = ((126u + (m >> 1)) << 23) | ((m & 1u) << 22);
  else bits = m ? 0x3F000000u : 0u;
  return __uint_as_float(bits | ((c & 8u) << 28));
}

// v_perm_b32: bytes 0-3 of the selector index come from `lo`, 4-7 from `hi`.
__device__ __forceinline__ uint32_t byte_perm(uint32_t hi, uint32_t lo, uint32_t sel) {
  return __builtin_amdgcn_perm(hi, lo, sel);
}

__host__ __device__ constexpr int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- the row tiles of a grouped product --------------------------------------
// Rows [offsets[e], offsets[e+1]) belong to expert e and are cut into tiles of
// `tile_rows` that never straddle two experts.  Which expert and which of its
// tiles is row tile `tile_m` of the whole product?  The wavefront looks at 64
// experts at a time, one a lane (two coalesced loads, a prefix sum over the
// lanes and a ballot), so that the search costs a few memory round trips
// whatever the number of experts -- walked one expert after the other it cost
// one round trip an expert in every workgroup's prologue.  Offsets are forced
// into [0, R] and non-decreasing whatever the array holds.  Every lane of the
// wavefront must be active; the results are the same in all of them.
struct RowTile {
  int e, lo, hi, idx;    // expert, its rows [lo, hi), the tile's number inside the expert
  int m_tiles;           // row tiles of the whole product
  bool found;            // false: tile_m is past the last tile
};

__device__ __forceinline__ RowTile find_row_tile(const int32_t* offsets, int E, int R, int tile_rows, int tile_m) {
  RowTile r{0, 0, 0, 0, 0, false};
  const int lane = (int)(threadIdx.x & 63);
  int base = 0;
  for (int e0 = 0; e0 < E; e0 += 64) {
    const int i = e0 + lane;
    int lo = 0, hi = 0;
    if (i < E) {
      lo = offsets[i];
      hi = offsets[i + 1];
      lo = lo < 0 ? 0 : (lo > R ? R : lo);
      hi = hi < lo ? lo : (hi > R ? R : hi);
    }
    const int tiles = (hi - lo + tile_rows - 1) / tile_rows;
    int incl = tiles;                               // tiles of experts e0 .. e0 + lane
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int v = __shfl_up(incl, d, 64);
      if (lane >= d) incl += v;
    }
    const int total = __shfl(incl, 63, 64);
    if (!r.found && tile_m >= base && tile_m < base + total) {
      const unsigned long long past = __ballot(base + incl > tile_m);    // lanes at or after the tile's expert
      const int L = __ffsll((long long)past) - 1;
      r.e = e0 + L;
      r.lo = __shfl(lo, L, 64);
      r.hi = __shfl(hi, L, 64);
      r.idx = tile_m - base - __shfl(incl - tiles, L, 64);
      r.found = true;
    }
    base += total;
  }
  r.e = __builtin_amdgcn_readfirstlane(r.e);
  r.lo = __builtin_amdgcn_readfirstlane(r.lo);
  r.hi = __builtin_amdgcn_readfirstlane(r.hi);
  r.idx = __builtin_amdgcn_readfirstlane(r.idx);
  r.m_tiles = __builtin_amdgcn_readfirstlane(base);
  return r;
}

// ---- host-side helpers ------------------------------------------------------

// Experiment switches (kernel overrides used while measuring).  The shipped
// library reads no environment: they exist only in a build with
// -DQMM_EXPERIMENTS.
inline const char* experiment_env(const char* name) {
#ifdef QMM_EXPERIMENTS
  return getenv(name);
#else
  (void)name;
  return nullptr;
#endif
}

// The status of the last failed launch set-up on this thread (hipSuccess when
// none); the C ABI turns it into QMM_ERR_HIP and clears it.
inline hipError_t& setup_error() {
  static thread_local hipError_t e = hipSuccess;
  return e;
}

// Raises kernel KERN's dynamic-LDS limit.  The HIP call is made once per
// process (the initialisation of a function-local static is thread-safe) and
// its status is kept: every later call reports the same status, so a launch
// behind a failed set-up is never attempted.  Returns true when the limit is set.
template <auto KERN>
inline bool lds_limit(size_t bytes) {
  static const size_t set_bytes = bytes;
  static const hipError_t rc = hipFuncSetAttribute(
      reinterpret_cast<const void*>(KERN), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  hipError_t r = rc;
  if (r == hipSuccess && bytes > set_bytes)      // a later call asking for more than the first did
    r = hipFuncSetAttribute(reinterpret_cast<const void*>(KERN),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (r != hipSuccess) setup_error() = r;
  return r == hipSuccess;
}

}  // namespace qmm
