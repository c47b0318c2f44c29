// Pieces shared by the prefill-regime kernels: tile constants, the LDS layout
// of a dequantized weight tile, the kernel arguments and the dequantization of
// one 16-byte piece.
#pragma once

#include "qmm_common.hpp"

namespace qmm {
namespace g2 {

constexpr int BN = 128, BK = 64;
constexpr int kRowBytes = BK * 2;                 // bf16 tile row
constexpr int kStage = BN * kRowBytes;            // 16 KB

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  const uint32_t n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}

__device__ __forceinline__ void lds_barrier() {   // orders LDS traffic only; global loads stay in flight
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// A bf16 tile row is 128 bytes = half of the 64 banks, so the parity of the
// row picks the half and 16-byte piece p of row r sits at p ^ ((r >> 1) & 7):
// the 16 lanes of one pass of a ds_read_b128 / ds_write_b128 (16 consecutive
// rows of one piece, or 8 rows x 2 halves of 4 pieces) then touch every bank
// once.  (With p ^ (r & 7) rows r and r + 8 shared their banks: every fragment
// read took two passes.)
__device__ __forceinline__ int swz(int row, int piece) {
  return row * kRowBytes + ((piece ^ ((row >> 1) & 7)) << 4);
}

// ---------------------------------------------------------------------------
struct Gemm2Args {
  const void* ax;        // re-laid activations
  const uint32_t* w;     // [E, N, K*bits/32]
  const void* s;         // [E, N, K/gs]
  const void* b;
  void* y;               // [R, N]
  const int32_t* row_offsets;   // [E+1] or null
  const int32_t* out_idx;       // optional row scatter for y
  int R, N, K, E, Rp;
  int gs, tab, y_dtype;
  int m_tiles;
  int tabfast;           // table rows are dword-aligned: fetch them as 16-byte windows
};

// How the tiles of a grouped product are dealt to the eight XCDs (workgroup
// b runs on XCD b % 8; l = b / 8 counts an XCD's workgroups).  A band of
// column tiles of every row tile per XCD keeps the row tiles of one expert
// and column on one L2 -- but with few column tiles the bands are uneven (11
// column tiles: five XCDs get two columns, one gets one, two get none), so
// when more than a sixteenth of the band slots would be empty the tiles go
// round the XCDs one by one instead, row tile after row tile.
__device__ __forceinline__ void deal_grouped_tile(int n_tiles, int xcd, int l, int& tile_m, int& tile_n) {
  const int band = (n_tiles + 7) / 8;
  if ((band * 8 - n_tiles) * 16 > n_tiles) {
    const int g = l * 8 + xcd;
    tile_m = g / n_tiles;
    tile_n = g % n_tiles;
  } else {
    tile_m = l / band;
    tile_n = xcd * band + l % band;       // may be past the last column tile: the caller checks
  }
}

// 32 codes (one row, one 32-group) -> four 16-byte pieces of bf16 weights
template <int MODE, int BITS>
__device__ __forceinline__ u32x4 dequant_piece(const uint32_t* q, int pc, float sc, float bi) {
  float f[8];
  if constexpr (MODE == 1) {
    // exact: the converter widens the two codes of a byte and applies the power-of-two scale
    const uint32_t w = q[pc];
    return u32x4{__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 0)),
                 __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 1)),
                 __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 2)),
                 __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 3))};
  } else if constexpr (BITS == 8) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint32_t w = q[2 * pc + h];
#pragma unroll
      for (int j = 0; j < 4; ++j) f[4 * h + j] = fmaf(sc, (float)((w >> (8 * j)) & 255u), bi);
    }
  } else {
    const uint32_t w = q[pc];
    uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;           // even / odd codes as bytes
    // kept opaque, so that each code is one byte-to-float conversion of lo / hi
    // (merged with the masks above they become a bit-field extract plus a conversion)
    asm("" : "+v"(lo));
    asm("" : "+v"(hi));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = fmaf(sc, (float)((lo >> (8 * j)) & 255u), bi);
      f[2 * j + 1] = fmaf(sc, (float)((hi >> (8 * j)) & 255u), bi);
    }
  }
  return u32x4{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
               pack_bf16x2(f[6], f[7])};
}

}  // namespace g2
}  // namespace qmm
