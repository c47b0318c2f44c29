// Prefill-regime quantized matmul (M > 16) and the grouped (per-expert) form,
// for gfx950: packed weight tile -> dequantize in registers -> bf16 tile in
// LDS -> v_mfma_f32_32x32x16_bf16.
//
// y[m, n] = sum_k x[m, k] * w[n, k].  Both operands are K-contiguous, so both
// LDS tiles are [rows][BK] and an MFMA fragment is "row i, 8 consecutive k" for
// either operand.  The bf16 weight tile is a single round-to-nearest-even of
// the float32 value fma(scale, q, bias) (affine) or the exact E2M1*2^e product
// (mxfp4, which is exact in bf16).
//
// Tile: BM x BN x BK = 128 x 128 x 64, 256 threads = 2 x 2 wavefronts, each
// owning a 64 x 64 sub-tile (2 x 2 MFMA tiles, 64 accumulator registers).  LDS
// rows are 128 bytes; the 16-byte chunk index is XOR-ed with (row & 7) so that
// the fragment reads of 8 consecutive lanes fall in distinct banks.  Global
// loads for K-tile t+1 are issued before the MFMAs of K-tile t and written to
// the other LDS buffer afterwards (one barrier per K-tile).
//
// Grouped form: rows [row_offsets[e], row_offsets[e+1]) belong to expert e; a
// workgroup walks the offsets to find its (expert, row-tile), so no host
// synchronization is needed and tiles never straddle an expert boundary.
#include "qmm_common.hpp"

namespace qmm {

namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int kThreads = 256;
constexpr int kRowBytes = BK * 2;                 // 128
constexpr int kTileBytes = BM * kRowBytes;        // 16 KiB per operand per stage

struct GemmArgs {
  const uint16_t* x;     // bf16 [R, K]
  const uint32_t* w;     // [E, N, K*bits/32]
  const void* s;         // [E, N, K/gs]
  const void* b;
  void* y;               // [R, N]
  const int32_t* row_offsets;   // [E+1] or null (one group of R rows)
  const int32_t* lhs_idx;       // optional row gather for x (null = identity)
  const int32_t* out_idx;       // optional row scatter for y (null = identity)
  int R, N, K, E;
  int gs, tab, y_dtype;
  int m_tiles;           // grid.y upper bound on row tiles
};

__device__ __forceinline__ int swz(int row, int chunk) { return row * kRowBytes + ((chunk ^ (row & 7)) << 4); }

// 16 codes (int8: one u32x4; int4 / e2m1: one u32x2) -> 16 bf16 (two u32x4)
template <int MODE, int BITS>
__device__ __forceinline__ void dequant16(const uint32_t* q, float sc, float bi, u32x4& lo, u32x4& hi) {
  float f[16];
  if constexpr (MODE == 1) {
#pragma unroll
    for (int j = 0; j < 16; ++j) f[j] = e2m1_to_f32((q[j >> 3] >> (4 * (j & 7))) & 15u) * sc;
  } else if constexpr (BITS == 4) {
#pragma unroll
    for (int j = 0; j < 16; ++j) f[j] = fmaf(sc, (float)((q[j >> 3] >> (4 * (j & 7))) & 15u), bi);
  } else {
#pragma unroll
    for (int j = 0; j < 16; ++j) f[j] = fmaf(sc, (float)((q[j >> 2] >> (8 * (j & 3))) & 255u), bi);
  }
  lo = u32x4{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
  hi = u32x4{pack_bf16x2(f[8], f[9]), pack_bf16x2(f[10], f[11]), pack_bf16x2(f[12], f[13]), pack_bf16x2(f[14], f[15])};
}

template <int MODE, int BITS>
__global__ __launch_bounds__(kThreads) void gemm_kernel(GemmArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sA = smem;                       // 2 stages
  unsigned char* sB = smem + 2 * kTileBytes;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- which (expert, row tile) is this workgroup?
  int e = 0, row_lo = 0, row_hi = a.R, mt = blockIdx.y;
  if (a.row_offsets) {
    int t = blockIdx.y;
    bool found = false;
    for (int i = 0; i < a.E; ++i) {
      const int lo = a.row_offsets[i], hi = a.row_offsets[i + 1];
      const int tiles = (hi - lo + BM - 1) / BM;
      if (t < tiles) { e = i; row_lo = lo; row_hi = hi; mt = t; found = true; break; }
      t -= tiles;
    }
    if (!found) return;
  }
  const int m0 = row_lo + mt * BM;
  if (m0 >= row_hi) return;
  const int n0 = blockIdx.x * BN;

  constexpr int WBITS = (MODE == 1) ? 4 : BITS;
  const int64_t wpr = (int64_t)a.K * WBITS / 32;
  const int64_t ng = (MODE == 1) ? a.K / 32 : a.K / a.gs;
  const int gs = (MODE == 1) ? 32 : a.gs;
  const int tabsz = (MODE == 1) ? 1 : (a.tab == QMM_F32 ? 4 : 2);
  const uint32_t* wb = a.w + (int64_t)e * a.N * wpr;
  const char* sb = static_cast<const char*>(a.s) + (int64_t)e * a.N * ng * tabsz;
  const char* bb = (MODE == 1) ? nullptr : static_cast<const char*>(a.b) + (int64_t)e * a.N * ng * tabsz;

  // ---- global -> register staging
  // A: 128 rows x 8 chunks of 16 B; thread handles chunk (tid & 7) of rows (tid >> 3) + 32*i
  const uint16_t* aptr[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int row = m0 + (tid >> 3) + 32 * i;
    if (row >= row_hi) row = row_hi - 1;
    const int64_t src = a.lhs_idx ? (int64_t)a.lhs_idx[row] : (int64_t)row;
    aptr[i] = a.x + src * a.K + (tid & 7) * 8;
  }
  // W: 128 rows x 4 pieces of 16 codes; thread handles piece (tid & 3) of rows (tid >> 2) + 64*i
  constexpr int WPP = 16 * WBITS / 32;            // words per piece: 2 (4-bit) or 4 (8-bit)
  const uint32_t* wptr[2];
  int64_t trow[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    int row = n0 + (tid >> 2) + 64 * i;
    if (row >= a.N) row = a.N - 1;
    wptr[i] = wb + row * wpr + (tid & 3) * WPP;
    trow[i] = row * ng;
  }

  u32x4 ra[4];
  uint32_t rw[2][WPP];
  float rs[2], rb[2];

  // A K-tile past the end of K (K % 64 == 32) is fed as zeros on both sides.
  auto load_tile = [&](int kt) {
    const int k0 = kt * BK;
    const bool a_in = k0 + (tid & 7) * 8 < a.K;
    const bool w_in = k0 + (tid & 3) * 16 < a.K;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[i] = u32x4{0u, 0u, 0u, 0u};
      if (a_in) ra[i] = *reinterpret_cast<const u32x4*>(aptr[i] + k0);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (!w_in) {
#pragma unroll
        for (int j = 0; j < WPP; ++j) rw[i][j] = 0u;
        rs[i] = 0.f;
        rb[i] = 0.f;
        continue;
      }
      const uint32_t* p = wptr[i] + (int64_t)k0 * WBITS / 32;
      if constexpr (WPP == 4) {
        u32x4 v = *reinterpret_cast<const u32x4*>(p);
        rw[i][0] = v[0]; rw[i][1] = v[1]; rw[i][2] = v[2]; rw[i][3] = v[3];
      } else {
        u32x2 v = *reinterpret_cast<const u32x2*>(p);
        rw[i][0] = v[0]; rw[i][1] = v[1];
      }
      const int64_t ti = trow[i] + (k0 + (tid & 3) * 16) / gs;
      if constexpr (MODE == 1) {
        rs[i] = e8m0_to_f32(reinterpret_cast<const uint8_t*>(sb)[ti]);
        rb[i] = 0.f;
      } else {
        rs[i] = load_table_rt(sb, ti, a.tab);
        rb[i] = load_table_rt(bb, ti, a.tab);
      }
    }
  };

  auto store_tile = [&](int stage) {
    unsigned char* pa = sA + stage * kTileBytes;
    unsigned char* pb = sB + stage * kTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *reinterpret_cast<u32x4*>(pa + swz((tid >> 3) + 32 * i, tid & 7)) = ra[i];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      u32x4 lo, hi;
      dequant16<MODE, BITS>(rw[i], rs[i], rb[i], lo, hi);
      const int row = (tid >> 2) + 64 * i, c = (tid & 3) * 2;
      *reinterpret_cast<u32x4*>(pb + swz(row, c)) = lo;
      *reinterpret_cast<u32x4*>(pb + swz(row, c + 1)) = hi;
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int KT = (a.K + BK - 1) / BK;
  load_tile(0);
  store_tile(0);
  __syncthreads();

  const int fr = lane & 31, fk = lane >> 5;       // fragment row, k-half
  for (int kt = 0; kt < KT; ++kt) {
    const int stage = kt & 1;
    if (kt + 1 < KT) load_tile(kt + 1);
    const unsigned char* pa = sA + stage * kTileBytes;
    const unsigned char* pb = sB + stage * kTileBytes;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      bf16x8 fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[i] = *reinterpret_cast<const bf16x8*>(pa + swz(wm * 64 + i * 32 + fr, ks * 2 + fk));
        fb[i] = *reinterpret_cast<const bf16x8*>(pb + swz(wn * 64 + i * 32 + fr, ks * 2 + fk));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) store_tile(stage ^ 1);
    __syncthreads();
  }

  // ---- epilogue: D[i][j] of a 32x32 tile: lane holds column j = lane % 32 and
  // rows (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5), r = 0..15
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5);
        if (m < row_hi && n < a.N) {
          const int64_t orow = a.out_idx ? (int64_t)a.out_idx[m] : (int64_t)m;
          store_out(a.y, orow * a.N + n, acc[i][j][r], a.y_dtype);
        }
      }
    }
}

template <int MODE, int BITS>
void launch(const GemmArgs& a, hipStream_t st) {
  dim3 grid((unsigned)ceil_div(a.N, BN), (unsigned)a.m_tiles);
  const size_t lds = 4 * kTileBytes;
  hipLaunchKernelGGL((gemm_kernel<MODE, BITS>), grid, dim3(kThreads), lds, st, a);
}

}  // namespace

// Rows a grouped launch must provision: every expert may add one ragged tile.
int64_t gemm_row_tile() { return BM; }

// Host entry used by the C ABI (shapes validated by the caller: x bf16,
// K % 32 == 0, K % group_size == 0).
void gemm_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                   int y_dtype, const int32_t* row_offsets, const int32_t* lhs_idx,
                   const int32_t* out_idx, int64_t R, int64_t E, int64_t N, int64_t K, int gs,
                   int bits, int mode, hipStream_t st) {
  GemmArgs a;
  a.x = static_cast<const uint16_t*>(x);
  a.w = static_cast<const uint32_t*>(w);
  a.s = s;
  a.b = b;
  a.y = y;
  a.row_offsets = row_offsets;
  a.lhs_idx = lhs_idx;
  a.out_idx = out_idx;
  a.R = (int)R;
  a.N = (int)N;
  a.K = (int)K;
  a.E = (int)E;
  a.gs = gs;
  a.tab = tab;
  a.y_dtype = y_dtype;
  a.m_tiles = (int)(row_offsets ? ceil_div(R, BM) + E : ceil_div(R, BM));
  if (R == 0 || N == 0) return;
  if (mode == QMM_MODE_MXFP4) launch<1, 4>(a, st);
  else if (bits == 4) launch<0, 4>(a, st);
  else launch<0, 8>(a, st);
}

}  // namespace qmm
