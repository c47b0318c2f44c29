// Prefill-regime quantized matmul (M > 16) and the grouped (per-expert) form,
// for gfx950: packed weight tile -> dequantize in registers -> bf16 tile in
// LDS -> v_mfma_f32_32x32x16_bf16.
//
// y[m, n] = sum_k x[m, k] * w[n, k].  Both operands are K-contiguous, so both
// LDS tiles are [rows][BK = 64 bf16 = 128 bytes] and an MFMA fragment is "row
// i, 8 consecutive k" for either operand.  The bf16 weight tile is a single
// round-to-nearest-even of the float32 value fma(scale, q, bias) (affine) or
// the exact E2M1 * 2^e product (mxfp4, exact in bf16).
//
// Tile BM x 128 x 64 (BM = 256 or 128), 256 threads = 2 x 2 wavefronts, each
// owning (BM/2) x 64 of the output: (BM/64) x 2 MFMA tiles of 32 x 32, so a
// k-step of 16 reads BM/64 + 2 fragments for 2*BM/64 MFMAs.
//
// Activation tile: fetched straight into LDS (buffer_load ... lds, 16 bytes a
// lane, no registers, no vector ALU work): per K-tile the lane offsets are
// loop-invariant and only a scalar offset advances.  Weight tile: each thread
// loads 32 codes of one row, dequantizes them and writes four 16-byte pieces.
// Both tiles use the same bank swizzle: the 16-byte piece p of row r lives at
// piece p ^ (r & 7); for the direct-to-LDS tile the swizzle is applied to the
// global address instead (lane l of a load owns LDS slot l), which keeps every
// group of four lanes inside one aligned 64-byte run.
//
// Three LDS stages.  While the MFMAs of K-tile t run, the DMA and the packed
// weight words of tile t+2 are in flight and the words of tile t+1 (fetched an
// iteration earlier) are dequantized into their stage, so every load has at
// least one full MFMA phase to land.  One workgroup barrier per K-tile.
//
// Grouped form: rows [row_offsets[e], row_offsets[e+1]) belong to expert e; a
// workgroup walks the offsets to find its (expert, row-tile), so no host
// synchronization is needed and tiles never straddle an expert boundary.
#include <type_traits>

#include "qmm_common.hpp"

namespace qmm {

namespace {

constexpr int BN = 128, BK = 64;
constexpr int kThreads = 256;
constexpr int kRowBytes = BK * 2;                 // 128

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
  int x_rows;            // rows of x (== R unless lhs_idx gathers from a larger array)
  int gs, tab, y_dtype;
  int m_tiles;           // grid.y upper bound on row tiles
};

__device__ __forceinline__ int swz(int row, int piece) { return row * kRowBytes + ((piece ^ (row & 7)) << 4); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  const uint32_t n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}
constexpr uint32_t kOutOfRange = 0x80000000u;

// Workgroup barrier that orders LDS traffic only: global loads (and the
// direct-to-LDS DMA, which is tracked by vmcnt) stay in flight across it.
// (A fence would also wait for the DMA, since that writes LDS; its completion
// is awaited explicitly with wait_vmcnt where a stage is about to be published.)
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {    // s_waitcnt vmcnt(N) only
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
}

// 8 codes of one word -> 8 float32 weights fma(sc, q, bi) / E2M1 * sc
template <int MODE, int BITS>
__device__ __forceinline__ void dequant_word8(uint32_t w, float sc, float bi, float* f) {
  if constexpr (MODE == 1) {
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = e2m1_to_f32((w >> (4 * j)) & 15u) * sc;
  } else {
    static_assert(BITS == 4, "8-bit words hold four codes");
    const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;   // even / odd codes as bytes
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = fmaf(sc, (float)((lo >> (8 * j)) & 255u), bi);
      f[2 * j + 1] = fmaf(sc, (float)((hi >> (8 * j)) & 255u), bi);
    }
  }
}

__device__ __forceinline__ void dequant_word4_i8(uint32_t w, float sc, float bi, float* f) {
#pragma unroll
  for (int j = 0; j < 4; ++j) f[j] = fmaf(sc, (float)((w >> (8 * j)) & 255u), bi);
}

template <int MODE, int BITS, int BM>
__global__ __launch_bounds__(kThreads) void gemm_kernel(GemmArgs a) {
  constexpr int kATile = BM * kRowBytes;           // bytes per stage
  constexpr int kBTile = BN * kRowBytes;
  constexpr int WM = BM / 2;                       // rows per wavefront
  constexpr int MT = WM / 32;                      // MFMA row tiles per wavefront
  constexpr int WBITS = (MODE == 1) ? 4 : BITS;
  constexpr int WPT = 32 * WBITS / 32;             // packed words per thread per K-tile: 4 | 8
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sA = smem;                        // 3 stages
  unsigned char* sB = smem + 3 * kATile;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // ---- which tile is this workgroup?  Workgroups are dealt to the 8 XCDs
  // round-robin in launch order, so XCD x is handed the contiguous run of
  // tiles [x * per, (x+1) * per) in column-fastest order: the workgroups that
  // share one L2 then walk a few activation row-tiles across all weight
  // columns, and each activation K-slice is fetched from beyond L2 once.
  const int n_tiles = (a.N + BN - 1) / BN;
  const int total = n_tiles * a.m_tiles;
  const int per = (total + 7) / 8;
  const int tile = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if (tile >= total) return;
  const int tile_n = tile % n_tiles, tile_m = tile / n_tiles;

  // ---- which (expert, row tile)?
  int e = 0, row_lo = 0, row_hi = a.R, mt = tile_m;
  if (a.row_offsets) {
    const RowTile rt = find_row_tile(a.row_offsets, a.E, a.R, BM, tile_m);
    if (!rt.found) return;
    e = rt.e; row_lo = rt.lo; row_hi = rt.hi; mt = rt.idx;
  }
  const int m0 = row_lo + mt * BM;
  if (m0 >= row_hi) return;
  const int n0 = tile_n * BN;

  const int64_t wpr = (int64_t)a.K * WBITS / 32;   // words per weight row
  const int64_t ng = (MODE == 1) ? a.K / 32 : a.K / a.gs;
  const int gs = (MODE == 1) ? 32 : a.gs;
  const int tabsz = (MODE == 1) ? 1 : (a.tab == QMM_F32 ? 4 : 2);
  const uint32_t* wb = a.w + (int64_t)e * a.N * wpr;
  const char* sb = static_cast<const char*>(a.s) + (int64_t)e * a.N * ng * tabsz;
  const char* bb = (MODE == 1) ? nullptr : static_cast<const char*>(a.b) + (int64_t)e * a.N * ng * tabsz;

  // ---- activation DMA: wavefront w fills rows [w*BM/4, (w+1)*BM/4) of the
  // stage, 8 rows an instruction; lane l owns slot l = (row l/8, piece l%8)
  // and fetches global piece (l%8) ^ (row & 7) of that row.
  constexpr int AI = BM / 32;                      // DMA instructions per wavefront per K-tile
  const auto rx = make_rsrc(a.x, (int64_t)a.x_rows * a.K * 2);
  uint32_t avo[AI];
#pragma unroll
  for (int j = 0; j < AI; ++j) {
    const int rl = lane >> 3;                      // (wave*BM/4 + j*8 + rl) & 7 == rl
    const int row = m0 + wave * (BM / 4) + j * 8 + rl;
    avo[j] = kOutOfRange;
    if (row < row_hi) {
      const int64_t src = a.lhs_idx ? (int64_t)a.lhs_idx[row] : (int64_t)row;
      avo[j] = (uint32_t)(src * a.K * 2 + (((lane & 7) ^ rl) << 4));
    }
  }
  // A row whose 64-element K-tile runs past K (K % 64 == 32) reads zeros for
  // the missing half through the descriptor only if it is the last row; mask
  // instead: pieces 4..7 of such a tile are fetched out of range.
  auto dma_a = [&](int kt, int stage) {
    const int k0 = kt * BK;
    const bool half = k0 + 32 == a.K;                      // uniform: only 32 valid elements
#pragma unroll
    for (int j = 0; j < AI; ++j) {
      uint32_t vo = avo[j];
      if (half && (((lane & 7) ^ (lane >> 3)) >= 4)) vo = kOutOfRange;
      unsigned char* dst = sA + stage * kATile + (wave * (BM / 4) + j * 8) * kRowBytes;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (__attribute__((address_space(3))) void*)dst, 16, vo,
                                               (uint32_t)k0 * 2, 0, 0);
    }
  };

  // ---- weight staging: thread -> (row tid/2, half tid%2): 32 codes a K-tile
  const int wrow = tid >> 1, whalf = tid & 1;
  int64_t wn_row = n0 + wrow;
  if (wn_row >= a.N) wn_row = a.N - 1;
  const uint32_t* wptr = wb + wn_row * wpr + whalf * WPT;
  const int64_t trow = wn_row * ng;
  struct WRegs { uint32_t q[WPT]; float s, b; };
  auto load_w = [&](int kt, WRegs& r) {
    const int k0 = kt * BK;
    if (k0 + whalf * 32 >= a.K) {                  // past the end of K: zeros
#pragma unroll
      for (int j = 0; j < WPT; ++j) r.q[j] = 0u;
      r.s = 0.f;
      r.b = 0.f;
      return;
    }
    const uint32_t* p = wptr + (int64_t)k0 * WBITS / 32;
#pragma unroll
    for (int j = 0; j < WPT; j += 4) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(p + j);
      r.q[j] = v[0]; r.q[j + 1] = v[1]; r.q[j + 2] = v[2]; r.q[j + 3] = v[3];
    }
    const int64_t ti = trow + (k0 + whalf * 32) / gs;
    if constexpr (MODE == 1) {
      r.s = e8m0_to_f32(reinterpret_cast<const uint8_t*>(sb)[ti]);
      r.b = 0.f;
    } else {
      r.s = load_table_rt(sb, ti, a.tab);
      r.b = load_table_rt(bb, ti, a.tab);
    }
  };
  auto store_w = [&](int stage, const WRegs& r) {
    unsigned char* pb = sB + stage * kBTile;
#pragma unroll
    for (int pc = 0; pc < 4; ++pc) {               // four pieces of 8 weights
      float f[8];
      if constexpr (MODE == 0 && BITS == 8) {
        dequant_word4_i8(r.q[2 * pc], r.s, r.b, f);
        dequant_word4_i8(r.q[2 * pc + 1], r.s, r.b, f + 4);
      } else {
        dequant_word8<MODE, BITS>(r.q[pc], r.s, r.b, f);
      }
      const u32x4 v = {pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                       pack_bf16x2(f[6], f[7])};
      *reinterpret_cast<u32x4*>(pb + swz(wrow, whalf * 4 + pc)) = v;
    }
  };

  f32x16 acc[MT][2];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Loads per K-tile that count against vmcnt: AI DMA instructions, then the
  // packed words (WPT/4 instructions) and two table entries (one for mxfp4).
  constexpr int kLoadsPerTile = AI + WPT / 4 + (MODE == 1 ? 1 : 2);
  const int KT = (a.K + BK - 1) / BK;
  const int fr = lane & 31, fk = lane >> 5;        // fragment row, k-half

  // Schedule.  Iteration t multiplies K-tile t from stage t % 3.  Its loads:
  // the packed words of tile t+2 first, then the DMA of tile t+2 into stage
  // (t+2) % 3.  The words of tile t+1 (issued in iteration t-1) are waited for
  // at the top of iteration t and dequantized into stage (t+1) % 3 in the
  // shadow of the MFMAs; the DMA of tile t+1 (issued in iteration t-1) is
  // waited for just before the barrier that ends iteration t.  Barriers fence
  // LDS only, so global loads stay in flight across them.
  WRegs w_cur, w_nxt;      // words of tile t+1 (ready / arriving), of tile t+2 (just issued)
  load_w(0, w_cur);
  dma_a(0, 0);
  if (KT > 1) {
    load_w(1, w_nxt);
    dma_a(1, 1);
    wait_vmcnt<kLoadsPerTile>();               // tile 0 landed
  } else {
    wait_vmcnt<0>();
  }
  store_w(0, w_cur);
  w_cur = w_nxt;
  lds_barrier();

  auto iteration = [&](int kt, auto has1_t, auto has2_t) {
    constexpr bool HAS1 = decltype(has1_t)::value, HAS2 = decltype(has2_t)::value;
    const int stage = kt % 3;
    // words of tile kt+1 must be here; its DMA (AI loads, issued after) may still fly
    if constexpr (HAS1) wait_vmcnt<AI>();
    if constexpr (HAS2) {
      load_w(kt + 2, w_nxt);
      dma_a(kt + 2, (kt + 2) % 3);
    }
    const unsigned char* pa = sA + stage * kATile;
    const unsigned char* pb = sB + stage * kBTile;
    bf16x8 fa[2][MT], fb[2][2];
    auto load_frags = [&](int ks, int set) {
#pragma unroll
      for (int i = 0; i < MT; ++i)
        fa[set][i] = *reinterpret_cast<const bf16x8*>(pa + swz(wm * WM + i * 32 + fr, ks * 2 + fk));
#pragma unroll
      for (int j = 0; j < 2; ++j)
        fb[set][j] = *reinterpret_cast<const bf16x8*>(pb + swz(wn * 64 + j * 32 + fr, ks * 2 + fk));
    };
    load_frags(0, 0);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      if (ks + 1 < BK / 16) load_frags(ks + 1, (ks + 1) & 1);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks & 1][i], fb[ks & 1][j], acc[i][j], 0, 0, 0);
    }
    if constexpr (HAS1) {
      store_w((kt + 1) % 3, w_cur);
      // the DMA of tile kt+1 must have landed before the barrier publishes its stage
      if constexpr (HAS2) wait_vmcnt<kLoadsPerTile>(); else wait_vmcnt<0>();
    }
    if constexpr (HAS2) w_cur = w_nxt;
    lds_barrier();
  };
  int kt = 0;
  for (; kt + 2 < KT; ++kt) iteration(kt, std::true_type{}, std::true_type{});
  if (kt + 1 < KT) { iteration(kt, std::true_type{}, std::false_type{}); ++kt; }
  if (kt < KT) iteration(kt, std::false_type{}, std::false_type{});

  // ---- epilogue: D[i][j] of a 32x32 tile: lane holds column j = lane % 32 and
  // rows (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5), r = 0..15
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * WM + i * 32 + (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5);
        if (m < row_hi && n < a.N) {
          const int64_t orow = a.out_idx ? (int64_t)a.out_idx[m] : (int64_t)m;
          store_out(a.y, orow * a.N + n, acc[i][j][r], a.y_dtype);
        }
      }
    }
}

template <int MODE, int BITS, int BM>
void launch(const GemmArgs& a0, hipStream_t st) {
  GemmArgs a = a0;
  a.m_tiles = (int)(a.row_offsets ? ceil_div(a.R, BM) + a.E : ceil_div(a.R, BM));
  const int64_t total = ceil_div(a.N, BN) * a.m_tiles;
  dim3 grid((unsigned)(ceil_div(total, 8) * 8));
  const size_t lds = 3 * (size_t)(BM + BN) * kRowBytes;
  constexpr auto kern = gemm_kernel<MODE, BITS, BM>;
  if (!lds_limit<kern>(lds)) return;
  hipLaunchKernelGGL(kern, grid, dim3(kThreads), lds, st, a);
}

template <int MODE, int BITS>
void launch_bm(const GemmArgs& a, int bm, hipStream_t st) {
  if (bm == 256) launch<MODE, BITS, 256>(a, st);
  else launch<MODE, BITS, 128>(a, st);
}

int env_int(const char* name) {
  const char* e = experiment_env(name);
  return e ? atoi(e) : 0;
}

}  // namespace

// Row tile of the launch that gemm_dispatch would choose (grouped launches
// provision one ragged tile per expert on top of ceil(R / tile)).
int64_t gemm_row_tile(int64_t R, int64_t E) {
  static const int env_bm = env_int("QMM_GEMM_BM");
  if (env_bm) return env_bm;
  // Grouped rows are ragged around R / E: once the mean nears 128 many experts
  // spill into a second 128-row tile that is almost empty, while a 256-row
  // tile takes each of them in one (and runs its short main loop for the
  // experts that fill at most half of it).
  const int64_t per_group = E > 0 ? R / E : R;
  if (E > 1) return per_group > 96 ? 256 : 128;
  return per_group >= 512 ? 256 : 128;
}

// Host entry used by the C ABI (shapes validated by the caller: x bf16,
// K % 32 == 0, K % group_size == 0).
void gemm_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                   int y_dtype, const int32_t* row_offsets, const int32_t* lhs_idx,
                   const int32_t* out_idx, int64_t R, int64_t x_rows, int64_t E, int64_t N,
                   int64_t K, int gs, int bits, int mode, hipStream_t st) {
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
  a.x_rows = (int)x_rows;
  a.gs = gs;
  a.tab = tab;
  a.y_dtype = y_dtype;
  a.m_tiles = 0;
  if (R == 0 || N == 0) return;
  const int bm = (int)gemm_row_tile(R, row_offsets ? E : 1);
  if (mode == QMM_MODE_MXFP4) launch_bm<1, 4>(a, bm, st);
  else if (bits == 4) launch_bm<0, 4>(a, bm, st);
  else launch_bm<0, 8>(a, bm, st);
}

}  // namespace qmm
