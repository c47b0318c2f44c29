// Decode-regime affine quantized matmul (M <= 16), LDS-staged: the fast path
// for the common layouts (group size 64 or 128, bf16 tables, K a multiple of
// the K-slice).
//
// Why staging.  The matrix-core operand layout wants lane l to hold weight row
// l % 16, so loading operands directly makes adjacent lanes touch rows that
// are a whole row pitch apart: every lane becomes its own L1 request and the
// kernel is bound by L1 tag lookups, not by HBM.  Here each wavefront instead
// loads its [16 rows x 256 packed bytes] tile with fully coalesced 16-byte
// lane loads (16 consecutive lanes = one row's 256 bytes), parks it in a
// wave-private LDS buffer, and reads it back in operand order.  The packed
// codes (not widened values) go through LDS, so LDS traffic is 2x the weight
// bytes and costs no vector ALU work.
//
// Work split.  A workgroup owns TILES*16 weight rows; wavefront w owns K-slice
// w, w+WAVES, ... (a slice is 256 packed bytes per row: 512 four-bit or 256
// eight-bit codes).  Per slice the activations are staged once (coalesced
// load -> LDS -> operand registers) and stay in registers for every tile.
//
// Arithmetic per 64-code chunk c and tile:
//     d_c      = sum_k x*q'          two v_mfma_f32_16x16x32_bf16 (exact products)
//     acc     += scale_c * d_c       four fused multiply-adds per lane
// where q' = q (8-bit) or 128+q (4-bit, one and-or per pair of codes).  The
// terms that do not involve the codes,
//     sum_c (bias_c - 128*scale_c) * xs_c,      xs_c = sum_k x  over chunk c,
// are themselves small matrix products over the chunk index and run on the
// matrix cores too: xs_c comes out of an MFMA against an all-ones operand
// already in operand layout, is split into three bf16 terms (24 significant
// bits), and multiplies the bias / scale table rows, which are bf16 and thus
// exact operands.
#include "qmm_gemv_common.hpp"

namespace qmm {

namespace {

constexpr int kSliceBytes = 256;            // packed bytes per row per K-slice
constexpr int kRowStride = 272;             // LDS row pitch (16-byte pad)
constexpr int kTileLds = 16 * kRowStride;   // wave-private staging buffer (codes / activations)
constexpr int kTabLds = 2 * 16 * 16;        // wave-private table rows: 16 scale rows, 16 bias rows

__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// float -> (hi, mid, lo) bf16 terms with hi + mid + lo == v to 24 bits.
__device__ __forceinline__ void split3(float v, float& hi, float& mid, float& lo) {
  hi = __uint_as_float(__float_as_uint(v) & 0xFFFF0000u);
  const float r1 = v - hi;
  mid = __uint_as_float(__float_as_uint(r1) & 0xFFFF0000u);
  lo = r1 - mid;                              // at most 8 significant bits: exact in bf16
}

__device__ __forceinline__ uint32_t hi16_pair(float a, float b) {      // (bf16(a), bf16(b)), truncating
  return byte_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}

// One tile's weight loads: instruction i covers rows 4i .. 4i+3 of the tile,
// 16 consecutive lanes one row's 256 bytes.  Rows at or past n_end read out of
// range (zeros, no memory traffic).
__device__ __forceinline__ void load_tile(u32x4 (&w)[4], __amdgpu_buffer_rsrc_t rw, int64_t row0,
                                          int64_t n_end, int64_t wpr, int lrow, int lpiece,
                                          uint32_t slice_off) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t n = row0 + 4 * i + lrow;
    const uint32_t vo = n < n_end ? (uint32_t)(n * wpr + lpiece * 16) : kOutOfRange;
    w[i] = __builtin_amdgcn_raw_buffer_load_b128(rw, vo, slice_off, 0);
  }
}

template <int BITS, int WAVES, int TMAX, int GSHIFT>
__global__ __launch_bounds__(kWave* WAVES) void skinny_affine_kernel(GemvArgs a, int rows_per_wg) {
  load_args_now(a);
  constexpr int KS = kSliceBytes * 8 / BITS;      // codes per slice: 512 | 256
  constexpr int CPS = KS / 64;                    // 64-code chunks per slice: 8 | 4
  constexpr int XR = KS / 128;                    // activation staging rounds (128 codes each)
  __shared__ __align__(16) unsigned char stage[WAVES][kTileLds + kTabLds];
  __shared__ float red[WAVES][TMAX][4][kWave];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, kg = lane >> 4;
  const int64_t bz = blockIdx.y;
  const int64_t n_begin = (int64_t)blockIdx.x * rows_per_wg;
  const int64_t n_end = n_begin + rows_per_wg < a.N ? n_begin + rows_per_wg : a.N;
  const int ntiles = (int)((n_end - n_begin + 15) / 16);        // uniform, <= TMAX
  const int64_t wpr = (int64_t)a.K * BITS / 8;                  // bytes per weight row
  const int64_t ng = (int64_t)(a.K / 64) >> GSHIFT;             // table entries per row
  const int slices = a.K / KS;

  int64_t xz = a.lhs_idx ? (int64_t)a.lhs_idx[bz] : bz;
  const int64_t wz = a.rhs_idx ? (int64_t)a.rhs_idx[bz] : bz;
  bool x_ok = true;
  if (a.rhs_idx) {                                  // gather form: indices are data
    if (wz < 0 || wz >= a.n_experts) return;        // uniform, before any barrier
    if (xz < 0 || xz >= a.n_xrows) { xz = 0; x_ok = false; }
  }
  const auto rx = make_rsrc(a.x + xz * a.M * (int64_t)a.K, x_ok ? (int64_t)a.M * a.K * 2 : 0);
  const auto rw = make_rsrc(reinterpret_cast<const char*>(a.w) + wz * a.N * wpr, a.N * wpr);
  const auto rs = make_rsrc(static_cast<const char*>(a.s) + wz * a.N * ng * 2, a.N * ng * 2);
  const auto rb = make_rsrc(static_cast<const char*>(a.b) + wz * a.N * ng * 2, a.N * ng * 2);

  unsigned char* buf = stage[wave];
  unsigned char* tbuf = buf + kTileLds;
  const int lrow = lane >> 4, lpiece = lane & 15;               // coalesced-load coordinates
  const uint32_t st_off = (uint32_t)(lrow * kRowStride + lpiece * 16);   // + i*4*kRowStride

  f32x4 acc[TMAX];
#pragma unroll
  for (int t = 0; t < TMAX; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  const uint32_t one = pin_vgpr(kOnesBf16x2);
  const bf16x8 ones = as_bf16x8(one, one, one, one);
  const uint32_t nib = pin_vgpr(0x000F000Fu), magic = pin_vgpr(0x43004300u);

  for (int sl = wave; sl < slices; sl += WAVES) {
    const uint32_t slice_off = (uint32_t)sl * kSliceBytes;
    const uint32_t tab_off = (uint32_t)((sl * CPS) >> GSHIFT) * 2;
    // ---- issue the global loads: the first tile (HBM, longest latency), the
    // activations (row blocks at or past M are not fetched), then the second tile
    u32x4 wl[TMAX][4], tvs[TMAX], tvb[TMAX];
    // Table rows: lanes 0-15 fetch the 16 scale rows of a tile, lanes 16-31 the
    // bias rows (one 16-byte run each); they reach every lane through LDS.
    auto load_tables = [&](int t, int set) {
      const int64_t n = n_begin + t * 16 + r;
      const uint32_t to = (uint32_t)(n * ng * 2);
      // (the two are merged where the tile is consumed, so that nothing waits here)
      tvs[set] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane < 16 && n < n_end ? to : kOutOfRange, tab_off, 0);
      tvb[set] = __builtin_amdgcn_raw_buffer_load_b128(rb, (lane & 48) == 16 && n < n_end ? to : kOutOfRange, tab_off, 0);
    };
    load_tile(wl[0], rw, n_begin, n_end, wpr, lrow, lpiece, slice_off);
    u32x4 xl[XR][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool any = 4 * i < a.M;                              // uniform
#pragma unroll
      for (int rd = 0; rd < XR; ++rd) {
        xl[rd][i] = u32x4{0u, 0u, 0u, 0u};
        if (any) {
          const int m = 4 * i + lrow;
          const uint32_t vo = m < a.M ? (uint32_t)(((int64_t)m * a.K) * 2 + lpiece * 16) : kOutOfRange;
          xl[rd][i] = __builtin_amdgcn_raw_buffer_load_b128(rx, vo, (uint32_t)(sl * KS + rd * 128) * 2, 0);
        }
      }
    }
    load_tables(0, 0);
    // every other tile of the slice: all of this wavefront's weight bytes are in
    // flight before the first one is consumed (tiles past the range read nothing)
#pragma unroll
    for (int t = 1; t < TMAX; ++t) {
      load_tile(wl[t], rw, n_begin + t * 16, n_end, wpr, lrow, lpiece, slice_off);
      load_tables(t, t);
    }

    // ---- activations: LDS round trip into operand layout, 128 codes a round
    bf16x8 xa[CPS][2];
#pragma unroll
    for (int rd = 0; rd < XR; ++rd) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<u32x4*>(buf + st_off + i * 4 * kRowStride) = xl[rd][i];
      wave_lds_fence();
#pragma unroll
      for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(buf + r * kRowStride + cc * 128 + kg * 32 + j * 16);
          if constexpr (BITS == 4) xa[rd * 2 + cc][j] = pair_stride4(v);
          else xa[rd * 2 + cc][j] = __builtin_bit_cast(bf16x8, v);
        }
      wave_lds_fence();
    }
    // xs_c for every chunk, in operand layout (lane l holds row l % 16), then
    // the three-term bf16 split packed as MFMA A operands over the chunk index.
    // Only the kg == 0 lanes carry them (the other k slots are zero).
    bf16x8 axh, axm, axo;
    {
      float xs[8], xh[8], xm[8], xo[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        xs[c] = 0.f;
        if (c < CPS) {
          f32x4 t4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xa[c][0], zero, 0, 0, 0);
          t4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xa[c][1], t4, 0, 0, 0);
          xs[c] = kg == 0 ? t4[0] : 0.f;
        }
        split3(xs[c], xh[c], xm[c], xo[c]);
      }
      axh = as_bf16x8(hi16_pair(xh[0], xh[1]), hi16_pair(xh[2], xh[3]), hi16_pair(xh[4], xh[5]), hi16_pair(xh[6], xh[7]));
      axm = as_bf16x8(hi16_pair(xm[0], xm[1]), hi16_pair(xm[2], xm[3]), hi16_pair(xm[4], xm[5]), hi16_pair(xm[6], xm[7]));
      axo = as_bf16x8(hi16_pair(xo[0], xo[1]), hi16_pair(xo[2], xo[3]), hi16_pair(xo[4], xo[5]), hi16_pair(xo[6], xo[7]));
    }

    // ---- tiles
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
      if (t < ntiles) {
        const int set = t;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          *reinterpret_cast<u32x4*>(buf + st_off + i * 4 * kRowStride) = wl[set][i];
        if (lane < 32) *reinterpret_cast<u32x4*>(tbuf + lane * 16) = tvs[set] | tvb[set];   // the lanes that miss read zeros
        wave_lds_fence();
        // table rows as B operands over the chunk index (lane's row, entries of this slice)
        u32x4 svt = *reinterpret_cast<const u32x4*>(tbuf + r * 16);
        u32x4 bvt = *reinterpret_cast<const u32x4*>(tbuf + 256 + r * 16);
        if constexpr (GSHIFT != 0) {   // group 128: one entry serves two chunks -> duplicate each bf16
          svt = u32x4{byte_perm(svt[0], svt[0], 0x01000100u), byte_perm(svt[0], svt[0], 0x03020302u),
                      byte_perm(svt[1], svt[1], 0x01000100u), byte_perm(svt[1], svt[1], 0x03020302u)};
          bvt = u32x4{byte_perm(bvt[0], bvt[0], 0x01000100u), byte_perm(bvt[0], bvt[0], 0x03020302u),
                      byte_perm(bvt[1], bvt[1], 0x01000100u), byte_perm(bvt[1], bvt[1], 0x03020302u)};
        }
        const bf16x8 bop = __builtin_bit_cast(bf16x8, bvt);
        f32x4 accb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(axh, bop, acc[t], 0, 0, 0);
        accb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(axm, bop, accb, 0, 0, 0);
        accb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(axo, bop, accb, 0, 0, 0);
        f32x4 accs = zero;
        if constexpr (BITS == 4) {
          const bf16x8 sop = __builtin_bit_cast(bf16x8, svt);
          accs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(axh, sop, zero, 0, 0, 0);
          accs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(axm, sop, accs, 0, 0, 0);
          accs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(axo, sop, accs, 0, 0, 0);
        }
        f32x4 at = accb;
#pragma unroll
        for (int c = 0; c < CPS; ++c) {
          f32x4 d;
          if constexpr (BITS == 4) {
            const u32x2 q = *reinterpret_cast<const u32x2*>(buf + r * kRowStride + c * 32 + kg * 8);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][0], widen_int4(q[0], nib, magic), zero, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][1], widen_int4(q[1], nib, magic), d, 0, 0, 0);
          } else {
            const u32x4 q = *reinterpret_cast<const u32x4*>(buf + r * kRowStride + c * 64 + kg * 16);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][0], widen_int8(q[0], q[1]), zero, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][1], widen_int8(q[2], q[3]), d, 0, 0, 0);
          }
          const uint32_t sw = svt[c >> 1];
          const float sc = __uint_as_float((c & 1) ? (sw & 0xFFFF0000u) : (sw << 16));
#pragma unroll
          for (int i = 0; i < 4; ++i) at[i] = fmaf(sc, d[i], at[i]);
        }
        if constexpr (BITS == 4) {
#pragma unroll
          for (int i = 0; i < 4; ++i) at[i] = fmaf(-128.f, accs[i], at[i]);
        }
        acc[t] = at;
        wave_lds_fence();
      }
    }
  }

  // ---- meet the K slices in LDS
#pragma unroll
  for (int t = 0; t < TMAX; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][t][i][lane] = acc[t][i];
  __syncthreads();
  for (int e = threadIdx.x; e < ntiles * 4 * kWave; e += kWave * WAVES) {
    const int l = e & 63, i = (e >> 6) & 3, t = e >> 8;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) v += red[wv][t][i][l];
    const int m = 4 * (l >> 4) + i;
    const int64_t n = n_begin + t * 16 + (l & 15);
    if (m < a.M && n < n_end) store_out(a.y, (bz * a.M + m) * (int64_t)a.N + n, v, a.y_dtype);
  }
}

template <int BITS, int WAVES, int TMAX>
void launch_k(const GemvArgs& a, int64_t batch, int rows_per_wg, hipStream_t st) {
  dim3 grid((unsigned)ceil_div(a.N, rows_per_wg), (unsigned)batch);
  if (a.gshift)
    hipLaunchKernelGGL((skinny_affine_kernel<BITS, WAVES, TMAX, 1>), grid, dim3(kWave * WAVES), 0, st, a, rows_per_wg);
  else
    hipLaunchKernelGGL((skinny_affine_kernel<BITS, WAVES, TMAX, 0>), grid, dim3(kWave * WAVES), 0, st, a, rows_per_wg);
}

template <int BITS>
void launch_g(const GemvArgs& a, int64_t batch, int waves, int rows_per_wg, hipStream_t st) {
  const int tmax = (rows_per_wg + 15) / 16;
#define QMM_CASE(WW, TT) if (waves == WW && tmax <= TT) return launch_k<BITS, WW, TT>(a, batch, rows_per_wg, st)
  QMM_CASE(8, 1); QMM_CASE(8, 2); QMM_CASE(8, 4);
  QMM_CASE(4, 1); QMM_CASE(4, 2); QMM_CASE(4, 4);
  QMM_CASE(2, 2); QMM_CASE(2, 4);
  QMM_CASE(1, 2); QMM_CASE(1, 4);
#undef QMM_CASE
}

int env_int(const char* name) {
  const char* e = experiment_env(name);
  return e ? atoi(e) : 0;
}

}  // namespace

// True when the staged kernel serves this problem (the caller falls back to
// the direct-load kernel otherwise).
bool skinny_supported(int64_t N, int64_t K, int gs, int bits, int mode, int tab, const void* s,
                      const void* b) {
  if (mode != QMM_MODE_AFFINE || (gs != 64 && gs != 128)) return false;
  if (tab != QMM_BF16) return false;       // table rows double as bf16 matrix operands
  const int64_t ks = (int64_t)kSliceBytes * 8 / bits;
  if (K % ks) return false;
  // table rows are read as dword-aligned 16-byte runs through bounds-checked descriptors
  if ((reinterpret_cast<uintptr_t>(s) & 3u) || (reinterpret_cast<uintptr_t>(b) & 3u)) return false;
  if (N * (K * bits / 8) >= 0x7FFFFFFFll) return false;       // 32-bit lane offsets
  return true;
}

// K slices per workgroup and rows per workgroup.  Rows are dealt so that the
// grid is about one workgroup per compute unit (each streams a contiguous row
// range, the last tile of a range may be partial), capped at four tiles.
void skinny_geometry(int64_t N, int64_t K, int bits, int* waves, int* rows_per_wg) {
  static const int env_w = env_int("QMM_SKINNY_WAVES"), env_r = env_int("QMM_SKINNY_ROWS");
  static const int cus = [] {
    int dev = 0, n = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
      hipDeviceProp_t p;
      if (hipGetDeviceProperties(&p, dev) == hipSuccess && p.multiProcessorCount > 0) n = p.multiProcessorCount;
    }
    return n;
  }();
  const int64_t slices = K / ((int64_t)kSliceBytes * 8 / bits);
  int w = slices >= 8 ? 8 : slices >= 4 ? 4 : slices >= 2 ? 2 : 1;
  int64_t rows = ceil_div(N, cus);
  if (rows < 16) rows = 16;
  if (rows > 64) rows = 64;
  if (env_w) w = env_w;
  if (env_r) rows = env_r;
  *waves = w;
  *rows_per_wg = (int)rows;
}

void skinny_dispatch(const GemvArgs& a0, int64_t batch, int gs, int bits, int tab, hipStream_t st) {
  GemvArgs a = a0;
  a.gshift = gs == 128 ? 1 : 0;
  int waves, rows;
  skinny_geometry(a.N, a.K, bits, &waves, &rows);
  (void)tab;
  if (bits == 4) launch_g<4>(a, batch, waves, rows, st);
  else launch_g<8>(a, batch, waves, rows, st);
}

}  // namespace qmm
