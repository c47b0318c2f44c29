// Decode-regime quantized matmul (M <= 16) for gfx950.
//
// y[m, n] = sum_k x[m, k] * w[n, k],  w = scales*q + biases (affine) or
// E2M1[q] * 2^(e-127) (mxfp4).  The kernel is HBM-bound: every packed weight
// byte is read exactly once with vector loads and unpacked in registers.
//
// Mapping.  One workgroup owns 16*T consecutive weight rows over the whole K;
// its WAVES wavefronts split K into contiguous slices and their partial sums
// meet in LDS at the end.  Inside a wavefront lane l = 16*kg + r holds weight
// row r of each tile and the kg-th quarter of a K-chunk (one quantization
// group of 64, or 32), so a row's chunk is one contiguous run of bytes split
// over four lanes.
//
// Arithmetic.  The integer codes are exact in bf16, so the per-chunk inner
// product sum_k x*q runs on the matrix cores (v_mfma_f32_16x16x32_bf16, the
// activations as the A operand: rows m, the codes as B: columns n) with exact
// products and float32 accumulation; an all-ones B operand yields sum_k x in
// the same register layout.  The affine map is applied once per chunk:
//     acc += scale * (sum_k x*q) + bias * (sum_k x)
// 4-bit codes are widened as the bf16 value 128+q (one and-or per pair), the
// 128 is folded into the bias; their pairs come out as (k, k+4), so the
// activation registers are byte-permuted to the same order.
#include "qmm_common.hpp"

namespace qmm {

namespace {

constexpr uint32_t kOnesBf16x2 = 0x3F803F80u;

__device__ __forceinline__ bf16x8 as_bf16x8(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  u32x4 v = {a, b, c, d};
  return __builtin_bit_cast(bf16x8, v);
}

// 8 four-bit codes -> four registers of bf16 pairs (128+q_t, 128+q_{t+4}).
__device__ __forceinline__ bf16x8 widen_int4(uint32_t w) {
  const uint32_t m = 0x000F000Fu, one28 = 0x43004300u;
  return as_bf16x8((w & m) | one28, ((w >> 4) & m) | one28, ((w >> 8) & m) | one28,
                   ((w >> 12) & m) | one28);
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

// 8 E2M1 codes -> bf16 pairs in natural order (q_2t, q_2t+1), exact: the
// hardware converter widens the two codes of one byte at a time.
__device__ __forceinline__ bf16x8 widen_e2m1(uint32_t w) {
  bf16x2 p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 0);
  bf16x2 p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 1);
  bf16x2 p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 2);
  bf16x2 p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, 1.0f, 3);
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
  const int32_t* lhs_idx;
  const int32_t* rhs_idx;
};

// MODE: 0 affine, 1 mxfp4.  BITS: 4 or 8.  CH: K-chunk per scale application
// (64 or 32; mxfp4: 32).  T: 16-row tiles per wavefront.  WAVES: K slices.
template <int MODE, int BITS, int CH, int T, int WAVES, int TAB>
__global__ __launch_bounds__(kWave* WAVES) void gemv_kernel(GemvArgs a) {
  constexpr int STEPS = CH / 32;                 // MFMA steps per chunk
  constexpr int WPL = CH * BITS / 128;           // packed words per lane per chunk
  constexpr int ROWS = 16 * T;
  __shared__ float red[WAVES][T][4][kWave];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15, kg = lane >> 4;
  const int64_t bz = blockIdx.y;
  const int64_t n0 = (int64_t)blockIdx.x * ROWS;
  const int64_t wpr = (int64_t)a.K * BITS / 32;  // words per weight row
  const int64_t ng = (int64_t)(a.K / CH) >> a.gshift;  // table entries per row

  const int64_t xz = a.lhs_idx ? (int64_t)a.lhs_idx[bz] : bz;
  const int64_t wz = a.rhs_idx ? (int64_t)a.rhs_idx[bz] : bz;
  const uint16_t* xb = a.x + xz * a.M * (int64_t)a.K;
  const uint32_t* wb = a.w + wz * a.N * wpr;
  const char* sb = static_cast<const char*>(a.s);
  const char* bb = static_cast<const char*>(a.b);
  constexpr int TABSZ = (MODE == 1) ? 1 : (TAB == QMM_F32 ? 4 : 2);
  sb += wz * a.N * ng * TABSZ;
  if (MODE == 0) bb += wz * a.N * ng * TABSZ;

  const int chunks = a.K / CH;
  const int c0 = (int)((int64_t)chunks * wave / WAVES);
  const int c1 = (int)((int64_t)chunks * (wave + 1) / WAVES);

  const uint32_t* wrow[T];
  int64_t trow[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int64_t n = n0 + t * 16 + r;
    if (n >= a.N) n = a.N - 1;
    wrow[t] = wb + n * wpr + kg * WPL;
    trow[t] = n * ng;
  }
  const bool xvalid = r < a.M;
  const uint16_t* xrow = xb + (int64_t)(xvalid ? r : 0) * a.K + kg * (CH / 4);

  f32x4 acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  const bf16x8 ones = as_bf16x8(kOnesBf16x2, kOnesBf16x2, kOnesBf16x2, kOnesBf16x2);


  for (int c = c0; c < c1; ++c) {
    // packed weights of this chunk, every tile
    uint32_t q[T][WPL];
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const uint32_t* p = wrow[t] + (int64_t)c * (CH * BITS / 32);
      if constexpr (WPL == 4) {
        u32x4 v = *reinterpret_cast<const u32x4*>(p);
        q[t][0] = v[0]; q[t][1] = v[1]; q[t][2] = v[2]; q[t][3] = v[3];
      } else if constexpr (WPL == 2) {
        u32x2 v = *reinterpret_cast<const u32x2*>(p);
        q[t][0] = v[0]; q[t][1] = v[1];
      } else {
        q[t][0] = *p;
      }
    }
    float sc[T], bi[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const int64_t ti = trow[t] + (c >> a.gshift);
      if constexpr (MODE == 1) {
        sc[t] = e8m0_to_f32(reinterpret_cast<const uint8_t*>(sb)[ti]);
        bi[t] = 0.f;
      } else {
        sc[t] = load_table<TAB>(sb, ti);
        bi[t] = load_table<TAB>(bb, ti);
        if constexpr (BITS == 4) bi[t] = fmaf(-128.f, sc[t], bi[t]);
      }
    }
    // activations of this chunk: lanes past M feed zeros
    u32x4 xr[STEPS];
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
      xr[j] = u32x4{0u, 0u, 0u, 0u};
      if (xvalid) xr[j] = *reinterpret_cast<const u32x4*>(xrow + (int64_t)c * CH + j * 8);
    }
    f32x4 d[T];
#pragma unroll
    for (int t = 0; t < T; ++t) d[t] = zero;
    f32x4 xs = zero;
#pragma unroll
    for (int j = 0; j < STEPS; ++j) {
      bf16x8 xa;
      if constexpr (MODE == 0 && BITS == 4) xa = pair_stride4(xr[j]);
      else xa = __builtin_bit_cast(bf16x8, xr[j]);
      if constexpr (MODE == 0)
        xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, ones, xs, 0, 0, 0);
#pragma unroll
      for (int t = 0; t < T; ++t) {
        bf16x8 wq;
        if constexpr (MODE == 1) wq = widen_e2m1(q[t][j]);
        else if constexpr (BITS == 4) wq = widen_int4(q[t][j]);
        else wq = widen_int8(q[t][2 * j], q[t][2 * j + 1]);
        d[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, wq, d[t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[t][i] = fmaf(sc[t], d[t][i], acc[t][i]);
        if constexpr (MODE == 0) acc[t][i] = fmaf(bi[t], xs[i], acc[t][i]);
      }
    }
  }

  // meet the K slices in LDS
#pragma unroll
  for (int t = 0; t < T; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[wave][t][i][lane] = acc[t][i];
  __syncthreads();
  for (int e = threadIdx.x; e < T * 4 * kWave; e += kWave * WAVES) {
    const int l = e & 63, i = (e >> 6) & 3, t = e >> 8;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) v += red[wv][t][i][l];
    const int m = 4 * (l >> 4) + i;
    const int64_t n = n0 + t * 16 + (l & 15);
    if (m < a.M && n < a.N) store_out(a.y, (bz * a.M + m) * (int64_t)a.N + n, v, a.y_dtype);
  }
}

template <int MODE, int BITS, int CH, int T, int WAVES, int TAB>
void launch(const GemvArgs& a, int64_t batch, hipStream_t st) {
  dim3 grid((unsigned)ceil_div(a.N, 16 * T), (unsigned)batch);
  hipLaunchKernelGGL((gemv_kernel<MODE, BITS, CH, T, WAVES, TAB>), grid, dim3(kWave * WAVES), 0,
                     st, a);
}

template <int MODE, int BITS, int CH, int TAB>
void launch_shape(const GemvArgs& a, int64_t batch, int t, int waves, hipStream_t st) {
  if (t == 1 && waves == 4) launch<MODE, BITS, CH, 1, 4, TAB>(a, batch, st);
  else if (t == 1 && waves == 8) launch<MODE, BITS, CH, 1, 8, TAB>(a, batch, st);
  else if (t == 2 && waves == 4) launch<MODE, BITS, CH, 2, 4, TAB>(a, batch, st);
  else if (t == 2 && waves == 8) launch<MODE, BITS, CH, 2, 8, TAB>(a, batch, st);
  else launch<MODE, BITS, CH, 1, 4, TAB>(a, batch, st);
}

template <int BITS, int CH>
void launch_affine(const GemvArgs& a, int64_t batch, int tab, int t, int waves, hipStream_t st) {
  if (tab == QMM_BF16) launch_shape<0, BITS, CH, QMM_BF16>(a, batch, t, waves, st);
  else if (tab == QMM_F32) launch_shape<0, BITS, CH, QMM_F32>(a, batch, t, waves, st);
  else launch_shape<0, BITS, CH, QMM_F16>(a, batch, t, waves, st);
}

}  // namespace

// Tile/slice choice.  Overridable for experiments through QMM_GEMV_T /
// QMM_GEMV_WAVES (read once).
void gemv_geometry(int64_t M, int64_t N, int64_t K, int* t, int* waves) {
  static const int env_t = [] { const char* e = getenv("QMM_GEMV_T"); return e ? atoi(e) : 0; }();
  static const int env_w = [] { const char* e = getenv("QMM_GEMV_WAVES"); return e ? atoi(e) : 0; }();
  int tt = (M > 8 && N >= 4096) ? 2 : 1;
  int ww = (K >= 4096) ? 8 : 4;
  if (env_t) tt = env_t;
  if (env_w) ww = env_w;
  *t = tt;
  *waves = ww;
}

// Host entry used by the C ABI.  Shapes were validated by the caller:
// M <= 16, K % 32 == 0, K % group_size == 0, x bf16.
void gemv_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                   int y_dtype, int64_t batch, int64_t M, int64_t N, int64_t K, int gs, int bits,
                   int mode, const int32_t* lhs_idx, const int32_t* rhs_idx, hipStream_t st) {
  GemvArgs a;
  a.x = static_cast<const uint16_t*>(x);
  a.w = static_cast<const uint32_t*>(w);
  a.s = s;
  a.b = b;
  a.y = y;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  a.y_dtype = y_dtype;
  a.lhs_idx = lhs_idx;
  a.rhs_idx = rhs_idx;
  int t, waves;
  gemv_geometry(M, N, K, &t, &waves);
  if (mode == QMM_MODE_MXFP4) {
    a.gshift = 0;
    launch_shape<1, 4, 32, QMM_BF16>(a, batch, t, waves, st);
    return;
  }
  const int ch = gs >= 64 ? 64 : 32;
  a.gshift = (gs == 128) ? 1 : 0;
  if (bits == 4) {
    if (ch == 64) launch_affine<4, 64>(a, batch, tab, t, waves, st);
    else launch_affine<4, 32>(a, batch, tab, t, waves, st);
  } else {
    if (ch == 64) launch_affine<8, 64>(a, batch, tab, t, waves, st);
    else launch_affine<8, 32>(a, batch, tab, t, waves, st);
  }
}

}  // namespace qmm
