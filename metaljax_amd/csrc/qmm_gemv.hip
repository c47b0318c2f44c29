// Decode-regime quantized matmul (M <= 16) for gfx950: the general kernel.
//
// y[m, n] = sum_k x[m, k] * w[n, k],  w = scales*q + biases (affine) or
// E2M1[q] * 2^(e-127) (mxfp4).  Every packed weight byte is read exactly once,
// straight into the matrix-core operand layout, and unpacked in registers.
// That layout makes each lane its own L1 request (lane = weight row), which
// bounds this kernel by L1 tag lookups rather than by HBM; the common layouts
// (group 64 / 128, bf16 tables, K a multiple of a slice) therefore run on the
// LDS-staged kernels of qmm_skinny.hip / qmm_skinny2.hip, and this one serves
// everything else: group 32, float32 / float16 tables, odd K, MXFP4.  The
// dispatcher at the end of the file chooses.
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
#include <type_traits>

#include "qmm_gemv_common.hpp"

namespace qmm {

namespace {

// Affine kernel.  BITS: 4 or 8.  CH: K-chunk per scale application (64, or 32
// for group size 32).  T: 16-row tiles per wavefront.  WAVES: K slices per
// workgroup.  U: chunks whose loads are all issued before any is consumed --
// the kernel lives on memory-level parallelism, a wavefront keeps U*T weight
// loads in flight.  VT: the U = 8 scales (and biases) of a block are one
// 16-byte load per row (16-bit tables, one table entry per chunk, aligned,
// every block full).
//
// Every address is "descriptor + 32-bit lane offset + uniform offset": the
// chunk index is wavefront-uniform, so stepping through K costs scalar
// instructions only.  Lanes past M read the activations out of range (zeros);
// chunks past the end of a ragged last block read their tables out of range,
// so their scale and bias are zero.
template <int BITS, int CH, int T, int WAVES, int TAB, int U, bool VT>
__global__ __launch_bounds__(kWave* WAVES) void gemv_affine_kernel(GemvArgs a) {
  load_args_now(a);
  constexpr int STEPS = CH / 32;                 // MFMA steps per chunk
  constexpr int WPL = CH * BITS / 128;           // packed words per lane per chunk
  constexpr int WPC = CH * BITS / 32;            // packed words per row per chunk
  constexpr int ROWS = 16 * T;
  constexpr int TABSZ = (TAB == QMM_F32) ? 4 : 2;
  __shared__ float red[WAVES][T][4][kWave];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, kg = lane >> 4;
  const int64_t bz = blockIdx.y;
  const int64_t n0 = (int64_t)blockIdx.x * ROWS;
  const int64_t wpr = (int64_t)a.K * BITS / 32;             // words per weight row
  const int64_t ng = (int64_t)((a.K / CH) >> a.gshift);     // table entries per row

  int64_t xz = a.lhs_idx ? (int64_t)a.lhs_idx[bz] : bz;
  int64_t wz = a.rhs_idx ? (int64_t)a.rhs_idx[bz] : bz;
  bool x_ok = true;
  int M = a.M, seg_lo = 0;
  if (a.segments) {                                 // grouped form: up to 16 sorted pairs of one expert
    if (bz >= a.segments[0]) return;                // uniform, before any barrier
    wz = a.segments[1 + 3 * bz];
    seg_lo = a.segments[2 + 3 * bz];
    M = a.segments[3 + 3 * bz];
    xz = 0;
  } else if (a.rhs_idx) {                           // gather form: indices are data
    if (wz < 0 || wz >= a.n_experts) return;        // uniform, before any barrier
    if (xz < 0 || xz >= a.n_xrows) { xz = 0; x_ok = false; }
  }
  const auto rx = a.segments ? make_rsrc(a.x, (int64_t)a.x_rows * a.K * 2)
                             : make_rsrc(a.x + xz * a.M * (int64_t)a.K, x_ok ? (int64_t)a.M * a.K * 2 : 0);
  const auto rw = make_rsrc(a.w + wz * a.N * wpr, a.N * wpr * 4);
  const auto rs = make_rsrc(static_cast<const char*>(a.s) + wz * a.N * ng * TABSZ, a.N * ng * TABSZ);
  const auto rb = make_rsrc(static_cast<const char*>(a.b) + wz * a.N * ng * TABSZ, a.N * ng * TABSZ);

  const int chunks = a.K / CH;
  const int c0 = (int)((int64_t)chunks * wave / WAVES);
  const int c1 = (int)((int64_t)chunks * (wave + 1) / WAVES);

  uint32_t woff[T], toff[T];                     // lane byte offsets
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int64_t n = n0 + t * 16 + r;
    if (n >= a.N) n = a.N - 1;
    woff[t] = (uint32_t)((n * wpr + kg * WPL) * 4);
    toff[t] = (uint32_t)(n * ng * TABSZ);
  }
  uint32_t xoff = r < M ? (uint32_t)(((int64_t)r * a.K + kg * (CH / 4)) * 2) : kOutOfRange;
  if (a.segments && r < M) {                        // row r of the segment is row src_row[first + r] of x
    const int64_t src = a.src_row[seg_lo + r];
    xoff = src >= 0 && src < a.x_rows ? (uint32_t)((src * a.K + kg * (CH / 4)) * 2) : kOutOfRange;
  }

  f32x4 acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  const uint32_t one = pin_vgpr(kOnesBf16x2);
  const bf16x8 ones = as_bf16x8(one, one, one, one);
  const uint32_t nib = pin_vgpr(0x000F000Fu), magic = pin_vgpr(0x43004300u);

  for (int cb = c0; cb < c1; cb += U) {
    uint32_t q[U][T][WPL];
    uint32_t sraw[U][T], braw[U][T];
    u32x4 svec[T], bvec[T];
    u32x4 xr[U][STEPS];
    // ---- every load of the block first
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = (VT || cb + u < c1) ? cb + u : c1 - 1;          // uniform
      const uint32_t so = (uint32_t)c * (WPC * 4);
#pragma unroll
      for (int t = 0; t < T; ++t) {
        if constexpr (WPL == 4) {
          u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rw, woff[t], so, 0);
          q[u][t][0] = v[0]; q[u][t][1] = v[1]; q[u][t][2] = v[2]; q[u][t][3] = v[3];
        } else if constexpr (WPL == 2) {
          u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rw, woff[t], so, 0);
          q[u][t][0] = v[0]; q[u][t][1] = v[1];
        } else {
          q[u][t][0] = __builtin_amdgcn_raw_buffer_load_b32(rw, woff[t], so, 0);
        }
      }
    }
    if constexpr (VT) {
#pragma unroll
      for (int t = 0; t < T; ++t) {
        svec[t] = __builtin_amdgcn_raw_buffer_load_b128(rs, toff[t], (uint32_t)cb * TABSZ, 0);
        bvec[t] = __builtin_amdgcn_raw_buffer_load_b128(rb, toff[t], (uint32_t)cb * TABSZ, 0);
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t so = cb + u < c1 ? (uint32_t)((cb + u) >> a.gshift) * TABSZ : kOutOfRange;
#pragma unroll
        for (int t = 0; t < T; ++t) {
          if constexpr (TAB == QMM_F32) {
            sraw[u][t] = __builtin_amdgcn_raw_buffer_load_b32(rs, toff[t], so, 0);
            braw[u][t] = __builtin_amdgcn_raw_buffer_load_b32(rb, toff[t], so, 0);
          } else {
            sraw[u][t] = __builtin_amdgcn_raw_buffer_load_b16(rs, toff[t], so, 0);
            braw[u][t] = __builtin_amdgcn_raw_buffer_load_b16(rb, toff[t], so, 0);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = (VT || cb + u < c1) ? cb + u : c1 - 1;
#pragma unroll
      for (int j = 0; j < STEPS; ++j)
        xr[u][j] = __builtin_amdgcn_raw_buffer_load_b128(rx, xoff, (uint32_t)(c * CH + j * 8) * 2, 0);
    }
    // ---- then the arithmetic
#pragma unroll
    for (int u = 0; u < U; ++u) {
      f32x4 d[T];
      f32x4 xs;
#pragma unroll
      for (int j = 0; j < STEPS; ++j) {
        bf16x8 xa;
        if constexpr (BITS == 4) xa = pair_stride4(xr[u][j]);
        else xa = __builtin_bit_cast(bf16x8, xr[u][j]);
        xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, ones, j ? xs : zero, 0, 0, 0);
#pragma unroll
        for (int t = 0; t < T; ++t) {
          bf16x8 wq;
          if constexpr (BITS == 4) wq = widen_int4(q[u][t][j], nib, magic);
          else wq = widen_int8(q[u][t][2 * j], q[u][t][2 * j + 1]);
          d[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, wq, j ? d[t] : zero, 0, 0, 0);
        }
      }
#pragma unroll
      for (int t = 0; t < T; ++t) {
        float sc, bi;
        if constexpr (VT) {
          const uint32_t sw = svec[t][u >> 1], bw = bvec[t][u >> 1];
          if constexpr (TAB == QMM_BF16) {
            sc = __uint_as_float((u & 1) ? (sw & 0xFFFF0000u) : (sw << 16));
            bi = __uint_as_float((u & 1) ? (bw & 0xFFFF0000u) : (bw << 16));
          } else {
            sc = f16_bits_to_f32((u & 1) ? (sw >> 16) : (sw & 0xFFFFu));
            bi = f16_bits_to_f32((u & 1) ? (bw >> 16) : (bw & 0xFFFFu));
          }
        } else if constexpr (TAB == QMM_F32) {
          sc = __uint_as_float(sraw[u][t]); bi = __uint_as_float(braw[u][t]);
        } else if constexpr (TAB == QMM_BF16) {
          sc = bf16_bits_to_f32(sraw[u][t]); bi = bf16_bits_to_f32(braw[u][t]);
        } else {
          sc = f16_bits_to_f32(sraw[u][t]); bi = f16_bits_to_f32(braw[u][t]);
        }
        if constexpr (BITS == 4) bi = fmaf(-128.f, sc, bi);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[t][i] = fmaf(sc, d[t][i], acc[t][i]);
          acc[t][i] = fmaf(bi, xs[i], acc[t][i]);
        }
      }
    }
  }

  // ---- meet the K slices in LDS
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
    if (m < M && n < a.N) {
      int64_t orow = bz * a.M + m;
      if (a.segments) orow = a.out_row[seg_lo + m];
      if (orow >= 0) store_out(a.y, orow * (int64_t)a.N + n, v, a.y_dtype);
    }
  }
}

// MXFP4 kernel.  A lane's 16-byte load is exactly one 32-element MX block, so
// the block's power-of-two scale rides along in the hardware fp4 -> bf16
// conversion (exact: an E2M1 value has one mantissa bit) and the products need
// no rescaling afterwards.  One macro chunk = 128 k = four MFMA steps.
template <int T, int WAVES, int U>
__global__ __launch_bounds__(kWave* WAVES) void gemv_mxfp4_kernel(GemvArgs a) {
  load_args_now(a);
  constexpr int ROWS = 16 * T;
  __shared__ float red[WAVES][T][4][kWave];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int r = lane & 15, kg = lane >> 4;
  const int64_t bz = blockIdx.y;
  const int64_t n0 = (int64_t)blockIdx.x * ROWS;
  const int64_t wpr = (int64_t)a.K / 8;
  const int nblk = a.K / 32;                       // MX blocks per row

  int64_t xz = a.lhs_idx ? (int64_t)a.lhs_idx[bz] : bz;
  int64_t wz = a.rhs_idx ? (int64_t)a.rhs_idx[bz] : bz;
  bool x_ok = true;
  int M = a.M, seg_lo = 0;
  if (a.segments) {                                 // grouped form: up to 16 sorted pairs of one expert
    if (bz >= a.segments[0]) return;                // uniform, before any barrier
    wz = a.segments[1 + 3 * bz];
    seg_lo = a.segments[2 + 3 * bz];
    M = a.segments[3 + 3 * bz];
    xz = 0;
  } else if (a.rhs_idx) {                           // gather form: indices are data
    if (wz < 0 || wz >= a.n_experts) return;        // uniform, before any barrier
    if (xz < 0 || xz >= a.n_xrows) { xz = 0; x_ok = false; }
  }
  const uint16_t* xb = a.x + xz * a.M * (int64_t)a.K;
  const uint32_t* wb = a.w + wz * a.N * wpr;
  const uint8_t* sb = static_cast<const uint8_t*>(a.s) + wz * a.N * (int64_t)nblk;

  const int chunks = (nblk + 3) / 4;               // macro chunks of 128 k
  const int c0 = (int)((int64_t)chunks * wave / WAVES);
  const int c1 = (int)((int64_t)chunks * (wave + 1) / WAVES);

  const uint32_t* wrow[T];
  const uint8_t* srow[T];
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int64_t n = n0 + t * 16 + r;
    if (n >= a.N) n = a.N - 1;
    wrow[t] = wb + n * wpr;
    srow[t] = sb + n * nblk;
  }
  bool xvalid = r < M && x_ok;
  const uint16_t* xrow = xb + (int64_t)(xvalid ? r : 0) * a.K;
  if (a.segments) {                                 // row r of the segment is row src_row[first + r] of x
    const int64_t src = r < M ? (int64_t)a.src_row[seg_lo + r] : -1;
    xvalid = src >= 0 && src < a.x_rows;
    xrow = a.x + (xvalid ? src : 0) * a.K;
  }

  f32x4 acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int cb = c0; cb < c1; cb += U) {
    u32x4 q[U][T];
    uint8_t sraw[U][T];
    u32x4 xr[U][4];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int blk = (cb + u) * 4 + kg;
      if (cb + u >= c1 || blk >= nblk) blk = nblk - 1;
#pragma unroll
      for (int t = 0; t < T; ++t)
        q[u][t] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wrow[t] + (int64_t)blk * 4));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int blk = (cb + u) * 4 + kg;
      if (cb + u >= c1 || blk >= nblk) blk = nblk - 1;
#pragma unroll
      for (int t = 0; t < T; ++t) sraw[u][t] = srow[t][blk];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int blk = (cb + u) * 4 + kg;
      const bool live = cb + u < c1 && blk < nblk;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        xr[u][j] = u32x4{0u, 0u, 0u, 0u};
        if (xvalid && live)
          xr[u][j] = *reinterpret_cast<const u32x4*>(xrow + (int64_t)blk * 32 + j * 8);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const float sc = e8m0_to_f32(sraw[u][t]);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bf16x8 xa = __builtin_bit_cast(bf16x8, xr[u][j]);   // zero where not live
          acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa, widen_e2m1(q[u][t][j], sc), acc[t], 0, 0, 0);
        }
      }
    }
  }

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
    if (m < M && n < a.N) {
      int64_t orow = bz * a.M + m;
      if (a.segments) orow = a.out_row[seg_lo + m];
      if (orow >= 0) store_out(a.y, orow * (int64_t)a.N + n, v, a.y_dtype);
    }
  }
}

struct Geometry { int t, waves, u; };

template <int BITS, int CH, int TAB, int T, int WAVES, int U>
void launch_affine_k(const GemvArgs& a, int64_t batch, hipStream_t st) {
  dim3 grid((unsigned)ceil_div(a.N, 16 * T), (unsigned)batch);
  // vector table loads: 16-bit tables, one entry per chunk, 16-byte aligned runs
  const int chunks = a.K / CH;
  bool vt = false;
  if constexpr (TAB != QMM_F32 && U == 8) {
    vt = a.gshift == 0 && chunks % (8 * WAVES) == 0 &&
         (reinterpret_cast<uintptr_t>(a.s) & 15u) == 0 && (reinterpret_cast<uintptr_t>(a.b) & 15u) == 0;
    if (vt) {
      hipLaunchKernelGGL((gemv_affine_kernel<BITS, CH, T, WAVES, TAB, U, true>), grid, dim3(kWave * WAVES), 0, st, a);
      return;
    }
  }
  hipLaunchKernelGGL((gemv_affine_kernel<BITS, CH, T, WAVES, TAB, U, false>), grid, dim3(kWave * WAVES), 0, st, a);
}

template <int BITS, int CH, int TAB>
void launch_affine_g(const GemvArgs& a, int64_t batch, Geometry g, hipStream_t st) {
#define QMM_CASE(TT, WW, UU) \
  if (g.t == TT && g.waves == WW && g.u == UU) return launch_affine_k<BITS, CH, TAB, TT, WW, UU>(a, batch, st)
  QMM_CASE(1, 4, 4); QMM_CASE(1, 4, 8); QMM_CASE(1, 8, 4); QMM_CASE(1, 8, 8);
  QMM_CASE(2, 4, 4); QMM_CASE(2, 4, 8); QMM_CASE(2, 8, 4); QMM_CASE(2, 8, 8);
  QMM_CASE(1, 16, 4); QMM_CASE(2, 16, 4);
#undef QMM_CASE
  launch_affine_k<BITS, CH, TAB, 1, 8, 8>(a, batch, st);
}

template <int BITS, int CH>
void launch_affine(const GemvArgs& a, int64_t batch, int tab, Geometry g, hipStream_t st) {
  if (tab == QMM_BF16) launch_affine_g<BITS, CH, QMM_BF16>(a, batch, g, st);
  else if (tab == QMM_F32) launch_affine_g<BITS, CH, QMM_F32>(a, batch, g, st);
  else launch_affine_g<BITS, CH, QMM_F16>(a, batch, g, st);
}

template <int T, int WAVES, int U>
void launch_mxfp4_k(const GemvArgs& a, int64_t batch, hipStream_t st) {
  dim3 grid((unsigned)ceil_div(a.N, 16 * T), (unsigned)batch);
  hipLaunchKernelGGL((gemv_mxfp4_kernel<T, WAVES, U>), grid, dim3(kWave * WAVES), 0, st, a);
}

void launch_mxfp4(const GemvArgs& a, int64_t batch, Geometry g, hipStream_t st) {
#define QMM_CASE(TT, WW, UU) \
  if (g.t == TT && g.waves == WW && g.u == UU) return launch_mxfp4_k<TT, WW, UU>(a, batch, st)
  QMM_CASE(1, 4, 4); QMM_CASE(1, 4, 8); QMM_CASE(1, 8, 4); QMM_CASE(1, 8, 8);
  QMM_CASE(2, 4, 4); QMM_CASE(2, 8, 4); QMM_CASE(2, 8, 8);
#undef QMM_CASE
  launch_mxfp4_k<1, 8, 4>(a, batch, st);
}

int env_int(const char* name) {
  const char* e = experiment_env(name);
  return e ? atoi(e) : 0;
}

}  // namespace

bool skinny_supported(int64_t N, int64_t K, int gs, int bits, int mode, int tab, const void* s,
                      const void* b);
void skinny_dispatch(const GemvArgs& a0, int64_t batch, int gs, int bits, int tab, hipStream_t st);
void skinny_geometry(int64_t N, int64_t K, int bits, int* waves, int* rows_per_wg);
bool skinny2_plan(int64_t M, int64_t N, int64_t K, int bits, int* rows_per_wg);
void skinny2_dispatch(const GemvArgs& a0, int64_t batch, int gs, int bits, int rows, hipStream_t st,
                      int tab, bool force_direct);
int skinny2_direct_rows(int64_t N);
bool skinny2_mx_supported(int64_t N, int64_t K, const void* s);
void skinny2_mx_dispatch(const GemvArgs& a0, int64_t batch, hipStream_t st);

// Tile / slice / unroll choice; QMM_GEMV_T, QMM_GEMV_WAVES and QMM_GEMV_U
// override it for experiments (read once).
void gemv_geometry(int64_t M, int64_t N, int64_t K, int* t, int* waves) {
  static const int env_t = env_int("QMM_GEMV_T"), env_w = env_int("QMM_GEMV_WAVES");
  // two 16-row tiles a workgroup only where that still leaves a workgroup per
  // compute unit (256 x 32 rows); below, one tile: 4096 x 11008 at M = 16
  // 24.3 against 33.4 us, 4096 x 14336 with groups of 32 32.3 against 49.9
  // (8192 x 11008: 45.0 against 35.6 the other way)
  int tt = (M > 8 && N >= 8192) ? 2 : 1;
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
                   int mode, const int32_t* lhs_idx, const int32_t* rhs_idx, int64_t n_experts,
                   int64_t n_xrows, hipStream_t st) {
  static const int env_u = env_int("QMM_GEMV_U");
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
  a.n_experts = (int)n_experts;
  a.n_xrows = (int)n_xrows;
  static const int no_skinny = env_int("QMM_NO_SKINNY");
  if (!no_skinny && skinny_supported(N, K, gs, bits, mode, tab, s, b)) {
    // big weights: the kernel with loader wavefronts (QMM_SKINNY_V1 keeps the
    // self-loading one everywhere, for comparison)
    static const int v1 = env_int("QMM_SKINNY_V1");
    int rows;
    if (!v1 && skinny2_plan(M, N, K, bits, &rows)) skinny2_dispatch(a, batch, gs, bits, rows, st, tab, false);
    else skinny_dispatch(a, batch, gs, bits, tab, st);
    return;
  }
  // float16 tables (what float16 models carry) and float32 tables (biases that
  // do not fit 16 bits): the loader-wavefront kernel reads them, the
  // self-loading one does not (from three K-slices a row on, as for bf16
  // tables; against the general kernel at M = 4: 16384 x 3072 with float16
  // tables 9.7 / 29.8 us, 37888 x 3584 with float32 tables 23.4 / 69.2)
  static const int no_f16 = env_int("QMM_NO_SKINNY_F16");
  if (!no_skinny && !no_f16 && (tab == QMM_F16 || tab == QMM_F32) && K * bits / 8 / 256 >= 3 &&
      skinny_supported(N, K, gs, bits, mode, QMM_BF16, s, b)) {
    int rows;
    const bool planned = skinny2_plan(M, N, K, bits, &rows);
    if (!planned) rows = skinny2_direct_rows(N);
    skinny2_dispatch(a, batch, gs, bits, rows, st, tab, !planned);
    return;
  }
  Geometry g;
  gemv_geometry(M, N, K, &g.t, &g.waves);
  g.u = env_u ? env_u : 8;
  if (mode == QMM_MODE_MXFP4) {
    a.gshift = 0;
    // big weights: the loader-wavefront kernel (activations fetched directly)
    if (!no_skinny && skinny2_mx_supported(N, K, s)) return skinny2_mx_dispatch(a, batch, st);
    if (!env_u) g.u = 4;
    launch_mxfp4(a, batch, g, st);
    return;
  }
  const int ch = gs >= 64 ? 64 : 32;
  a.gshift = (gs == 128) ? 1 : 0;
  if (bits == 4) {
    if (ch == 64) launch_affine<4, 64>(a, batch, tab, g, st);
    else launch_affine<4, 32>(a, batch, tab, g, st);
  } else {
    if (ch == 64) launch_affine<8, 64>(a, batch, tab, g, st);
    else launch_affine<8, 32>(a, batch, tab, g, st);
  }
}

// The general kernels would serve this shape (no staged decode kernel does).
bool gemv_runs_general(int64_t N, int64_t K, int gs, int bits, int mode, int tab, const void* s, const void* b) {
  if (skinny_supported(N, K, gs, bits, mode, tab, s, b)) return false;
  if ((tab == QMM_F16 || tab == QMM_F32) && K * bits / 8 / 256 >= 8 &&
      skinny_supported(N, K, gs, bits, mode, QMM_BF16, s, b))
    return false;
  if (mode == QMM_MODE_MXFP4 && skinny2_mx_supported(N, K, s)) return false;
  return true;
}

// Expert-indexed pairs sorted by expert (segments / src_row / out_row as the
// routing pass writes them) on the general kernels: one decode product per
// expert and sixteen pairs, so that an expert's weights are read once for all
// of its pairs instead of once per pair.  `max_segments` rows of workgroups
// are launched; the ones past the list's count exit at once.
void gemv_grouped_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                           int y_dtype, const int32_t* segments, const int32_t* src_row,
                           const int32_t* out_row, int64_t max_segments, int64_t x_rows, int64_t N,
                           int64_t K, int gs, int bits, int mode, hipStream_t st) {
  GemvArgs a;
  a.x = static_cast<const uint16_t*>(x);
  a.w = static_cast<const uint32_t*>(w);
  a.s = s;
  a.b = b;
  a.y = y;
  a.M = 16;
  a.N = (int)N;
  a.K = (int)K;
  a.y_dtype = y_dtype;
  a.lhs_idx = nullptr;
  a.rhs_idx = nullptr;
  a.segments = segments;
  a.src_row = src_row;
  a.out_row = out_row;
  a.x_rows = (int)x_rows;
  Geometry g;
  gemv_geometry(16, N, K, &g.t, &g.waves);
  if (mode == QMM_MODE_MXFP4) {
    a.gshift = 0;
    g.u = 4;
    launch_mxfp4(a, max_segments, g, st);
    return;
  }
  g.u = 8;
  const int ch = gs >= 64 ? 64 : 32;
  a.gshift = (gs == 128) ? 1 : 0;
  if (bits == 4) {
    if (ch == 64) launch_affine<4, 64>(a, max_segments, tab, g, st);
    else launch_affine<4, 32>(a, max_segments, tab, g, st);
  } else {
    if (ch == 64) launch_affine<8, 64>(a, max_segments, tab, g, st);
    else launch_affine<8, 32>(a, max_segments, tab, g, st);
  }
}

}  // namespace qmm
