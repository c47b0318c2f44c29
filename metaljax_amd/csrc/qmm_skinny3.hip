// Decode-regime affine quantized matmul (M <= 16), sixteen self-loading
// wavefronts a workgroup.
//
// Same arithmetic as qmm_skinny.hip (codes exact in bf16, two
// v_mfma_f32_16x16x32_bf16 per 64-code chunk, the scale applied to the chunk's
// dot, the code-independent terms as small MFMAs over the chunk index), same
// wave-private LDS round trip from coalesced loads to operand order.  What
// differs is how the memory system is kept busy.  A launch that only reads the
// weight of the 4096 x 14336 case takes 6.7 us on this machine with every
// byte requested at once from registers, whereas four loader wavefronts with
// a four-slot LDS ring hold one 32 KB tile a compute unit in flight.  Here a
// workgroup is sixteen wavefronts (four a SIMD), wavefront w owns the K-slices
// w, w + 16, ... of 128 packed bytes per row, and
//   * every wavefront requests its activations and its first two tiles at
//     once, and tile t + 2 as soon as tile t has left its registers for LDS:
//     up to 12 KB a wavefront, 192 KB a compute unit, are in flight;
//   * nothing synchronises the wavefronts until the K-slices meet at the end:
//     while one waits for data or sits in the issue of a load, the other three
//     of its SIMD compute.
// A row's 128 bytes of a slice are one cache line; a 16-row tile is two load
// instructions (eight rows each), its table share 8 bytes a row and kind.
#include "qmm_gemv_common.hpp"

namespace qmm {

namespace {

constexpr int kWaves3 = 16;
constexpr int kXStride = 272;                    // LDS pitch of an activation round's row (256 bytes + pad)
constexpr int kWStride = 144;                    // LDS pitch of a tile row (128 bytes + pad): conflict-free 8-byte reads
constexpr int kStage3 = 16 * kXStride;           // wave-private staging (activation round | tile)
constexpr int kTab3 = 2 * 16 * 8;                // wave-private table rows: 16 x 8 bytes of scales, of biases
constexpr int kPart3 = 4 * 4 * kWave * 4;         // wave-private partial sums: up to four tiles x 4 components x 64 lanes
constexpr int kWaveLds3 = kStage3 + kTab3 + kPart3;   // 8704

__device__ __forceinline__ void wave_fence3() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ void split3b(float v, float& hi, float& mid, float& lo) {
  hi = __uint_as_float(__float_as_uint(v) & 0xFFFF0000u);
  const float r1 = v - hi;
  mid = __uint_as_float(__float_as_uint(r1) & 0xFFFF0000u);
  lo = r1 - mid;                                 // at most 8 significant bits: exact in bf16
}

__device__ __forceinline__ uint32_t hi16_pair3(float a, float b) {
  return byte_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}

// GSHIFT: 0 = groups of 64, 1 = groups of 128 (bf16 tables).
template <int BITS, int TMAX, int GSHIFT>
__global__ __launch_bounds__(kWave* kWaves3) void skinny3_kernel(GemvArgs a, int rows_per_wg) {
  constexpr int SB = 128;                        // packed bytes per row per K-slice
  constexpr int KS = SB * 8 / BITS;              // codes per slice: 256 | 128
  constexpr int CPS = KS / 64;                   // 64-code chunks per slice: 4 | 2
  constexpr int XR = KS / 128;                   // activation staging rounds (128 codes each): 2 | 1
  constexpr int TE = CPS >> GSHIFT;              // table entries per row and slice: 4 | 2 | 1
  static_assert(TE >= 2, "a row's table share of a slice is fetched as whole dwords");
  extern __shared__ __align__(16) unsigned char smem3[];

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
  const char* sbase = static_cast<const char*>(a.s) + wz * a.N * ng * 2;
  const char* bbase = static_cast<const char*>(a.b) + wz * a.N * ng * 2;

  unsigned char* buf = smem3 + wave * kWaveLds3;
  unsigned char* tbuf = buf + kStage3;
  float* part = reinterpret_cast<float*>(tbuf + kTab3);          // [tile][component][lane]
  const int xrow4 = lane >> 4, xpiece = lane & 15;              // activation loads: 4 rows x 256 bytes
  const int wrow8 = lane >> 3, wpiece = lane & 7;               // tile loads: 8 rows x 128 bytes
  const uint32_t xst = (uint32_t)(xrow4 * kXStride + xpiece * 16);     // + i * 4 * kXStride
  const uint32_t wst = (uint32_t)(wrow8 * kWStride + wpiece * 16);     // + i * 8 * kWStride

  static_assert(TMAX <= 4, "the partial-sum area holds four tiles");
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  const uint32_t one = pin_vgpr(kOnesBf16x2);
  const bf16x8 ones = as_bf16x8(one, one, one, one);
  const uint32_t nib = pin_vgpr(0x000F000Fu), magic = pin_vgpr(0x43004300u);

  for (int sl = wave; sl < slices; sl += kWaves3) {
    const uint32_t slice_off = (uint32_t)sl * SB;
    const uint32_t tab_off = (uint32_t)((sl * CPS) >> GSHIFT) * 2;
    u32x4 wl[2][2];                               // two tiles in flight: [slot][instruction]
    u32x2 tv[2];                                  // their table runs (scale rows in lanes 0-15, bias rows in 16-31)
    auto load_tile = [&](int t, int slot) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int64_t n = n_begin + t * 16 + 8 * i + wrow8;
        const uint32_t vo = t < ntiles && n < n_end ? (uint32_t)(n * wpr + wpiece * 16) : kOutOfRange;
        wl[slot][i] = __builtin_amdgcn_raw_buffer_load_b128(rw, vo, slice_off, 0);
      }
      // lanes 0-15: the scale run of row r; lanes 16-31: the bias run; one
      // instruction over two base pointers (the other lanes fetch nothing)
      const int64_t n = n_begin + t * 16 + r;
      tv[slot] = u32x2{0u, 0u};
      if (t < ntiles && n < n_end && lane < 32) {
        const char* tp = (lane < 16 ? sbase : bbase) + n * ng * 2 + tab_off;
        if constexpr (TE == 4) tv[slot] = *reinterpret_cast<const u32x2*>(tp);
        else tv[slot][0] = *reinterpret_cast<const uint32_t*>(tp);
      }
    };
    // ---- requests: the first tile (HBM, longest latency), the activations
    // (row blocks at or past M are not fetched), the second tile
    load_tile(0, 0);
    u32x4 xl[XR][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool any = 4 * i < a.M;                              // uniform
#pragma unroll
      for (int rd = 0; rd < XR; ++rd) {
        xl[rd][i] = u32x4{0u, 0u, 0u, 0u};
        if (any) {
          const int m = 4 * i + xrow4;
          const uint32_t vo = m < a.M ? (uint32_t)(((int64_t)m * a.K) * 2 + xpiece * 16) : kOutOfRange;
          xl[rd][i] = __builtin_amdgcn_raw_buffer_load_b128(rx, vo, (uint32_t)(sl * KS + rd * 128) * 2, 0);
        }
      }
    }
    load_tile(1, 1);

    // ---- activations: LDS round trip into operand layout, 128 codes a round
    bf16x8 xa[CPS][2];
#pragma unroll
    for (int rd = 0; rd < XR; ++rd) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<u32x4*>(buf + xst + i * 4 * kXStride) = xl[rd][i];
      wave_fence3();
#pragma unroll
      for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(buf + r * kXStride + cc * 128 + kg * 32 + j * 16);
          if constexpr (BITS == 4) xa[rd * 2 + cc][j] = pair_stride4(v);
          else xa[rd * 2 + cc][j] = __builtin_bit_cast(bf16x8, v);
        }
      wave_fence3();
    }
    // xs_c = sum_k x over chunk c in operand layout, split into three bf16
    // terms and packed as MFMA A operands over the chunk index (kg == 0 lanes;
    // chunk slots past CPS hold zeros)
    bf16x8 axh, axm, axo;
    {
      float xh[8], xm[8], xo[8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float xs = 0.f;
        if (c < CPS) {
          f32x4 t4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xa[c][0], zero, 0, 0, 0);
          t4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xa[c][1], t4, 0, 0, 0);
          xs = kg == 0 ? t4[0] : 0.f;
        }
        split3b(xs, xh[c], xm[c], xo[c]);
      }
      axh = as_bf16x8(hi16_pair3(xh[0], xh[1]), hi16_pair3(xh[2], xh[3]), hi16_pair3(xh[4], xh[5]), hi16_pair3(xh[6], xh[7]));
      axm = as_bf16x8(hi16_pair3(xm[0], xm[1]), hi16_pair3(xm[2], xm[3]), hi16_pair3(xm[4], xm[5]), hi16_pair3(xm[6], xm[7]));
      axo = as_bf16x8(hi16_pair3(xo[0], xo[1]), hi16_pair3(xo[2], xo[3]), hi16_pair3(xo[4], xo[5]), hi16_pair3(xo[6], xo[7]));
    }

    // ---- tiles
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
      if (t < ntiles) {
        const int slot = t & 1;
#pragma unroll
        for (int i = 0; i < 2; ++i)
          *reinterpret_cast<u32x4*>(buf + wst + i * 8 * kWStride) = wl[slot][i];
        if (lane < 32) *reinterpret_cast<u32x2*>(tbuf + lane * 8) = tv[slot];
        wave_fence3();
        if (t + 2 < TMAX) load_tile(t + 2, slot);            // its registers are free again
        // table rows as B operands over the chunk index (this lane's row);
        // the chunk slots past this slice's entries are zero
        const u32x2 sv2 = *reinterpret_cast<const u32x2*>(tbuf + r * 8);
        const u32x2 bv2 = *reinterpret_cast<const u32x2*>(tbuf + 128 + r * 8);
        u32x4 svt, bvt;
        if constexpr (GSHIFT == 0) {
          svt = u32x4{sv2[0], sv2[1], 0u, 0u};
          bvt = u32x4{bv2[0], bv2[1], 0u, 0u};
        } else {                                  // groups of 128: one entry serves two chunks
          svt = u32x4{byte_perm(sv2[0], sv2[0], 0x01000100u), byte_perm(sv2[0], sv2[0], 0x03020302u), 0u, 0u};
          bvt = u32x4{byte_perm(bv2[0], bv2[0], 0x01000100u), byte_perm(bv2[0], bv2[0], 0x03020302u), 0u, 0u};
        }
        const bf16x8 bop = __builtin_bit_cast(bf16x8, bvt);
        f32x4 prev = zero;                        // this wavefront's sums of earlier passes
        if (sl >= kWaves3) {
#pragma unroll
          for (int i = 0; i < 4; ++i) prev[i] = part[(t * 4 + i) * kWave + lane];
        }
        f32x4 accb = __builtin_amdgcn_mfma_f32_16x16x32_bf16(axh, bop, prev, 0, 0, 0);
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
            const u32x2 q = *reinterpret_cast<const u32x2*>(buf + r * kWStride + c * 32 + kg * 8);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][0], widen_int4(q[0], nib, magic), zero, 0, 0, 0);
            d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][1], widen_int4(q[1], nib, magic), d, 0, 0, 0);
          } else {
            const u32x4 q = *reinterpret_cast<const u32x4*>(buf + r * kWStride + c * 64 + kg * 16);
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
#pragma unroll
        for (int i = 0; i < 4; ++i) part[(t * 4 + i) * kWave + lane] = at[i];
        wave_fence3();
      }
    }
  }

  // ---- the K-slices meet: every wavefront's partial sums lie in its own LDS area
  __syncthreads();
  for (int e = threadIdx.x; e < ntiles * 4 * kWave; e += kWave * kWaves3) {
    const int l = e & 63, i = (e >> 6) & 3, t = e >> 8;
    float v = 0.f;
#pragma unroll
    for (int wv = 0; wv < kWaves3; ++wv)
      v += reinterpret_cast<const float*>(smem3 + wv * kWaveLds3 + kStage3 + kTab3)[(t * 4 + i) * kWave + l];
    const int m = 4 * (l >> 4) + i;
    const int64_t n = n_begin + t * 16 + (l & 15);
    if (m < a.M && n < n_end) store_out(a.y, (bz * a.M + m) * (int64_t)a.N + n, v, a.y_dtype);
  }
}

template <int BITS, int TMAX, int GSHIFT>
void launch3(const GemvArgs& a, int64_t batch, int rows_per_wg, hipStream_t st) {
  dim3 grid((unsigned)ceil_div(a.N, rows_per_wg), (unsigned)batch);
  constexpr size_t lds = (size_t)kWaves3 * kWaveLds3;
  constexpr auto kern = skinny3_kernel<BITS, TMAX, GSHIFT>;
  if (!lds_limit<kern>(lds)) return;
  hipLaunchKernelGGL(kern, grid, dim3(kWave * kWaves3), lds, st, a, rows_per_wg);
}

template <int BITS, int GSHIFT>
void launch3_t(const GemvArgs& a, int64_t batch, int rows_per_wg, hipStream_t st) {
  const int tmax = (rows_per_wg + 15) / 16;
  if (tmax <= 2) launch3<BITS, 2, GSHIFT>(a, batch, rows_per_wg, st);
  else launch3<BITS, 4, GSHIFT>(a, batch, rows_per_wg, st);
}

}  // namespace

// Shapes this kernel serves: bf16 tables, every wavefront of a workgroup with
// a K-slice of its own in every pass, at most four tiles a workgroup.
bool skinny3_supported(int64_t N, int64_t K, int gs, int bits, int rows_per_wg) {
  if (bits == 8 && gs != 64) return false;       // a row's table share of a slice must be whole dwords
  const int64_t ks = 128 * 8 / bits;
  return K % (ks * kWaves3) == 0 && rows_per_wg <= 64 && N * (K * bits / 8) < 0x7FFFFFFFll;
}

// Where the kernel is used.  QMM_SKINNY3 (experiments build): 1 = wherever it
// can run, 0 = nowhere.
bool skinny3_wanted(int64_t M, int64_t N, int64_t K, int gs, int bits, int* rows_per_wg) {
  static const char* const env = experiment_env("QMM_SKINNY3");
  static const int cus = [] {
    int dev = 0, n = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
      hipDeviceProp_t p;
      if (hipGetDeviceProperties(&p, dev) == hipSuccess && p.multiProcessorCount > 0) n = p.multiProcessorCount;
    }
    return n;
  }();
  int64_t rows = ceil_div(N, (int64_t)cus);
  if (rows < 16) rows = 16;
  *rows_per_wg = (int)rows;
  if (!skinny3_supported(N, K, gs, bits, (int)rows)) return false;
  if (env) return env[0] == '1';
  (void)M;
  return false;
}

void skinny3_dispatch(const GemvArgs& a0, int64_t batch, int gs, int bits, int rows_per_wg,
                      hipStream_t st) {
  GemvArgs a = a0;
  a.gshift = gs == 128 ? 1 : 0;
  if (bits == 4) {
    if (gs == 128) launch3_t<4, 1>(a, batch, rows_per_wg, st);
    else launch3_t<4, 0>(a, batch, rows_per_wg, st);
  } else {
    launch3_t<8, 0>(a, batch, rows_per_wg, st);
  }
}

}  // namespace qmm
