// MXFP4 quantized matmul on the gfx950 block-scaled matrix cores
// (v_mfma_scale_f32_32x32x64_f8f6f4), for M > 16 and K a multiple of 512.
//
// y[m, n] = sum_k x[m, k] * E2M1[code[n, k]] * 2^(scale[n, k/32] - 127)
//
// The weight operand goes to the matrix core exactly as stored: 32 four-bit
// codes (16 bytes) a lane plus the E8M0 byte of that 32-block, so the
// dequantized weight is exact by construction.  The instruction needs the
// other operand in a block-scaled narrow format too, so the bf16 activations
// are split once per call into two FP6 (E2M3) terms, each with one E8M0 scale
// per 32 elements:
//     x = hi + lo + eps,   hi = fp6(x),  lo = fp6(x - hi)   (x - hi is exact)
// which leaves |eps| around 3e-4 of |x| (rms over a 32-block), far inside the
// output tolerance, at the cost of issuing two MFMAs per useful one.
//
// Kernel 1 (mx_split_kernel): x [R, K] bf16 -> the two FP6 terms in the order
// the matrix core reads them.  A lane's operand is one row's 32-block: 24
// bytes a term, 48 bytes for both = three 16-byte planes (hi | lo back to
// back).  For K-step ks (128 elements = 32-blocks kb = 0..3; one 32x32x64 MFMA
// covers blocks 2u, 2u+1):
//     aq[ks][plane][kb][row]     (16 bytes each, rows contiguous)
// so a wavefront's operand load is two 512-byte runs for any first row, and
//     as[ks/4][t][kb][row]       (4 bytes: the E8M0 bytes of K-steps 4q..4q+3)
// so one scale register serves four K-steps through the instruction's byte
// select.
//
// Kernel 2 (mxfp4_mfma_kernel): one workgroup = a 64 x 128 output tile, four
// wavefronts that split K (wavefront w owns K-quads w, w+4, ...; a quad is
// four K-steps) and are summed through LDS at the end.  No barrier in the main
// loop: each wavefront stages its own weight codes.
//   * weight codes: direct-to-LDS loads, 16 bytes a lane, four lanes = one
//     row's 64 bytes of a K-step (coalesced), into a 4-deep ring; read back
//     with ds_read_b128 in operand order (lane = column i, block 2u + lane/32).
//     The 16-byte piece p of row i sits at piece p ^ ((i >> 2) & 3), applied on
//     the global side of the load, so a 16-lane read phase covers all banks.
//   * weight scales: 16 bytes a row per K-quad, direct-to-LDS, double buffered;
//     the lane shifts its block's byte to bits 0-7.
//   * activation terms: straight from global (L2-resident) into operand
//     registers, one K-step ahead.
// Per K-step a wavefront issues 32 MFMAs of 32x32x64 (2 K-halves x 2 terms x 2
// row tiles x 4 column tiles) against 24 + 8 loads.  (The 16x16x128 form of
// the instruction sustains well under half the rate of the 32x32x64 form.)
#include <type_traits>
#include <utility>

#include "qmm_common.hpp"

namespace qmm {

namespace {

typedef __attribute__((ext_vector_type(32))) __bf16 bf16x32;
typedef __attribute__((ext_vector_type(32))) float f32x32;
typedef __attribute__((ext_vector_type(16))) unsigned u32x16;
typedef __attribute__((ext_vector_type(6))) unsigned u32x6;

constexpr int TM = 64, TN = 128;
constexpr int kStageBytes = TN * 64;             // 128 rows x 64 bytes of codes: one K-step
constexpr int kStages = 4;
constexpr int kScaleBytes = TN * 16;             // 128 rows x 16 scale bytes: one K-quad
constexpr int kWaveLds = kStages * kStageBytes + 2 * kScaleBytes;   // 36864
constexpr int kLds = 4 * kWaveLds;               // 147456
constexpr uint32_t kOutOfRange = 0x80000000u;
constexpr int kFp6 = 2, kFp4 = 4;                // matrix-core format selectors (E2M3, E2M1)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  const uint32_t n = bytes > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {    // s_waitcnt vmcnt(N) only; also a compiler barrier
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
  asm volatile("" ::: "memory");
}

typedef __attribute__((address_space(3))) void lds_void;

__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t r, unsigned char* dst, uint32_t voff,
                                      uint32_t soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)dst, 16, voff, soff, 0, 0);
}

// E8M0 byte of the scale that maps a block whose largest magnitude has float
// exponent field `e` into the FP6 E2M3 range (largest binade 4 .. 7.5).
__device__ __forceinline__ uint32_t block_scale_byte(uint32_t e) {
  const int b = (int)e - 2;
  return (uint32_t)(b < 1 ? 1 : (b > 254 ? 254 : b));
}

// ---------------------------------------------------------------------------
// x [x_rows, K] bf16 (rows optionally gathered through lhs_idx) -> two FP6
// terms + scales in matrix-core operand order.
// One thread = one (row, 32-block); consecutive threads = consecutive rows.
__global__ __launch_bounds__(256) void mx_split_kernel(const uint16_t* __restrict__ x,
                                                       const int32_t* __restrict__ lhs_idx,
                                                       u32x4* __restrict__ aq,
                                                       uint8_t* __restrict__ as, int R, int x_rows,
                                                       int K, int Rp) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int row = (int)(idx % Rp);
  const int blk = (int)(idx / Rp);
  if (blk >= K / 32 || row >= R) return;
  const int64_t srow = lhs_idx ? (int64_t)lhs_idx[row] : (int64_t)row;
  const bool ok = srow >= 0 && srow < x_rows;      // an index outside x gathers a zero row
  const u32x4* src = reinterpret_cast<const u32x4*>(x + (ok ? srow : 0) * K + blk * 32);
  u32x16 raw;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const u32x4 v = ok ? src[i] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 4; ++j) raw[4 * i + j] = v[j];
  }
  uint32_t amax = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t lo = raw[i] & 0x7FFFu, hi = (raw[i] >> 16) & 0x7FFFu;
    amax = max(amax, max(lo, hi));
  }
  const uint32_t byte_hi = block_scale_byte(amax >> 7);
  const float scale_hi = __uint_as_float(byte_hi << 23);
  const bf16x32 xv = __builtin_bit_cast(bf16x32, raw);
  const u32x6 hi6 = __builtin_amdgcn_cvt_scalef32_pk32_fp6_bf16(xv, scale_hi);
  const f32x32 back = __builtin_amdgcn_cvt_scalef32_pk32_f32_fp6(hi6, scale_hi);
  // residual: exact in float32, and representable in bf16 (a multiple of
  // ulp(x) that is smaller than x), so the truncation below loses nothing
  u32x16 res;
  uint32_t rmax = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float r0 = __uint_as_float(raw[i] << 16) - back[2 * i];
    const float r1 = __uint_as_float(raw[i] & 0xFFFF0000u) - back[2 * i + 1];
    const uint32_t b0 = __float_as_uint(r0), b1 = __float_as_uint(r1);
    rmax = max(rmax, max(b0 & 0x7FFFFFFFu, b1 & 0x7FFFFFFFu));
    res[i] = (b0 >> 16) | (b1 & 0xFFFF0000u);
  }
  const uint32_t byte_lo = block_scale_byte(rmax >> 23);
  const float scale_lo = __uint_as_float(byte_lo << 23);
  const u32x6 lo6 = __builtin_amdgcn_cvt_scalef32_pk32_fp6_bf16(__builtin_bit_cast(bf16x32, res), scale_lo);

  const int ks = blk >> 2, kb = blk & 3;
  const u32x4 planes[3] = {u32x4{hi6[0], hi6[1], hi6[2], hi6[3]}, u32x4{hi6[4], hi6[5], lo6[0], lo6[1]},
                           u32x4{lo6[2], lo6[3], lo6[4], lo6[5]}};
#pragma unroll
  for (int p = 0; p < 3; ++p) aq[(((int64_t)ks * 3 + p) * 4 + kb) * Rp + row] = planes[p];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int64_t so = ((((int64_t)(ks >> 2) * 2 + t) * 4 + kb) * Rp + row) * 4 + (ks & 3);
    as[so] = (uint8_t)(t ? byte_lo : byte_hi);
  }
}

// ---------------------------------------------------------------------------
struct MxArgs {
  const void* aq;        // split activations (see the file comment)
  const void* as;
  const void* w;         // uint8 [N, K/2]
  const void* s;         // uint8 [N, K/32]
  void* y;               // [R, N]
  const int32_t* row_offsets;   // [E+1] or null: rows [o[e], o[e+1]) use expert e's weight
  const int32_t* out_idx;       // optional row scatter for y
  int R, N, K, Rp, E;
  int y_dtype;
  int m_tiles, n_tiles;  // provisioned row tiles (>= the tiles that exist when grouped)
};

// The two FP6 terms of a lane's 48 bytes (three 16-byte planes, hi | lo).
__device__ __forceinline__ i32x8 fp6_term(const u32x4 (&p)[3], int term) {
  if (term == 0) return i32x8{(int)p[0][0], (int)p[0][1], (int)p[0][2], (int)p[0][3], (int)p[1][0], (int)p[1][1], 0, 0};
  return i32x8{(int)p[1][2], (int)p[1][3], (int)p[2][0], (int)p[2][1], (int)p[2][2], (int)p[2][3], 0, 0};
}

__device__ __forceinline__ i32x8 as_fp4_operand(u32x4 v) {
  return i32x8{(int)v[0], (int)v[1], (int)v[2], (int)v[3], 0, 0, 0, 0};
}

__global__ __launch_bounds__(256) void mxfp4_mfma_kernel(MxArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 31, kh = lane >> 5;       // operand row / column, 32-block within a 64-wide MFMA

  // Workgroups are dealt to the 8 XCDs round-robin in launch order; XCD x is
  // handed a contiguous run of tiles, row-tile fastest, so the workgroups that
  // share one L2 share weight column tiles.
  // Grouped: the grid is provisioned for the worst raggedness; the row tiles
  // that exist are counted first and only those are dealt; a tile never
  // straddles two experts.
  int m_tiles = a.m_tiles;
  if (a.row_offsets) m_tiles = find_row_tile(a.row_offsets, a.E, a.R, TM, -1).m_tiles;   // counted only
  if (m_tiles == 0) return;
  const int total = m_tiles * a.n_tiles;
  const int per = (total + 7) / 8;
  const int tile = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per || tile >= total) return;
  int e = 0, row_hi = a.R, m0 = (tile % m_tiles) * TM;
  const int n0 = (tile / m_tiles) * TN;
  if (a.row_offsets) {
    const RowTile rt = find_row_tile(a.row_offsets, a.E, a.R, TM, tile % m_tiles);
    if (!rt.found) return;
    e = rt.e; m0 = rt.lo + rt.idx * TM; row_hi = rt.hi;
  }

  const int nquads = a.K / 512;
  const int nq = nquads > wave ? (nquads - wave + 3) / 4 : 0;       // this wavefront's quads
  const int last_step = 4 * nq - 1;
  auto kstep_of = [&](int i) {                    // wave-local step -> K-step (clamped)
    i = i < last_step ? i : last_step;
    return 4 * (wave + 4 * (i >> 2)) + (i & 3);
  };

  const int64_t wpitch = a.K / 2, spitch = a.K / 32;
  const auto rw = make_rsrc(static_cast<const char*>(a.w) + (int64_t)e * a.N * wpitch, (int64_t)a.N * wpitch);
  const auto rs = make_rsrc(static_cast<const char*>(a.s) + (int64_t)e * a.N * spitch, (int64_t)a.N * spitch);
  const auto ra = make_rsrc(a.aq, (int64_t)(a.K / 128) * 192 * a.Rp);
  const auto rsa = make_rsrc(a.as, (int64_t)nquads * 32 * a.Rp);

  unsigned char* wbase = smem + wave * kWaveLds;
  unsigned char* sbase = wbase + kStages * kStageBytes;

  // loop-invariant lane offsets
  uint32_t wvo[8];                                // weight codes: row 16j + lane/4, piece swizzled
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int n = n0 + 16 * j + (lane >> 2);
    const int gp = (lane & 3) ^ ((lane >> 4) & 3);
    wvo[j] = n < a.N ? (uint32_t)(n * wpitch + gp * 16) : kOutOfRange;
  }
  uint32_t svo[2];                                // weight scales: row 64h + lane
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int n = n0 + 64 * h + lane;
    svo[h] = n < a.N ? (uint32_t)(n * spitch) : kOutOfRange;
  }
  const uint32_t avo = (uint32_t)((kh * a.Rp + m0 + li) * 16);      // + mt*512; block 2u+kh via the scalar offset
  const uint32_t savo = (uint32_t)((kh * a.Rp + m0 + li) * 4);      // + mt*128
  // codes of row r, block kb sit at r*64 + ((kb ^ ((r >> 2) & 3)) << 4)
  const uint32_t rd_row = (uint32_t)(li * 64);
  const uint32_t rd_swz = (uint32_t)((li >> 2) & 3);
  const uint32_t rd_off[2] = {rd_row + (((0u + kh) ^ rd_swz) << 4), rd_row + (((2u + kh) ^ rd_swz) << 4)};
  const uint32_t sh[2] = {(uint32_t)kh * 8, (uint32_t)kh * 8 + 16};  // this lane's scale byte within a K-step's dword

  f32x16 acc[2][4];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][nt][r] = 0.f;

  u32x4 areg[4][2][2][3];                         // [buffer][u][mt][plane]
  uint32_t sa[2][2][2], sa_nxt[2][2][2];          // [u][mt][term]
  u32x4 sbq[4];

  // The 12 activation loads and 8 weight loads of a K-step are issued in four
  // parts (g = 0..3) so they can be spread between the MFMAs of another step.
  auto issue_a_part = [&](int ks, u32x4 (&dst)[2][2][3], int g) {
#pragma unroll
    for (int j = 3 * g; j < 3 * g + 3; ++j) {
      const int p = j >> 2, u = (j >> 1) & 1, mt = j & 1;
      const uint32_t so = (uint32_t)(((ks * 3 + p) * 4 + 2 * u) * 16) * (uint32_t)a.Rp;
      dst[u][mt][p] = __builtin_amdgcn_raw_buffer_load_b128(ra, avo + mt * 512, so, 0);
    }
  };
  auto issue_a = [&](int ks, u32x4 (&dst)[2][2][3]) {
#pragma unroll
    for (int g = 0; g < 4; ++g) issue_a_part(ks, dst, g);
  };
  auto issue_sa = [&](int quad, uint32_t (&dst)[2][2][2]) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const uint32_t so = (uint32_t)(((quad * 2 + t) * 4 + 2 * u) * 4) * (uint32_t)a.Rp;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
          dst[u][mt][t] = __builtin_amdgcn_raw_buffer_load_b32(rsa, savo + mt * 128, so, 0);
      }
  };
  auto dma_w_part = [&](int ks, int stage, int g) {
#pragma unroll
    for (int j = 2 * g; j < 2 * g + 2; ++j)
      dma16(rw, wbase + stage * kStageBytes + j * 1024, wvo[j], (uint32_t)ks * 64);
  };
  auto dma_w = [&](int ks, int stage) {
#pragma unroll
    for (int g = 0; g < 4; ++g) dma_w_part(ks, stage, g);
  };
  auto dma_s = [&](int quad, int par) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
      dma16(rs, sbase + par * kScaleBytes + h * 1024, svo[h], (uint32_t)quad * 16);
  };
  auto quad_of = [&](int qi) { return wave + 4 * (qi < nq - 1 ? qi : nq - 1); };

  // Loads retire in order, so a wait can only say "all but the newest n have
  // landed": the order of issue has to be the order of use.  A K-step i uses
  // its activation terms A(i) and its weight codes W(i); step i issues A(i+1)
  // during its first two MFMA groups and W(i+2) during its last two, and
  // before its last group waits for W(i+1) and reads its fragments, so that a
  // step starts with its weight operands already in registers.  The prologue issues in the same
  // order (W0 A0 W1), which keeps every count in the loop valid on its
  // first pass.  A step issues 20 loads, the first of a quad 10 more (its
  // activation scales and the next quad's weight scales).  (Asking further
  // ahead -- A(i+2), W(i+3) -- measured 2 % slower on C4: a wavefront keeps
  // about sixteen loads in flight and sits in issue beyond that.)
  i32x8 bfq[2][2][4];                             // [step parity][u][nt] weight fragments
  auto read_bf = [&](int stage, i32x8 (&dst)[2][4]) {
    const unsigned char* st = wbase + stage * kStageBytes;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
        dst[u][nt] = as_fp4_operand(*reinterpret_cast<const u32x4*>(st + rd_off[u] + nt * 2048));
  };
  auto read_sbq = [&](int par) {
    const unsigned char* sq = sbase + par * kScaleBytes + li * 16;
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) sbq[nt] = *reinterpret_cast<const u32x4*>(sq + nt * 512);
  };
  if (nq > 0) {
    issue_sa(quad_of(0), sa);
    dma_s(quad_of(0), 0);
    dma_w(kstep_of(0), 0);
    issue_a(kstep_of(0), areg[0]);
    dma_w(kstep_of(1), 1);
    wait_vmcnt<20>();                              // W0 and the first scales
    read_bf(0, bfq[0]);
    read_sbq(0);
    auto step = [&](int qi, auto tc) __attribute__((always_inline)) {
      constexpr int t = decltype(tc)::value;
      const int i = 4 * qi + t;
      // A(i) has landed once at most W(i+1), the loads issued after it, are out
      wait_vmcnt<8>();
      const int ks_a = kstep_of(i + 1), ks_w = kstep_of(i + 2);
      int sb[2][4];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) sb[u][nt] = (int)(sbq[nt][t] >> sh[u]);
      // Four groups of 8 MFMAs, each followed by a share of the loads for later
      // steps, so that load issue hides under the matrix-core work of this
      // single wavefront per SIMD.
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int u = g >> 1, term = g & 1;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const i32x8 af = fp6_term(areg[t][u][mt], term);
#pragma unroll
          for (int nt = 0; nt < 4; ++nt) {
            acc[mt][nt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                af, bfq[t & 1][u][nt], acc[mt][nt], kFp6, kFp4, t, (int)sa[u][mt][term], 0, sb[u][nt]);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (g < 2) {
          issue_a_part(ks_a, areg[(t + 1) & 3], 2 * g);
          issue_a_part(ks_a, areg[(t + 1) & 3], 2 * g + 1);
          if (t == 0 && g == 0) {
            issue_sa(quad_of(qi + 1), sa_nxt);
            dma_s(quad_of(qi + 1), (qi + 1) & 1);
          }
        } else {
          dma_w_part(ks_w, (t + 2) & 3, 2 * (g - 2));
          dma_w_part(ks_w, (t + 2) & 3, 2 * (g - 2) + 1);
        }
        if (g == 2) {
          // W(i+1): everything but the previous step's loads and this step's so far;
          // the fragment reads then run under the last MFMA group
          wait_vmcnt<(t == 0 ? 26 : 16)>();
          read_bf((t + 1) & 3, bfq[(t + 1) & 1]);
          if (t == 3) read_sbq((qi + 1) & 1);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (t == 3) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int mt = 0; mt < 2; ++mt) {
            sa[u][mt][0] = sa_nxt[u][mt][0];
            sa[u][mt][1] = sa_nxt[u][mt][1];
          }
      }
    };
    for (int qi = 0; qi < nq; ++qi) {
      step(qi, std::integral_constant<int, 0>{});
      step(qi, std::integral_constant<int, 1>{});
      step(qi, std::integral_constant<int, 2>{});
      step(qi, std::integral_constant<int, 3>{});
    }
  }
  // every direct-to-LDS load (including the clamped repeats) must have landed
  // before the staging area is reused for the reduction
  wait_vmcnt<0>();
  __syncthreads();

  // ---- sum the four K-slices: red[wave][tile = mt*4+nt][r][lane]
  float* red = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        red[(((wave * 8 + mt * 4 + nt) * 16) + r) * 64 + lane] = acc[mt][nt][r];
  __syncthreads();
  // wavefront w finishes tiles 2w and 2w+1 (row tile w/2, column tiles 2(w%2), +1)
  const int mt = wave >> 1, nh = wave & 1;
  float v[2][16];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) t += red[(((w * 8 + 2 * wave + h) * 16) + r) * 64 + lane];
      v[h][r] = t;
    }
  const bool wide = a.y_dtype != QMM_F32 && (a.N & 7) == 0 &&
                    (reinterpret_cast<uintptr_t>(a.y) & 15u) == 0;
  if (wide) {
    // 16-bit outputs: transpose this wavefront's 32 x 64 block through the LDS
    // left over beside `red`, then store 16 bytes a lane (128 bytes a row)
    uint16_t* o16 = reinterpret_cast<uint16_t*>(smem + 4 * 8 * 16 * 64 * 4) + wave * (32 * 64);
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int rl = 8 * (r >> 2) + 4 * kh + (r & 3), cl = 32 * h + li;
        o16[rl * 64 + cl] = (uint16_t)(a.y_dtype == QMM_BF16 ? f32_to_bf16_bits(v[h][r]) : f32_to_f16_bits(v[h][r]));
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int idx = q * 64 + lane, rl = idx >> 3, pc = idx & 7;
      const int row = m0 + 32 * mt + rl, col = n0 + 64 * nh + pc * 8;
      if (row < row_hi && col < a.N) {
        const int64_t orow = a.out_idx ? (int64_t)a.out_idx[row] : (int64_t)row;
        *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(a.y) + orow * a.N + col) =
            *reinterpret_cast<const u32x4*>(o16 + rl * 64 + pc * 8);
      }
    }
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + 32 * mt + 8 * (r >> 2) + 4 * kh + (r & 3), col = n0 + 32 * (2 * nh + h) + li;
        if (row < row_hi && col < a.N) {
          const int64_t orow = a.out_idx ? (int64_t)a.out_idx[row] : (int64_t)row;
          store_out(a.y, orow * a.N + col, v[h][r], a.y_dtype);
        }
      }
  }
}


// ---------------------------------------------------------------------------
// The eight-wavefront form (K a multiple of 2048).  What bounds the kernel
// above is not the matrix core: with the MFMAs compiled out it is 10 % faster,
// with the weight loads emptied 40 %.  A wavefront keeps about sixteen loads in
// flight, so four wavefronts have 64 KB a compute unit out against latencies of
// 0.8 us (activation terms out of L2) to 1.6 us and more (weight lines), and a
// wavefront that sits in issue behind its loads issues no MFMA either.  Here
// the same 64 x 128 tile is worked by eight wavefronts, two a SIMD: K quarter
// kq = wave % 4 as before, and the tile's rows in halves mh = wave / 4, so a
// wavefront multiplies 32 x 128 (64 accumulator registers, 16 MFMAs a K-step)
// and the SIMD has the other wavefront's MFMAs to issue while one waits.
//   * weight codes: the two wavefronts of a K quarter share one ring of two
//     stages, a stage = 128 rows x 128 bytes = two K-steps, i.e. whole cache
//     lines (the 64-byte halves of the form above fetch every line twice);
//     each of the two requests half of the rows; piece p of row r at position
//     p ^ ((r >> 1) & 7), so that a 16-lane read pass covers every bank once.
//   * one workgroup barrier a stage: before it a wavefront waits for its share
//     of the stage's codes and finishes its reads of the stage before; after
//     it the stage before is refilled with the stage after.
//   * activation terms: straight into registers as above, two K-steps ahead.
constexpr int kStage8 = TN * 128;
constexpr int kKqLds8 = 2 * kStage8 + 2 * kScaleBytes;     // 36864
constexpr int kLds8 = 4 * kKqLds8;                         // 147456

__device__ __forceinline__ void stage_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__global__ __launch_bounds__(512) void mxfp4_mfma8_kernel(MxArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kq = wave & 3, mh = wave >> 2;
  const int li = lane & 31, kh = lane >> 5;

  int m_tiles = a.m_tiles;
  if (a.row_offsets) m_tiles = find_row_tile(a.row_offsets, a.E, a.R, TM, -1).m_tiles;   // counted only
  if (m_tiles == 0) return;
  const int total = m_tiles * a.n_tiles;
  const int per = (total + 7) / 8;
  const int tile = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
  if ((int)(blockIdx.x >> 3) >= per || tile >= total) return;
  int e = 0, row_hi = a.R, m0 = (tile % m_tiles) * TM;
  const int n0 = (tile / m_tiles) * TN;
  if (a.row_offsets) {
    const RowTile rt = find_row_tile(a.row_offsets, a.E, a.R, TM, tile % m_tiles);
    if (!rt.found) return;
    e = rt.e; m0 = rt.lo + rt.idx * TM; row_hi = rt.hi;
  }

  const int nq = a.K / 2048;                      // quads of this K quarter: kq, kq + 4, ...
  const int64_t wpitch = a.K / 2, spitch = a.K / 32;
  const auto rw = make_rsrc(static_cast<const char*>(a.w) + (int64_t)e * a.N * wpitch, (int64_t)a.N * wpitch);
  const auto rs = make_rsrc(static_cast<const char*>(a.s) + (int64_t)e * a.N * spitch, (int64_t)a.N * spitch);
  const auto ra = make_rsrc(a.aq, (int64_t)(a.K / 128) * 192 * a.Rp);
  const auto rsa = make_rsrc(a.as, (int64_t)(a.K / 512) * 32 * a.Rp);

  unsigned char* wring = smem + kq * kKqLds8;
  unsigned char* sring = wring + 2 * kStage8;

  // weight codes: request j of this wavefront covers rows 64 mh + 8 j + lane / 8, a row's 128 bytes
  uint32_t wvo[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int row = 64 * mh + 8 * j + (lane >> 3);
    const int n = n0 + row;
    const int gp = (lane & 7) ^ ((row >> 1) & 7);
    wvo[j] = n < a.N ? (uint32_t)(n * wpitch + gp * 16) : kOutOfRange;
  }
  const int sn = n0 + 64 * mh + lane;             // weight scales: this lane's row
  const uint32_t svo = sn < a.N ? (uint32_t)(sn * spitch) : kOutOfRange;
  const uint32_t avo = (uint32_t)((kh * a.Rp + m0 + 32 * mh + li) * 16);
  const uint32_t savo = (uint32_t)((kh * a.Rp + m0 + 32 * mh + li) * 4);
  // codes of tile row r, piece p (16 bytes = one 32-block; a K-step is four) at r*128 + ((p ^ ((r >> 1) & 7)) << 4)
  const uint32_t rd_row = (uint32_t)(li * 128);
  const uint32_t rd_swz = (uint32_t)((li >> 1) & 7);

  f32x16 acc[4];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nt][r] = 0.f;

  u32x4 areg[4][2][3];                            // [K-step of the quad][u][plane]
  uint32_t sa[2][2], sa_nxt[2][2];                // [u][term]

  // (Requests past the last quad repeat the last quad's: every wavefront issues the same number of
  // loads a stage whatever its position, the waits count loads.)
  auto issue_a = [&](int i, int tq, u32x4 (&dst)[2][3]) {      // K-step tq of this wavefront's quad i
    const int ks = 4 * (kq + 4 * (i < nq ? i : nq - 1)) + tq;
#pragma unroll
    for (int p = 0; p < 3; ++p)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const uint32_t so = (uint32_t)(((ks * 3 + p) * 4 + 2 * u) * 16) * (uint32_t)a.Rp;
        dst[u][p] = __builtin_amdgcn_raw_buffer_load_b128(ra, avo, so, 0);
      }
  };
  auto issue_scales = [&](int i) {                // activation and weight scales of quad i: 5 loads
    const int quad = kq + 4 * (i < nq ? i : nq - 1);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const uint32_t so = (uint32_t)(((quad * 2 + t) * 4 + 2 * u) * 4) * (uint32_t)a.Rp;
        sa_nxt[u][t] = __builtin_amdgcn_raw_buffer_load_b32(rsa, savo, so, 0);
      }
    dma16(rs, sring + (i & 1) * kScaleBytes + mh * 1024, svo, (uint32_t)quad * 16);
  };
  auto dma_w = [&](int i, int h) {                // stage (quad i, half h) into slot h: 8 loads
    const uint32_t so = (uint32_t)((kq + 4 * (i < nq ? i : nq - 1)) * 256 + h * 128);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      dma16(rw, wring + h * kStage8 + mh * 8192 + j * 1024, wvo[j], so);
  };

  // Loads retire in order; the order of issue is
  //   [scales of quad 0] W(0) A(0) A(1) | after barrier s: [scales of the next quad, in the second
  //   stage of a quad] W(s+1), then A(2s+2) and A(2s+3) during the stage's two K-steps,
  // so before barrier s only this stage's two A sets (12 loads) may be out, and before K-step t of a
  // stage the A set after it, W(s+1) and the scale loads: 14 or 19.
  issue_scales(0);
  dma_w(0, 0);
  issue_a(0, 0, areg[0]);
  issue_a(0, 1, areg[1]);

  auto stage = [&](int i, auto hc) __attribute__((always_inline)) {
    constexpr int h = decltype(hc)::value;
    wait_vmcnt<12>();
    stage_barrier();
    if constexpr (h == 0) {
#pragma unroll
      for (int u = 0; u < 2; ++u) { sa[u][0] = sa_nxt[u][0]; sa[u][1] = sa_nxt[u][1]; }
    } else {
      issue_scales(i + 1);
    }
    if constexpr (h == 0) dma_w(i, 1); else dma_w(i + 1, 0);
    const unsigned char* st = wring + h * kStage8;
    const unsigned char* sq = sring + (i & 1) * kScaleBytes + li * 16;
    auto kstep = [&](auto tc) __attribute__((always_inline)) {
      constexpr int t = decltype(tc)::value;
      constexpr int tq = 2 * h + t;
      wait_vmcnt<(h == 1 ? 19 : 14)>();
      if constexpr (tq < 2) issue_a(i, tq + 2, areg[(tq + 2) & 3]); else issue_a(i + 1, tq - 2, areg[(tq + 2) & 3]);
      uint32_t sbw[4];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) sbw[nt] = *reinterpret_cast<const uint32_t*>(sq + nt * 512 + tq * 4);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        i32x8 bf[4];
        const uint32_t pc = (uint32_t)(4 * t + 2 * u + kh);
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
          bf[nt] = as_fp4_operand(*reinterpret_cast<const u32x4*>(st + nt * 4096 + rd_row + ((pc ^ rd_swz) << 4)));
#pragma unroll
        for (int term = 0; term < 2; ++term) {
          const i32x8 af = fp6_term(areg[tq][u], term);
#pragma unroll
          for (int nt = 0; nt < 4; ++nt) {
            acc[nt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                af, bf[nt], acc[nt], kFp6, kFp4, tq, (int)sa[u][term], 0, (int)(sbw[nt] >> (8 * kh + 16 * u)));
          }
        }
      }
    };
    kstep(std::integral_constant<int, 0>{});
    kstep(std::integral_constant<int, 1>{});
  };
  for (int i = 0; i < nq; ++i) {
    stage(i, std::integral_constant<int, 0>{});
    stage(i, std::integral_constant<int, 1>{});
  }
  wait_vmcnt<0>();
  __syncthreads();

  // ---- sum the four K quarters: red[wave][nt][r][lane]
  float* red = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) red[(((wave * 4 + nt) * 16) + r) * 64 + lane] = acc[nt][r];
  __syncthreads();
  // wavefront w finishes the 32 x 32 block of row half w / 4, column block w % 4
  const int fm = wave >> 2, fn = wave & 3;
  float v[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    float t = 0.f;
#pragma unroll
    for (int q = 0; q < 4; ++q) t += red[((((q + 4 * fm) * 4 + fn) * 16) + r) * 64 + lane];
    v[r] = t;
  }
  const bool wide = a.y_dtype != QMM_F32 && (a.N & 7) == 0 && (reinterpret_cast<uintptr_t>(a.y) & 15u) == 0;
  if (wide) {
    // 16-bit outputs: transpose the block through the LDS left over beside `red`, store 16 bytes a lane
    uint16_t* o16 = reinterpret_cast<uint16_t*>(smem + 8 * 4 * 16 * 64 * 4) + wave * (32 * 32);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int rl = 8 * (r >> 2) + 4 * kh + (r & 3);
      o16[rl * 32 + li] = (uint16_t)(a.y_dtype == QMM_BF16 ? f32_to_bf16_bits(v[r]) : f32_to_f16_bits(v[r]));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int idx = q * 64 + lane, rl = idx >> 2, pc = idx & 3;
      const int row = m0 + 32 * fm + rl, col = n0 + 32 * fn + pc * 8;
      if (row < row_hi && col < a.N) {
        const int64_t orow = a.out_idx ? (int64_t)a.out_idx[row] : (int64_t)row;
        *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(a.y) + orow * a.N + col) =
            *reinterpret_cast<const u32x4*>(o16 + rl * 32 + pc * 8);
      }
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = m0 + 32 * fm + 8 * (r >> 2) + 4 * kh + (r & 3), col = n0 + 32 * fn + li;
      if (row < row_hi && col < a.N) {
        const int64_t orow = a.out_idx ? (int64_t)a.out_idx[row] : (int64_t)row;
        store_out(a.y, orow * a.N + col, v[r], a.y_dtype);
      }
    }
  }
}

}  // namespace

// Rows of the split-activation workspace (row count rounded up to the tile).
// (a tile of a row group may start at any row, so a full tile past the last row is provisioned)
static int64_t mx_rows(int64_t R) { return ceil_div(R + TM, TM) * TM; }

bool mxfp4_mfma_supported(int64_t R, int64_t N, int64_t K) {
  if (experiment_env("QMM_NO_MXFP4_MFMA")) return false;
  return K > 0 && K % 512 == 0 && N * (K / 2) < (1ll << 31) && mx_rows(R) * K * 3 / 2 < (1ll << 32) &&
         mx_rows(R) * 4 * 8 < (1ll << 31);
}

size_t mxfp4_workspace_bytes(int64_t R, int64_t K) {
  const int64_t rp = mx_rows(R);
  return (size_t)(rp * K * 3 / 2 + (K / 512) * 32 * rp);
}

void mxfp4_geometry(int64_t R, int64_t N, int64_t K, int* grid, int* block) {
  const int64_t tiles = ceil_div(R, TM) * ceil_div(N, TN);
  *grid = (int)(ceil_div(tiles, 8) * 8);
  *block = K % 2048 == 0 ? 512 : 256;            // the eight-wavefront form | the four-wavefront form
}

// x bf16 [x_rows, K] (rows gathered through lhs_idx when given); w uint8 [E, N, K/2];
// s uint8 [E, N, K/32]; y [R, N] (rows scattered through out_idx when given);
// row_offsets [E+1] or null (one weight); workspace as sized above.
void mxfp4_mfma_dispatch(const void* x, const void* w, const void* s, void* y, int y_dtype,
                         const int32_t* row_offsets, const int32_t* lhs_idx,
                         const int32_t* out_idx, int64_t R, int64_t x_rows, int64_t E, int64_t N,
                         int64_t K, void* workspace, hipStream_t st) {
  const int64_t rp = mx_rows(R);
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  void* aq = ws;
  void* as = ws + rp * K * 3 / 2;
  const int64_t threads = rp * (K / 32);
  hipLaunchKernelGGL(mx_split_kernel, dim3((unsigned)ceil_div(threads, 256)), dim3(256), 0, st,
                     static_cast<const uint16_t*>(x), lhs_idx, static_cast<u32x4*>(aq),
                     static_cast<uint8_t*>(as), (int)R, (int)x_rows, (int)K, (int)rp);
  MxArgs a;
  a.aq = aq; a.as = as; a.w = w; a.s = s; a.y = y;
  a.row_offsets = row_offsets; a.out_idx = out_idx;
  a.R = (int)R; a.N = (int)N; a.K = (int)K; a.Rp = (int)rp; a.E = (int)E;
  a.y_dtype = y_dtype;
  a.m_tiles = (int)(ceil_div(R, TM) + (row_offsets ? E : 0));
  a.n_tiles = (int)ceil_div(N, TN);
  const int grid = (int)(ceil_div((int64_t)a.m_tiles * a.n_tiles, 8) * 8), block = 256;
  if (K % 2048 == 0) {
    if (!lds_limit<mxfp4_mfma8_kernel>(kLds8)) return;
    hipLaunchKernelGGL(mxfp4_mfma8_kernel, dim3(grid), dim3(512), kLds8, st, a);
    return;
  }
  if (!lds_limit<mxfp4_mfma_kernel>(kLds)) return;
  hipLaunchKernelGGL(mxfp4_mfma_kernel, dim3(grid), dim3(block), kLds, st, a);
}

}  // namespace qmm
