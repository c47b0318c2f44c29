// Decode-regime affine quantized matmul (M <= 16) with loader wavefronts.
//
// Same arithmetic as qmm_skinny.hip (codes exact in bf16, two
// v_mfma_f32_16x16x32_bf16 per 64-code chunk, scale applied to the chunk's
// dot, the code-independent terms as small MFMAs over the chunk index); what
// differs is who moves the bytes.
//
// A compute unit cannot keep its whole share of the weight (about 130 KB for
// the 4096 x 14336 case) in flight: vector-memory instructions are accepted at
// the pace the memory system returns data, and a wavefront that issues all its
// loads first spends most of the streaming time blocked in issue, computing
// only afterwards.  Here NL loader wavefronts do nothing but issue
// direct-to-LDS loads (they are the ones that block), and CW compute
// wavefronts never touch global memory until the final store: they consume
// "items" from a four-slot LDS ring as the loaders complete them.
//
// Two variants (template flag XD):
//
// * ring variant (XD = 0; more than eight rows of activations on a weight of
//   at most 64 rows per compute unit, where the direct variant has no room
//   for its staging patches or K takes several passes): activations and
//   weight tiles both travel through the ring, as described below;
// * direct variant (every one-pass shape, and several passes with few rows or
//   wide weights): each compute wavefront fetches its own K-slice of the
//   activations when a pass begins -- straight into MFMA operand registers up
//   to four rows, with whole-line loads through a wave-private LDS patch from
//   five rows on -- every ring slot holds a weight tile, and the loaders' tile
//   loop is a real loop.  XD = 1, K exactly one pass: the compute wavefronts'
//   tile loop is a real loop too, any number of tiles, a tile's sums leave for
//   LDS at once; XD = 2, several passes: the tiles' sums stay in registers
//   from pass to pass (at most eight tiles, unrolled).  The host deals up to
//   128 rows a workgroup, so that a 28672-row weight is still one workgroup
//   per compute unit.  The loaders keep two tiles requested: tile g+1 before
//   tile g is published, tile g+2 right after.  A wavefront holds about
//   sixteen loads in flight, so two tiles are all four loaders can have out,
//   and a wavefront blocked in issue cannot publish; more in flight (every
//   tile up front with flags in LDS, eight loaders with three tiles out) was
//   built and measured slower every time: what ends the launch early is the
//   next needed tile landing early, and more requests share the bandwidth
//   among later tiles.  Measured on 4096 x 14336 four-bit weights: 9.6 us a
//   launch at one row, 10.4-10.7 us at sixteen (ring variant: 11.2 / 12.0 us).
//
// The direct variants also serve MXFP4 weights (template value GSHIFT = 2): the
// hardware converter widens two E2M1 codes at a time with the 32-block's
// power-of-two scale applied (exact in bf16), the chunks chain through the
// MFMA accumulator, and a row's table share of a slice is its 16 scale bytes.
//
// Items of one pass (a pass = CW consecutive K-slices, one per compute
// wavefront; a slice = 256 packed bytes per row):
//   XR activation rounds  [CW slices][16 rows m][256 bytes = 128 codes of x]
//   TMAX weight tiles     [CW slices][16 rows n][256 packed bytes] + table rows
// Every item is CW * 4 KB.  Inside a slice's 4 KB, row r holds its 16-byte
// piece p at position p ^ (r & 15): the loader lane that fills position
// (r, lp) fetches global piece lp ^ (r & 15), so the global access stays inside
// the row's 256 bytes (coalesced) and the operand-order readback (lane = row
// l % 16: sixteen rows of one piece in a pass) touches sixteen different
// positions, i.e. every bank once, without padding.  (With p ^ (r & 7) rows r
// and r + 8 shared their banks: SQ_LDS_BANK_CONFLICT was 36 % of
// SQ_LDS_IDX_ACTIVE.)
//
// Synchronisation is one workgroup barrier per item: a loader wavefront
// arrives after its share of item i has landed, a compute wavefront after it
// has finished item i-1; past the barrier the loaders refill the slot of item
// i-1.  Every wavefront executes the same number of barriers whatever its
// role, the tile count or the slice count.
//
// (Items half this size -- eight half tiles, eight slots -- shorten the
// arithmetic left after the last byte lands, but measured 0.6 us slower: each
// barrier puts the twelve wavefronts in lockstep.)
//
// Order of issue.  The first byte of a kernel arrives 2-3 us after it starts
// and the weight stream is what bounds the kernel, so the first weight tile is
// requested at once, between the activation rounds: x0 x1 t0 x2 (the four
// slots), then one item per freed slot: x3 t1 t2 t3, running on into the next
// pass (K > CW slices) without draining the ring.  Loads retire in order, so
// "item i has landed" is a wait on the number of loads issued after it; the
// schedule and those counts are worked out at compile time (struct Sched),
// the slot of every item is a small piece of scalar bookkeeping that both
// roles run identically.
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "qmm_gemv_common.hpp"

namespace qmm {

namespace {

typedef __attribute__((address_space(3))) void lds_void;

template <int N>
__device__ __forceinline__ void wait_vmcnt() {    // s_waitcnt vmcnt(N) only; also a compiler barrier
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
  asm volatile("" ::: "memory");
}

// Direct-to-LDS load, 16 bytes a lane.  AUX = 2 marks the lines non-temporal:
// weights and their tables are read once per launch (a read-only launch over
// 32 MiB measures 6.5 us with the hint against 7.5 us without).
constexpr int kStream = 2;
template <int AUX = 0>
__device__ __forceinline__ void dma16(__amdgpu_buffer_rsrc_t r, unsigned char* dst, uint32_t voff,
                                      uint32_t soff) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lds_void*)dst, 16, voff, soff, 0, AUX);
}

// Clock stamps (builds with -DQMM_TIMELINE only): lane 0 of every wavefront
// writes the constant 100 MHz clock into g_stamps[workgroup][wavefront][i];
// qmm_debug_stamps copies the array out.
#ifdef QMM_TIMELINE
constexpr int kStampWgs = 256, kStampWaves = 12, kStampSlots = 16;
__device__ uint64_t g_stamps[kStampWgs * kStampWaves * kStampSlots];
#define QMM_STAMP(i)                                                                              \
  do {                                                                                            \
    if ((threadIdx.x & 63) == 0 && blockIdx.x < kStampWgs && blockIdx.y == 0)                     \
      g_stamps[(blockIdx.x * kStampWaves + wave) * kStampSlots + (i)] =                           \
          __builtin_amdgcn_s_memrealtime();                                                       \
  } while (0)
#else
#define QMM_STAMP(i) do {} while (0)
#endif

// all LDS traffic of this wavefront done, then the workgroup barrier
__device__ __forceinline__ void item_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ void split3(float v, float& hi, float& mid, float& lo) {
  hi = __uint_as_float(__float_as_uint(v) & 0xFFFF0000u);
  const float r1 = v - hi;
  mid = __uint_as_float(__float_as_uint(r1) & 0xFFFF0000u);
  lo = r1 - mid;                              // at most 8 significant bits: exact in bf16
}

__device__ __forceinline__ uint32_t hi16_pair(float a, float b) {      // (bf16(a), bf16(b)), truncating
  return byte_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}

// The static schedule of one pass: XR activation rounds (items 0 .. XR-1) and
// TMAX weight tiles (items XR ..), consumed in that order, issued in the order
// x0 x1 t0 x2 .. t1 ..; LX / LT loads per loader wavefront per item.
template <int XR, int TMAX, int LX, int LT>
struct Sched {
  static constexpr int NI = XR + TMAX;
  static constexpr int B = XR == 0 || NI >= 4 ? 4 : NI;     // ring slots (= items issued up front by the ring variant)
  static constexpr int item_at(int j) {                     // the item issued j-th
    if (XR == 0 || j < 2) return j;
    if (j == 2) return XR;
    if (j < XR + 1) return j - 1;
    return j;
  }
  static constexpr int pos(int item) {
    for (int j = 0; j < NI; ++j)
      if (item_at(j) == item) return j;
    return -1;
  }
  static constexpr int loads(int item) { return item < XR ? LX : LT; }
  // Loads that may still be outstanding when item k of a pass is declared
  // landed, `end` issue positions (counted from the start of that pass, running
  // on into the next pass, whose items repeat the order) having been issued.
  static constexpr int allowed(int k, int end) {
    int n = 0;
    for (int j = pos(k) + 1; j < end; ++j) n += loads(item_at(j % NI));
    return n > 63 ? 63 : n;
  }
};

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

template <int BITS, int CW, int NL, int TMAX, int GSHIFT, int XD>
__global__ __launch_bounds__(kWave*(CW + NL)) void skinny2_kernel(GemvArgs a, int rows_per_wg) {
  load_args_now(a);
  asm volatile("" ::"s"(rows_per_wg));
  constexpr int KS = 2048 / BITS;                 // codes per slice: 512 | 256
  constexpr int CPS = KS / 64;                    // 64-code chunks per slice: 8 | 4
  constexpr int XR = XD ? 0 : KS / 128;           // activation rounds per slice through the ring: 4 | 2, or none
  constexpr int NI = XR + TMAX;                   // items per pass
  constexpr int kItem = CW * 4096;
  // Table kind (GSHIFT): 0 / 1 = bf16 tables, groups of 64 / 128; 2 = MXFP4
  // (E2M1 codes, one E8M0 byte per 32 codes); 3 / 4 = float16 tables; 5 / 6 =
  // float32 tables.  A row's table share of a slice is 16 bytes, except for
  // float32 tables with groups of 64 (eight 4-byte entries: 32 bytes, WIDE).
  constexpr bool WIDE = GSHIFT == 5;
  constexpr int kTabKind = (CW >= 4 ? CW * 256 : 1024) * (WIDE ? 2 : 1);   // scale rows | bias rows of one tile
  constexpr int kTab = 2 * kTabKind;
  constexpr int NTAB = 2 * (CW >= 4 ? CW / 4 : 1) * (WIDE ? 2 : 1);        // table load instructions per tile
  static_assert((CW * 4) % NL == 0 && NTAB % NL == 0, "loader shares must be whole");
  constexpr int QI = CW * 4 / NL;                 // code / activation loads per loader wavefront per item
  constexpr int QT = NTAB / NL;                   // table loads per loader wavefront per tile
  constexpr int LX = QI, LT = QI + QT;            // loads per loader wavefront: activation item | tile item
  typedef Sched<XR, TMAX, LX, LT> S;
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* ring = smem;
  unsigned char* tabs = smem + S::B * kItem;
  // Direct variants: behind the ring and the tables, a 1 KB patch a compute
  // wavefront (staging of activations that come in with whole-line loads).
  unsigned char* patches = smem + 4 * (kItem + kTab);

  const int lane = threadIdx.x & 63;
  // (Wavefronts start in the order of their hardware index, a whole workgroup
  // over about 0.4 us.  The compute wavefronts come first on purpose: data
  // returns in the order of the requests, and their activations -- cache hits
  // -- must not queue behind the first weight tile; with the loaders first
  // 4096 x 14336 measured 10.6 against 9.9 us at one row, 13.3 against 11.4 us
  // at sixteen.)
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t bz = blockIdx.y;
  const int64_t n_begin = (int64_t)blockIdx.x * rows_per_wg;
  const int64_t n_end = n_begin + rows_per_wg < a.N ? n_begin + rows_per_wg : a.N;
  const int ntiles = (int)((n_end - n_begin + 15) / 16);        // uniform, <= TMAX
  const int64_t wpr = (int64_t)a.K * BITS / 8;                  // bytes per weight row
  // float16 / float32 entries are split into two / three bf16 terms, exactly,
  // where they have to be matrix operands.
  // GSHIFT = 7: MXFP4 whose K is any multiple of 64 up to one pass (the hidden
  // size 2880 of gpt-oss: five and a half slices a row, 90 scale bytes a row):
  // the last slice is ragged -- the code pieces and activation chunks past K are
  // requested out of range and read as zeros -- and a tile's scale rows, which
  // are not dword-aligned one by one, come in as the one contiguous run they
  // are in memory and are picked apart by byte offset.
  constexpr bool MXR = GSHIFT == 7;
  constexpr bool MX = GSHIFT == 2 || MXR;
  constexpr bool F16T = GSHIFT == 3 || GSHIFT == 4;
  constexpr bool F32T = GSHIFT == 5 || GSHIFT == 6;
  static_assert(!MXR || XD == 1, "the ragged MXFP4 form is a one-pass direct variant");
  constexpr int ES = F32T ? 4 : 2;                             // bytes per table entry
  constexpr int GLOG = (GSHIFT == 1 || GSHIFT == 4 || GSHIFT == 6) ? 1 : 0;   // log2(group / 64)
  static_assert(!MX || (BITS == 4 && XD != 0), "MXFP4: four-bit codes, direct variants");
  const int64_t ng = MX ? (int64_t)(a.K / 64) : (int64_t)(a.K / 64) >> GLOG;   // table row = ng * ES bytes (MXFP4: K/32 bytes)
  const int slices = MXR ? (a.K + KS - 1) / KS : a.K / KS;
  const int passes = (slices + CW - 1) / CW;
  const int tail_codes = MXR ? a.K % KS : 0;                   // codes of a ragged last slice (0: it is whole)
  const int tailp = tail_codes / 32, tailc = tail_codes / 64;  // its 16-byte pieces | its 64-code chunks
  const uint32_t spitch = (uint32_t)(ng * ES);                 // bytes of a table row

  int64_t xz = a.lhs_idx ? (int64_t)a.lhs_idx[bz] : bz;
  int64_t wz = a.rhs_idx ? (int64_t)a.rhs_idx[bz] : bz;
  bool x_ok = true;
  if (a.rhs_idx) {                                  // gather form: indices are data
    if (wz < 0 || wz >= a.n_experts) return;        // uniform, before any barrier
    if (xz < 0 || xz >= a.n_xrows) { xz = 0; x_ok = false; }
  }
  // Rows of activations of this workgroup: a.M, or in the grouped form (direct
  // variants only) those of segment blockIdx.y.
  int M = a.M;
  const int32_t* src_row = nullptr;
  const int32_t* out_row = nullptr;
  if (XD != 0 && a.segments) {
    if (bz >= a.segments[0]) return;              // uniform: before any barrier
    const int lo = a.segments[2 + 3 * bz];
    M = a.segments[3 + 3 * bz];
    src_row = a.src_row + lo;
    out_row = a.out_row + lo;
    xz = 0;
    wz = a.segments[1 + 3 * bz];
  }

  f32x4 acc[TMAX];
#pragma unroll
  for (int t = 0; t < TMAX; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  // Row packing (several passes, direct variant): the operand's sixteen rows
  // hold the activations of every pass at once -- rows [q*PK, q*PK + M) are
  // the M rows of x over pass q's K-slices -- so nothing is fetched between
  // passes.  A tile of pass p then yields meaningful sums only in row block p
  // (the other blocks multiply another pass's activations with this pass's
  // weights and are masked off), and the blocks are added up at the end.
  const int PK = XD != 2 ? 0 : (passes <= 2 && M <= 8) ? 8 : (passes <= 4 && M <= 4) ? 4 : 0;

  if (wave >= CW) {
    // ------------------------------------------------------------ loaders ----
    const int lw = wave - CW;
    const auto rx = make_rsrc(a.x + xz * a.M * (int64_t)a.K, x_ok ? (int64_t)a.M * a.K * 2 : 0);
    const auto rw = make_rsrc(reinterpret_cast<const char*>(a.w) + wz * a.N * wpr, a.N * wpr);
    const auto rs = make_rsrc(static_cast<const char*>(a.s) + wz * a.N * ng * ES, a.N * ng * ES);
    const auto rb = make_rsrc(static_cast<const char*>(a.b) + wz * a.N * ng * ES, a.N * ng * ES);
    const int lrow = lane >> 4, lp = lane & 15;
    // Load q of this wavefront is instruction j = lw + q*NL of the item: slice
    // j / 4, row quad j % 4 = (lw + o) % 4 with o = q*NL % 4 known at compile
    // time, so the lane offsets are kept per o.
    uint32_t wv[4], xv[4], wvt[4];
    int wrow[4];
#pragma unroll
    for (int o = 0; o < 4; ++o) {
      const int rq = (lw + o) & 3;
      const int row = 4 * rq + lrow;
      const uint32_t gp = (uint32_t)(lp ^ (row & 15));
      wrow[o] = row;
      wv[o] = (uint32_t)((n_begin + row) * wpr) + gp * 16;
      wvt[o] = MXR && tailp != 0 && (int)gp >= tailp ? kOutOfRange : wv[o];   // in a ragged last slice
      xv[o] = row < a.M ? (uint32_t)((int64_t)row * a.K * 2) + gp * 16 : kOutOfRange;
    }
    const int trow = lane & 15, tsl = lane >> 4;  // table loads: lane = (slice within four, row)

    // weight tile t of pass `p`, and its table rows, into ring slot `slot`
    auto issue_tile = [&](int p, int t, int slot) __attribute__((always_inline)) {
      unsigned char* base = ring + slot * kItem;
      // (The wavefront-uniform offset must depend on uniform values only, or
      // every load turns into a loop over its distinct values: a row past the
      // end is a lane offset out of range, a slice past the end both.)
      const bool full = n_begin + t * 16 + 16 <= n_end;                // uniform
      uint32_t vt[4], vtt[4];
#pragma unroll
      for (int o = 0; o < 4; ++o) {
        vt[o] = full || n_begin + t * 16 + wrow[o] < n_end ? wv[o] : kOutOfRange;
        vtt[o] = full || n_begin + t * 16 + wrow[o] < n_end ? wvt[o] : kOutOfRange;
      }
      const uint32_t tile_off = (uint32_t)(t * 16 * wpr);
      // The table rows go first (their sixteen quarter lines are the slow part
      // of a tile's requests; ahead of the codes they measured 0.1-0.2 us a
      // launch better than behind them).
      unsigned char* tb = tabs + slot * kTab;
#pragma unroll
      for (int q = 0; q < QT; ++q) {
        const int jt = lw + q * NL;               // uniform
        if constexpr (MXR) {
          // the tile's scale rows as the contiguous run they are: request jt covers its bytes [1024 jt, 1024 jt + 1024)
          const int64_t n0t = n_begin + t * 16;
          const int rows_here = n_end - n0t < 16 ? (int)(n_end - n0t) : 16;
          const uint32_t off = (uint32_t)(jt * 1024 + lane * 16);
          const uint32_t vo = rows_here > 0 && off < (uint32_t)rows_here * spitch ? (uint32_t)(n0t * spitch) + off
                                                                                   : kOutOfRange;
          dma16<kStream>(rs, tb + jt * 1024, vo, 0u);
          continue;
        }
        const int kind = jt / (NTAB / 2), rem = jt % (NTAB / 2);
        const int h = WIDE ? rem >> 1 : rem, h2 = WIDE ? rem & 1 : 0;   // four-slice group; 16-byte half of a wide row
        const int sloc = 4 * h + tsl;
        const int sl = p * CW + sloc;
        const int64_t n = n_begin + t * 16 + trow;
        const bool ok = sloc < CW && sl < slices && n < n_end;
        const uint32_t vo = ok ? (uint32_t)(n * ng * ES) + (uint32_t)((sl * CPS) >> (MX ? 0 : GLOG)) * (uint32_t)ES + (uint32_t)h2 * 16u
                               : kOutOfRange;
        unsigned char* tdst = tb + kind * kTabKind + (WIDE ? h * 2048 + h2 * 1024 : h * 1024);
        // (MXFP4 has no second table: the load still goes out, fetching nothing,
        // so that every loader wavefront issues the same number per tile -- the
        // waits count loads)
        if constexpr (MX) dma16<kStream>(rs, tdst, kind == 0 ? vo : kOutOfRange, 0u);
        else dma16<kStream>(kind ? rb : rs, tdst, vo, 0u);
      }
      static_for<QI>([&](auto qc) __attribute__((always_inline)) {
        constexpr int q = decltype(qc)::value;
        constexpr int o = (q * NL) & 3;
        const int j = lw + q * NL;                // uniform
        const int sloc = j >> 2, rq = j & 3;
        const int sl = p * CW + sloc;
        const bool sok = sl < slices;             // uniform; false for passes past the last
        const uint32_t so = sok ? (uint32_t)sl * 256u + tile_off : 0u;
        const bool rag = MXR && sl == slices - 1;  // uniform
        dma16<kStream>(rw, base + sloc * 4096 + rq * 1024, sok ? (rag ? vtt[o] : vt[o]) : kOutOfRange, so);
      });
    };
    // item `i` (compile-time kind) of pass `p` into ring slot `slot`
    auto issue_item = [&](int p, auto ic, int slot) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value;
      if constexpr (i < XR) {
        unsigned char* base = ring + slot * kItem;
        static_for<QI>([&](auto qc) __attribute__((always_inline)) {
          constexpr int q = decltype(qc)::value;
          constexpr int o = (q * NL) & 3;
          const int j = lw + q * NL;              // uniform
          const int sloc = j >> 2, rq = j & 3;
          const int sl = p * CW + sloc;
          const bool ok = sl < slices;            // also false for passes past the last
          const uint32_t so = ok ? (uint32_t)(sl * KS + i * 128) * 2u : 0u;
          dma16(rx, base + sloc * 4096 + rq * 1024, ok ? xv[o] : kOutOfRange, so);
        });
      } else {
        issue_tile(p, i - XR, slot);
      }
    };
    // The K slices of tile t meet here: after the barrier that follows the
    // tile's consumption the loaders (otherwise idle) add up the compute
    // wavefronts' partial sums and store the 16 x 16 results, under the next
    // item's arithmetic.  Lane l, component e of an accumulator is output row
    // 4*(l/16) + e, column l % 16 of the tile.
    auto reduce_tile = [&](int p, int t, int slot) __attribute__((always_inline)) {
      if (p != passes - 1 || t >= ntiles) return;
      const float* part = reinterpret_cast<const float*>(ring + slot * kItem);
#pragma unroll
      for (int e = lw; e < 4; e += NL) {
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < CW; ++wv) v += part[wv * 1024 + e * kWave + lane];
        if constexpr (XD == 2) {
          if (PK != 0) {                            // row blocks of the passes -> rows [0, PK)
            v += __shfl_xor(v, 32);
            if (PK == 4) v += __shfl_xor(v, 16);
          }
        }
        const int m = 4 * (lane >> 4) + e;
        const int64_t n = n_begin + t * 16 + (lane & 15);
        const bool row_ok = m < M && (PK == 0 || m < PK);
        int64_t yrow = bz * a.M + m;
        if (out_row) yrow = row_ok ? (int64_t)out_row[m] : -1;
        if (row_ok && yrow >= 0 && n < n_end) store_out(a.y, yrow * (int64_t)a.N + n, v, a.y_dtype);
      }
    };
    if constexpr (XD) {
      // Every item is a tile: tile g lives in slot g % 4.  A load
      // instruction is accepted at the pace at which data comes back (issuing
      // a tile takes about as long as receiving one), and a wavefront stuck in
      // issue cannot publish what has already landed: so the loaders keep two
      // items out -- item g+1 is requested before item g is published, g+2
      // right after -- and no more (refilling two slots after a publication
      // measured 0.5 us slower).
      // Item g = pass g / ntiles, tile g % ntiles, in slot g % 4; any number of
      // tiles with one pass, up to TMAX (accumulators in registers) with more.
      static_assert(!XD || S::B == 4, "two items in flight, one being consumed, one being reduced");
      const int G = passes * ntiles;
      auto issue = [&](int g) __attribute__((always_inline)) {
        const int p = g / ntiles;
        issue_tile(p, g - p * ntiles, g & 3);
      };
      QMM_STAMP(0);
      issue(0);
      QMM_STAMP(1);
      if (G > 1) issue(1);
      QMM_STAMP(2);
#pragma nounroll
      for (int g = 0; g < G; ++g) {
        // item g has landed: only item g+1 may still be out (a store in
        // between only tightens the wait)
        if (g + 1 < G) wait_vmcnt<LT>(); else wait_vmcnt<0>();
        if (g < 4) QMM_STAMP(3 + 3 * g);
        item_barrier();                           // item g published; item g-1 consumed
        if (g < 4) QMM_STAMP(4 + 3 * g);
        if (g + 2 < G) issue(g + 2);              // that slot's last tile was consumed (and, in the last pass, reduced) a step ago
        if (g >= 1 && g - 1 >= G - ntiles) reduce_tile(passes - 1, g - 1 - (G - ntiles), (g - 1) & 3);
        if (g < 4) QMM_STAMP(5 + 3 * g);
      }
      item_barrier();                             // everything consumed
      reduce_tile(passes - 1, ntiles - 1, (G - 1) & 3);
      QMM_STAMP(15);
      return;
    }
    // Slot of every item of the current pass (by order of use) and of the next
    // pass's items issued ahead; both roles keep this bookkeeping identically.
    int sl_cur[NI], sl_nxt[NI], prev_last = 0;
#pragma unroll
    for (int k = 0; k < NI; ++k) sl_cur[k] = sl_nxt[k] = 0;
    static_for<S::B>([&](auto jc) __attribute__((always_inline)) {
      constexpr int j = decltype(jc)::value;
      sl_cur[S::item_at(j)] = j;
      issue_item(0, std::integral_constant<int, S::item_at(j)>{}, j);
    });
    for (int p = 0; p < passes; ++p) {
      const bool last = p == passes - 1;
      // publication of item k: wait until it has landed, barrier, refill the
      // slot of the item used just before with the next item in issue order
      auto publish = [&](auto kc) __attribute__((always_inline)) {
        constexpr int k = decltype(kc)::value;
        constexpr int e = S::B + k - 1;           // issue positions out when item k (not the very first) is awaited
        if constexpr (k == 0) {
          if (p == 0) wait_vmcnt<S::allowed(0, S::B)>();
          else wait_vmcnt<S::allowed(0, e)>();
        } else {
          if (last) wait_vmcnt<S::allowed(k, e < NI ? e : NI)>();
          else wait_vmcnt<S::allowed(k, e)>();
        }
        item_barrier();
        const int freed = k >= 1 ? sl_cur[k >= 1 ? k - 1 : 0] : prev_last;
        if (k >= 1 || p >= 1) {
          if constexpr (e < NI) {
            sl_cur[S::item_at(e)] = freed;
            issue_item(p, std::integral_constant<int, S::item_at(e)>{}, freed);
          } else if (!last) {
            sl_nxt[S::item_at(e - NI)] = freed;
            issue_item(p + 1, std::integral_constant<int, S::item_at(e - NI)>{}, freed);
          }
        }
      };
      static_for<XR + 1>(publish);                // the activation rounds and the first tile
      // The other tiles, and the barrier that ends the last pass, as a real
      // loop: after its barrier, step k sums the K-slices of the tile used just
      // before (item k-1), and that code is then the same, already fetched,
      // copy for every tile -- a kernel that runs each instruction once pays an
      // instruction-cache miss for every new block, and at the very end of the
      // kernel nothing hides it (measured: 1.2 us for the last tile's sum as a
      // separate copy, 0.3 us for a second run of the same code).
#pragma nounroll
      for (int k = XR + 1; k <= NI; ++k) {
        if (k == NI) {
          if (!last) break;
          item_barrier();                         // everything consumed
        } else {
          if (k == XR + 1) { if constexpr (TMAX > 1) publish(std::integral_constant<int, XR + 1>{}); }
          else if (k == XR + 2) { if constexpr (TMAX > 2) publish(std::integral_constant<int, (TMAX > 2 ? XR + 2 : 0)>{}); }
          else { if constexpr (TMAX > 3) publish(std::integral_constant<int, (TMAX > 3 ? XR + 3 : 0)>{}); }
        }
        const int t = k - 1 - XR;
        int slot = sl_cur[XR];
        if constexpr (TMAX > 1) slot = t == 1 ? sl_cur[XR + 1] : slot;
        if constexpr (TMAX > 2) slot = t == 2 ? sl_cur[XR + (TMAX > 2 ? 2 : 0)] : slot;
        if constexpr (TMAX > 3) slot = t == 3 ? sl_cur[XR + (TMAX > 3 ? 3 : 0)] : slot;
        reduce_tile(p, t, slot);
      }
      static_assert(XD || TMAX <= 4, "the tile loop names at most four tiles");
      prev_last = sl_cur[NI - 1];
#pragma unroll
      for (int k = 0; k < NI; ++k) sl_cur[k] = sl_nxt[k];
    }
  } else {
    // ----------------------------------------------------- compute wavefronts
    const int r = lane & 15, kg = lane >> 4;
    const uint32_t swz = (uint32_t)(r & 15);
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    const uint32_t one = pin_vgpr(kOnesBf16x2);
    const bf16x8 ones = as_bf16x8(one, one, one, one);
    const uint32_t nib = pin_vgpr(0x000F000Fu), magic = pin_vgpr(0x43004300u);
    // The K-slice this wavefront works on.  In the one-pass variant the
    // assignment rotates with the workgroup (and so does the order in which a
    // wavefront asks for its slice's chunks, below): every workgroup reads all
    // of the activations, and 256 of them walking through the same lines in
    // the same order at the same time wait on one another's misses -- 128 KB
    // that are not in L2 take a compute unit 2.6 us in lockstep, 1.85 us
    // rotated (measured with a fetch-only kernel).  The slices' sums are added
    // in slice order whoever computed them, so the results do not change.
    static_assert((CW & (CW - 1)) == 0, "slice rotation");
    const int sw = XD == 1 ? (wave + (int)(blockIdx.x >> 3)) & (CW - 1) : wave;
    const uint32_t rowb = (uint32_t)(sw * 4096 + r * 256);      // this lane's row inside its slice's 4 KB
    // the operand row r of this lane is row xrow(r) of x (gathered in the grouped form)
    const int tab_row = MXR ? 0 : (sw >> 2) * (WIDE ? 2048 : 1024) + (sw & 3) * 256 + r * 16;   // this lane's table row inside a kind
    // chunks of this wavefront's slice that lie inside K (a ragged last slice has fewer)
    const int vc = MXR && tailc != 0 && sw == slices - 1 ? tailc : CPS;
    const int64_t xrows = src_row ? (int64_t)a.x_rows : (int64_t)a.M;
    const auto rxc = make_rsrc(a.x + xz * a.M * (int64_t)a.K, x_ok ? xrows * a.K * 2 : 0);
    auto xrow = [&](int m) -> int64_t {
      if (m >= M) return -1;
      if (!src_row) return m;
      const int64_t sr = src_row[m];
      return sr < xrows ? sr : -1;
    };
    const int64_t xr0 = xrow(r);
    const uint32_t xlane = xr0 >= 0 ? (uint32_t)(xr0 * a.K * 2) + (uint32_t)kg * 32u : kOutOfRange;
    int sl_cur[NI], sl_nxt[NI], prev_last = 0;     // the loaders' slot bookkeeping, mirrored
#pragma unroll
    for (int k = 0; k < NI; ++k) sl_cur[k] = sl_nxt[k] = 0;
    static_for<S::B>([&](auto jc) __attribute__((always_inline)) {
      constexpr int j = decltype(jc)::value;
      sl_cur[S::item_at(j)] = j;
    });
    bf16x8 xa[CPS][2];
    // The code-independent part of a tile's sums is sum_c t_c * xs_c over the
    // chunks c of the slice, xs_c = sum_k x over chunk c, for every table entry
    // t that multiplies a constant: the bias, and for four-bit codes (widened
    // as 128 + q) the scale times -128.  It runs on the matrix cores with the
    // chunk index as the K dimension: xs_c is split into three bf16 terms
    // (24 bits, exact), a float16 / float32 table entry into two / three.  A
    // slice has eight chunks and the instruction's K is 32, so four (x term,
    // table term) pairs share one MFMA, one per lane quarter kg: pair g =
    // (kind, table term, x term) sits in MFMA g / 4, quarter g % 4.  The A
    // operands depend on the activations only and are built once; bf16 tables
    // with four-bit codes take two MFMAs a tile this way instead of six.
    constexpr int NT = F32T ? 3 : F16T ? 2 : 1;     // bf16 terms per table entry
    constexpr int NG = (BITS == 4 ? 2 : 1) * NT * 3;
    constexpr int NA = (NG + 3) / 4;
    bf16x8 ax[NA];
    auto chunk_sums = [&]() __attribute__((always_inline)) {
      float xt[3][8];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float xs = 0.f;
        if (c < CPS) {
          f32x4 t4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xa[c][0], zero, 0, 0, 0);
          t4 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xa[c][1], t4, 0, 0, 0);
          xs = t4[0];                               // every row of the product holds the column's sum
        }
        split3(xs, xt[0][c], xt[1][c], xt[2][c]);
      }
      static_for<NA>([&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        float v[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) v[c] = 0.f;
        static_for<4>([&](auto qc) __attribute__((always_inline)) {
          constexpr int g = 4 * i + decltype(qc)::value;
          if constexpr (g < NG) {
            constexpr float f = g / (3 * NT) ? -128.f : 1.f;      // exact: a power of two
#pragma unroll
            for (int c = 0; c < 8; ++c) v[c] = kg == (g & 3) ? f * xt[g % 3][c] : v[c];
          }
        });
        ax[i] = as_bf16x8(hi16_pair(v[0], v[1]), hi16_pair(v[2], v[3]), hi16_pair(v[4], v[5]), hi16_pair(v[6], v[7]));
      });
    };
    // acc + this wavefront's K-slice of one tile: `base` is the lane's row in
    // the slice's 4 KB of codes, `tb` its table row
    auto tile_math = [&](const unsigned char* base, const unsigned char* tb, f32x4 acc_in) __attribute__((always_inline)) {
      if constexpr (MX) {
        // E2M1 codes: the converter widens two codes at a time and multiplies
        // by the 32-block's power-of-two scale (exact in bf16), so the chunks
        // chain straight through the MFMA accumulator.  Lane kg holds codes
        // [16 kg, 16 kg + 16) of the chunk: block 2c + kg/2 of the slice.
        u32x4 sv;
        if constexpr (MXR) {
          // this row's sixteen scale bytes of the slice, at an even byte offset of the tile's run
          const uint32_t off = (uint32_t)r * spitch + 16u * (uint32_t)sw;
          const uint32_t* pw = reinterpret_cast<const uint32_t*>(tb + (off & ~3u));
          const uint32_t d0 = pw[0], d1 = pw[1], d2 = pw[2], d3 = pw[3], d4 = pw[4];
          const uint32_t sh = (off & 2u) * 8u;
          sv = u32x4{__builtin_amdgcn_alignbit(d1, d0, sh), __builtin_amdgcn_alignbit(d2, d1, sh),
                     __builtin_amdgcn_alignbit(d3, d2, sh), __builtin_amdgcn_alignbit(d4, d3, sh)};
        } else {
          sv = *reinterpret_cast<const u32x4*>(tb);
        }
        f32x4 at = acc_in;
#pragma unroll
        for (int c = 0; c < CPS; ++c) {
          const uint32_t pc = (uint32_t)(2 * c + (kg >> 1));
          const u32x2 q = *reinterpret_cast<const u32x2*>(base + ((pc ^ swz) << 4) + (kg & 1) * 8);
          float sc = e8m0_to_f32((sv[c >> 1] >> (16 * (c & 1) + 8 * (kg >> 1))) & 255u);
          if constexpr (MXR) sc = c < vc ? sc : 1.0f;        // past K: zero codes times a finite scale
          at = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][0], widen_e2m1(q[0], sc), at, 0, 0, 0);
          at = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][1], widen_e2m1(q[1], sc), at, 0, 0, 0);
        }
        return at;
      }
      u32x4 svt = *reinterpret_cast<const u32x4*>(tb);
      u32x4 bvt = *reinterpret_cast<const u32x4*>(tb + kTabKind);
      if constexpr (GLOG == 1 && !F32T) {   // group 128: one entry serves two chunks -> duplicate each 16-bit entry
        svt = u32x4{byte_perm(svt[0], svt[0], 0x01000100u), byte_perm(svt[0], svt[0], 0x03020302u),
                    byte_perm(svt[1], svt[1], 0x01000100u), byte_perm(svt[1], svt[1], 0x03020302u)};
        bvt = u32x4{byte_perm(bvt[0], bvt[0], 0x01000100u), byte_perm(bvt[0], bvt[0], 0x03020302u),
                    byte_perm(bvt[1], bvt[1], 0x01000100u), byte_perm(bvt[1], bvt[1], 0x03020302u)};
      }
      // eight table entries as matrix operands over the chunk index: one bf16
      // operand, or for float16 tables two (hi + lo, exact: 11 significant bits)
      auto split_f16 = [&](const u32x4& t, bf16x8& hi, bf16x8& lo) __attribute__((always_inline)) {
        uint32_t h[4], l[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float f0 = f16_bits_to_f32(t[i] & 0xFFFFu), f1 = f16_bits_to_f32(t[i] >> 16);
          const float h0 = __uint_as_float(__float_as_uint(f0) & 0xFFFF0000u);
          const float h1 = __uint_as_float(__float_as_uint(f1) & 0xFFFF0000u);
          h[i] = hi16_pair(h0, h1);
          l[i] = hi16_pair(f0 - h0, f1 - h1);     // at most three significant bits: exact in bf16
        }
        hi = as_bf16x8(h[0], h[1], h[2], h[3]);
        lo = as_bf16x8(l[0], l[1], l[2], l[3]);
      };
      // float32 tables: the entries of the eight chunks as floats (group 128: one
      // entry serves two chunks), and as matrix operands three bf16 terms each
      float sf[8], bfv[8];
      if constexpr (F32T) {
        if constexpr (WIDE) {
          const u32x4 s1 = *reinterpret_cast<const u32x4*>(tb + 1024);
          const u32x4 b1 = *reinterpret_cast<const u32x4*>(tb + kTabKind + 1024);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            sf[i] = __uint_as_float(svt[i]); sf[4 + i] = __uint_as_float(s1[i]);
            bfv[i] = __uint_as_float(bvt[i]); bfv[4 + i] = __uint_as_float(b1[i]);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            sf[2 * i] = sf[2 * i + 1] = __uint_as_float(svt[i]);
            bfv[2 * i] = bfv[2 * i + 1] = __uint_as_float(bvt[i]);
          }
        }
      }
      // the bf16 terms of the table entries as matrix operands over the chunk
      // index: tt[kind * NT + term], kind 0 = bias, 1 = scale
      bf16x8 tt[2 * NT];
      if constexpr (F32T) {
        auto terms = [&](const float (&v)[8], bf16x8* out) __attribute__((always_inline)) {
          float h[8], m[8], l[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) split3(v[i], h[i], m[i], l[i]);
          out[0] = as_bf16x8(hi16_pair(h[0], h[1]), hi16_pair(h[2], h[3]), hi16_pair(h[4], h[5]), hi16_pair(h[6], h[7]));
          out[1] = as_bf16x8(hi16_pair(m[0], m[1]), hi16_pair(m[2], m[3]), hi16_pair(m[4], m[5]), hi16_pair(m[6], m[7]));
          out[2] = as_bf16x8(hi16_pair(l[0], l[1]), hi16_pair(l[2], l[3]), hi16_pair(l[4], l[5]), hi16_pair(l[6], l[7]));
        };
        terms(bfv, tt);
        if constexpr (BITS == 4) terms(sf, tt + NT);
      } else if constexpr (F16T) {
        split_f16(bvt, tt[0], tt[1]);
        if constexpr (BITS == 4) split_f16(svt, tt[2], tt[3]);
      } else {
        tt[0] = __builtin_bit_cast(bf16x8, bvt);
        if constexpr (BITS == 4) tt[1] = __builtin_bit_cast(bf16x8, svt);
      }
      f32x4 at = acc_in;
      static_for<NA>([&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        bf16x8 op = tt[(4 * i) / 3];
        static_for<3>([&](auto qc) __attribute__((always_inline)) {
          constexpr int g = 4 * i + 1 + decltype(qc)::value;
          if constexpr (g < NG && g / 3 != (g - 1) / 3) {        // the table term changes at this quarter
            const bf16x8 nx = tt[g / 3];
            op = kg >= (g & 3) ? nx : op;
          }
        });
        at = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ax[i], op, at, 0, 0, 0);
      });
#pragma unroll
      for (int c = 0; c < CPS; ++c) {
        f32x4 d;
        if constexpr (BITS == 4) {
          const uint32_t pc = (uint32_t)(2 * c + (kg >> 1));
          const u32x2 q = *reinterpret_cast<const u32x2*>(base + ((pc ^ swz) << 4) + (kg & 1) * 8);
          d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][0], widen_int4(q[0], nib, magic), zero, 0, 0, 0);
          d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][1], widen_int4(q[1], nib, magic), d, 0, 0, 0);
        } else {
          const uint32_t pc = (uint32_t)(4 * c + kg);
          const u32x4 q = *reinterpret_cast<const u32x4*>(base + ((pc ^ swz) << 4));
          d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][0], widen_int8(q[0], q[1]), zero, 0, 0, 0);
          d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[c][1], widen_int8(q[2], q[3]), d, 0, 0, 0);
        }
        const uint32_t sw = svt[c >> 1];
        float sc;
        if constexpr (F32T) sc = sf[c];
        else if constexpr (F16T) sc = f16_bits_to_f32((c & 1) ? sw >> 16 : sw & 0xFFFFu);
        else sc = __uint_as_float((c & 1) ? (sw & 0xFFFF0000u) : (sw << 16));
#pragma unroll
        for (int e = 0; e < 4; ++e) at[e] = fmaf(sc, d[e], at[e]);
      }
      return at;
    };
    if constexpr (XD) {
      // This wavefront's slice of pass p of the activations straight from
      // global memory (L2 after the first workgroup) into operand layout: lane
      // (r, kg) takes pieces 2*kg and 2*kg + 1 of every chunk of row r.
      auto fetch_x = [&](int p, bool active, uint32_t lane_off) __attribute__((always_inline)) {
        u32x4 raw[CPS][2];
        const uint32_t so = active ? (uint32_t)((p * CW + sw) * KS) * 2u : 0u;
#pragma unroll
        for (int c = 0; c < CPS; ++c)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            raw[c][j] = __builtin_amdgcn_raw_buffer_load_b128(
                rxc, active && (!MXR || c < vc) ? lane_off + (uint32_t)(c * 128 + j * 16) : kOutOfRange, so, 0);
#pragma unroll
        for (int c = 0; c < CPS; ++c)
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            if constexpr (BITS == 4 && !MX) xa[c][j] = pair_stride4(raw[c][j]);
            else xa[c][j] = __builtin_bit_cast(bf16x8, raw[c][j]);
          }
        if constexpr (!MX) {
          if (active) chunk_sums();
        }
      };
      // More than eight rows of activations: the direct load above makes every
      // lane a cache-line request of its own (sixteen rows a quarter line each
      // per instruction), which at sixteen rows costs more than it saves.
      // Here the slice comes in with whole-line loads instead -- instruction
      // (c, h) fetches the 128 bytes of chunk c of rows 8h .. 8h+7 -- all of
      // them requested at once, and each takes a round trip through a 1 KB
      // wave-private LDS patch into operand order (piece p of row r at
      // position p ^ ((r >> 1) & 3): both the 16-lane write and read passes
      // touch every bank once; the lanes whose operand row is in the other
      // half read along and keep what they had).
      // (pk != 0, the row packing of the several-pass variant: operand row
      // q*pk + m is row m of x over the K-slice of pass q.)
      auto fetch_x_staged = [&](auto rotc, int p, bool active, int pk) __attribute__((always_inline)) {
        constexpr int ROT = decltype(rotc)::value % CPS;          // chunk asked for first
        unsigned char* stg = patches + wave * 1024;
        const int srow = lane >> 3, sp = lane & 7;
        u32x4 raw[CPS][2];
        uint32_t lo[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int rr = 8 * h + srow;
          int64_t xr;
          uint32_t pass_off = 0u;
          if (pk == 0) {
            xr = active ? xrow(rr) : -1;
          } else {
            const int q = pk == 8 ? rr >> 3 : rr >> 2, m = rr - q * pk;
            xr = active && q * CW + wave < slices ? xrow(m) : -1;
            pass_off = (uint32_t)(q * CW * KS) * 2u;
          }
          lo[h] = xr >= 0 ? (uint32_t)(xr * a.K * 2) + pass_off + (uint32_t)sp * 16u : kOutOfRange;
        }
        const uint32_t so = active ? (uint32_t)((p * CW + sw) * KS) * 2u : 0u;
#pragma unroll
        for (int c = 0; c < CPS; ++c)
#pragma unroll
          for (int h = 0; h < 2; ++h)
            raw[c][h] = __builtin_amdgcn_raw_buffer_load_b128(
                rxc, !MXR || (c + ROT) % CPS < vc ? lo[h] : kOutOfRange, so + (uint32_t)(((c + ROT) % CPS) * 128), 0);
        const uint32_t wr = (uint32_t)(srow * 128 + ((sp ^ ((srow >> 1) & 3)) << 4));
        const uint32_t rkey = (uint32_t)((r >> 1) & 3);
        const bool upper = r >= 8;
#pragma unroll
        for (int c = 0; c < CPS; ++c)
#pragma unroll
          for (int h = 0; h < 2; ++h) {                          // rows 8h .. 8h+7 of chunk c
            *reinterpret_cast<u32x4*>(stg + wr) = raw[c][h];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const uint32_t pc = (uint32_t)(kg * 2 + j);
              const u32x4 v = *reinterpret_cast<const u32x4*>(stg + (r & 7) * 128 + ((pc ^ rkey) << 4));
              bf16x8 o;
              if constexpr (BITS == 4 && !MX) o = pair_stride4(v);
              else o = __builtin_bit_cast(bf16x8, v);
              if (upper == (h == 1)) xa[(c + ROT) % CPS][j] = o;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          }
        if constexpr (!MX) {
          if (active) chunk_sums();
        }
      };
      // Five to eight rows, through the same patch with whole-line loads.  The
      // direct fetch above makes every live lane a cache-line request of its
      // own: at eight rows 512 requests a wavefront for 64 lines of data, all
      // in front of the loaders' first tile in a vector-memory path that serves
      // a compute unit's requests in order.  Here an instruction covers R rows
      // with 1024 / R consecutive bytes each, so a slice takes R of them, every
      // instruction's 1 KB goes through the patch (piece p of row r at position
      // p ^ key(r): conflict-free both ways) and comes back in operand order.
      // 4096 x 14336, four-bit, same box: eight rows 9.8 against 10.7 us a
      // launch, four rows (R = 4) 10.1 against 10.35 and 5.5 against 5.8 on
      // 4096 x 4096; with one or two rows it is a wash (R = 1: 9.93 against
      // 9.93, 5.72 against 5.56) and the direct fetch stays.
      auto fetch_x_lines = [&](auto rc, bool active) __attribute__((always_inline)) {
        constexpr int SB = CPS * 128;                             // bytes of a row's slice
        constexpr int R = decltype(rc)::value * SB < 1024 ? 1024 / SB : decltype(rc)::value;
        constexpr int W = 1024 / R;                               // bytes a row and instruction
        constexpr int NI = SB / W;                                // instructions a slice
        constexpr int CPI = W / 128;                              // chunks an instruction
        constexpr int LPR = W / 16;                               // lanes a row
        unsigned char* stg = patches + wave * 1024;
        const int srow = lane / LPR, sp = lane % LPR;
        auto key = [](int row) { return R == 8 ? (row >> 1) & 3 : row; };
        const int64_t xr = active ? xrow(srow) : -1;
        const uint32_t lo = xr >= 0 ? (uint32_t)(xr * a.K * 2) + (uint32_t)sp * 16u : kOutOfRange;
        const uint32_t so = active ? (uint32_t)(sw * KS) * 2u : 0u;
        u32x4 raw[NI];
#pragma unroll
        for (int i = 0; i < NI; ++i)
          raw[i] = __builtin_amdgcn_raw_buffer_load_b128(
              rxc, !MXR || i * CPI + (sp >> 3) < vc ? lo : kOutOfRange, so + (uint32_t)(i * W), 0);
        const uint32_t wr = (uint32_t)(srow * W + ((sp ^ key(srow)) << 4));
        const int rr = r % R;
        const uint32_t rd = (uint32_t)(rr * W), rkey = (uint32_t)key(rr);
        const bool live = r < R;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
          *reinterpret_cast<u32x4*>(stg + wr) = raw[i];
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
          for (int cc = 0; cc < CPI; ++cc)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const uint32_t pc = (uint32_t)(cc * 8 + kg * 2 + j);
              u32x4 v = *reinterpret_cast<const u32x4*>(stg + rd + ((pc ^ rkey) << 4));
              if (!live) v = u32x4{0u, 0u, 0u, 0u};
              if constexpr (BITS == 4 && !MX) xa[i * CPI + cc][j] = pair_stride4(v);
              else xa[i * CPI + cc][j] = __builtin_bit_cast(bf16x8, v);
            }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        if constexpr (!MX) {
          if (active) chunk_sums();
        }
      };
      if constexpr (XD == 1) {
        // One pass (the host sees to it).  The tiles as a real loop (any number of them): a tile's sums leave
        // for its slot at once, where the loaders add up the slices.
        const bool active = sw < slices;          // uniform
        QMM_STAMP(0);
        if constexpr (!WIDE) {                    // (wide table rows leave no LDS for the staging patches)
          if (M > 8) {
            switch ((blockIdx.x >> 6) & 3) {
              case 0: fetch_x_staged(std::integral_constant<int, 0>{}, 0, active, 0); break;
              case 1: fetch_x_staged(std::integral_constant<int, 2>{}, 0, active, 0); break;
              case 2: fetch_x_staged(std::integral_constant<int, 4>{}, 0, active, 0); break;
              default: fetch_x_staged(std::integral_constant<int, 6>{}, 0, active, 0); break;
            }
          }
          else if (M > 4) fetch_x_lines(std::integral_constant<int, 8>{}, active);
          else if (M > 2) fetch_x_lines(std::integral_constant<int, 4>{}, active);
          else fetch_x(0, active, xlane);
        } else {
          fetch_x(0, active, xlane);
        }
        QMM_STAMP(2);
#pragma nounroll
        for (int g = 0; g < ntiles; ++g) {
          item_barrier();
          if (g < 4) QMM_STAMP(3 + 2 * g);
          const int slot = g & 3;
          f32x4 at = zero;
          if (active) at = tile_math(ring + slot * kItem + rowb, tabs + slot * kTab + tab_row, zero);
          float* part = reinterpret_cast<float*>(ring + slot * kItem + sw * 4096);
#pragma unroll
          for (int e = 0; e < 4; ++e) part[e * kWave + lane] = at[e];
          if (g < 4) QMM_STAMP(4 + 2 * g);
        }
      } else {
        // Several passes: the tiles' sums stay in registers from pass to pass
        // (at most TMAX tiles, unrolled); the next pass's activations are
        // fetched when the pass begins.
        QMM_STAMP(0);
        if (PK != 0) {
          // every pass's activations at once: lane row r = q*PK + m reads row m
          // over the K-slice of pass q (lanes past M, past the passes or past
          // the last slice read zeros)
          const int q = r / PK, m = r - q * PK;
          const int64_t xr = q * CW + wave < slices ? xrow(m) : -1;
          const uint32_t off = xr >= 0 ? (uint32_t)(xr * a.K * 2) + (uint32_t)kg * 32u + (uint32_t)(q * CW * KS) * 2u
                                       : kOutOfRange;
          // more than eight live operand rows: whole-line loads through the
          // patch, as in the one-pass variant (the direct fetch asks for a
          // quarter line a lane: sixteen live rows are sixteen line requests
          // an instruction).  Same box, direct against staged: 8192 x 8192
          // at eight rows 13.3 / 11.7 us, 4096 x 14336 at four rows 11.4 /
          // 11.0; with eight live rows it goes either way (8192 x 8192 at
          // four rows 11.35 / 10.9, 4096 x 14336 at two rows 9.7 / 10.2).
          bool staged = false;
          if constexpr (!WIDE) staged = M * passes > 8;
          if (staged) fetch_x_staged(std::integral_constant<int, 0>{}, 0, wave < slices, PK);
          else fetch_x(0, wave < slices, off);
        }
        const int my_pass = PK == 8 ? kg >> 1 : kg;   // the pass whose sums this lane's accumulator rows hold
        QMM_STAMP(2);
        for (int p = 0; p < passes; ++p) {
          const bool active = p * CW + wave < slices;   // uniform
          if (PK == 0) fetch_x(p, active, xlane);
          static_for<TMAX>([&](auto tc) __attribute__((always_inline)) {
            constexpr int t = decltype(tc)::value;
            if (t < ntiles) {
              item_barrier();
              if (p * ntiles + t < 4) QMM_STAMP(3 + 2 * (p * ntiles + t));
              const int slot = (p * ntiles + t) & 3;
              if (active) {
                const f32x4 d = tile_math(ring + slot * kItem + rowb, tabs + slot * kTab + tab_row, zero);
                const bool mine = PK == 0 || my_pass == p;
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[t][e] += mine ? d[e] : 0.f;
              }
              if (p == passes - 1) {
                float* part = reinterpret_cast<float*>(ring + slot * kItem + wave * 4096);
#pragma unroll
                for (int e = 0; e < 4; ++e) part[e * kWave + lane] = acc[t][e];
              }
              if (p * ntiles + t < 4) QMM_STAMP(4 + 2 * (p * ntiles + t));
            }
          });
        }
      }
      item_barrier();                             // everything consumed
      return;
    }
    for (int p = 0; p < passes; ++p) {
      const bool last = p == passes - 1;
      const bool active = p * CW + wave < slices;               // uniform
      auto consume = [&](auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        item_barrier();
        const int slot = sl_cur[i];
        const unsigned char* base = ring + slot * kItem + rowb;
        if constexpr (i < XR) {
          // activations of chunks 2i, 2i+1 into operand layout
          if (active) {
#pragma unroll
            for (int cc = 0; cc < 2; ++cc)
#pragma unroll
              for (int j = 0; j < 2; ++j) {
                const uint32_t pc = (uint32_t)(cc * 8 + kg * 2 + j);
                const u32x4 v = *reinterpret_cast<const u32x4*>(base + ((pc ^ swz) << 4));
                if constexpr (BITS == 4) xa[i * 2 + cc][j] = pair_stride4(v);
                else xa[i * 2 + cc][j] = __builtin_bit_cast(bf16x8, v);
              }
          }
          if constexpr (i == XR - 1) {
            if (active) chunk_sums();
          }
        } else {
          constexpr int t = i - XR;
          if (active && t < ntiles)
            acc[t] = tile_math(base, tabs + slot * kTab + tab_row, acc[t]);
          // Last pass: this wavefront's partial sums of tile t go where its own
          // slice of the tile was (nobody else reads that region, and a tile's
          // slot is not refilled within a pass); the loaders add the slices up.
          if (p == passes - 1 && t < ntiles) {
            float* part = reinterpret_cast<float*>(ring + slot * kItem + wave * 4096);
#pragma unroll
            for (int e = 0; e < 4; ++e) part[e * kWave + lane] = acc[t][e];
          }
        }
        // mirror of the loaders' issue after this item's barrier
        constexpr int e = S::B + i - 1;
        const int freed = i >= 1 ? sl_cur[i >= 1 ? i - 1 : 0] : prev_last;
        if (i >= 1 || p >= 1) {
          if constexpr (e < NI) sl_cur[S::item_at(e)] = freed;
          else if (!last) sl_nxt[S::item_at(e - NI)] = freed;
        }
      };
      static_for<NI>(consume);
      prev_last = sl_cur[NI - 1];
      if (last) item_barrier();                   // everything consumed
#pragma unroll
      for (int k = 0; k < NI; ++k) sl_cur[k] = sl_nxt[k];
    }
  }
}

template <int BITS, int CW, int NL, int TMAX, int GSHIFT, int XD>
void launch_one(const GemvArgs& a, int64_t batch, int rows_per_wg, hipStream_t st, int chunks = 1) {
  dim3 grid((unsigned)ceil_div(a.N, rows_per_wg), (unsigned)batch, (unsigned)chunks);
  constexpr int kTabKind = (CW >= 4 ? CW * 256 : 1024) * (GSHIFT == 5 ? 2 : 1);
  constexpr int XR = XD ? 0 : 2048 / BITS / 128;
  // (direct variants: plus a 1 KB patch a compute wavefront for staging activations)
  const size_t lds = (size_t)(XD || XR + TMAX >= 4 ? 4 : XR + TMAX) * (CW * 4096 + 2 * kTabKind) +
                     (XD != 0 && GSHIFT != 5 ? (size_t)CW * 1024 : 0);
  constexpr auto kern = skinny2_kernel<BITS, CW, NL, TMAX, GSHIFT, XD>;
  if (!lds_limit<kern>(lds)) return;
  hipLaunchKernelGGL(kern, grid, dim3(kWave * (CW + NL)), lds, st, a, rows_per_wg);
}

template <int BITS, int CW, int NL, int TMAX, int XD>
void launch_k(const GemvArgs& a, int64_t batch, int rows_per_wg, hipStream_t st, int chunks = 1) {
  if constexpr (BITS == 4 && XD != 0) {
    if (a.gshift == 2) return launch_one<BITS, CW, NL, TMAX, 2, XD>(a, batch, rows_per_wg, st, chunks);
  }
  if constexpr (BITS == 4 && XD == 1) {
    if (a.gshift == 7) return launch_one<BITS, CW, NL, TMAX, 7, XD>(a, batch, rows_per_wg, st, chunks);
  }
  switch (a.gshift) {
    case 1: return launch_one<BITS, CW, NL, TMAX, 1, XD>(a, batch, rows_per_wg, st, chunks);
    case 3: return launch_one<BITS, CW, NL, TMAX, 3, XD>(a, batch, rows_per_wg, st, chunks);
    case 4: return launch_one<BITS, CW, NL, TMAX, 4, XD>(a, batch, rows_per_wg, st, chunks);
    case 5: return launch_one<BITS, CW, NL, TMAX, 5, XD>(a, batch, rows_per_wg, st, chunks);
    case 6: return launch_one<BITS, CW, NL, TMAX, 6, XD>(a, batch, rows_per_wg, st, chunks);
    default: return launch_one<BITS, CW, NL, TMAX, 0, XD>(a, batch, rows_per_wg, st, chunks);
  }
}

int device_cus() {
  static const int cus = [] {
    int dev = 0, n = 256;
    if (hipGetDevice(&dev) == hipSuccess) {
      hipDeviceProp_t p;
      if (hipGetDeviceProperties(&p, dev) == hipSuccess && p.multiProcessorCount > 0) n = p.multiProcessorCount;
    }
    return n;
  }();
  return cus;
}

// One pass (K is exactly the eight slices of the compute wavefronts) and few
// rows of activations: the variant whose compute wavefronts fetch their own
// activations.  Its tile loop is a real loop, so a workgroup takes as many
// rows as make the grid one workgroup per compute unit (or a whole number of
// such rounds), up to 128.  With more than eight rows of activations their
// direct fetch costs 2-4 us more than the ring's rounds, which still pays
// where the ring variant (at most 64 rows a workgroup) would need a second
// round of workgroups (28672 x 4096 at M = 16: 17 against 22 us).
bool direct_x(int64_t M, int64_t N, int64_t K, int bits) {
  static const char* const env = experiment_env("QMM_SKINNY2_XD");   // 0 | 1 overrides the choice (experiments)
  static const int force = env ? atoi(env) : -1;
  if (force >= 0) return force != 0;
  const int64_t per = ceil_div(N, (int64_t)device_cus());
  // More than eight rows of activations on a weight of at most 64 rows per
  // compute unit: with one pass over K the direct variant stages the
  // activations through LDS patches (whole-line loads) and is ahead of the
  // ring (4096 x 14336 at M = 16: 12.1 against 12.9 us a launch, 4096 x 4096:
  // 6.5 against 7.6; fewer than eight slices: 9216 x 3072 8.6 against 12.2 on
  // the self-loading kernel); with several passes the ring variant stays.
  if (M > 8 && per <= 64 && K * bits / 8 / 256 > 8) return false;
  // Several passes over K: the next pass's activations are fetched when the
  // pass begins, which costs about 0.8 us a pass; measured against the other
  // kernels at M = 4 (us): 28672 x 8192 30.8 / 38.4, 57344 x 8192 61 / 79,
  // 10240 x 8192 16.1 / 18.3, eight-bit 14336 x 4096 16.7 / 18.6 and 22016 x
  // 4096 25.2 / 30.8, but 8192 x 8192 14.2 / 12.9 and 4096 x 14336 15.3 / 12.3:
  // it pays from three tiles a workgroup on.
  const int64_t slices = K * bits / 8 / 256;
  if (slices > 8) {
    // ... unless the kernel can pack every pass's activations into the sixteen
    // operand rows at once (passes x M <= 16), which takes the fetches away
    const int64_t passes = ceil_div(slices, (int64_t)8);
    const bool packs = (passes <= 2 && M <= 8) || (passes <= 4 && M <= 4);
    return per > 32 || packs;
  }
  return true;
}

}  // namespace

void skinny_geometry(int64_t N, int64_t K, int bits, int* waves, int* rows_per_wg);

// Does the loader-wavefront kernel serve this shape, and with how many rows a
// workgroup?  The ring variant pays off where a workgroup streams three or
// four tiles over eight K-slices at a time (with two tiles a workgroup its
// activation items outweigh the tiles and the self-loading kernel is 13 %
// faster).  Eight compute and four loader wavefronts either way.
bool skinny2_plan(int64_t M, int64_t N, int64_t K, int bits, int* rows_per_wg) {
  int waves, rows;
  skinny_geometry(N, K, bits, &waves, &rows);
  if (waves != 8) {
    // Three to seven K-slices a row (K = 1536 ... 3584 with four-bit codes):
    // the one-pass direct variant with some of its compute wavefronts idle is
    // still well ahead of the self-loading kernel, whose four wavefronts a
    // workgroup keep too little in flight (M = 4, us a launch: 37888 x 3584
    // 21.2 against 27.4, 16384 x 3072 9.0 / 13.6, 20480 x 2560 9.6 / 15.9,
    // 8192 x 2048 5.6 / 6.2, 32768 x 1536 11.7 / 15.4, eight-bit 16384 x 1536
    // 7.5 / 10.4; with two slices it loses on large weights: 65536 x 1024
    // 19.9 / 13.7).
    static const bool off = experiment_env("QMM_S2_NO_FEW_SLICES") != nullptr;
    const int64_t slices = K * bits / 8 / 256;
    if (off || slices < 3 || !direct_x(M, N, K, bits)) return false;
  }
  if (direct_x(M, N, K, bits)) {
    const int64_t cus = device_cus();
    const int64_t per = ceil_div(N, cus);
    const int64_t rounds = ceil_div(per, 128);
    int64_t r = ceil_div(N, cus * rounds);
    if (r < 16) r = 16;
    *rows_per_wg = (int)r;
    return true;
  }
  *rows_per_wg = rows;
  return rows > 32 && rows <= 64;
}

// Rows a workgroup for the direct variants whatever the shape (float16 tables:
// the self-loading kernel does not read them).
int skinny2_direct_rows(int64_t N) {
  const int64_t cus = device_cus();
  const int64_t rounds = ceil_div(ceil_div(N, cus), (int64_t)128);
  const int64_t r = ceil_div(N, cus * rounds);
  return (int)(r < 16 ? 16 : r);
}

// tab: QMM_BF16 or QMM_F16 tables; force_direct: a direct variant even where
// the ring variant or the self-loading kernel would be chosen
void skinny2_dispatch(const GemvArgs& a0, int64_t batch, int gs, int bits, int rows, hipStream_t st,
                      int tab, bool force_direct) {
  GemvArgs a = a0;
  a.gshift = (gs == 128 ? 1 : 0) + (tab == QMM_F16 ? 3 : tab == QMM_F32 ? 5 : 0);
  bool xd = force_direct || direct_x(a.M, a.N, a.K, bits);
  // float32 tables with groups of 64 fill the LDS with table rows: no room for
  // the staging patches, and direct loads of more than eight rows lose to the ring
  if (xd && !force_direct && a.M > 8 && rows <= 64 && tab == QMM_F32 && gs == 64) xd = false;
  if (xd) {                                       // up to eight tiles' sums in registers over several passes
    const bool one_pass = a.K * bits / 8 / 256 <= 8;
    if (one_pass) {
      if (bits == 4) launch_k<4, 8, 4, 4, 1>(a, batch, rows, st);
      else launch_k<8, 8, 4, 4, 1>(a, batch, rows, st);
    } else {
      if (bits == 4) launch_k<4, 8, 4, 8, 2>(a, batch, rows, st);
      else launch_k<8, 8, 4, 8, 2>(a, batch, rows, st);
    }
    return;
  }
  if (bits == 4) launch_k<4, 8, 4, 4, 0>(a, batch, rows, st);
  else launch_k<8, 8, 4, 4, 0>(a, batch, rows, st);
}

bool skinny_supported(int64_t N, int64_t K, int gs, int bits, int mode, int tab, const void* s,
                      const void* b);

// Grouped decode: the pairs of an expert-indexed product, sorted by expert
// (segments / src_row / out_row as the routing pass writes them), as one
// decode product per segment (an expert's rows, sixteen at a time): every
// expert's weight is streamed once per sixteen pairs that name it.  Grid y =
// segment, provisioned for the most there can be (workgroups past the count
// leave at once; an empty workgroup still costs about a microsecond of a
// compute unit, which is why the grid is not expert x chunk).
bool skinny2_mx_supported(int64_t N, int64_t K, const void* s);
static int64_t mx_rows_per_wg(int64_t N, int64_t K, int64_t products);

bool skinny2_grouped_supported(int64_t N, int64_t K, int gs, int bits, int mode, int tab,
                               const void* s, const void* b, int64_t E) {
  // (MXFP4 whose K is no whole number of slices has no other staged kernel to go to: its ragged
  // one-pass form takes the grouped decode from three slices on)
  if (mode == QMM_MODE_MXFP4) return (K / 512 >= 8 || K % 512 != 0) && skinny2_mx_supported(N, K, s);
  if (!skinny_supported(N, K, gs, bits, mode, QMM_BF16, s, b)) return false;   // bf16, float16 and float32 tables alike
  return K * bits / 8 / 256 >= 8;
}

int64_t skinny2_max_segments(int64_t P, int64_t E) { return (E < P ? E : P) + P / 16; }

void skinny2_grouped_dispatch(const void* x, const void* w, const void* s, const void* b, void* y,
                              int y_dtype, const int32_t* segments, const int32_t* src_row,
                              const int32_t* out_row, int64_t P, int64_t T, int64_t E, int64_t N,
                              int64_t K, int gs, int bits, int mode, int tab, hipStream_t st) {
  GemvArgs a;
  a.x = static_cast<const uint16_t*>(x);
  a.w = static_cast<const uint32_t*>(w);
  a.s = s;
  a.b = b;
  a.y = y;
  a.M = 1; a.N = (int)N; a.K = (int)K;
  a.gshift = mode == QMM_MODE_MXFP4 ? (K % 512 ? 7 : 2)
                                    : (gs == 128 ? 1 : 0) + (tab == QMM_F16 ? 3 : tab == QMM_F32 ? 5 : 0);
  a.y_dtype = y_dtype;
  a.lhs_idx = nullptr;
  a.rhs_idx = nullptr;
  a.segments = segments;
  a.src_row = src_row;
  a.out_row = out_row;
  a.x_rows = (int)T;
  const int64_t cus = device_cus();
  const int64_t rounds = ceil_div(ceil_div(N, cus), (int64_t)128);
  int64_t rows = ceil_div(N, cus * rounds);
  if (rows < 16) rows = 16;
  if (mode == QMM_MODE_MXFP4) rows = mx_rows_per_wg(N, K, P < E ? P : E);
  const int64_t segs = skinny2_max_segments(P, E);
  if (K * bits / 8 / 256 <= 8) {
    if (bits == 4) launch_k<4, 8, 4, 4, 1>(a, segs, (int)rows, st);
    else launch_k<8, 8, 4, 4, 1>(a, segs, (int)rows, st);
  } else {
    if (bits == 4) launch_k<4, 8, 4, 8, 2>(a, segs, (int)rows, st);
    else launch_k<8, 8, 4, 8, 2>(a, segs, (int)rows, st);
  }
}

// MXFP4 decode on the direct variants: K a multiple of 512 with at least
// three slices (with fewer than eight some compute wavefronts idle; M = 4, us
// a launch against the general kernel: 16384 x 3072 8.2 / 16.4, 37888 x 3584
// 19.4 / 33.3, 32768 x 1536 9.9 / 13.6), scale rows dword-aligned (they are
// fetched as 16-byte runs).
bool skinny2_mx_supported(int64_t N, int64_t K, const void* s) {
  static const bool off = experiment_env("QMM_NO_SKINNY_MX") != nullptr;
  if (off || N * (K / 2) >= 0x7FFFFFFFll) return false;       // 32-bit lane offsets
  if (K % 512 == 0) return K / 512 >= 3 && (reinterpret_cast<uintptr_t>(s) & 3u) == 0;
  // the ragged one-pass form: K any multiple of 64 between three and eight slices, a tile's
  // scale rows a 16-byte-aligned run (every expert's table a multiple of 16 bytes, rows dealt by eights)
  return K % 64 == 0 && K > 1024 && K < 4096 && (N * (K / 32)) % 16 == 0 &&
         (reinterpret_cast<uintptr_t>(s) & 15u) == 0;
}

// Rows a workgroup for the MXFP4 decode: `products` decode products run side by side (batch entries,
// the segments of a grouped product), so each gets its share of the compute units -- a workgroup's
// fixed cost (its first tile lands about 3.5 us after it starts) is then paid once a compute unit, not
// once per product.  For the ragged form a multiple of eight (see above).
static int64_t mx_rows_per_wg(int64_t N, int64_t K, int64_t products) {
  const int64_t cus = device_cus();
  if (products < 1) products = 1;
  const int64_t wgs = products >= cus ? 1 : cus / products;      // workgroups a product
  int64_t rows = ceil_div(N, wgs);
  if (rows > 128) rows = ceil_div(N, ceil_div(N, (int64_t)128));
  if (rows < 16) rows = 16;
  if (K % 512) rows = ceil_div(rows, (int64_t)8) * 8;
  return rows;
}

// For the plan query: whether a dense MXFP4 decode product of this shape runs here (tables taken as
// aligned), and with how many rows a workgroup.
bool skinny2_mx_plan(int64_t N, int64_t K, int* rows_per_wg) {
  if (!skinny2_mx_supported(N, K, nullptr)) return false;
  *rows_per_wg = (int)mx_rows_per_wg(N, K, 1);
  return true;
}

void skinny2_mx_dispatch(const GemvArgs& a0, int64_t batch, hipStream_t st) {
  GemvArgs a = a0;
  a.gshift = a.K % 512 ? 7 : 2;
  const int64_t rows = mx_rows_per_wg(a.N, a.K, batch);
  if (a.K <= 4096) launch_k<4, 8, 4, 4, 1>(a, batch, (int)rows, st);
  else launch_k<4, 8, 4, 8, 2>(a, batch, (int)rows, st);
}

}  // namespace qmm

#ifdef QMM_TIMELINE
extern "C" int qmm_debug_stamps(void* out, size_t bytes) {
  if (bytes > sizeof(qmm::g_stamps)) bytes = sizeof(qmm::g_stamps);
  return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(qmm::g_stamps), bytes);
}
#endif

