// Prefill-regime quantized matmul on gfx950 with the wavefronts' roles split:
// the grouped (per-expert) product that the reference hands to mx.gather_qmm
// (src/metaljax/moe.py:1283-1340) and the dense product of
// mx.quantized_matmul (src/metaljax/qmm.py:2491) at M > 16, with the
// dequantization semantics of src/metaljax/qmm.py:71-79 (w = scale * q + bias
// as one fma).
//
// Why a second kernel.  In the general kernel every wavefront both
// dequantizes and multiplies, and a single wavefront a SIMD issues one
// instruction per four clocks, of any kind: the dequantization of a K-tile
// (about 100 vector ALU instructions per thread, the LDS writes, the loads
// that feed them) stands in the way of its own MFMAs.  With short row groups
// that is most of the time (a K-tile of a 128-row tile took 0.78 us of which
// the MFMAs were a third).
//
// So the roles are split, as in the decode kernel.  A workgroup is eight
// wavefronts, two a SIMD:
//   * producers (wavefronts 4-7) load the packed words and the scale / bias
//     windows, dequantize a K-tile (float32 fma, one round-to-nearest-even
//     to bf16: the reference's tile, bit for bit) two K-tiles ahead of its use
//     and write it to LDS one K-tile ahead;
//   * consumers (wavefronts 0-3) load their activation fragments (the re-laid
//     ax[k/8][row] form of the general kernel), read the weight fragments of
//     K-tile t from LDS and issue the MFMAs.
// One workgroup barrier per K-tile publishes tile t+1 and frees the stage of
// tile t-1 (three stages).
//
// Tile: up to 256 rows x 128 columns, and the rows a tile really holds pick
// one of three loops.  Up to 128 rows: consumer w multiplies row block w
// (32 rows) with the whole weight tile.  Up to 160: rows 128..159 are a fifth
// block split by columns, consumer w multiplies it with column block w.  More:
// consumer w multiplies row blocks w and w + 4 (every weight fragment read
// from LDS then feeds two MFMAs).  Longer experts take several tiles.
#include <type_traits>

#include "qmm_gemm2_common.hpp"

namespace qmm {

namespace {

using namespace g2;

constexpr int kS = 3;                 // LDS stages: K-tile t lives in stage t % 3
constexpr int kTileRows = 256;        // eight row blocks, two a consumer
constexpr int kAR = 3;                // activation fragments: K-tile t lives in ring slot t % 3 (t % 2 on full tiles)

// Table rows staged in LDS (a row's scales / biases of the whole K when they
// fit 128 bytes): 128 + 16 bytes a row, so that eight rows fall on different banks.
constexpr int kTabRow = 144;
constexpr int kTabKind = BN * kTabRow;

// TLDS: a tile's table rows are fetched once, into LDS (each row's line comes
// in once instead of once per four K-tiles); otherwise 16-byte windows per
// four K-tiles in registers.
template <int MODE, int BITS, bool G64, bool TLDS>
__global__ __launch_bounds__(512) void gemm2s_kernel(Gemm2Args a) {
  static_assert(!G64 || MODE == 0, "one group a K-tile is an affine layout");
  constexpr int WBITS = (MODE == 1) ? 4 : BITS;
  constexpr int WPT = 32 * WBITS / 32;             // packed words per producer thread and K-tile: 4 | 8
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- which tile?  The grid is provisioned for the worst raggedness and
  // only the row tiles that exist are dealt (deal_grouped_tile: a band of
  // column tiles of every expert per XCD, expert after expert, or one by one
  // round the XCDs when the bands would be uneven).
  const int n_tiles = (a.N + BN - 1) / BN;
  const int xcd = blockIdx.x & 7, l = blockIdx.x >> 3;
  int tile_m, tile_n;
  deal_grouped_tile(n_tiles, xcd, l, tile_m, tile_n);
  int e = 0, row_lo = 0, row_hi = a.R, mt_idx = 0;
  if (!a.row_offsets) {
    // one expert of all rows: an eighth of the grid takes a contiguous run of
    // tiles, column tile fastest, so its workgroups share few activation rows
    const int m_tiles = (a.R + kTileRows - 1) / kTileRows;
    const int total = n_tiles * m_tiles, per = (total + 7) / 8;
    const int t = xcd * per + l;
    if (l >= per || t >= total) return;
    tile_m = t / n_tiles;
    tile_n = t % n_tiles;
    mt_idx = tile_m;
  } else {
    if (tile_n >= n_tiles) return;
    const RowTile rt = find_row_tile(a.row_offsets, a.E, a.R, kTileRows, tile_m);
    if (!rt.found) return;
    e = rt.e; row_lo = rt.lo; row_hi = rt.hi; mt_idx = rt.idx;
  }
  const int m0 = row_lo + mt_idx * kTileRows;
  if (m0 >= row_hi) return;
  const int m_end = row_hi < m0 + kTileRows ? row_hi : m0 + kTileRows;
  const int n0 = tile_n * BN;
  const int KT = a.K / BK;
  auto clampk = [&](int kt) { return kt < KT ? kt : KT - 1; };

  if (wave >= 4) {
    // ======================= producers: the weight tile ====================
    const int ptid = tid - 256;
    const int wrow = ptid >> 1, whalf = ptid & 1;  // weight row of the tile, 32-code half of its K-tile
    const int64_t wpr = (int64_t)a.K * WBITS / 32;
    const int gs = (MODE == 1) ? 32 : a.gs;
    const int64_t ng = a.K / gs;
    constexpr int tabsz = (MODE == 1) ? 1 : 2;     // E8M0 bytes | bf16
    const uint32_t* wb = a.w + (int64_t)e * a.N * wpr;
    const char* sb = static_cast<const char*>(a.s) + (int64_t)e * a.N * ng * tabsz;
    const char* bb = (MODE == 1) ? sb : static_cast<const char*>(a.b) + (int64_t)e * a.N * ng * tabsz;
    int64_t wn_row = n0 + wrow;
    if (wn_row >= a.N) wn_row = a.N - 1;           // rows past N are computed and never stored
    const auto rw = make_rsrc(wb, (int64_t)a.N * wpr * 4);
    const uint32_t wvo = (uint32_t)((wn_row * wpr + whalf * WPT) * 4);
    struct WRegs { uint32_t q[WPT]; };
    auto load_w = [&](int kt, WRegs& r) {
      const uint32_t so = (uint32_t)kt * (BK * WBITS / 8);
#pragma unroll
      for (int j = 0; j < WPT; j += 4) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rw, wvo + j * 4, so, 0);
        r.q[j] = v[0]; r.q[j + 1] = v[1]; r.q[j + 2] = v[2]; r.q[j + 3] = v[3];
      }
    };
    // scale / bias window: the entries of four K-tiles of this thread's row
    // (at most 16 bytes a table), fetched once per four K-tiles
    struct TabWin { u32x4 s, b; };
    const auto rs = make_rsrc(sb, (int64_t)a.N * ng * tabsz);
    const auto rb = make_rsrc(bb, (int64_t)a.N * ng * tabsz);
    const uint32_t tvo = (uint32_t)(wn_row * ng * tabsz);
    const int gshift = gs == 32 ? 5 : (gs == 64 ? 6 : 7);
    auto load_win = [&](int quad, TabWin& tw) {
      const uint32_t so = (uint32_t)(((quad * 4 * BK) >> gshift) * tabsz);
      tw.s = __builtin_amdgcn_raw_buffer_load_b128(rs, tvo, so, 0);
      if constexpr (MODE == 0) tw.b = __builtin_amdgcn_raw_buffer_load_b128(rb, tvo, so, 0);
    };
    uint32_t eidx[4];                              // entry of K-tile t' inside its window, for this thread's half
#pragma unroll
    for (int t = 0; t < 4; ++t) eidx[t] = (uint32_t)((t * BK + whalf * 32) >> gshift);
    auto pick = [&](const u32x4& w, uint32_t ei) -> float {
      const uint32_t byte = ei * (uint32_t)tabsz;
      const uint32_t d = byte >> 2;
      uint32_t v = w[0];
      v = d == 1 ? w[1] : v;
      v = d == 2 ? w[2] : v;
      v = d == 3 ? w[3] : v;
      v >>= (byte & 3u) * 8u;
      if constexpr (MODE == 1) return e8m0_to_f32(v & 255u);
      return __uint_as_float(v << 16);
    };
    unsigned char* tabs = smem + kS * kStage + wrow * kTabRow;
    auto entry = [&](int kt, auto tqc, const TabWin& tw, float& sc, float& bi) {
      constexpr int tq = decltype(tqc)::value;
      if constexpr (TLDS) {
        const int ei = (kt * BK + whalf * 32) >> gshift;
        if constexpr (MODE == 1) {
          sc = e8m0_to_f32(tabs[ei]);
          bi = 0.f;
        } else {
          sc = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(tabs)[ei]);
          bi = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(tabs + kTabKind)[ei]);
        }
      } else if constexpr (G64) {                          // one group a K-tile: entry tq for every thread
        const uint32_t vs = tw.s[tq >> 1], vb = tw.b[tq >> 1];
        sc = __uint_as_float((tq & 1) ? (vs & 0xFFFF0000u) : (vs << 16));
        bi = __uint_as_float((tq & 1) ? (vb & 0xFFFF0000u) : (vb << 16));
      } else {
        sc = pick(tw.s, eidx[tq]);
        bi = MODE == 1 ? 0.f : pick(tw.b, eidx[tq]);
      }
    };
    // Pipeline of a weight tile: its words are requested a quad at a time,
    // seven to ten K-tiles before it is published, it is dequantized into
    // registers two K-tiles before, and written to LDS at the start of the
    // step before (the write then has the whole step to finish before the
    // barrier that publishes it).
    auto dequant_tile = [&](u32x4 (&dst)[4], const WRegs& r, float sc, float bi) {
#pragma unroll
      for (int pc = 0; pc < 4; ++pc) dst[pc] = dequant_piece<MODE, BITS>(r.q, pc, sc, bi);
    };
    auto write_tile = [&](int stage, const u32x4 (&src)[4]) {
#pragma unroll
      for (int pc = 0; pc < 4; ++pc)
        *reinterpret_cast<u32x4*>(smem + stage * kStage + swz(wrow, whalf * 4 + pc)) = src[pc];
    };
    TabWin tw_cur, tw_nxt;
    // Words of K-tile t live in wr[t % 12].  They are requested a quad (four
    // K-tiles) at a time: the four 16-byte pieces that a thread needs for a
    // quad lie in one 128-byte line of its row (four-bit codes; two lines with
    // eight-bit codes), and asked for one K-tile at a time the line came in
    // four times, each time evicted again by the 36 KB a K-tile moves through
    // the 32 KB L1.
    WRegs wr[12];
    u32x4 pend[4];                                  // the dequantized tile that the next step writes
    auto load_quad = [&](int kt0, auto sc0) __attribute__((always_inline)) {
      constexpr int s0 = decltype(sc0)::value;      // ring slot of tile kt0
#pragma unroll
      for (int i = 0; i < 4; ++i) load_w(clampk(kt0 + i), wr[(s0 + i) % 12]);
    };
    if constexpr (TLDS) {
      // this thread's half (64 bytes) of its row's table, per kind; the other
      // half is its neighbour lane's, and a wavefront's LDS accesses stay in order
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t o = (uint32_t)(whalf * 64 + i * 16);
        *reinterpret_cast<u32x4*>(tabs + o) = __builtin_amdgcn_raw_buffer_load_b128(rs, tvo + o, 0, 0);
        if constexpr (MODE == 0)
          *reinterpret_cast<u32x4*>(tabs + kTabKind + o) = __builtin_amdgcn_raw_buffer_load_b128(rb, tvo + o, 0, 0);
      }
    } else {
      load_win(0, tw_cur);
    }
    load_quad(0, std::integral_constant<int, 0>{});
    load_quad(4, std::integral_constant<int, 4>{});
    tw_nxt = tw_cur;
    {
      float sc, bi;
      entry(0, std::integral_constant<int, 0>{}, tw_cur, sc, bi);
      dequant_tile(pend, wr[0], sc, bi);
      write_tile(0, pend);
      entry(clampk(1), std::integral_constant<int, 1>{}, tw_cur, sc, bi);
      dequant_tile(pend, wr[1], sc, bi);
    }
    lds_barrier();                                  // tile 0 is published
    __builtin_amdgcn_sched_barrier(0);
    // step kt runs beside the consumers' K-tile kt: it publishes tile kt + 1 and
    // dequantizes tile kt + 2 (past the last tile: clamped repeats into stages
    // that nobody reads)
    auto pstep = [&](int kt, auto tc) __attribute__((always_inline)) {
      constexpr int t12 = decltype(tc)::value;      // kt % 12
      constexpr int t = t12 & 3;
      write_tile((kt + 1) % kS, pend);
      if constexpr (t == 0) {
        // the quad two ahead, into the slots of the quad before this one
        // (its last tile was dequantized three steps ago)
        load_quad(kt + 8, std::integral_constant<int, (t12 + 8) % 12>{});
        if constexpr (!TLDS) {
          const int q = (kt >> 2) + 1;              // next quad's windows (clamped at the end)
          load_win(q * 4 < KT ? q : (kt >> 2), tw_nxt);
        }
      }
      float sc, bi;
      entry(clampk(kt + 2), std::integral_constant<int, (t + 2) & 3>{}, t >= 2 ? tw_nxt : tw_cur, sc, bi);
      // the step's barrier as soon as the write has landed (the consumers reach
      // theirs before their last k-step); the next tile's arithmetic after it
      lds_barrier();
      __builtin_amdgcn_sched_barrier(0);
      dequant_tile(pend, wr[(t12 + 2) % 12], sc, bi);
      if (t == 3) tw_cur = tw_nxt;
      __builtin_amdgcn_sched_barrier(0);
    };
    int kt = 0;
    for (; kt + 12 <= KT; kt += 12) {
      pstep(kt, std::integral_constant<int, 0>{});
      pstep(kt + 1, std::integral_constant<int, 1>{});
      pstep(kt + 2, std::integral_constant<int, 2>{});
      pstep(kt + 3, std::integral_constant<int, 3>{});
      pstep(kt + 4, std::integral_constant<int, 4>{});
      pstep(kt + 5, std::integral_constant<int, 5>{});
      pstep(kt + 6, std::integral_constant<int, 6>{});
      pstep(kt + 7, std::integral_constant<int, 7>{});
      pstep(kt + 8, std::integral_constant<int, 8>{});
      pstep(kt + 9, std::integral_constant<int, 9>{});
      pstep(kt + 10, std::integral_constant<int, 10>{});
      pstep(kt + 11, std::integral_constant<int, 11>{});
    }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 0>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 1>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 2>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 3>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 4>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 5>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 6>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 7>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 8>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 9>{}); ++kt; }
    if (kt < KT) { pstep(kt, std::integral_constant<int, 10>{}); ++kt; }
    return;
  }

  // ========================= consumers: the MFMAs ==========================
  const int wm = wave;                             // row block, and column block of the fifth
  const int li = lane & 31, kh = lane >> 5;
  // How many rows the tile holds decides the loop, for the whole workgroup:
  //   0: up to 128, one row block a consumer;
  //   1: up to 160, plus a fifth block split by columns;
  //   2: up to 256, two row blocks a consumer (w and w + 4).
  const int path = m_end - m0 <= 128 ? 0 : (m_end - m0 <= 160 ? 1 : 2);
  const bool five = path == 1, two = path == 2;
  // lane (row li, k-half kh) of k-step ks reads ax[(kt*8 + ks*2 + kh) * Rp + row]
  const auto ra = make_rsrc(a.ax, (int64_t)(a.K / 8) * a.Rp * 16);
  const uint32_t avo = (uint32_t)((kh * a.Rp + m0 + wm * 32 + li) * 16);
  // the second block: the fifth block's rows, or row block w + 4
  const uint32_t avo1 = avo + (uint32_t)(five ? (4 - wm) * 512 : 128 * 16);
  typedef u32x4 AFrag[4][2];
  auto load_a_part = [&](int kt, AFrag& dst, int ks, auto nac) __attribute__((always_inline)) {
    const uint32_t so = (uint32_t)((kt * 8 + ks * 2) * 16) * (uint32_t)a.Rp;
    dst[ks][0] = __builtin_amdgcn_raw_buffer_load_b128(ra, avo, so, 0);
    if constexpr (decltype(nac)::value == 2) dst[ks][1] = __builtin_amdgcn_raw_buffer_load_b128(ra, avo1, so, 0);
  };

  f32x16 acc[4], acc2[4];                           // acc2[0] doubles as the fifth block's accumulator
#pragma unroll
  for (int r = 0; r < 16; ++r) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[j][r] = 0.f;
      acc2[j][r] = 0.f;
    }
  }
  AFrag af[kAR];
  bf16x8 fb[2][4], fbx[2];                          // B fragments: k-step ks in set ks & 1
  auto read_b = [&](const unsigned char* pbase, int ks, int set, auto fc) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      fb[set][j] = *reinterpret_cast<const bf16x8*>(pbase + swz(j * 32 + li, ks * 2 + kh));
    if constexpr (decltype(fc)::value)
      fbx[set] = *reinterpret_cast<const bf16x8*>(pbase + swz(wm * 32 + li, ks * 2 + kh));
  };

  auto run = [&](auto pathc) __attribute__((always_inline)) {
    constexpr int PATH = decltype(pathc)::value;
    constexpr bool FIVE = PATH == 1, TWO = PATH == 2;
    // activation K-tiles in registers: three (two K-tiles ahead), or two on a
    // full tile, whose 128 accumulator registers leave room for no more
    constexpr int AR = TWO ? 2 : 3;
    const std::integral_constant<int, PATH == 0 ? 1 : 2> nac;
    const std::integral_constant<bool, FIVE> fc;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) load_a_part(0, af[0], ks, nac);
    if constexpr (AR == 3) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) load_a_part(clampk(1), af[1], ks, nac);
    }
    lds_barrier();                                  // tile 0 is published
    read_b(smem, 0, 0, fc);
    auto cstep = [&](int kt, auto tc, auto ac) __attribute__((always_inline)) {
      constexpr int t = decltype(tc)::value;        // kt % 3: the LDS stage
      constexpr int as = decltype(ac)::value;       // kt % AR: the activation slot
      const unsigned char* pb = smem + t * kStage;
      constexpr int nstage = (t + 1) % kS;
      const int ktn = clampk(kt + AR - 1);
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        // the next k-step's fragments; in the last k-step those of the next
        // tile, which the barrier below has published (past the last tile: a
        // stage that nobody reads)
        if (ks < 3) read_b(pb, ks + 1, (ks + 1) & 1, fc);
        else read_b(smem + nstage * kStage, 0, 0, fc);
        load_a_part(ktn, af[(as + AR - 1) % AR], ks, nac);
        // the fragment read last feeds the first MFMA: one LDS wait a k-step
        if constexpr (FIVE)
          acc2[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[as][ks][1]),
                                                            fbx[ks & 1], acc2[0], 0, 0, 0);
        const bf16x8 fa = __builtin_bit_cast(bf16x8, af[as][ks][0]);
#pragma unroll
        for (int j = 3; j >= 0; --j)
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb[ks & 1][j], acc[j], 0, 0, 0);
        if constexpr (TWO) {
          const bf16x8 fa1 = __builtin_bit_cast(bf16x8, af[as][ks][1]);
#pragma unroll
          for (int j = 3; j >= 0; --j)
            acc2[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa1, fb[ks & 1][j], acc2[j], 0, 0, 0);
        }
        // order inside the k-step: the next k-step's fragment reads first (their
        // latency hides under this k-step's MFMAs), the loads spread between the MFMAs
        constexpr int NM = TWO ? 8 : (FIVE ? 5 : 4);
        __builtin_amdgcn_sched_group_barrier(0x100, FIVE ? 5 : 4, 0);
#pragma unroll
        for (int m = 0; m < NM; ++m) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (m < (PATH == 0 ? 1 : 2)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // One barrier a K-tile, before its last k-step: tile kt + 1 is
        // published (its producers wrote it at the start of their step), and
        // the producers learn that tile kt - 1 is read (they reuse its stage
        // in their next step).  The last k-step then fetches the next tile's
        // first fragments under its own MFMAs.
        if (ks == 2) lds_barrier();
      }
    };
    using std::integral_constant;
    int kt = 0;
    if constexpr (AR == 3) {
      for (; kt + 3 <= KT; kt += 3) {
        cstep(kt, integral_constant<int, 0>{}, integral_constant<int, 0>{});
        cstep(kt + 1, integral_constant<int, 1>{}, integral_constant<int, 1>{});
        cstep(kt + 2, integral_constant<int, 2>{}, integral_constant<int, 2>{});
      }
      if (kt < KT) { cstep(kt, integral_constant<int, 0>{}, integral_constant<int, 0>{}); ++kt; }
      if (kt < KT) { cstep(kt, integral_constant<int, 1>{}, integral_constant<int, 1>{}); ++kt; }
    } else {
      for (; kt + 6 <= KT; kt += 6) {
        cstep(kt, integral_constant<int, 0>{}, integral_constant<int, 0>{});
        cstep(kt + 1, integral_constant<int, 1>{}, integral_constant<int, 1>{});
        cstep(kt + 2, integral_constant<int, 2>{}, integral_constant<int, 0>{});
        cstep(kt + 3, integral_constant<int, 0>{}, integral_constant<int, 1>{});
        cstep(kt + 4, integral_constant<int, 1>{}, integral_constant<int, 0>{});
        cstep(kt + 5, integral_constant<int, 2>{}, integral_constant<int, 1>{});
      }
      if (kt < KT) { cstep(kt, integral_constant<int, 0>{}, integral_constant<int, 0>{}); ++kt; }
      if (kt < KT) { cstep(kt, integral_constant<int, 1>{}, integral_constant<int, 1>{}); ++kt; }
      if (kt < KT) { cstep(kt, integral_constant<int, 2>{}, integral_constant<int, 0>{}); ++kt; }
      if (kt < KT) { cstep(kt, integral_constant<int, 0>{}, integral_constant<int, 1>{}); ++kt; }
      if (kt < KT) { cstep(kt, integral_constant<int, 1>{}, integral_constant<int, 0>{}); ++kt; }
    }
  };
  if (two) run(std::integral_constant<int, 2>{});
  else if (five) run(std::integral_constant<int, 1>{});
  else run(std::integral_constant<int, 0>{});

  // ---- epilogue.  D of a 32x32 tile: lane holds column lane % 32 and rows
  // (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5), r = 0..15.  Block 0 is row block
  // w over all columns; block 1 the fifth block's column block w, or row
  // block w + 4 over all columns.
  const bool wide = a.y_dtype != QMM_F32 && (a.N & 7) == 0 &&
                    (reinterpret_cast<uintptr_t>(a.y) & 15u) == 0;
  if (wide) {
    // 16-bit outputs: transpose each 32-row block through this wavefront's
    // share of LDS (free after the last barrier), store 16 bytes a lane
    uint16_t* o16 = reinterpret_cast<uint16_t*>(smem) + wave * (32 * BN);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (i == 1 && !five && !two) break;
      const int ncb = (i == 0 || two) ? 4 : 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j >= ncb) break;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int rl = (r & 3) + 8 * (r >> 2) + 4 * kh;
          const float v = i == 0 ? acc[j][r] : acc2[j][r];
          o16[rl * BN + j * 32 + li] =
              (uint16_t)(a.y_dtype == QMM_BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v));
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int ppr = ncb * 4;                      // 16-byte pieces per row
      for (int q = 0; q < (32 * ppr) / 64; ++q) {
        const int idx = q * 64 + lane, rl = idx / ppr, pc = idx % ppr;
        const int m = m0 + (i == 0 ? wm : (two ? wm + 4 : 4)) * 32 + rl;
        const int n = n0 + ((i == 0 || two) ? 0 : wm * 32) + pc * 8;
        if (m < m_end && n < a.N) {
          const int64_t orow = a.out_idx ? (int64_t)a.out_idx[m] : (int64_t)m;
          *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(a.y) + orow * a.N + n) =
              *reinterpret_cast<const u32x4*>(o16 + rl * BN + pc * 8);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  } else {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (i == 1 && !five && !two) break;
      const int ncb = (i == 0 || two) ? 4 : 1;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j >= ncb) break;
        const int n = n0 + ((i == 0 || two) ? j : wm) * 32 + li;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + (i == 0 ? wm : (two ? wm + 4 : 4)) * 32 + (r & 3) + 8 * (r >> 2) + 4 * kh;
          if (m < m_end && n < a.N) {
            const int64_t orow = a.out_idx ? (int64_t)a.out_idx[m] : (int64_t)m;
            store_out(a.y, orow * a.N + n, i == 0 ? acc[j][r] : acc2[j][r], a.y_dtype);
          }
        }
      }
    }
  }
}

template <int MODE, int BITS, bool G64, bool TLDS>
void launch_k(const Gemm2Args& a, hipStream_t st) {
  const int64_t m_tiles = ceil_div(a.R, kTileRows) + a.E;      // provisioned: a tile never straddles an expert
  int64_t total = ceil_div(ceil_div(a.N, BN), 8) * 8 * m_tiles;
  if (!a.row_offsets) total = ceil_div(ceil_div(a.N, BN) * ceil_div(a.R, kTileRows), 8) * 8;
  const size_t epi = (size_t)4 * 32 * BN * 2;
  const size_t need = (size_t)(kS * kStage) + (TLDS ? 2 * kTabKind : 0);
  const size_t lds = epi > need ? epi : need;
  constexpr auto kern = gemm2s_kernel<MODE, BITS, G64, TLDS>;
  if (!lds_limit<kern>(lds)) return;
  hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(512), lds, st, a);
}

template <int MODE, int BITS, bool G64>
void launch_s(const Gemm2Args& a, hipStream_t st) {
  // a row's table of the whole K in one 128-byte line per kind?
  const int64_t row_bytes = MODE == 1 ? a.K / 32 : (int64_t)(a.K / a.gs) * 2;
  static const bool no_tlds = experiment_env("QMM_GEMM2S_NOTLDS") != nullptr;
  if (row_bytes <= 128 && !no_tlds) launch_k<MODE, BITS, G64, true>(a, st);
  else launch_k<MODE, BITS, G64, false>(a, st);
}

}  // namespace

// Products whose tables can be fetched as 16-byte windows of bf16 (E8M0 for
// MXFP4) entries and whose K is a multiple of four K-tiles; everything else
// stays on the general kernel.
bool gemm2s_wanted(const g2::Gemm2Args& a, int mode, int bits) {
  static const char* env = experiment_env("QMM_GEMM2S");   // "0": never, "2": short experts only
  if (env && env[0] == '0') return false;
  const bool can = (a.row_offsets ? a.E > 0 : a.E == 1) && a.tabfast && a.K % 256 == 0 &&
                   (mode == QMM_MODE_MXFP4 || (a.tab == QMM_BF16 && (bits == 4 || bits == 8)));
  if (!can) return false;
  if (env && env[0] == '2') return a.row_offsets && a.R / a.E <= 144;
  return true;
}

void gemm2s_launch(const g2::Gemm2Args& a, int mode, int bits, hipStream_t st) {
  if (mode == QMM_MODE_MXFP4) launch_s<1, 4, false>(a, st);
  else if (bits == 4) { if (a.gs == 64) launch_s<0, 4, true>(a, st); else launch_s<0, 4, false>(a, st); }
  else { if (a.gs == 64) launch_s<0, 8, true>(a, st); else launch_s<0, 8, false>(a, st); }
}

}  // namespace qmm
