// Prefill-regime quantized matmul (M > 16) and the grouped (per-expert) form
// for gfx950, second generation: activations reach the matrix cores straight
// from global memory, only the dequantized weight tile goes through LDS.
//
// Why.  With both operand tiles in LDS a 256 x 128 x 64 step moves 144 KB
// through LDS (48 KB of writes, 96 KB of fragment reads) for 1024 clocks of
// v_mfma_f32_32x32x16_bf16 work per SIMD: more than the 128 B/clk the LDS can
// deliver, so the matrix cores wait.  The activation fragments have no reuse
// inside a wavefront row block, so they do not need LDS at all, provided a
// lane's 16 bytes (row i, 8 consecutive k) can be fetched coalesced.  A short
// pre-pass therefore re-lays x once per call:
//     ax[k/8][row]   16 bytes each (8 consecutive k of one row), rows contiguous
// so the lanes of a fragment load (32 rows x 2 k-halves) read two 512-byte
// runs, for any first row (grouped tiles start at arbitrary rows).  The row
// gather of the expert-sorted form (lhs_idx) is folded into the same pass.
//
// Main kernel.  Workgroup tile BM x 128, BK = 64, four wavefronts stacked in M
// (each (BM/4) x 128: MT x 4 MFMA tiles of 32 x 32).  Per K-tile:
//   * every thread loads 32 packed codes of one weight row (row tid/2, k-half
//     tid%2), dequantizes them with the row's scale/bias of that 32-group
//     (float32 fma, one round-to-nearest-even to bf16: the reference's tile
//     semantics, bit for bit) and writes four 16-byte pieces of the bf16 tile
//     to LDS (piece p of row r at p ^ ((r >> 1) & 7): every 16-lane pass covers all banks);
//   * every wavefront reads the whole weight tile back as B fragments and
//     multiplies it with its own activation fragments (registers).
// Schedule: the packed words of tile t+4 (they come from HBM and are consumed
// three K-tiles later) and the activation fragments of tile t+2 (from L2) are
// loaded while tile t is multiplied; tile t+1 is dequantized between the MFMAs
// of tile t; three LDS stages, one LDS-only barrier per K-tile.
#include <type_traits>

#include "qmm_gemm2_common.hpp"

namespace qmm {

// the grouped kernel for short row groups (qmm_gemm2s.hip)
bool gemm2s_wanted(const g2::Gemm2Args& a, int mode, int bits);
void gemm2s_launch(const g2::Gemm2Args& a, int mode, int bits, hipStream_t st);

namespace {

using namespace g2;

constexpr int kStages = 4;                        // stage of K-tile t = t & 3: a compile-time LDS offset

// ---------------------------------------------------------------------------
// x [x_rows, K] bf16 (rows optionally gathered through lhs_idx) -> ax[K/8][Rp]
// One thread = one 16-byte piece.  A wavefront covers 8 rows x 8 pieces, so
// that both sides move whole 128-byte lines: 8 lanes read one row's line, and
// the 8 rows of one piece are written as one 128-byte run.  A workgroup is
// four such wavefronts side by side along K (512 contiguous bytes a row).
__global__ __launch_bounds__(256) void gemm_prep_kernel(const uint16_t* __restrict__ x,
                                                        const int32_t* __restrict__ lhs_idx,
                                                        u32x4* __restrict__ ax, int R, int x_rows,
                                                        int K, int Rp) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pieces = K / 8;
  const int pblocks = (pieces + 31) / 32;
  const int rb = blockIdx.x / pblocks, pb = blockIdx.x % pblocks;
  const int row = rb * 8 + (lane >> 3);
  const int piece = pb * 32 + wave * 8 + (lane & 7);
  if (row >= R || piece >= pieces) return;
  const int64_t src = lhs_idx ? (int64_t)lhs_idx[row] : (int64_t)row;
  const bool ok = src >= 0 && src < x_rows;        // an index outside x gathers a zero row
  u32x4 v = {0u, 0u, 0u, 0u};
  if (ok) v = reinterpret_cast<const u32x4*>(x + src * K)[piece];
  ax[(int64_t)piece * Rp + row] = v;
}

// MT x NT MFMA tiles (32 x 32) per wavefront; WMW wavefronts stacked in M and
// NWAVES / WMW side by side in N, which always spans the 128 weight rows of a tile:
//   MT=2 NT=4 WMW=4 NWAVES=4: 256 x 128 workgroup tile, one wavefront a SIMD
//                    (every wavefront reads the whole weight tile, activations
//                    are private);
//   MT=1 NT=2 WMW=4 NWAVES=8: 128 x 128 for short row groups, two wavefronts a
//                    SIMD (one's vector ALU and load issue fill the other's
//                    MFMA shadow) at a quarter of the work each.
//
// RAG (ragged row groups: the grouped launches) deals a wavefront's row blocks
// round-robin (block wm + i*WMW instead of wm*MT + i), so that a tile whose
// rows end in its first half leaves every wavefront's second block empty and
// runs a main loop without it.
//
// TF selects how scales / biases are fetched.  1..3: as 16-byte windows (four
// K-tiles of a row at once), with the entry type fixed at compile time --
// 1 = two-byte bf16 (one-byte E8M0 for MXFP4), 2 = float32, 3 = float16 -- so
// that picking an entry is a handful of selects and the K loop has no branch
// in it (a branch would end the region the MFMAs are interleaved in).
// 0: any layout, one load per entry, types read at run time (unaligned or
// short tables).
//
// G64 (bf16 tables, groups of 64): a K-tile is one group, so the entry of
// K-tile t' of a window is its t'-th, the same for every thread: no selects.
template <int MODE, int BITS, int MT, int NT, int WMW, int NWAVES, bool RAG, int TF, bool G64>
__global__ __launch_bounds__(64 * NWAVES) void gemm2_kernel(Gemm2Args a) {
  static_assert(!G64 || (TF == 1 && MODE == 0), "the one-group-a-K-tile form reads bf16 windows");
  constexpr int WNW = NWAVES / WMW;
  static_assert(WNW * NT * 32 == BN, "the wavefronts must span the weight tile");
  constexpr int WM = MT * 32;                      // rows per wavefront
  constexpr int BM = WMW * WM;                     // rows per workgroup
  constexpr int WBITS = (MODE == 1) ? 4 : BITS;
  constexpr int TPR = NWAVES / 2;                  // threads per weight row: 2 | 4
  constexpr int CPT = BK / TPR;                    // codes per thread per K-tile: 32 | 16
  constexpr int PPT = CPT / 8;                     // 16-byte bf16 pieces per thread: 4 | 2
  constexpr int WPT = CPT * WBITS / 32;            // packed words per thread per K-tile
  constexpr int RB0 = RAG ? 1 : MT;                // row block of (wm, i) = wm*RB0 + i*RBI
  constexpr int RBI = RAG ? WMW : 1;
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WNW, wn = wave % WNW;
  const int li = lane & 31, kh = lane >> 5;

  // ---- which tile?  Workgroups are dealt round-robin over the 8 XCDs.
  // Dense: XCD x gets a contiguous run of tiles, column tile fastest, so the
  // workgroups sharing an L2 share activation row blocks.
  // Grouped: XCD x gets a band of column tiles of every expert, expert after
  // expert.  Experts differ in rows (a tile that is at most half full runs the
  // short main loop), and this way every XCD sees the same mix, while the
  // workgroups in flight on one XCD still share an expert's rows.
  const int n_tiles = (a.N + BN - 1) / BN;
  int tile_n, tile_m;
  int e = 0, row_lo = 0, row_hi = a.R, mt_idx = 0;
  if (a.row_offsets) {
    // the grid is provisioned for the worst raggedness: only the row tiles that exist are dealt
    deal_grouped_tile(n_tiles, blockIdx.x & 7, blockIdx.x >> 3, tile_m, tile_n);
    if (tile_n >= n_tiles) return;
    const RowTile rt = find_row_tile(a.row_offsets, a.E, a.R, BM, tile_m);
    if (!rt.found) return;
    e = rt.e; row_lo = rt.lo; row_hi = rt.hi; mt_idx = rt.idx;
  } else {
    const int total = n_tiles * a.m_tiles;
    const int per = (total + 7) / 8;
    const int tile = (blockIdx.x & 7) * per + (blockIdx.x >> 3);
    if (tile >= total) return;
    tile_n = tile % n_tiles;
    tile_m = tile / n_tiles;
    mt_idx = tile_m;
  }
  const int m0 = row_lo + mt_idx * BM;
  if (m0 >= row_hi) return;
  const int n0 = tile_n * BN;

  const int64_t wpr = (int64_t)a.K * WBITS / 32;
  const int gs = (MODE == 1) ? 32 : a.gs;
  const int64_t ng = a.K / gs;
  const int tabsz = (MODE == 1) ? 1 : (TF == 2 ? 4 : TF != 0 ? 2 : (a.tab == QMM_F32 ? 4 : 2));
  const uint32_t* wb = a.w + (int64_t)e * a.N * wpr;
  const char* sb = static_cast<const char*>(a.s) + (int64_t)e * a.N * ng * tabsz;
  const char* bb = (MODE == 1) ? nullptr : static_cast<const char*>(a.b) + (int64_t)e * a.N * ng * tabsz;

  // ---- activation fragments: lane (row li, k-half kh) of row tile i, k-step ks
  // reads ax[(kt*8 + ks*2 + kh) * Rp + m0 + (wm*RB0 + i*RBI)*32 + li]
  const auto ra = make_rsrc(a.ax, (int64_t)(a.K / 8) * a.Rp * 16);
  const uint32_t avo = (uint32_t)((kh * a.Rp + m0 + wm * (RB0 * 32) + li) * 16);
  // Ragged tiles by the rows they hold (uniform over the workgroup): at most
  // WMW row blocks -> every wavefront multiplies one block; one block more ->
  // that fifth block is split by columns, wavefront w taking its column block
  // w (five MFMAs a k-step for everyone instead of eight for wavefront 0 and a
  // barrier wait for the others); beyond that the full tile.
  const bool half_tile = RAG && MT == 2 && m0 + WMW * 32 >= row_hi;
  constexpr bool kFifth = RAG && MT == 2 && WNW == 1 && WMW * 32 == BN;   // one column block a wavefront
  const bool five_tile = kFifth && !half_tile && m0 + (WMW + 1) * 32 >= row_hi;
  const uint32_t avo1 = five_tile ? avo + (uint32_t)((WMW - wm) * 512) : avo + RBI * 512;   // second fragment's rows
  typedef u32x4 AFrag[4][MT];
  auto load_a_part = [&](int kt, AFrag& dst, int ks, auto ac) __attribute__((always_inline)) {   // the fragments of one k-step
    constexpr int ACT = decltype(ac)::value;
    const uint32_t so = (uint32_t)((kt * 8 + ks * 2) * 16) * (uint32_t)a.Rp;
#pragma unroll
    for (int i = 0; i < ACT; ++i)
      dst[ks][i] = __builtin_amdgcn_raw_buffer_load_b128(ra, i == 0 ? avo : avo1, so, 0);
  };
  auto load_a = [&](int kt, AFrag& dst, auto ac) __attribute__((always_inline)) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) load_a_part(kt, dst, ks, ac);
  };

  // ---- weight staging: thread -> (row tid/TPR, k-part tid%TPR): CPT codes a K-tile
  const int wrow = tid / TPR, whalf = tid % TPR;
  int64_t wn_row = n0 + wrow;
  if (wn_row >= a.N) wn_row = a.N - 1;             // rows past N are computed and never stored
  const auto rw = make_rsrc(wb, (int64_t)a.N * wpr * 4);
  const uint32_t wvo = (uint32_t)((wn_row * wpr + whalf * WPT) * 4);
  const int64_t trow = wn_row * ng;
  struct WRegs { uint32_t q[WPT]; };
  auto load_w = [&](int kt, WRegs& r) {
    const uint32_t so = (uint32_t)kt * (BK * WBITS / 8);
    if constexpr (WPT == 2) {
      const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rw, wvo, so, 0);
      r.q[0] = v[0]; r.q[1] = v[1];
    } else {
#pragma unroll
      for (int j = 0; j < WPT; j += 4) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rw, wvo + j * 4, so, 0);
        r.q[j] = v[0]; r.q[j + 1] = v[1]; r.q[j + 2] = v[2]; r.q[j + 3] = v[3];
      }
    }
  };

  // ---- scale / bias entries.  A window = the entries of four K-tiles of this
  // thread's row (32 bytes a table, fetched once per four K-tiles); the entry
  // of K-tile t' = kt & 3 is picked out of it with per-thread constants.
  struct TabWin { u32x4 s[2], b[2]; };
  const auto rs = make_rsrc(sb, (int64_t)a.N * ng * tabsz);
  const auto rb = make_rsrc(MODE == 1 ? sb : bb, (int64_t)a.N * ng * tabsz);
  const uint32_t tvo = (uint32_t)(trow * tabsz);
  const int gshift = gs == 32 ? 5 : (gs == 64 ? 6 : 7);
  auto load_win = [&](int quad, TabWin& tw) {
    const uint32_t so = (uint32_t)(((quad * 4 * BK) >> gshift) * tabsz);
    tw.s[0] = __builtin_amdgcn_raw_buffer_load_b128(rs, tvo, so, 0);
    if constexpr (TF == 2) tw.s[1] = __builtin_amdgcn_raw_buffer_load_b128(rs, tvo + 16, so, 0);
    if constexpr (MODE == 0) {
      tw.b[0] = __builtin_amdgcn_raw_buffer_load_b128(rb, tvo, so, 0);
      if constexpr (TF == 2) tw.b[1] = __builtin_amdgcn_raw_buffer_load_b128(rb, tvo + 16, so, 0);
    }
  };
  // entry index of K-tile t' inside its window, for this thread's k-half
  uint32_t eidx[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) eidx[t] = (uint32_t)((t * BK + whalf * CPT) >> gshift);
  auto pick = [&](const u32x4 (&w)[2], uint32_t e) -> float {
    // entry e (0..7) of a window of 1-, 2- or 4-byte entries (TF != 0 only)
    constexpr uint32_t TS = (MODE == 1) ? 1u : (TF == 2 ? 4u : 2u);
    const uint32_t byte = e * TS;
    const uint32_t d = byte >> 2;
    uint32_t v = w[0][0];
    v = d == 1 ? w[0][1] : v;
    v = d == 2 ? w[0][2] : v;
    v = d == 3 ? w[0][3] : v;
    if constexpr (TF == 2) {
      v = d == 4 ? w[1][0] : v;
      v = d == 5 ? w[1][1] : v;
      v = d == 6 ? w[1][2] : v;
      v = d == 7 ? w[1][3] : v;
      return __uint_as_float(v);
    }
    v >>= (byte & 3u) * 8u;
    if constexpr (MODE == 1) return e8m0_to_f32(v & 255u);
    if constexpr (TF == 3) return f16_bits_to_f32(v & 0xFFFFu);
    return __uint_as_float(v << 16);
  };
  // (scale, bias) of K-tile kt for this thread; tq = kt & 3 at compile time
  // (a clamped kt past the last tile only feeds a stage that nobody reads)
  auto entry = [&](int kt, auto tqc, const TabWin& tw, float& sc, float& bi) {
    constexpr int tq = decltype(tqc)::value;
    if constexpr (G64) {
      const uint32_t vs = tw.s[0][tq >> 1], vb = tw.b[0][tq >> 1];
      sc = __uint_as_float((tq & 1) ? (vs & 0xFFFF0000u) : (vs << 16));
      bi = __uint_as_float((tq & 1) ? (vb & 0xFFFF0000u) : (vb << 16));
    } else if constexpr (TF != 0) {
      sc = pick(tw.s, eidx[tq]);
      bi = MODE == 1 ? 0.f : pick(tw.b, eidx[tq]);
    } else {
      const int64_t ti = trow + ((kt * BK + whalf * CPT) >> gshift);
      if constexpr (MODE == 1) {
        sc = e8m0_to_f32(reinterpret_cast<const uint8_t*>(sb)[ti]);
        bi = 0.f;
      } else {
        sc = load_table_rt(sb, ti, a.tab);
        bi = load_table_rt(bb, ti, a.tab);
      }
    }
  };
  auto store_piece = [&](int stage, const WRegs& r, int pc, float sc, float bi) {
    *reinterpret_cast<u32x4*>(smem + stage * kStage + swz(wrow, whalf * PPT + pc)) =
        dequant_piece<MODE, BITS>(r.q, pc, sc, bi);
  };

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int KT = a.K / BK;
  AFrag af[4];                                    // K-tile t lives in af[t & 3]
  WRegs wr[4];                                    // words of K-tile t live in wr[t & 3]
  auto clampk = [&](int kt) { return kt < KT ? kt : KT - 1; };

  // prologue: tile 0 dequantized, tiles 0..1 of the activations and the words
  // of tiles 1..3 in flight
  TabWin tw_cur, tw_nxt;
  if constexpr (TF != 0) load_win(0, tw_cur);
  // Issue order matters: a wait counts the loads issued after the one it needs,
  // and the waits inside the loop must also hold on its first pass.  The words
  // that the loop dequantizes first (tiles 1, 2, 3) therefore go out before the
  // sixteen activation loads, as they do in steady state.
  load_w(0, wr[0]);
  load_w(clampk(1), wr[1]);
  load_w(clampk(2), wr[2]);
  load_w(clampk(3), wr[3]);
  if (half_tile) {
    load_a(0, af[0], std::integral_constant<int, 1>{});
    load_a(clampk(1), af[1], std::integral_constant<int, 1>{});
  } else {
    load_a(0, af[0], std::integral_constant<int, MT>{});
    load_a(clampk(1), af[1], std::integral_constant<int, MT>{});
  }
  {
    float sc, bi;
    entry(0, std::integral_constant<int, 0>{}, tw_cur, sc, bi);
#pragma unroll
    for (int pc = 0; pc < PPT; ++pc) store_piece(0, wr[0], pc, sc, bi);
  }
  lds_barrier();

  bf16x8 fb[2][NT];                               // B fragments: k-step ks in set ks & 1
  auto read_b = [&](const unsigned char* pbase, int ks, int set) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
      fb[set][j] = *reinterpret_cast<const bf16x8*>(pbase + swz(wn * (NT * 32) + j * 32 + li, ks * 2 + kh));
  };
  bf16x8 fbx[2];                                  // fifth-block tiles: column block wm of the weight tile
  auto read_bx = [&](const unsigned char* pbase, int ks, int set) {
    fbx[set] = *reinterpret_cast<const bf16x8*>(pbase + swz(wm * 32 + li, ks * 2 + kh));
  };
  read_b(smem, 0, 0);
  if constexpr (kFifth) read_bx(smem, 0, 0);

  // One K-tile.  A single wavefront per SIMD has to keep its matrix core busy
  // by itself, and both a vector-memory instruction (about 64 clocks to issue
  // 1 KB) and a run of vector ALU work stall the next MFMA if they sit in one
  // lump; so each k-step's eight MFMAs are interleaved, instruction by
  // instruction, with a quarter of everything else the tile needs: the loads
  // of tile kt+2, one piece of tile kt+1's dequantization, the fragment reads
  // of the next k-step.  (Dequantizing two tiles ahead and reading fragments
  // two k-steps ahead was measured too: no faster, more registers.)
  auto step = [&](int kt, auto tc, auto ac) __attribute__((always_inline)) {
    constexpr int t = decltype(tc)::value;         // kt & 3
    constexpr int ACV = decltype(ac)::value;       // row blocks this wavefront multiplies; 3 = one and a quarter
    constexpr bool FIVE = ACV == 3;
    constexpr int ACT = FIVE ? 1 : ACV;
    constexpr int NM = FIVE ? NT + 1 : ACT * NT;   // MFMAs a k-step
    const std::integral_constant<int, FIVE ? 2 : ACT> na;   // fragments loaded a k-step
    const unsigned char* pb = smem + t * kStage;
    constexpr int nstage = (t + 1) % kStages;
    const bool has_next = kt + 1 < KT;             // uniform
    const int kt2 = clampk(kt + 2), kt4 = clampk(kt + 4);
    float sc, bi;                                  // of tile kt+1 (the first tile of the next quad at t == 3)
    entry(clampk(kt + 1), std::integral_constant<int, (t + 1) & 3>{}, t == 3 ? tw_nxt : tw_cur, sc, bi);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      if (ks < 3) {
        read_b(pb, ks + 1, (ks + 1) & 1);
        if constexpr (FIVE) read_bx(pb, ks + 1, (ks + 1) & 1);
      }
      load_a_part(kt2, af[(t + 2) & 3], ks, na);
      if (ks == 0) load_w(kt4, wr[t & 3]);          // three K-tiles ahead of its dequantization
      if (TF != 0 && ks == 1 && t == 0) {          // next quad's table window (clamped at the end)
        const int q = (kt >> 2) + 1;
        load_win(q * 4 < KT ? q : (kt >> 2), tw_nxt);
      }
      // The fragment read last is used first: LDS reads return in order, so
      // one wait covers the k-step instead of one before every MFMA (a single
      // wavefront a SIMD issues one instruction per four clocks, waits included).
      if constexpr (FIVE)
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[t][ks][1]),
                                                             fbx[ks & 1], acc[1][0], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < ACT; ++i) {
        const bf16x8 fa = __builtin_bit_cast(bf16x8, af[t][ks][i]);
#pragma unroll
        for (int j = NT - 1; j >= 0; --j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa, fb[ks & 1][j], acc[i][j], 0, 0, 0);
      }
      // (after the last tile this writes a stage nobody reads: cheaper than a branch,
      // which would split the scheduling region)
      if (PPT == 4 || (ks & 1) == 0) store_piece(nstage, wr[(t + 1) & 3], PPT == 4 ? ks : ks / 2, sc, bi);
      // order inside the k-step: fragment reads first, then MFMA / ALU / load slots
      __builtin_amdgcn_sched_group_barrier(0x100, FIVE ? NT + 1 : NT, 0);      // ds reads
#pragma unroll
      for (int m = 0; m < NM; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, (32 + NM - 1) / NM, 0);   // a few vector ALU instructions
        if (m < 4) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // one vector-memory load
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (t == 3) tw_cur = tw_nxt;
    lds_barrier();
    if (has_next) {
      read_b(smem + nstage * kStage, 0, 0);
      if constexpr (FIVE) read_bx(smem + nstage * kStage, 0, 0);
    }
  };
  auto run = [&](auto ac) __attribute__((always_inline)) {
    int kt = 0;
    for (; kt + 4 <= KT; kt += 4) {
      step(kt, std::integral_constant<int, 0>{}, ac);
      step(kt + 1, std::integral_constant<int, 1>{}, ac);
      step(kt + 2, std::integral_constant<int, 2>{}, ac);
      step(kt + 3, std::integral_constant<int, 3>{}, ac);
    }
    if (kt < KT) { step(kt, std::integral_constant<int, 0>{}, ac); ++kt; }
    if (kt < KT) { step(kt, std::integral_constant<int, 1>{}, ac); ++kt; }
    if (kt < KT) { step(kt, std::integral_constant<int, 2>{}, ac); ++kt; }
  };
  if constexpr (RAG && MT == 2) {
    if (half_tile) run(std::integral_constant<int, 1>{});
    else if (kFifth && five_tile) run(std::integral_constant<int, kFifth ? 3 : MT>{});
    else run(std::integral_constant<int, MT>{});
  } else {
    run(std::integral_constant<int, MT>{});
  }

  // ---- epilogue.  D[i][j] of a 32x32 tile: lane holds column lane % 32 and
  // rows (r & 3) + 8 * (r >> 2) + 4 * (lane >> 5), r = 0..15.
  const bool wide = a.y_dtype != QMM_F32 && (a.N & 7) == 0 &&
                    (reinterpret_cast<uintptr_t>(a.y) & 15u) == 0;
  if (wide) {
    // 16-bit outputs: transpose each 32 x (NT*32) block through this wavefront's
    // share of LDS (free after the last barrier), store 16 bytes a lane
    constexpr int WC = NT * 32;                    // columns per wavefront
    uint16_t* o16 = reinterpret_cast<uint16_t*>(smem) + wave * (32 * WC);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      // a fifth-block tile's second block: rows of block WMW, the 32 columns of block wm
      const bool fifth = i == 1 && five_tile;
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int rl = (r & 3) + 8 * (r >> 2) + 4 * kh;
          const float v = acc[i][j][r];
          o16[rl * WC + j * 32 + li] =
              (uint16_t)(a.y_dtype == QMM_BF16 ? f32_to_bf16_bits(v) : f32_to_f16_bits(v));
        }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int q = 0; q < WC / 16; ++q) {          // 32 rows x WC/8 pieces over 64 lanes
        const int idx = q * 64 + lane, rl = idx / (WC / 8), pc = idx % (WC / 8);
        const int m = m0 + (fifth ? WMW : wm * RB0 + i * RBI) * 32 + rl;
        const int n = n0 + wn * WC + pc * 8 + (fifth ? wm * 32 : 0);
        if (fifth && pc >= 4) continue;            // only column block 0 of the staging area holds results
        if (m < row_hi && n < a.N) {
          const int64_t orow = a.out_idx ? (int64_t)a.out_idx[m] : (int64_t)m;
          *reinterpret_cast<u32x4*>(static_cast<uint16_t*>(a.y) + orow * a.N + n) =
              *reinterpret_cast<const u32x4*>(o16 + rl * WC + pc * 8);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  } else {
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const bool fifth = i == 1 && five_tile;
        if (fifth && j > 0) continue;
        const int n = n0 + wn * (NT * 32) + j * 32 + li + (fifth ? wm * 32 : 0);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + (fifth ? WMW : wm * RB0 + i * RBI) * 32 + (r & 3) + 8 * (r >> 2) + 4 * kh;
          if (m < row_hi && n < a.N) {
            const int64_t orow = a.out_idx ? (int64_t)a.out_idx[m] : (int64_t)m;
            store_out(a.y, orow * a.N + n, acc[i][j][r], a.y_dtype);
          }
        }
      }
  }
}

template <int MODE, int BITS, int MT, int NT, int WMW, int NWAVES, bool RAG, int TF, bool G64 = false>
void launch2_k(const Gemm2Args& a0, hipStream_t st) {
  constexpr int BM = WMW * MT * 32;
  Gemm2Args a = a0;
  a.m_tiles = (int)(a.row_offsets ? ceil_div(a.R, BM) + a.E : ceil_div(a.R, BM));
  // dense: tiles rounded up to the 8 XCDs; grouped: 8 bands of column tiles x provisioned row tiles
  const int64_t total = a.row_offsets ? ceil_div(ceil_div(a.N, BN), 8) * 8 * a.m_tiles
                                      : ceil_div(ceil_div(a.N, BN) * a.m_tiles, 8) * 8;
  dim3 grid((unsigned)total);
  // three weight stages; the epilogue transposes 32 x NT*32 sixteen-bit results per wavefront there
  const size_t epi = (size_t)NWAVES * 32 * NT * 32 * 2;
  const size_t lds = epi > (size_t)(kStages * kStage) ? epi : (size_t)(kStages * kStage);
  constexpr auto kern = gemm2_kernel<MODE, BITS, MT, NT, WMW, NWAVES, RAG, TF, G64>;
  if (!lds_limit<kern>(lds)) return;
  hipLaunchKernelGGL(kern, grid, dim3(64 * NWAVES), lds, st, a);
}

template <int MODE, int BITS, int MT, int NT, int WMW, int NWAVES, bool RAG>
void launch2_tf(const Gemm2Args& a, hipStream_t st) {
  if (!a.tabfast) return launch2_k<MODE, BITS, MT, NT, WMW, NWAVES, RAG, 0>(a, st);
  if constexpr (MODE == 1) {
    launch2_k<MODE, BITS, MT, NT, WMW, NWAVES, RAG, 1>(a, st);
  } else {
    if (a.tab == QMM_BF16 && a.gs == 64) launch2_k<MODE, BITS, MT, NT, WMW, NWAVES, RAG, 1, true>(a, st);
    else if (a.tab == QMM_BF16) launch2_k<MODE, BITS, MT, NT, WMW, NWAVES, RAG, 1>(a, st);
    else if (a.tab == QMM_F32) launch2_k<MODE, BITS, MT, NT, WMW, NWAVES, RAG, 2>(a, st);
    else launch2_k<MODE, BITS, MT, NT, WMW, NWAVES, RAG, 3>(a, st);
  }
}

template <int MODE, int BITS, int MT, int NT, int WMW, int NWAVES>
void launch2(const Gemm2Args& a, hipStream_t st) {
  if (a.row_offsets) launch2_tf<MODE, BITS, MT, NT, WMW, NWAVES, true>(a, st);
  else launch2_tf<MODE, BITS, MT, NT, WMW, NWAVES, false>(a, st);
}

template <int MODE, int BITS>
void launch2_mt(const Gemm2Args& a, int mt, hipStream_t st) {
  if (mt == 2) launch2<MODE, BITS, 2, 4, 4, 4>(a, st);     // 256 x 128, four wavefronts
  else launch2<MODE, BITS, 1, 2, 4, 8>(a, st);             // 128 x 128, eight wavefronts
}

int64_t prep_rows(int64_t R) { return ceil_div(R + 256, 64) * 64; }   // a tile may start at any row

}  // namespace

bool gemm2_supported(int64_t R, int64_t N, int64_t K) {
  if (experiment_env("QMM_GEMM_V1")) return false;
  return K > 0 && K % 64 == 0 && prep_rows(R) * K * 2 < (1ll << 32) && N * K < (1ll << 31);
}

size_t gemm2_workspace_bytes(int64_t R, int64_t K) { return (size_t)(prep_rows(R) * K * 2); }

// x bf16 [x_rows, K] (rows gathered through lhs_idx when given); the rest as gemm_dispatch.
void gemm2_dispatch(const void* x, const void* w, const void* s, const void* b, int tab, void* y,
                    int y_dtype, const int32_t* row_offsets, const int32_t* lhs_idx,
                    const int32_t* out_idx, int64_t R, int64_t x_rows, int64_t E, int64_t N,
                    int64_t K, int gs, int bits, int mode, int row_tile, void* workspace,
                    hipStream_t st) {
  if (R == 0 || N == 0) return;
  const int64_t rp = prep_rows(R);
  const int64_t prep_blocks = ceil_div(R, 8) * ceil_div(K / 8, 32);
  hipLaunchKernelGGL(gemm_prep_kernel, dim3((unsigned)prep_blocks), dim3(256), 0, st,
                     static_cast<const uint16_t*>(x), lhs_idx, static_cast<u32x4*>(workspace),
                     (int)R, (int)x_rows, (int)K, (int)rp);
  Gemm2Args a;
  a.ax = workspace;
  a.w = static_cast<const uint32_t*>(w);
  a.s = s;
  a.b = b;
  a.y = y;
  a.row_offsets = row_offsets;
  a.out_idx = out_idx;
  a.R = (int)R; a.N = (int)N; a.K = (int)K; a.E = (int)E; a.Rp = (int)rp;
  a.gs = gs; a.tab = tab; a.y_dtype = y_dtype;
  a.m_tiles = 0;
  {
    const int esz = mode == QMM_MODE_MXFP4 ? 1 : (tab == QMM_F32 ? 4 : 2);
    const int g = mode == QMM_MODE_MXFP4 ? 32 : gs;
    const bool aligned = ((K / g) * esz) % 4 == 0 && (reinterpret_cast<uintptr_t>(s) & 3u) == 0 &&
                         (mode == QMM_MODE_MXFP4 || (reinterpret_cast<uintptr_t>(b) & 3u) == 0);
    a.tabfast = aligned && K % 256 == 0 && N * (K / g) * esz < (1ll << 31) && !experiment_env("QMM_G2_NOTABFAST");
  }
  if (gemm2s_wanted(a, mode, bits)) return gemm2s_launch(a, mode, bits, st);
  const int mt = row_tile >= 256 ? 2 : 1;
  if (mode == QMM_MODE_MXFP4) launch2_mt<1, 4>(a, mt, st);
  else if (bits == 4) launch2_mt<0, 4>(a, mt, st);
  else launch2_mt<0, 8>(a, mt, st);
}

}  // namespace qmm
