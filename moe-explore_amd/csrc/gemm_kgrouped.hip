// K-grouped GEMM on gfx950 matrix cores: the expert weight gradients
//     out[e] = sum over expert e's sorted positions p of  a[arow(p), :]^T (x) b[brow(p), :]
// (dW1 = Xg^T dH with the token rows gathered, dW2 = (s*A)^T dOut with the dOut rows
// gathered).  The reference is forward-only; this is the transpose-side product
// that autograd takes of its per-expert matmuls (functional/topk_moe.py:88-92).
//
// A workgroup (8 wavefronts, 2 x 4 or 4 x 2) computes 256 x 256 tiles of out[e], walking the
// expert's row segment 64 positions at a time.  Both operands are stored with
// the contraction index as the row, so both LDS tiles are [64 positions][256
// features] and both fragment kinds are read with the LDS transpose load
// (ds_read_b64_tr_b16) into the operand layout of v_mfma_f32_16x16x32 (that shape draws
// less power per FLOP than 32x32x16, and the clock under this load is set by power).  Rows are copied global -> LDS directly
// (global_load_lds_dwordx4); positions past the end of the segment copy from a
// page of zeros, so the ragged tail contributes nothing.  Row indices of a
// gathered operand are fetched one step ahead.  The output tile leaves through
// LDS so that every global store instruction writes whole 128-byte row pieces.
// Experts without rows store zeros.  Workgroups are persistent (one per CU) and
// run the K steps of all their tiles as one pipeline.
//
// K-major operand (MOE_KGEMM_A_KMAJOR / MOE_KGEMM_B_KMAJOR): the small operand of a weight
// gradient is a set of gathered token rows that the caller has to materialise anyway.  Given
// feature-major instead ([features, columns], the contraction index contiguous; written by
// moe_row_gather_kmajor with every expert's segment starting on a multiple of 64 columns and
// zero-filled up to the next one), its LDS tile is [256 features][64 positions] and its
// fragments are plain 16-byte reads instead of two transpose loads each: with both operands
// read through transpose loads the LDS, not the matrix cores, sets the pace of a K step.
#include "gemm_mfma.h"

#include <mutex>
#include <set>
#include <utility>

namespace moe {
namespace {

using namespace mfma;

typedef __attribute__((address_space(3))) void lds_void;

constexpr int KBM = 256, KBN = 256;  // out tile: KBM features of a x KBN features of b
constexpr int TILE_BYTES = BK * 256 * 2;  // 32 KiB per operand per stage
constexpr int KSTAGE_BYTES = 2 * TILE_BYTES;

__device__ __attribute__((aligned(512))) char g_zero_page[512];

__device__ __forceinline__ void copy16_to_lds(const void* src, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_addr), "v"(src)
               : "memory");
}
__device__ __forceinline__ void wait_copies_and_barrier() {
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// As above, but the YOUNGEST vector memory operations of this wavefront (issued last;
// they complete in order) may stay in flight.
template <int YOUNGEST>
__device__ __forceinline__ void wait_copies_keep_youngest_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(YOUNGEST) : "memory");
}

struct KSched {
  int MT, NT, GM, GN, nblk_m, nblk_n;
  int tiles;      // MT * NT, the tiles of one expert
  int rows_last;  // tile rows of the last row of blocks (GM in the others)
  // The divisions of the tile lookup, which every tile pays three times (two copy cursors
  // and the multiply): a multiply and a shift each instead of the ~40 instructions of an
  // integer division by a run-time value.
  FastDiv by_tiles, by_band, by_blk_full, by_blk_last, by_rows_full, by_rows_last;
};

// Chunk lists for uneven experts.  A chunk is one tile for every workgroup of an XCD (consecutive
// tiles: they share operand panels through that XCD's L2), and a tile's K loop is as long as its
// expert has rows.  Dealt round-robin, the chunks of a large expert leave some XCDs with far
// more K steps than others, and a chunk that straddles a long and a short expert leaves the
// workgroups of an XCD out of step with each other for the rest of the launch.  When the
// experts differ by more than an eighth, every workgroup therefore builds the same tables in
// LDS before its pipeline starts (the LDS is idle then): the experts ranked by rows, longest
// first, the tiles numbered in that order (so a straddling chunk joins experts of similar
// length and the chunks come out heaviest first), and every chunk handed to the XCD with the
// least work so far among those with room in their list.  Returns this XCD's number of chunks,
// its list in a register (lane i: the i-th chunk) and the ranking in two more (lane i of
// experts[i / 64]: the expert of rank i), or returns -1 when the round-robin deal in expert
// order stays (even experts, or more experts / chunks than the tables hold).
constexpr int kBalMaxExperts = 128, kBalMaxRounds = 64, kBalMaxChunks = kNumXcd * kBalMaxRounds;
constexpr int kBalStoreSteps = 6;  // what a tile costs beside its K loop (store, first copies), in K steps

__device__ __forceinline__ int balance_chunks(char* smem, const int32_t* group_indices, int E,
                                              int P, FastDiv by_tiles, int wpx, int nch, int xcd,
                                              int& list, int (&experts)[2]) {
  if (E > kBalMaxExperts || nch > kBalMaxChunks || nch <= kNumXcd) return -1;
  int* const kt = reinterpret_cast<int*>(smem);          // [kBalMaxExperts] K steps of an expert
  int* const ranked = kt + kBalMaxExperts;               // [kBalMaxExperts] experts, longest first
  int* const cnt = ranked + kBalMaxExperts;              // [kNumXcd] chunks of an XCD, then:
  int* const ext = cnt + kNumXcd;                        // [2] longest and shortest expert
  int* const lists = ext + 2;                            // [kNumXcd][kBalMaxRounds]
  const int tid = threadIdx.x;
  if (tid == 0) {
    ext[0] = 0;
    ext[1] = 0x7fffffff;
  }
  __syncthreads();
  for (int e = tid; e < E; e += kThreads) {
    int lo = group_indices[e], hi = group_indices[e + 1];
    lo = lo < 0 ? 0 : lo;
    hi = hi > P ? P : hi;
    const int k = hi > lo ? (hi - lo + BK - 1) / BK : 0;
    kt[e] = k;
    atomicMax(&ext[0], k);
    atomicMin(&ext[1], k);
  }
  __syncthreads();
  const int longest = ext[0], shortest = ext[1];
  if ((longest - shortest) * 8 <= longest) return -1;  // (uniform: every thread leaves here)
  for (int e = tid; e < E; e += kThreads) {
    const int k = kt[e];
    int rank = 0;
    for (int o = 0; o < E; ++o) {
      const int ko = kt[o];
      rank += (ko > k || (ko == k && o < e)) ? 1 : 0;
    }
    ranked[rank] = e;
  }
  __syncthreads();
  if (tid == 0) {
    int load[kNumXcd], n[kNumXcd];
#pragma unroll
    for (int q = 0; q < kNumXcd; ++q) load[q] = n[q] = 0;
    for (int c = 0; c < nch; ++c) {
      // the first tile of a chunk is its longest (and chunk c is no lighter than chunk c + 1)
      const int k = kt[ranked[by_tiles.div(c * wpx)]];
      const int w = k > 0 ? k + kBalStoreSteps : 1;  // (tiles of empty experts are zero-filled)
      // the XCD with the least work among those whose list has room (nch <= 8 lists: one has)
      int best = -1, least = 0x7fffffff;
#pragma unroll
      for (int q = 0; q < kNumXcd; ++q)
        if (n[q] < kBalMaxRounds && load[q] < least) {
          least = load[q];
          best = q;
        }
      int at = 0;
#pragma unroll
      for (int q = 0; q < kNumXcd; ++q)
        if (q == best) {
          at = n[q];
          load[q] += w;
          n[q] += 1;
        }
      if (best >= 0) lists[best * kBalMaxRounds + at] = c;
    }
#pragma unroll
    for (int q = 0; q < kNumXcd; ++q) cnt[q] = n[q];
  }
  __syncthreads();
  const int mine = cnt[xcd];
  const int lane = tid & 63;
  static_assert(kBalMaxRounds == 64 && kBalMaxExperts == 128, "one lane a round, two an expert");
  list = lane < mine ? lists[xcd * kBalMaxRounds + lane] : 0;
  experts[0] = lane < E ? ranked[lane] : 0;
  experts[1] = 64 + lane < E ? ranked[64 + lane] : 0;
  return mine;
}

// GA / GB: the rows of a / b are gathered by token (at most one of the two).
// gridDim.x is a multiple of the XCD count: workgroup w belongs to XCD w % 8 and takes
// tile w / 8 of every chunk of that XCD (a chunk: gridDim.x / 8 consecutive tiles; the
// tile order has no padding).  Experts in index order and chunks round-robin over the XCDs,
// or both by balance_chunks when the experts are uneven.  The K steps of
// successive tiles form ONE pipeline: the rows of the first step of the next tile
// are copied during the last step of the current one, so the only work between two
// tiles is the store of the finished accumulators (through the LDS stage that was
// consumed last).  A segment of ~1000 rows is only 16 steps long: with a workgroup
// per tile, launch + first-copy latency + store would be paid every 16 steps.
// Tiles of experts without rows are zero-filled by the copy cursor when it passes
// them.
constexpr int SHORT_BASE = 0;                // two stages of the operand copied one step ahead
constexpr int LONG_BASE = 2 * TILE_BYTES;    // three stages of the operand copied two steps ahead
constexpr int KLDS_BYTES = 5 * TILE_BYTES;   // 160 KiB, the whole LDS of a CU

typedef const __attribute__((address_space(4))) int32_t* const_i32p;

// KM: 0 = both operands position-major; 1 = a is K-major; 2 = b is K-major (then no gather).
// WA: wavefronts along the a features, 2 (wave tiles of 128 a x 64 b features) or 4 (64 x 128).
// The K-major operand is the wide side of the wave tile: eight of a wavefront's twelve fragments
// per K half are then plain 16-byte reads and four are transpose-load pairs, for dW2 (b K-major)
// as for dW1 (a K-major).
template <typename T, bool GA, bool GB, int KM, int WA = 2>
__global__ __launch_bounds__(kThreads) void k_grouped_persistent_kernel(KGemmArgs g, KSched s,
                                                                        int ntiles) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  constexpr bool gathered = GA || GB;
  static_assert(KM == 0 || !gathered, "a K-major operand is gathered by the caller");
  // The gathered operand (token rows: small, cache resident) is the SHORT one: two
  // LDS stages, copied one K step ahead.  The other operand streams from HBM: three
  // stages, copied two steps ahead.  Without a gather, a is the short one; a K-major
  // operand always is.
  constexpr bool A_SHORT = KM == 1 ? true : (KM == 2 ? false : !GB);
  constexpr bool SKM = KM != 0;  // the short operand is K-major
  const int wpx = gridDim.x / kNumXcd;  // workgroups of an XCD = tiles of a chunk
  const int xcd = blockIdx.x % kNumXcd, within = blockIdx.x / kNumXcd;
  const int nch = (ntiles + wpx - 1) / wpx;
  int chunk_list = 0, ranked_experts[2] = {0, 0};
  int rounds = balance_chunks(smem, g.group_indices, g.E, static_cast<int>(g.P), s.by_tiles, wpx,
                              nch, xcd, chunk_list, ranked_experts);
  const bool listed = rounds >= 0;
  if (!listed) rounds = nch > xcd ? (nch - xcd + kNumXcd - 1) / kNumXcd : 0;
  __syncthreads();  // the lists are read; from here on the LDS belongs to the copy pipeline
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  static_assert(WA == 2 || WA == 4, "2 x 4 or 4 x 2 wavefronts");
  constexpr int WB = 8 / WA;
  constexpr int WTM = KBM / WA, WTN = KBN / WB;  // wave tile: a features x b features
  const int wm0 = (wave / WB) * WTM, wn0 = (wave % WB) * WTN;

  struct Tile {
    int e, mt, nt, lo, hi, KT;
    int qs;  // first column of the expert's segment in a K-major operand
  };
  // round of this workgroup -> tile; false for the positions that pad the last chunk.  The
  // tiles of an expert are numbered block by block (blocks of GM x GN tiles, smaller ones at
  // the right and lower edge), experts one after the other, without gaps, so that the tiles
  // of a chunk share operand panels and every workgroup gets the same number of tiles
  // whatever MT and NT are.
  auto decode = [&](int round, Tile& t) -> bool {
    int chunk = round * kNumXcd + xcd;
    if (listed) chunk = __builtin_amdgcn_readlane(chunk_list, round);
    const int pos = chunk * wpx + within;
    if (pos >= ntiles) return false;
    const int nth = s.by_tiles.div(pos);  // the expert's place in the tile order
    int r = pos - nth * s.tiles;
    t.e = nth;
    if (listed)
      t.e = __builtin_amdgcn_readlane(nth < 64 ? ranked_experts[0] : ranked_experts[1], nth & 63);
    const int band = s.GM * s.NT;  // tiles of a full row of blocks
    int bm = s.by_band.div(r);
    bm = bm < s.nblk_m ? bm : s.nblk_m - 1;
    r -= bm * band;
    const bool last_band = bm == s.nblk_m - 1;
    const int rows_in = last_band ? s.rows_last : s.GM;
    int bn = last_band ? s.by_blk_last.div(r) : s.by_blk_full.div(r);
    bn = bn < s.nblk_n ? bn : s.nblk_n - 1;
    r -= bn * rows_in * s.GN;
    const int col = last_band ? s.by_rows_last.div(r) : s.by_rows_full.div(r);
    t.mt = bm * s.GM + (r - col * rows_in);
    t.nt = bn * s.GN + col;
    // scalar loads (the expert is wave-uniform): a vector load would have to be awaited
    // with vmcnt(0), and with it every copy in flight
    const const_i32p gi = (const_i32p)(uintptr_t)g.group_indices;
    int lo = gi[t.e], hi = gi[t.e + 1];
    lo = lo < 0 ? 0 : lo;
    hi = hi > g.P ? static_cast<int>(g.P) : hi;
    t.lo = lo;
    t.hi = hi;
    t.KT = t.hi > t.lo ? (t.hi - t.lo + BK - 1) / BK : 0;
    t.qs = 64 * ((lo >> 6) + t.e);
    return true;
  };
  auto store_zero_tile = [&](const Tile& t) {
    T* out = static_cast<T*>(g.out) + static_cast<int64_t>(t.e) * g.Ka * g.Nb;
    const int64_t col = static_cast<int64_t>(t.nt) * KBN + (tid & 31) * 8;
    for (int r = tid >> 5; r < KBM; r += kThreads / 32) {
      const int64_t row = static_cast<int64_t>(t.mt) * KBM + r;
      if (row < g.Ka && col < g.Nb)
        *reinterpret_cast<uint4*>(out + row * g.Nb + col) = make_uint4(0, 0, 0, 0);
    }
  };

  // ---- copy geometry: instruction i of wavefront w fills positions 2*(8i+w), +1 ----------
  // (instruction i is 16 positions after instruction 0, and the column swizzle, which
  // depends on k & 3 and k & 8 only, is the same for all four: one position, one byte
  // offset and one source pointer per operand describe them all)
  const int p_first = 2 * wave + (lane >> 5);
  const int lbyte = ((lane & 31) * 16) ^ nmajor16_swizzle(p_first);
  auto p_local = [&](int i) __attribute__((always_inline)) { return p_first + 16 * i; };
  const int zero_off = (lane & 31) * 16;
  const unsigned lds0 =
      __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<size_t>((lds_void*)smem))) +
      wave * 1024;
  // K-major short operand: tile [256 features][64 positions], 128-byte rows; instruction i of
  // wavefront w fills feature rows 64*i + 8*w .. +7 (lane -> row lane / 8, 16-byte chunk
  // (lane & 7) ^ swizzle of the row, which is the same for all four instructions)
  const int km_row = 8 * wave + (lane >> 3);
  const int km_chunk = (lane & 7) ^ ((km_row >> 1) & 7);
  int km_f0 = 0, km_last = 0;  // first feature row of the short cursor's tile, last row of the matrix
  const int64_t lda2 = g.lda * 2, ldb2 = g.ldb * 2;
  const int64_t ld_s2 = A_SHORT ? lda2 : ldb2, ld_l2 = A_SHORT ? ldb2 : lda2;
  const int s_last = static_cast<int>((A_SHORT ? g.a_rows : g.b_rows) - 1);

  // A copy cursor: the next K step (tile, kt) of one operand that will be copied, and
  // this lane's source of row `lo + p_local[i]` (plain) or of row 0 (gathered) of
  // that tile's feature columns.
  struct Cursor {
    Tile t;
    int id, kt;  // id: the round (chunk of this XCD) the tile belongs to
    bool valid;
  };
  Cursor cs, cl;
  const char* s_plain;  // source of copy instruction 0; instruction i is 16 rows further
  const char* l_plain;
  auto set_bases = [&](const Tile& t, bool is_a, const char*& plain) {
    const int64_t f0 = static_cast<int64_t>(is_a ? t.mt : t.nt) * (is_a ? KBM : KBN);
    const int64_t width = is_a ? g.Ka : g.Nb;
    if (SKM && is_a == A_SHORT) {
      km_f0 = static_cast<int>(f0);
      km_last = static_cast<int>(width - 1);
      plain = static_cast<const char*>(is_a ? g.a : g.b) + (static_cast<int64_t>(t.qs) + km_chunk * 8) * 2;
      return;
    }
    const bool gath = is_a ? GA : GB;
    const int64_t ld2 = is_a ? lda2 : ldb2;
    const char* base = static_cast<const char*>(is_a ? g.a : g.b);
    // feature columns past the matrix only feed outputs that are not stored
    const int64_t col = (f0 + lbyte / 2 < width) ? f0 * 2 + lbyte : 0;
    const int64_t p = t.lo + p_first;
    plain = base + (gath ? 0 : p * ld2) + col;
  };
  // moves a cursor to the next tile that has rows; the short cursor zero-fills the
  // tiles of experts without rows on its way
  auto next_tile = [&](Cursor& c, bool is_short) {
    c.valid = false;
    for (;;) {
      c.id += 1;
      if (c.id >= rounds) return;
      if (!decode(c.id, c.t)) continue;
      if (c.t.KT == 0) {
        if (is_short) store_zero_tile(c.t);
        continue;
      }
      break;
    }
    c.valid = true;
    c.kt = 0;
    if (is_short) set_bases(c.t, A_SHORT, s_plain);
    else set_bases(c.t, !A_SHORT, l_plain);
  };
  auto advance = [&](Cursor& c, bool is_short) {
    if (c.kt + 1 < c.t.KT) ++c.kt;
    else next_tile(c, is_short);
  };

  // Slot ids of the gathered rows under the short cursor, one per copy instruction of
  // this lane: loaded right after the short copies of a step, used at the top of the
  // next one.  (The compiler waits for them with vmcnt(0) there, and so also for the
  // long copies issued in between; loads hidden in inline assembly would avoid that
  // but would rest on the register allocator never moving their destination before
  // they land.  The layer gathers the rows beforehand where that is faster.)
  int32_t slot[4] = {0, 0, 0, 0};
  auto fetch_slots = [&]() {
    if (!gathered || !cs.valid) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      int p = cs.t.lo + cs.kt * BK + p_local(i);
      p = p < cs.t.hi ? p : cs.t.hi - 1;
      slot[i] = load_index32(g.indices, g.idx_bytes, p);
    }
  };

  auto issue_short = [&](int stage) {
    const unsigned base = lds0 + SHORT_BASE + stage * TILE_BYTES;
    const bool tail = cs.kt + 1 == cs.t.KT;
    if constexpr (SKM) {
      // (the columns past the end of the segment hold zeros: nothing to mask)
      // (feature rows past the matrix only feed outputs that are not stored)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int f = km_f0 + km_row + 64 * i;
        f = f < km_last ? f : km_last;
        copy16_to_lds(s_plain + f * ld_s2 + cs.kt * (BK * 2), base + i * 8192);
      }
      advance(cs, true);
      return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const char* src;
      if constexpr (gathered) {
        int t = g.by_topk.div(slot[i]);
        t = t > s_last ? s_last : t;
        src = s_plain + t * ld_s2;
      } else {
        src = s_plain + static_cast<int64_t>(cs.kt * BK + 16 * i) * ld_s2;
      }
      if (tail && cs.t.lo + cs.kt * BK + p_local(i) >= cs.t.hi) src = g_zero_page + zero_off;
      copy16_to_lds(src, base + i * 8192);
    }
    advance(cs, true);
    fetch_slots();
  };
  auto issue_long = [&](int stage) {
    const unsigned base = lds0 + LONG_BASE + stage * TILE_BYTES;
    const bool tail = cl.kt + 1 == cl.t.KT;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const char* src = l_plain + static_cast<int64_t>(cl.kt * BK + 16 * i) * ld_l2;
      if (tail && cl.t.lo + cl.kt * BK + p_local(i) >= cl.t.hi) src = g_zero_page + zero_off;
      copy16_to_lds(src, base + i * 8192);
    }
    advance(cl, false);
  };

  // ---- fragment reads ----------------------------------------------------------------------
  // 16 x 16 x 32 MFMAs: the wavefront's 128 x 64 (64 x 128) tile is 8 x 4 (4 x 8) blocks of
  // 16 x 16.  A K step is four units of 16 MFMAs: unit u = K half (u >> 1), half of the a
  // blocks (u & 1); the b fragments of a K half serve both of its units.  A fragment of a
  // position-major tile is two transpose loads: the 16-lane group lg fetches k rows 8*lg + i
  // and + 4 of a 16-column block.
  constexpr int MB16 = WTM / 16, NB16 = WTN / 16, HB = MB16 / 2, NH = NB16 / 2;
  const int l16 = lane & 15, lg = lane >> 4;
  const int tr_i = (lane >> 2) & 3, tr_q = lane & 3;
  const int tr_c = 4 * tr_q;
  const int tr_k = 8 * lg + tr_i;
  auto read_tr = [&](const char* tile, int kh, int col0) __attribute__((always_inline)) -> s16x8 {
    const int k = kh * 32 + tr_k;
    const int cbyte = (col0 + tr_c) * 2;
    s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + nmajor16_off(k, cbyte)));
    s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + nmajor16_off(k + 4, cbyte)));
    return __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto read_km = [&](const char* tile, int kh, int row0) __attribute__((always_inline)) -> s16x8 {
    return *reinterpret_cast<const s16x8*>(tile + kmajor_off(row0 + l16, kh * 4 + lg));
  };
  auto read_unit_a = [&](int sstage, int lstage, int u, s16x8 (&af)[HB]) __attribute__((always_inline)) {
    const char* at = A_SHORT ? smem + SHORT_BASE + sstage * TILE_BYTES : smem + LONG_BASE + lstage * TILE_BYTES;
#pragma unroll
    for (int mb = 0; mb < HB; ++mb) {
      if constexpr (KM == 1) af[mb] = read_km(at, u >> 1, wm0 + ((u & 1) * HB + mb) * 16);
      else af[mb] = read_tr(at, u >> 1, wm0 + ((u & 1) * HB + mb) * 16);
    }
  };
  // b blocks [NH*half, NH*half + NH) of K half kh
  auto read_unit_b = [&](int sstage, int lstage, int kh, int half, s16x8 (&bf)[NB16]) __attribute__((always_inline)) {
    const char* bt = A_SHORT ? smem + LONG_BASE + lstage * TILE_BYTES : smem + SHORT_BASE + sstage * TILE_BYTES;
#pragma unroll
    for (int nb = NH * half; nb < NH * half + NH; ++nb) {
      if constexpr (KM == 2) bf[nb] = read_km(bt, kh, wn0 + nb * 16);
      else bf[nb] = read_tr(bt, kh, wn0 + nb * 16);
    }
  };
  f32x4 acc[MB16][NB16];
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int mb = 0; mb < MB16; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB16; ++nb) acc[mb][nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  };
  // b features as the first MFMA operand, a features as the second: a lane then owns one
  // out row (an a feature) and four consecutive out columns (b features) per block.  The first
  // half of the column blocks comes first: the fragments of the second half are read at the
  // start of the unit that first needs them, so that every unit reads the same 6 KiB.
  auto multiply_unit = [&](int rh, s16x8 (&af)[HB], s16x8 (&bf)[NB16]) __attribute__((always_inline)) {
#pragma unroll
    for (int nb = 0; nb < NB16; ++nb)
#pragma unroll
      for (int mb = 0; mb < HB; ++mb) {
        if (rh == 0) acc[mb][nb] = mfma16<T>(bf[nb], af[mb], acc[mb][nb]);
        else acc[HB + mb][nb] = mfma16<T>(bf[nb], af[mb], acc[HB + mb][nb]);
      }
  };
  auto interleave_unit = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < HB * NB16; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // accumulators -> out tile of `t`, PR rows of every wave tile at a time through `epi`
  // (rows of WTN columns + pad: conflict-free writes)
  constexpr int EPI_ROW_BYTES = WTN * 2 + 8;
  constexpr int PR = WTN == 64 ? 32 : 16;
  constexpr int EPI_WAVE_BYTES = PR * EPI_ROW_BYTES;
  constexpr int ROW_LANES = WTN / 8;  // lanes that store one row piece, 16 bytes each
  auto store_acc = [&](const Tile& t, char* epi) __attribute__((always_inline)) {
    T* out = static_cast<T*>(g.out) + static_cast<int64_t>(t.e) * g.Ka * g.Nb;
    const int64_t m0 = static_cast<int64_t>(t.mt) * KBM, n0 = static_cast<int64_t>(t.nt) * KBN;
    const int64_t col = n0 + wn0 + (lane % ROW_LANES) * 8;
#pragma unroll
    for (int pass = 0; pass < WTM / PR; ++pass) {
#pragma unroll
      for (int mbh = 0; mbh < PR / 16; ++mbh)
#pragma unroll
        for (int nb = 0; nb < NB16; ++nb) {
          T v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = from_f32<T>(acc[pass * (PR / 16) + mbh][nb][j]);
          *reinterpret_cast<uint2*>(epi + (mbh * 16 + l16) * EPI_ROW_BYTES + (nb * 16 + lg * 4) * 2) =
              *reinterpret_cast<const uint2*>(v);
        }
#pragma unroll
      for (int it = 0; it < PR * ROW_LANES / 64; ++it) {
        const int r = it * (64 / ROW_LANES) + lane / ROW_LANES;
        const char* src = epi + r * EPI_ROW_BYTES + (lane % ROW_LANES) * 16;
        uint2 v0 = *reinterpret_cast<const uint2*>(src);
        uint2 v1 = *reinterpret_cast<const uint2*>(src + 8);
        const int64_t row = m0 + wm0 + pass * PR + r;
        if (row < g.Ka && col < g.Nb)
          *reinterpret_cast<uint4*>(out + row * g.Nb + col) = make_uint4(v0.x, v0.y, v1.x, v1.y);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- the pipeline --------------------------------------------------------------------------
  // K step number gs (counted over all tiles of this workgroup) lives in short stage
  // gs % 2 and long stage gs % 3.
  cs.id = cl.id = -1;
  next_tile(cs, true);
  if (!cs.valid) return;
  next_tile(cl, false);
  fetch_slots();
  issue_short(0);
  issue_long(0);
  if (cl.valid) {
    issue_long(1);
    wait_copies_keep_youngest_and_barrier<4>();
  } else {
    wait_copies_and_barrier();
  }
  s16x8 afA[HB], afB[HB], bfP[NB16], bfQ[NB16];
  read_unit_a(0, 0, 0, afA);
  read_unit_b(0, 0, 0, 0, bfP);
  Tile tc;
  int id_c = -1;
  int sstage = 0, lstage = 0;
  for (;;) {
    // next tile with rows (the order the cursors took)
    bool found = false;
    for (;;) {
      id_c += 1;
      if (id_c >= rounds) break;
      if (decode(id_c, tc) && tc.KT > 0) {
        found = true;
        break;
      }
    }
    if (!found) break;
    zero_acc();
    bool more = true;
    for (int kt = 0; kt < tc.KT; ++kt) {
      const int lnext = lstage == 2 ? 0 : lstage + 1;
      const int lahead = lnext == 2 ? 0 : lnext + 1;
      more = cs.valid;                // a step gs+1 exists (of this tile or of the next one)
      const bool ahead = cl.valid;    // a step gs+2 exists
      if (more) issue_short(sstage ^ 1);
      __builtin_amdgcn_s_setprio(2);
      __builtin_amdgcn_sched_barrier(0);
      read_unit_b(sstage, lstage, 0, 1, bfP);
      read_unit_a(sstage, lstage, 1, afB);
      multiply_unit(0, afA, bfP);
      interleave_unit();
      read_unit_b(sstage, lstage, 1, 0, bfQ);
      read_unit_a(sstage, lstage, 2, afA);
      multiply_unit(1, afB, bfP);
      interleave_unit();
      if (ahead) issue_long(lahead);
      __builtin_amdgcn_sched_barrier(0);
      read_unit_b(sstage, lstage, 1, 1, bfQ);
      read_unit_a(sstage, lstage, 3, afB);
      multiply_unit(0, afA, bfQ);
      interleave_unit();
      __builtin_amdgcn_s_setprio(0);
      if (more) {
        // step gs+1 must have landed; the long copies of step gs+2, the youngest four
        // copy instructions of this wavefront, may still fly
        if (ahead) wait_copies_keep_youngest_and_barrier<4>();
        else wait_copies_and_barrier();
        read_unit_a(sstage ^ 1, lnext, 0, afA);
        read_unit_b(sstage ^ 1, lnext, 0, 0, bfP);
      }
      multiply_unit(1, afB, bfQ);
      interleave_unit();
      sstage ^= 1;
      lstage = lnext;
    }
    // The two stages of the last step are free now (every wavefront passed the barrier
    // above, or there is no later step and nothing else in flight): wavefronts 0-3 stage
    // their rows in the short one, 4-7 in the long one.
    if (!more) __syncthreads();
    const int lprev = lstage == 0 ? 2 : lstage - 1;
    char* epi = wave < 4 ? smem + SHORT_BASE + (sstage ^ 1) * TILE_BYTES + wave * EPI_WAVE_BYTES
                         : smem + LONG_BASE + lprev * TILE_BYTES + (wave - 4) * EPI_WAVE_BYTES;
    store_acc(tc, epi);
    if (more) __syncthreads();  // later steps copy into the stages just used for the store
  }
}


// Gathers token rows into the K-major operand layout of the weight-gradient kernel:
//     dst[f, qs(e) + (p - lo(e))] = src[idx[p] / div, f]      p in [lo(e), hi(e))
// with qs(e) = 64 * (lo(e) / 64 + e), and zeros from the end of the expert's segment up to the
// next multiple of 64 columns.  A workgroup moves 64 positions x 256 features through LDS, 64 x 64
// at a time: 128-byte row pieces in (gathered rows of src), 128-byte row pieces out (feature rows
// of dst).  The expert lookup and the row ids are paid once for the four feature blocks and
// all their loads are in flight together: with one 64 x 64 block a workgroup the launch was
// bound by that latency chain, not by memory.
constexpr int kGatherFB = 4;  // 64-feature blocks a workgroup
template <typename T>
__global__ __launch_bounds__(256) void row_gather_kmajor_kernel(
    const T* __restrict__ src, int64_t src_rows, int64_t src_stride, const void* __restrict__ idx,
    int idx_bytes, FastDiv by_div, const int32_t* __restrict__ gi, int E, int P,
    T* __restrict__ dst, int64_t ld_dst, int64_t features) {
  __shared__ int sh[3];
  // (rows of 64 + 12 elements and eight-position groups in the transposing reads below: the four
  // groups of a wavefront then read different banks; with 64 + 8 and sixteen-position groups
  // every 2-byte read was a four-way bank conflict and the launch was bound by them)
  __shared__ __attribute__((aligned(16))) T tile[kGatherFB][64][64 + 12];
  if (threadIdx.x < 64) find_tile<64>(gi, E, P, static_cast<int>(blockIdx.x), sh);
  __syncthreads();
  const int e = sh[0];
  if (e < 0) return;
  const int row0 = sh[1], end = sh[2];
  int lo = gi[e];
  lo = lo < 0 ? 0 : lo;
  const int64_t col0 = 64 * static_cast<int64_t>((lo >> 6) + e) + (row0 - lo);
  const int64_t f0 = static_cast<int64_t>(blockIdx.y) * (64 * kGatherFB);
  const int t = threadIdx.x;
  {  // in: position t / 4, features 16 * (t % 4) .. +15 of every block
    const int pos = t >> 2;
    const int p = row0 + pos;
    int64_t srow = 0;
    if (p < end) srow = clamp_index(by_div.div(load_index32(idx, idx_bytes, p)), src_rows);
    uint4 v[kGatherFB][2];
#pragma unroll
    for (int fb = 0; fb < kGatherFB; ++fb)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int64_t c = f0 + fb * 64 + (t & 3) * 16 + h * 8;
        v[fb][h] = make_uint4(0, 0, 0, 0);
        if (p < end && c < features) v[fb][h] = *reinterpret_cast<const uint4*>(src + srow * src_stride + c);
      }
#pragma unroll
    for (int fb = 0; fb < kGatherFB; ++fb)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint2* dst2 = reinterpret_cast<uint2*>(&tile[fb][pos][(t & 3) * 16 + h * 8]);  // 8-byte aligned rows
        dst2[0] = make_uint2(v[fb][h].x, v[fb][h].y);
        dst2[1] = make_uint2(v[fb][h].z, v[fb][h].w);
      }
  }
  __syncthreads();
  {  // out: feature t / 4 of every block, positions 8 * (t % 4) .. +7 and 32 + those
    const int f = t >> 2;
#pragma unroll
    for (int fb = 0; fb < kGatherFB; ++fb) {
      const int64_t row = f0 + fb * 64 + f;
      if (row >= features) continue;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int q = (t & 3) * 8 + h * 32;
        T v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = tile[fb][q + j][f];
        *reinterpret_cast<uint4*>(dst + row * ld_dst + col0 + q) = *reinterpret_cast<const uint4*>(v);
      }
    }
  }
}

}  // namespace

bool k_grouped_mfma_supported(const KGemmArgs& g) {
  if (g.dtype != MOE_DTYPE_BF16 && g.dtype != MOE_DTYPE_F16) return false;
  if (g.Ka % 8 != 0 || g.Nb % 8 != 0) return false;
  if (g.lda % 8 != 0 || g.ldb % 8 != 0) return false;
  if ((g.flags & (MOE_KGEMM_A_KMAJOR | MOE_KGEMM_B_KMAJOR)) && (g.flags & (MOE_KGEMM_GATHER_A | MOE_KGEMM_GATHER_B)))
    return false;
  if (!aligned16(g.a) || !aligned16(g.b) || !aligned16(g.out)) return false;
  if (g.P == 0) return false;  // nothing to contract: the scalar kernel writes the zeros
  return true;
}

int launch_k_grouped_mfma(const KGemmArgs& g, hipStream_t stream) {
  KSched s;
  s.MT = static_cast<int>((g.Ka + KBM - 1) / KBM);
  s.NT = static_cast<int>((g.Nb + KBN - 1) / KBN);
  s.GM = s.MT < 4 ? s.MT : 4;
  s.GN = s.NT < 8 ? s.NT : 8;
  s.nblk_m = (s.MT + s.GM - 1) / s.GM;
  s.nblk_n = (s.NT + s.GN - 1) / s.GN;
  s.tiles = s.MT * s.NT;
  s.rows_last = s.MT - (s.nblk_m - 1) * s.GM;
  s.by_tiles = FastDiv(static_cast<uint32_t>(s.tiles));
  s.by_band = FastDiv(static_cast<uint32_t>(s.GM * s.NT));
  s.by_blk_full = FastDiv(static_cast<uint32_t>(s.GM * s.GN));
  s.by_blk_last = FastDiv(static_cast<uint32_t>(s.rows_last * s.GN));
  s.by_rows_full = FastDiv(static_cast<uint32_t>(s.GM));
  s.by_rows_last = FastDiv(static_cast<uint32_t>(s.rows_last));
  const int64_t ntiles = static_cast<int64_t>(g.E) * s.tiles;
  if (ntiles > 0x3fffffff) return fail(MOE_ERR_UNSUPPORTED, "grid too large");
  int cus = num_cus();
  if (cus <= 0) return MOE_ERR_HIP;
  cus = cus / kNumXcd * kNumXcd;
  if (cus < kNumXcd) cus = kNumXcd;
  const int64_t wanted = (ntiles + kNumXcd - 1) / kNumXcd * kNumXcd;
  const dim3 grid(static_cast<unsigned>(wanted < cus ? wanted : cus));
  const int total = static_cast<int>(ntiles);
  constexpr size_t lds = KLDS_BYTES;
  auto launch = [&](auto kernel) -> int {
    const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds);
    if (rc != MOE_OK) return rc;
    kernel<<<grid, kThreads, lds, stream>>>(g, s, total);
    return MOE_OK;
  };
  const bool ga = g.flags & MOE_KGEMM_GATHER_A, gb = g.flags & MOE_KGEMM_GATHER_B;
  const int km = (g.flags & MOE_KGEMM_A_KMAJOR) ? 1 : ((g.flags & MOE_KGEMM_B_KMAJOR) ? 2 : 0);
  int rc;
  if (g.dtype == MOE_DTYPE_BF16) {
    if (km == 1) rc = launch(k_grouped_persistent_kernel<bf16_t, false, false, 1>);
    else if (km == 2) rc = launch(k_grouped_persistent_kernel<bf16_t, false, false, 2, 4>);
    else rc = ga ? launch(k_grouped_persistent_kernel<bf16_t, true, false, 0>)
                 : (gb ? launch(k_grouped_persistent_kernel<bf16_t, false, true, 0>)
                       : launch(k_grouped_persistent_kernel<bf16_t, false, false, 0>));
  } else {
    if (km == 1) rc = launch(k_grouped_persistent_kernel<f16_t, false, false, 1>);
    else if (km == 2) rc = launch(k_grouped_persistent_kernel<f16_t, false, false, 2, 4>);
    else rc = ga ? launch(k_grouped_persistent_kernel<f16_t, true, false, 0>)
                 : (gb ? launch(k_grouped_persistent_kernel<f16_t, false, true, 0>)
                       : launch(k_grouped_persistent_kernel<f16_t, false, false, 0>));
  }
  if (rc != MOE_OK) return rc;
  return check_launch("k_grouped_gemm (MFMA kernel)");
}

int launch_row_gather_kmajor(const void* src, int64_t src_rows, int64_t src_stride, const void* idx,
                             int idx_bytes, int idx_div, const int32_t* group_indices, int E,
                             int64_t P, void* dst, int64_t ld_dst, int64_t features, int dtype,
                             hipStream_t stream) {
  const int64_t blocks = P / 64 + E;  // static bound on the 64-position blocks of all experts
  const int64_t fgroups = (features + 64 * kGatherFB - 1) / (64 * kGatherFB);
  if (blocks > 0x7fffffff || fgroups > 65535) return fail(MOE_ERR_UNSUPPORTED, "grid too large");
  const dim3 grid(static_cast<unsigned>(blocks), static_cast<unsigned>(fgroups));
  const FastDiv by_div(static_cast<uint32_t>(idx_div));
  if (dtype == MOE_DTYPE_BF16)
    row_gather_kmajor_kernel<bf16_t><<<grid, 256, 0, stream>>>(
        static_cast<const bf16_t*>(src), src_rows, src_stride, idx, idx_bytes, by_div, group_indices, E,
        static_cast<int>(P), static_cast<bf16_t*>(dst), ld_dst, features);
  else
    row_gather_kmajor_kernel<f16_t><<<grid, 256, 0, stream>>>(
        static_cast<const f16_t*>(src), src_rows, src_stride, idx, idx_bytes, by_div, group_indices, E,
        static_cast<int>(P), static_cast<f16_t*>(dst), ld_dst, features);
  return check_launch("row_gather_kmajor");
}

}  // namespace moe
