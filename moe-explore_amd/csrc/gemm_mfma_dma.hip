// M-grouped GEMM, main kernel: as gemm_mfma.hip (same tiles, layouts, epilogue,
// device-side tile map) but global memory is copied straight into LDS
// (global_load_lds_dwordx4), so no VGPRs or ds_write issue slots are spent on
// staging, and the LDS -> register fragment reads run one K sub-step (16) ahead of
// the MFMAs that consume them.  Takes K that is a multiple of 64 and outputs that
// can be stored 16 bytes at a time (they leave through LDS); the rest goes to the
// register-staged kernel.
//
// One workgroup per compute unit stays resident and draws work items from a queue (see
// g_tile_queues).  A work item is s.tpw adjacent column tiles of one row block, computed one
// after the other as ONE stream of K steps: the token addresses stay, the weight addresses move
// on, and the copies of the first steps of the next tile are in flight while the
// accumulators of the finished tile are stored (through the two LDS stages consumed
// last).  Tile lookup, index fetch and first-copy latency are paid once a work item.
//
// One K step (64) of a workgroup is four parts of equal MFMA time (256 cycles): K
// sub-steps of 16 on 32 x 32 x 16 MFMAs (128-row tiles), or units of 16 MFMAs of
// 16 x 16 x 32 (256-row tiles: K half x token-row half; see the kernel's comment):
//     issue the token copies of the next step and the weight copies of the step after
//     it, a few instructions at a time between the parts
//     parts 0..2: read fragments of part i+1, multiply part i
//     wait for own copies and own LDS reads; workgroup barrier
//     read fragments of part 0 of the next step; multiply part 3
// The barrier thus sits in front of the last quarter of a step's MFMAs, which cover
// the LDS latency of the first reads of the next one.
//
// The copy instruction writes lane i's 16 bytes at (M0 base) + 16*i: the LDS
// image of one instruction is 1 KiB contiguous, so the XOR swizzles of the tile
// layouts are applied to the global source address of each lane instead.
#include "gemm_mfma.h"

#include <mutex>
#include <unordered_map>

namespace moe {
namespace {

using namespace mfma;

typedef __attribute__((address_space(3))) void lds_void;

// 16 bytes per lane, global -> LDS.  `lds_addr` must be wave-uniform.  The
// compiler is not told that this is a memory-to-LDS copy: it would otherwise make
// every later LDS read wait for all copies in flight.  Completion is awaited by
// wait_copies_and_barrier().
// The source is a wave-uniform base plus a 32-bit byte offset per lane: one address register
// per copy instead of two (the launcher sends operands that span 4 GiB or more elsewhere).
__device__ __forceinline__ void copy16_to_lds(const void* base, uint32_t offset, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(offset), "s"(base)
               : "memory");
}

__device__ __forceinline__ void wait_copies_and_barrier() {
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// As above, but the YOUNGEST copies (issued last; loads complete in order) may stay
// in flight: they fill a stage that is not read before the next barrier.
template <int YOUNGEST>
__device__ __forceinline__ void wait_copies_keep_youngest_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(YOUNGEST) : "memory");
}

// WVM x WVN wavefronts share the BM x 256 tile: 2 x 4, a wave tile of BM/2 x 64.  (2 x 2
// with BM/2 x 128 wave tiles and one wavefront per SIMD reads a third less from LDS but
// measured 7 % slower: a lone wavefront per SIMD stalls the matrix pipe whenever one of
// its copy instructions waits for room in the memory pipeline.)
// The MFMAs are 16 x 16 x 32: the wavefront's (BM/2) x 64 tile is MB16 x 4 blocks of 16 x 16, a
// K step is four units (K half x token-row half) of 16 MFMAs (8 for BM = 128), the fragments
// of the next unit are read while a unit is multiplied, and the weight fragments of a K half
// serve both of its units.
// ACT: epilogue code, or kGluBwd + the GLU code for the fused GLU backward
// (store_tile_glu_bwd16).
constexpr int kGluBwd = 16;

// `next`: thread 0 draws the id of the workgroup's next work item right before the last store
// of this one, so that the atomic's round trip runs under the store instead of after it.
template <typename T, int BM, int WVM, int WVN, int WL, int ACT>
__device__ __forceinline__ void m_grouped_dma_tile(MGemmArgs g, const Sched s, const int id,
                                                   NextDraw& next) {
  constexpr int NWAVES = WVM * WVN;
  constexpr int WM = BM / WVM, WNN = BN / WVN;
  constexpr int NBX = WNN / 32;
  constexpr int MB16 = WM / 16, NB16 = WNN / 16;  // 16-row and 16-column blocks of a wavefront
  constexpr int HB = MB16 / 2;                    // token blocks of one unit
  static_assert(WVM == 2 && WVN == 4 && HB >= 1, "2 x 4 wavefronts");
  constexpr int A_INSTR = BM / 8 / NWAVES;  // 1 KiB copy instructions per wavefront, token tile
  constexpr int W_INSTR = 32 / NWAVES;
  constexpr int A_BYTES = BM * BK * 2, W_BYTES = BN * BK * 2;
  // LDS: two token stages, then three weight stages (weights are copied two K
  // steps ahead, tokens one): 160 KiB for BM = 256, the whole LDS of a CU.
  constexpr int W_BASE = 2 * A_BYTES;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  // tile descriptor: lives in the third weight stage, which is first written after
  // every wavefront has passed the first barrier of the main loop
  int* const sh_tile = reinterpret_cast<int*>(smem + W_BASE + 2 * W_BYTES);

  int mt, nt;
  {
    const int ch = s.GM * s.GN;
    const int xcd = id % kNumXcd, j = id / kNumXcd;
    const int jb = s.by_block.div(j);
    const int blk = jb * kNumXcd + xcd, within = j - jb * ch;
    const int blk_m = s.by_nblk_n.div(blk), blk_n = blk - blk_m * s.nblk_n;
    const int wq = s.by_gm.div(within);
    mt = blk_m * s.GM + (within - wq * s.GM);
    nt = blk_n * s.GN + wq;
    if (nt >= s.NT) return;
  }
  // a K part of a tile is scheduled like a column tile of its own
  const int real_nt = s.real_nt;
  const int kpart = s.by_real_nt.div(nt);
  nt -= kpart * real_nt;
  const int KT = static_cast<int>(g.K / BK) / s.ksplit;  // K steps of this part
  const int kt0 = kpart * KT;
  g.c = static_cast<char*>(g.c) + static_cast<int64_t>(kpart) * g.c_split_stride * sizeof(T);
  if (threadIdx.x < 64) find_tile<BM>(g.group_indices, g.E, static_cast<int>(g.P), mt, sh_tile, s.even_tail != 0, s.band);
  __syncthreads();
  const int expert = __builtin_amdgcn_readfirstlane(sh_tile[0]);
  if (expert < 0) return;
  const int row0 = sh_tile[1], end = sh_tile[2];
  // column tiles nt0 .. nt0 + ntiles - 1 of this row block
  const int nt0 = nt * s.tpw;
  const int col_tiles = static_cast<int>((g.N + BN - 1) / BN);
  const int ntiles = col_tiles - nt0 < s.tpw ? col_tiles - nt0 : s.tpw;

  // (opaque: what depends only on the thread id would otherwise be computed once for all the
  // tiles of the workgroup and held in registers across them, next to the accumulators)
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WVN) * WM, wn0 = (wave % WVN) * WNN;

  // ---- global source address of every copy instruction ----------------------------
  // token tile: instruction i of wavefront w fills rows 8*(8i + w) .. +7, lane -> (row, chunk)
  uint32_t a_src[A_INSTR];  // byte offsets from g.a
#pragma unroll
  for (int i = 0; i < A_INSTR; ++i) {
    const int r = 8 * (NWAVES * i + wave) + (lane >> 3);
    const int c = (lane & 7) ^ ((r >> 1) & 7);
    int p = row0 + r;
    p = p < end ? p : end - 1;
    int64_t arow = p;
    if (g.flags & MOE_GEMM_GATHER_A) arow = g.by_topk.div(load_index32(g.indices, g.idx_bytes, p));
    arow = clamp_index(arow, g.a_rows);
    a_src[i] = static_cast<uint32_t>((arow * g.lda + c * 8) * 2);
  }
  uint32_t w_src[W_INSTR];  // byte offsets from wbase, the weight matrix of this expert
  const char* wbase = static_cast<const char*>(g.w) + static_cast<int64_t>(expert) * g.ldw_e * 2;
  const uint32_t w_step = static_cast<uint32_t>(WL == 0 ? static_cast<int64_t>(BK) * g.ldw_k * 2 : BK * 2);  // bytes per K step
  auto set_w_src = [&](int tile) __attribute__((always_inline)) {  // weight sources of column tile nt0 + tile
    const int64_t n0 = static_cast<int64_t>(nt0 + tile) * BN;
    if constexpr (WL == 0) {
      // N-contiguous tile [64][256]: instruction i fills k rows 2*(8i + w), +1
#pragma unroll
      for (int i = 0; i < W_INSTR; ++i) {
        const int k = 2 * (NWAVES * i + wave) + (lane >> 5);
        const int lb = ((lane & 31) * 16) ^ nmajor16_swizzle(k);
        int64_t n = n0 + lb / 2;
        n = n < g.N ? n : 0;  // columns past N only feed outputs that are not stored
        w_src[i] = static_cast<uint32_t>((static_cast<int64_t>(k) * g.ldw_k + n) * 2);
      }
    } else {
      // K-contiguous tile [256][64]
#pragma unroll
      for (int i = 0; i < W_INSTR; ++i) {
        const int r = 8 * (NWAVES * i + wave) + (lane >> 3);
        const int c = (lane & 7) ^ ((r >> 1) & 7);
        int64_t n = n0 + r;
        n = n < g.N ? n : g.N - 1;
        w_src[i] = static_cast<uint32_t>((n * g.ldw_n + c * 8) * 2);
      }
    }
  };
  set_w_src(0);
  const unsigned lds0 =
      __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<size_t>((lds_void*)smem))) +
      wave * 1024;

  // Copy instructions [first, last) of a tile; the main loop spreads them over the
  // sub-steps of a K step so that they do not queue up in front of the MFMAs.
  // A copy instruction whose eight token rows all lie past the end of the group is
  // not issued: those LDS rows keep stale data and only feed rows that are never
  // stored.  The last row block of a group is mostly such rows.
  const int rows_here = __builtin_amdgcn_readfirstlane(end - row0);
  auto issue_token_copies = [&](int stage, int kt, int first, int last) __attribute__((always_inline)) {
    const unsigned base = lds0 + stage * A_BYTES;
#pragma unroll
    for (int i = 0; i < A_INSTR; ++i)
      if (i >= first && i < last && 8 * (NWAVES * i + wave) < rows_here)
        copy16_to_lds(g.a, a_src[i] + static_cast<uint32_t>(kt0 + kt) * (BK * 2),
                      base + i * (NWAVES * 1024));
  };
  auto issue_weight_copies = [&](int wstage, int kt, int first, int last) __attribute__((always_inline)) {
    const unsigned base = lds0 + W_BASE + wstage * W_BYTES;
#pragma unroll
    for (int i = 0; i < W_INSTR; ++i)
      if (i >= first && i < last)
        copy16_to_lds(wbase, w_src[i] + static_cast<uint32_t>(kt0 + kt) * w_step,
                      base + i * (NWAVES * 1024));
  };

  // ---- LDS -> fragment addresses --------------------------------------------------
  const int tr_i = (lane >> 2) & 3, tr_q = lane & 3;  // transpose load: k row and column quad

  // 16-row blocks of this wavefront that hold rows of the group.  The last row block of a
  // group is mostly empty: the K loop is compiled for 0, MB16/4, MB16/2 and MB16 blocks, and a
  // wavefront runs the smallest that covers its own (every variant copies and synchronises
  // alike, so the wavefronts of a workgroup may run different ones).  A loop that tested each
  // block at run time took 350 instructions and 47 branches a K step and was bound by their
  // issue: 1.0 us a step for 8 MFMAs.
  int live = (end - row0 - wm0 + 15) / 16;
  live = live < 0 ? 0 : (live > MB16 ? MB16 : live);
  live = __builtin_amdgcn_readfirstlane(live);

  // unit u of a K step = K half (u >> 1), token-row half (u & 1)
  const int l16 = lane & 15, lg = lane >> 4;
  // transpose load of a 16-column block: group lg of 16 lanes fetches k rows 8*lg + i (+4)
  const int tr16_n = wn0 + 4 * tr_q;
  const int tr16_k = 8 * lg + tr_i;
  auto read_unit_t = [&](int stage, int u, s16x8 (&tf)[HB], auto blocks) __attribute__((always_inline)) {
    constexpr int LC = decltype(blocks)::value;
    const char* at = smem + stage * A_BYTES;
    const int kh = u >> 1, rh = u & 1;
#pragma unroll
    for (int mb = 0; mb < HB; ++mb)
      if (rh * HB + mb < LC)
        tf[mb] = *reinterpret_cast<const s16x8*>(
            at + kmajor_off(wm0 + (rh * HB + mb) * 16 + l16, kh * 4 + lg));
  };
  // column blocks [2*half, 2*half + 2) of K half kh: half 0 before the unit of token-row half
  // 0, half 1 at its start (a wavefront with at most HB live blocks has no other unit)
  auto read_unit_w = [&](int wstage, int kh, int half, s16x8 (&wf)[NB16], auto blocks) __attribute__((always_inline)) {
    constexpr int LC = decltype(blocks)::value;
    if (LC == 0) return;
    const char* wt = smem + W_BASE + wstage * W_BYTES;
#pragma unroll
    for (int nb = 2 * half; nb < 2 * half + 2; ++nb) {
      if constexpr (WL == 0) {
        const int k = kh * 32 + tr16_k;
        const int nbyte = (tr16_n + nb * 16) * 2;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(wt + nmajor16_off(k, nbyte)));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(wt + nmajor16_off(k + 4, nbyte)));
        wf[nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      } else {
        wf[nb] = *reinterpret_cast<const s16x8*>(wt + kmajor_off(wn0 + nb * 16 + l16, kh * 4 + lg));
      }
    }
  };

  f32x4 acc16[MB16][NB16];
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int mb = 0; mb < MB16; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB16; ++nb) acc16[mb][nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  };
  zero_acc();
  // the 16 MFMAs of unit (.., rh): token blocks rh*HB .. +HB-1 against the four column
  // blocks, column blocks 0 and 1 first: the fragments of blocks 2 and 3 are read at the start
  // of the unit that first needs them (every unit then reads 6 KiB: four token fragments and
  // two weight fragments, as evenly as the 32 x 32 x 16 schedule)
  auto multiply_unit = [&](int rh, s16x8 (&tf)[HB], s16x8 (&wf)[NB16], auto blocks) __attribute__((always_inline)) {
    constexpr int LC = decltype(blocks)::value;
#pragma unroll
    for (int nb = 0; nb < NB16; ++nb) {
#pragma unroll
      for (int mb = 0; mb < HB; ++mb) {
        if (rh == 0 && mb < LC) acc16[mb][nb] = mfma16<T>(wf[nb], tf[mb], acc16[mb][nb]);
        if (rh == 1 && HB + mb < LC) acc16[HB + mb][nb] = mfma16<T>(wf[nb], tf[mb], acc16[HB + mb][nb]);
      }
    }
  };
  auto interleave_unit = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < HB * NB16; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  s16x8 tfA[HB], tfB[HB], wfP[NB16], wfQ[NB16];
  // The accumulators of column tile `tile` leave through LDS regions that no copy in
  // flight writes: wavefronts 0..NWAVES/2-1 through the token stage `a_free` (BM = 256;
  // a spare region for BM = 128, whose token stages are too small), the others through
  // the weight stage `w_free`.
  constexpr int EPI_BYTES = epi_wave_bytes<NBX, 32>();
  constexpr int SPARE_BASE = W_BASE + 3 * W_BYTES;
  const int row0_wg = row0, end_wg = end, lane_wg = lane;
  auto store_acc = [&](int tile, int a_free, int w_free) __attribute__((always_inline)) {
    const int64_t n0 = static_cast<int64_t>(nt0 + tile) * BN;
    // The rows are the same for every tile of the workgroup, so the compiler would
    // compute the row addresses of the store (and load the scatter indices) once, ahead
    // of the K loop, and keep them in registers next to the accumulators: dozens of
    // VGPRs that spill.  Opaque copies of the row range and the lane id tie that work to
    // this call.
    int row0 = row0_wg, end = end_wg, lane = lane_wg;
    asm volatile("" : "+s"(row0), "+s"(end), "+v"(lane));
    char* epi;
    if (wave < NWAVES / 2)
      epi = smem + (BM == 256 ? a_free * A_BYTES : SPARE_BASE) + wave * EPI_BYTES;
    else
      epi = smem + W_BASE + w_free * W_BYTES + (wave - NWAVES / 2) * EPI_BYTES;
    if constexpr (ACT >= kGluBwd)
      // (launched with one column tile a workgroup: nothing is in flight after the last K
      // step, and every wavefront parks its G piece in a region of its own)
      store_tile_glu_bwd16<T, ACT - kGluBwd, MB16, NB16>(g, acc16, smem + wave * (WM * glu_bwd_pitch), row0,
                                                         end, n0, wm0, wn0, lane);
    else
      store_tile_lds16<T, ACT, MB16, NB16>(g, acc16, epi, row0, end, n0, wm0, wn0, lane);
  };
  auto main_loop = [&](auto blocks) __attribute__((always_inline)) {
    const int S = ntiles * KT;   // K steps of this workgroup; step gs is step gs % KT of tile gs / KT
    int kt_a = 0;                // copy cursors: K step (within its tile) to copy next
    int kt_w = 0, tile_w = 0;
    auto advance_a = [&]() __attribute__((always_inline)) { kt_a = kt_a + 1 == KT ? 0 : kt_a + 1; };
    auto advance_w = [&]() __attribute__((always_inline)) {
      if (++kt_w == KT) {
        kt_w = 0;
        if (++tile_w < ntiles) set_w_src(tile_w);
      }
    };
    issue_token_copies(0, kt_a, 0, A_INSTR);
    advance_a();
    issue_weight_copies(0, kt_w, 0, W_INSTR);
    advance_w();
    if (S > 1) {
      issue_weight_copies(1, kt_w, 0, W_INSTR);
      advance_w();
      wait_copies_keep_youngest_and_barrier<W_INSTR>();
    } else {
      wait_copies_and_barrier();
    }
    read_unit_t(0, 0, tfA, blocks);
    read_unit_w(0, 0, 0, wfP, blocks);
    int stage = 0, wcur = 0;  // token stage gs % 2, weight stage gs % 3
    int kt = 0, tile = 0;
    constexpr int AH = (A_INSTR + 1) / 2, WH = (W_INSTR + 1) / 2;
    for (int gs = 0; gs < S; ++gs) {
      const int wnext = wcur == 2 ? 0 : wcur + 1;
      const int wahead = wnext == 2 ? 0 : wnext + 1;
      const bool more = gs + 1 < S, ahead = gs + 2 < S;
      const bool tile_ends = kt + 1 == KT;
      if (more) issue_token_copies(stage ^ 1, kt_a, 0, AH);
      __builtin_amdgcn_s_setprio(2);
      __builtin_amdgcn_sched_barrier(0);
      read_unit_w(wcur, 0, 1, wfP, blocks);
      read_unit_t(stage, 1, tfB, blocks);
      multiply_unit(0, tfA, wfP, blocks);
      interleave_unit();
      if (more) {
        issue_token_copies(stage ^ 1, kt_a, AH, A_INSTR);
        advance_a();
      }
      __builtin_amdgcn_sched_barrier(0);
      read_unit_w(wcur, 1, 0, wfQ, blocks);
      read_unit_t(stage, 2, tfA, blocks);
      multiply_unit(1, tfB, wfP, blocks);
      interleave_unit();
      if (ahead) issue_weight_copies(wahead, kt_w, 0, WH);
      __builtin_amdgcn_sched_barrier(0);
      read_unit_w(wcur, 1, 1, wfQ, blocks);
      read_unit_t(stage, 3, tfB, blocks);
      multiply_unit(0, tfA, wfQ, blocks);
      interleave_unit();
      if (ahead) {
        issue_weight_copies(wahead, kt_w, WH, W_INSTR);
        advance_w();
      }
      __builtin_amdgcn_s_setprio(0);
      if (more) {
        // the token copies of step gs+1 and the weight copies of step gs+1 (issued a
        // step earlier) must have landed; the weight copies of step gs+2 may still fly
        if (ahead) wait_copies_keep_youngest_and_barrier<W_INSTR>();
        else wait_copies_and_barrier();
        // (the first fragments of a next tile are read after the store of this one:
        // held across the store they would crowd the register file)
        if (!tile_ends) {
          read_unit_t(stage ^ 1, 0, tfA, blocks);
          read_unit_w(wnext, 0, 0, wfP, blocks);
        }
      }
      multiply_unit(1, tfB, wfQ, blocks);
      interleave_unit();
      if (tile_ends) {
        // every wavefront is past the barrier above (or no later step exists and
        // nothing is in flight): the stages of this step are free
        if (!more) {
          __syncthreads();
          if (threadIdx.x == 0 && next.slot != nullptr) {
            next.value = atomicAdd(next.slot, 1u);
            next.drawn = true;
          }
        }
        store_acc(tile, stage, wcur);
        // (leaving here, instead of through the loop condition, tells the compiler that the
        // accumulators are dead during the store: their registers are the store's to use)
        if (!more) break;
        {
          __syncthreads();  // later steps copy into the stages just used for the store
          zero_acc();
          read_unit_t(stage ^ 1, 0, tfA, blocks);
          read_unit_w(wnext, 0, 0, wfP, blocks);
        }
        kt = 0;
        ++tile;
      } else {
        ++kt;
      }
      stage ^= 1;
      wcur = wnext;
    }
  };
  // The loop exists for 0, MB16/4, MB16/2 and MB16 live blocks; a wavefront takes the smallest
  // that covers its own (blocks past the end of the group then multiply stale LDS rows into
  // accumulators that are never stored: a token row only feeds its own output row).
  if (live == 0) main_loop(std::integral_constant<int, 0>{});
  else if (live <= MB16 / 4) main_loop(std::integral_constant<int, MB16 / 4>{});
  else if (live <= MB16 / 2) main_loop(std::integral_constant<int, MB16 / 2>{});
  else main_loop(std::integral_constant<int, MB16>{});
}

// Tile queues.  The kernel is launched with one workgroup per compute unit (its LDS use allows
// no more) and every workgroup draws tile ids until none is left.  Left to the hardware
// dispatcher, a compute unit idled 15 us on average between two workgroups once their durations
// differed (a group's last row block is short), 3 us between equal ones.  Tile id j * 8 + q
// belongs to queue q.  A workgroup draws from the queue of the XCD it runs on (the ids of a
// queue share the weight tiles they stream, and an XCD has its own L2), then from the other
// queues, so every id is drawn whatever XCDs the launch lands on.  Word 8 of a queue set counts
// the workgroups that are done; the last one clears the set for the next launch that uses it.
// A queue set belongs to ONE stream of one device: launches on a stream run one after the
// other, so they can share a set, and launches on different streams never do.  A launch that is
// being captured into a graph takes no set at all (queue == nullptr: workgroup b takes the ids
// b, b + gridDim.x, ... in order): a graph may be replayed on any stream, several times at once
// and next to eager launches, so nothing it runs may own device state.  The same holds for a
// process that uses more than kQueueSets streams on one device.
constexpr int kQueueSets = 1024;
constexpr int kQueueWords = 16;
static_assert((kNumXcd & (kNumXcd - 1)) == 0 && kNumXcd < kQueueWords, "queue per XCD, then the counter");
__device__ unsigned g_tile_queues[kQueueSets * kQueueWords];

struct DmaKernelArgs {
  MGemmArgs g;
  Sched s;
  unsigned* queue;
};
typedef __attribute__((address_space(4))) const DmaKernelArgs* kernarg_ptr;

template <typename T, int BM, int WVM, int WVN, int WL, int ACT>
__global__ __launch_bounds__(64 * WVM * WVN) void m_grouped_dma_kernel(DmaKernelArgs ka) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // (beside the tile descriptor that m_grouped_dma_tile keeps in the third weight stage)
  int* const sh_next = reinterpret_cast<int*>(smem + 2 * (BM * BK * 2) + 2 * (BN * BK * 2)) + 8;
  // hardware register XCC_ID: the XCD this workgroup runs on
  const int home = __builtin_amdgcn_s_getreg((31 << 11) | 20) & (kNumXcd - 1);
  int tried = 0;  // queues found empty so far, the home queue first
  NextDraw next{nullptr, 0u, false};
  int64_t static_id = blockIdx.x;  // launches without a queue set: ids in strides of the grid
  for (;;) {
    // The arguments are read from the kernel argument segment again for every tile: held in
    // scalar registers across the tiles they crowd out what the K loop keeps there.
    kernarg_ptr kp = (kernarg_ptr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(kp));
    const DmaKernelArgs* const args = (const DmaKernelArgs*)kp;
    __syncthreads();  // every wavefront is done with the LDS of the tile before
    if (threadIdx.x == 0 && args->queue == nullptr) {
      *sh_next = static_id < args->s.wgs ? static_cast<int>(static_id) : -1;
      static_id += gridDim.x;
    } else if (threadIdx.x == 0) {
      *sh_next = draw_work_item(args->queue, static_cast<int>(args->s.wgs), home, tried, next);
    }
    __syncthreads();
    const int id = __builtin_amdgcn_readfirstlane(*sh_next);
    if (id < 0) break;
    m_grouped_dma_tile<T, BM, WVM, WVN, WL, ACT>(args->g, args->s, id, next);
  }
  // (every workgroup ends here: each queue runs dry after s.wgs / 8 draws)
  if (threadIdx.x == 0 && ka.queue != nullptr) leave_queues(ka.queue);
}

// The queue set of `stream` on the current device and the number of compute units of that
// device.  *queue stays nullptr (ids in strides of the grid, no device state) while the stream
// is being captured and when the device has handed out all its sets.  Every device holds its
// own copy of g_tile_queues.  Returns MOE_OK or the status of fail().
int queue_set_of(hipStream_t stream, unsigned** queue, int* cus) {
  struct DeviceQueues {
    unsigned* base = nullptr;
    int cus = 0;
    std::unordered_map<hipStream_t, unsigned> set_of_stream;
  };
  constexpr int kMaxDevices = 64;
  static DeviceQueues per_device[kMaxDevices];
  static std::mutex lock;
  *queue = nullptr;
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(MOE_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(err));
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  err = hipStreamIsCapturing(stream, &capture);
  if (err != hipSuccess) return fail(MOE_ERR_HIP, "hipStreamIsCapturing: %s", hipGetErrorString(err));
  std::lock_guard<std::mutex> hold(lock);
  DeviceQueues& dq = per_device[dev];
  if (dq.base == nullptr) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(g_tile_queues));
    if (err != hipSuccess || p == nullptr)
      return fail(MOE_ERR_HIP, "hipGetSymbolAddress(tile queues): %s", hipGetErrorString(err));
    int n = 0;
    err = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess || n < 1)
      return fail(MOE_ERR_HIP, "hipDeviceGetAttribute(compute units): %s", hipGetErrorString(err));
    dq.cus = n;
    dq.base = static_cast<unsigned*>(p);
  }
  *cus = dq.cus;
  if (capture != hipStreamCaptureStatusNone) return MOE_OK;
  auto it = dq.set_of_stream.find(stream);
  if (it == dq.set_of_stream.end()) {
    if (dq.set_of_stream.size() >= static_cast<size_t>(kQueueSets)) return MOE_OK;
    it = dq.set_of_stream.emplace(stream, static_cast<unsigned>(dq.set_of_stream.size())).first;
  }
  *queue = dq.base + static_cast<size_t>(it->second) * kQueueWords;
  return MOE_OK;
}

// Sets the kernel's dynamic LDS limit on first use (per device) and launches it with one workgroup per
// compute unit (fewer if there are fewer work items).
template <auto Kernel>
int launch_kernel(const MGemmArgs& g, const Sched& s, dim3 grid, int threads, size_t lds,
                  hipStream_t stream) {
  int rc = allow_dynamic_lds(reinterpret_cast<const void*>(Kernel), lds);
  if (rc != MOE_OK) return rc;
  int cus = 0;
  unsigned* queue = nullptr;
  rc = queue_set_of(stream, &queue, &cus);
  if (rc != MOE_OK) return rc;
  DmaKernelArgs ka;
  ka.g = g;
  ka.s = s;
  ka.queue = queue;
  // (a multiple of the XCD count, so that ids taken in strides of the grid stay on their XCD)
  unsigned wgs = static_cast<unsigned>(cus) / kNumXcd * kNumXcd;
  if (wgs == 0) wgs = static_cast<unsigned>(cus);
  if (grid.x < wgs) wgs = grid.x;
  Kernel<<<dim3(wgs), threads, lds, stream>>>(ka);
  return MOE_OK;
}

template <typename T, int BM, int WVM, int WVN, int WL>
int launch_act(const MGemmArgs& g, hipStream_t stream) {
  // two column tiles a workgroup where that still leaves several rounds of workgroups
  const int64_t tiles = ((g.P + BM - 1) / BM + g.E / 2) * ((g.N + BN - 1) / BN) * (g.ksplit < 1 ? 1 : g.ksplit);
  // (the fused GLU backward stores through the whole LDS: one column tile a workgroup)
  const int tpw = (g.flags & MOE_GEMM_GLU_BWD) ? 1 : (tiles >= 2048 ? 2 : 1);
  // Tile order.  With long K a column tile's weight panel is megabytes, and what the launch
  // fetches through the fabric depends on which tiles run together (Mixtral shape, random
  // routing: 7.7 GB a gate/up launch against 2.8 GB with evenly loaded experts, and every full
  // tile 7 % slower).  Launches that keep K whole take expert-aligned bands (5.1 GB; gate/up
  // -4 %, fused GLU backward -2 %); launches with split K, whose work items are few and long,
  // gain more from an even last pair of row blocks (dX -5.5 %, down -3 %: a workgroup's items
  // are then closer to equal).  Either rule applied to the other kind of launch loses 1-3 %, and
  // with K below 4096 (panels of 1 MiB and less) neither changes anything.
  const bool split = g.ksplit > 1;
  Sched s = make_sched(g, BM, tpw, !split && g.K >= 4096 ? 4 : 0);
  s.even_tail = split;
  if (s.wgs > 0x7fffffff) return fail(MOE_ERR_UNSUPPORTED, "grid too large");
  // 2 token + 3 weight stages; BM = 128 adds room for the store staging of half the wavefronts
  const size_t lds = 2 * (BM * BK * 2) + 3 * (BN * BK * 2) +
                     (BM == 256 ? 0 : (WVM * WVN / 2) * epi_wave_bytes<BN / WVN / 32, 32>());
  const dim3 grid(static_cast<unsigned>(s.wgs));
  constexpr int threads = 64 * WVM * WVN;
  if (g.flags & MOE_GEMM_GLU_BWD) {
    if constexpr (WL == 1) {  // the fused GLU backward is built for K-contiguous weights only
      const int rc =
          g.epilogue == MOE_ACT_SWIGLU
              ? launch_kernel<m_grouped_dma_kernel<T, BM, WVM, WVN, WL, kGluBwd + MOE_ACT_SWIGLU>>(g, s, grid, threads, lds, stream)
              : launch_kernel<m_grouped_dma_kernel<T, BM, WVM, WVN, WL, kGluBwd + MOE_ACT_GEGLU>>(g, s, grid, threads, lds, stream);
      if (rc != MOE_OK) return rc;
      return check_launch("m_grouped_gemm (fused GLU backward)");
    } else {
      return fail(MOE_ERR_UNSUPPORTED, "fused GLU backward needs K-contiguous weights");
    }
  }
  MOE_DISPATCH_ACT(g.epilogue, ACT, {
    const int rc = launch_kernel<m_grouped_dma_kernel<T, BM, WVM, WVN, WL, ACT>>(g, s, grid, threads, lds, stream);
    if (rc != MOE_OK) return rc;
  });
  return check_launch("m_grouped_gemm (MFMA kernel, direct-to-LDS copies)");
}

}  // namespace

int tile_queue_set_of(hipStream_t stream, unsigned** queue, int* cus) {
  return queue_set_of(stream, queue, cus);
}

bool m_grouped_mfma_dma_supported(const MGemmArgs& g) {
  // stores through LDS only; copy sources are 32-bit byte offsets from the token matrix
  // and from the weight matrix of one expert
  if (!(g.dtype == MOE_DTYPE_BF16 ? lds_epilogue_ok<bf16_t>(g) : lds_epilogue_ok<f16_t>(g))) return false;
  const int64_t limit = int64_t(1) << 32;
  const int64_t a_span = g.a_rows * g.lda * 2;
  const int64_t w_span = ((g.K - 1) * g.ldw_k + (g.N - 1) * g.ldw_n + 256 * (g.ldw_k + g.ldw_n)) * 2;
  return g.K % BK == 0 && a_span < limit && w_span < limit;
}

int launch_m_grouped_mfma_dma(const MGemmArgs& g, hipStream_t stream) {
  if (!m_grouped_mfma_dma_supported(g))
    return fail(MOE_ERR_UNSUPPORTED, "operands outside the reach of the direct-to-LDS kernel");
  const bool nmajor = g.ldw_n == 1 && g.ldw_k % 8 == 0;
  // 256-row tiles from an average of 256 rows an expert: a group of ~256 rows is then one full
  // row block and a short one (whose dead 16-row blocks are not multiplied) instead of two or
  // three 128-row blocks that each stream the weight panel (measured: +22 % at 8 experts x 256
  // rows, K = 4096; +21 % at 64 x 256, K = 2048; +8 % at 128 x 256, K = 768; at 128 rows an
  // expert the 128-row tiles are 3-10 % faster)
  const bool big = g.P / g.E >= 256;
  if (g.dtype == MOE_DTYPE_BF16) {
    if (nmajor) return big ? launch_act<bf16_t, 256, 2, 4, 0>(g, stream) : launch_act<bf16_t, 128, 2, 4, 0>(g, stream);
    return big ? launch_act<bf16_t, 256, 2, 4, 1>(g, stream) : launch_act<bf16_t, 128, 2, 4, 1>(g, stream);
  }
  if (nmajor) return big ? launch_act<f16_t, 256, 2, 4, 0>(g, stream) : launch_act<f16_t, 128, 2, 4, 0>(g, stream);
  return big ? launch_act<f16_t, 256, 2, 4, 1>(g, stream) : launch_act<f16_t, 128, 2, 4, 1>(g, stream);
}

}  // namespace moe
