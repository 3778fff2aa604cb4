// Pieces shared by the MFMA grouped-GEMM kernels: fragment types, LDS tile
// layouts, the device-side tile -> (expert, row block) map and the epilogue.
#pragma once
#include "gemm.h"

#include <type_traits>

namespace moe {
namespace mfma {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

constexpr int BN = 256, BK = 64;
constexpr int kThreads = 512;
constexpr int WAVES_M = 2, WAVES_N = 4;
constexpr int WN = BN / WAVES_N;  // 64 columns per wavefront
constexpr int NB = WN / 32;       // 2 column blocks per wavefront
constexpr int kNumXcd = 8;

template <typename T>
__device__ __forceinline__ f32x16 mfma32(s16x8 w, s16x8 t, f32x16 acc) {
  if constexpr (sizeof(T) == 2 && __is_same(T, bf16_t)) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, w),
                                                   __builtin_bit_cast(bf16x8, t), acc, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, w),
                                                  __builtin_bit_cast(f16x8, t), acc, 0, 0, 0);
  }
}

// 16 x 16 x 32: operands are 16 rows x 32 K (lane: row lane % 16, K chunk lane / 16 of
// eight values); the result has column lane % 16 and rows 4 * (lane / 16) + {0..3}.
// With random operands this shape draws less power per FLOP than 32 x 32 x 16, and the
// shader clock under a GEMM load is set by power: measured +9..13 % throughput.
template <typename T>
__device__ __forceinline__ f32x4 mfma16(s16x8 w, s16x8 t, f32x4 acc) {
  if constexpr (sizeof(T) == 2 && __is_same(T, bf16_t)) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w),
                                                   __builtin_bit_cast(bf16x8, t), acc, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, w),
                                                  __builtin_bit_cast(f16x8, t), acc, 0, 0, 0);
  }
}

// Byte offset of 16-byte chunk `c` of row `r` in a [rows][64]-element tile.
__device__ __forceinline__ int kmajor_off(int r, int c) {
  return r * 128 + ((c ^ ((r >> 1) & 7)) << 4);
}
// Byte offset of element (k, n) in a [64][256]-element N-contiguous tile; the
// swizzle moves 64-byte groups so that the four k rows of one transpose load
// fall into different banks.
__device__ __forceinline__ int nmajor_off(int k, int nbyte) {
  return k * 512 + (nbyte ^ ((k & 3) << 6) ^ (((k >> 2) & 1) << 5));
}

// The same tile for the 16 x 16 x 32 kernels, whose transpose loads fetch k rows
// 8g + i (+4) for the four 16-lane groups g of an instruction: the 32-byte bit follows
// k bit 3, so that the two groups served together read different banks.
__device__ __forceinline__ int nmajor16_swizzle(int k) {
  return ((k & 3) << 6) ^ (((k >> 3) & 1) << 5);
}
__device__ __forceinline__ int nmajor16_off(int k, int nbyte) {
  return k * 512 + (nbyte ^ nmajor16_swizzle(k));
}

// Tile order of one launch, fixed on the host.
struct Sched {
  int tpw;     // adjacent column tiles that one workgroup computes one after the other
  int NT;      // groups of tpw column tiles (times ksplit: a K part is scheduled like a group)
  int ksplit;  // parts the K loop is cut into (each part stores to its own copy of c)
  int GM, GN;  // tile block handed to one XCD at a time
  int nblk_n;  // blocks per band of rows
  int64_t wgs; // workgroups to launch
  // the divisions of the id -> tile lookup as multipliers (an integer division by a run-time
  // value is ~40 instructions): by GM * GN, nblk_n, GM and NT / ksplit
  int real_nt;  // NT / ksplit
  FastDiv by_block, by_nblk_n, by_gm, by_real_nt;
  int band;       // > 0: bands of that many row blocks stay inside one expert (see make_sched)
  int even_tail;  // the last two row blocks of a group share their rows evenly (see find_tile)
};

// The grid is a static bound: cdiv(P, BM) + E row blocks times the column tiles,
// padded so that the GM x GN blocks tile it and their count is a multiple of 8.
// band > 0: a band of `band` row blocks never crosses from one expert into the next (an expert
// of n row blocks has cdiv(n, band) bands, the last one padded with empty slots), so that the
// band x GN tiles an XCD works on at a time share GN weight panels instead of up to 2 GN; the
// bound on the bands is then cdiv(cdiv(P, BM), band) + E.
inline Sched make_sched(const MGemmArgs& g, int BM, int tpw = 1, int band = 0) {
  Sched s;
  s.tpw = tpw;
  s.ksplit = g.ksplit < 1 ? 1 : g.ksplit;
  s.NT = (static_cast<int>((g.N + BN - 1) / BN) + tpw - 1) / tpw * s.ksplit;
  int MT = static_cast<int>((g.P + BM - 1) / BM) + g.E;
  if (band > 0) MT = band * (static_cast<int>(((g.P + BM - 1) / BM + band - 1) / band) + g.E);
  s.band = band;
  s.even_tail = 0;
  const int gm = band > 0 ? band : 4;
  s.GM = MT < gm ? MT : gm;
  s.GN = s.NT < 8 ? s.NT : 8;
  const int nblk_m = (MT + s.GM - 1) / s.GM;
  s.nblk_n = (s.NT + s.GN - 1) / s.GN;
  const int64_t nblk = (static_cast<int64_t>(nblk_m) * s.nblk_n + kNumXcd - 1) / kNumXcd * kNumXcd;
  s.wgs = nblk * s.GM * s.GN;
  s.real_nt = s.NT / s.ksplit;
  s.by_block = FastDiv(static_cast<uint32_t>(s.GM * s.GN));
  s.by_nblk_n = FastDiv(static_cast<uint32_t>(s.nblk_n));
  s.by_gm = FastDiv(static_cast<uint32_t>(s.GM));
  s.by_real_nt = FastDiv(static_cast<uint32_t>(s.real_nt < 1 ? 1 : s.real_nt));
  return s;
}

// ---- tile queues of the persistent kernels ---------------------------------------------
// A launch has one resident workgroup per compute unit; every workgroup draws work item ids
// until none is left.  Id 8 j + q belongs to queue q: a workgroup draws from the queue of the
// XCD it runs on (its ids share the panels they stream, and an XCD has its own L2), then from
// the other queues, so every id is drawn whatever XCDs the launch lands on.  A queue set is 16
// words: eight draw counters, then the count of workgroups that are done; the last one clears
// the set for the next launch that uses it (sets belong to one stream: gemm.h).
struct NextDraw {
  unsigned* slot;   // queue word the next draw goes to (nullptr: every queue has run dry)
  unsigned value;   // what a draw made ahead of time returned (thread 0)
  bool drawn;
};

// Thread 0: the next id of this workgroup, or -1.  `tried`: queues found dry so far, the home
// queue first.  A draw made ahead of time (during the last store of the item before, so that the
// atomic's round trip runs under the store) is in `next`.
__device__ __forceinline__ int draw_work_item(unsigned* queue, int total, int home, int& tried,
                                              NextDraw& next) {
  int id = -1;
  while (tried < kNumXcd) {
    const int q = (home + tried) & (kNumXcd - 1);
    const unsigned got = next.drawn ? next.value : atomicAdd(&queue[q], 1u);
    next.drawn = false;
    const int64_t cand = static_cast<int64_t>(got) * kNumXcd + q;
    if (cand < total) {
      id = static_cast<int>(cand);
      break;
    }
    ++tried;
    // A queue that has run dry stays dry for the rest of the launch: look at all the
    // counters at once (one round trip) and pass over the dry ones, instead of finding
    // each of them empty with an atomic of its own when the launch drains.
    unsigned seen[kNumXcd];
#pragma unroll
    for (int i = 0; i < kNumXcd; ++i)
      seen[i] = __hip_atomic_load(&queue[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while (tried < kNumXcd) {
      const int qq = (home + tried) & (kNumXcd - 1);
      unsigned c = 0;
#pragma unroll
      for (int i = 0; i < kNumXcd; ++i) c = i == qq ? seen[i] : c;
      if (static_cast<int64_t>(c) * kNumXcd + qq < total) break;
      ++tried;
    }
  }
  next.slot = tried < kNumXcd ? &queue[(home + tried) & (kNumXcd - 1)] : nullptr;
  return id;
}

// Thread 0 of a workgroup that has run out of work (each queue runs dry after total / 8 draws).
__device__ __forceinline__ void leave_queues(unsigned* queue) {
  __threadfence();
  if (atomicAdd(&queue[kNumXcd], 1u) == gridDim.x - 1) {
    for (int q = 0; q <= kNumXcd; ++q) atomicExch(&queue[q], 0u);
  }
}

// Wavefront 0 finds the expert whose row blocks contain block `mt`: sh[0] = expert (-1: none),
// sh[1] = first row of the block, sh[2] = end of the block's rows.
// EVEN_TAIL: a group of n rows has cdiv(n, BM) blocks either way, but when its last block would
// hold at most BM / 2 rows, the last TWO blocks share their BM + r rows about evenly instead
// (BM / 2 + ceil(r / 2) rounded up to 16, and the rest).  A block of few rows costs a workgroup
// most of what a full one does (it streams the same weight panel; the matrix cores idle), while
// two blocks of little more than BM / 2 rows each skip the multiplies of their dead 16-row
// blocks and take about as long as each other and as a full block, which keeps the work items
// of a launch with few, long items alike.
// BAND > 0: `mt` counts slots of expert-aligned bands of BAND row blocks (make_sched with
// band): slot mt is row block (mt / BAND - bands before the expert) * BAND + mt % BAND of its
// expert, or nothing when the expert has fewer row blocks.
template <int BM>
__device__ __forceinline__ void find_tile(const int32_t* __restrict__ gi, int E, int P, int mt,
                                          int* sh, bool EVEN_TAIL = false, int BAND = 0) {
  const int lane = threadIdx.x;
  const int band = BAND > 0 ? mt / BAND : 0;
  const int in_band = BAND > 0 ? mt - band * BAND : 0;
  int run = 0;
  bool done = false;
  for (int base = 0; base < E && !done; base += 64) {
    const int e = base + lane;
    int lo = 0, hi = 0;
    if (e < E) {
      lo = gi[e];
      hi = gi[e + 1];
      lo = lo < 0 ? 0 : lo;
      hi = hi > P ? P : hi;
    }
    const int tiles = hi > lo ? (hi - lo + BM - 1) / BM : 0;
    // what the scan counts: row blocks, or bands of them
    const int units = BAND > 0 ? (tiles + BAND - 1) / BAND : tiles;
    int incl = units;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      int v = __shfl_up(incl, off, 64);
      if (lane >= off) incl += v;
    }
    const int excl = run + incl - units;
    const int at = BAND > 0 ? band : mt;
    const bool here = at >= excl && at < excl + units;
    const int b = BAND > 0 ? (band - excl) * BAND + in_band : mt - excl;
    const bool mine = here && b < tiles;
    if (mine) {
      int first = lo + b * BM, last = hi;
      if (EVEN_TAIL && tiles >= 2 && b >= tiles - 2) {
        const int r = hi - lo - (tiles - 1) * BM;  // rows of the last block: 1 .. BM
        if (r <= BM / 2) {
          const int cut = lo + (tiles - 2) * BM + BM / 2 + (((r + 1) / 2 + 15) & ~15);
          if (b == tiles - 2) last = cut;
          else first = cut;
        }
      }
      sh[0] = e;
      sh[1] = first;
      sh[2] = last;
    }
    done = __ballot(here) != 0;
    if (done && __ballot(mine) == 0 && lane == 0) sh[0] = -1;  // a padding slot of the expert's last band
    run += __shfl(incl, 63, 64);
  }
  if (!done && lane == 0) sh[0] = -1;
}

// Epilogue shared by the MFMA kernels.  A lane owns token row (lane & 31) of each
// 32-row block and, per 32-column block, four runs of four consecutive columns:
// n = 8*run + 4*(lane >> 5) + {0..3}; a gate/up pair of the interleaved GLU layout
// is two neighbouring accumulator registers.
template <typename T, int ACT, int MB, int NBX = NB>
__device__ __forceinline__ void store_tile(const MGemmArgs& g, f32x16 (&acc)[MB][NBX], int row0,
                                           int end, int64_t n0, int wm0, int wn0, int l32,
                                           int lhi) {
  constexpr bool GLU = act_is_glu(ACT);
  // lane owns token row (l32) of each row block and, per column block, four runs of
  // four consecutive columns: n = 8*run + 4*lhi + {0..3}
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int p = row0 + wm0 + mb * 32 + l32;
    if (p >= end) continue;
    int64_t slot = p;
    if (g.flags & (MOE_GEMM_SCATTER_C | MOE_GEMM_SCATTER_ADD))
      slot = load_index(g.indices, g.idx_bytes, p);
    float wgt = 1.0f;
    int64_t crow;
    if (g.flags & MOE_GEMM_SCATTER_ADD) {
      crow = clamp_index(g.by_topk.div(static_cast<int32_t>(slot)), g.c_rows);
      if (g.scales != nullptr) wgt = to_f32(static_cast<const T*>(g.scales)[clamp_index(slot, g.P)]);
    } else {
      crow = clamp_index(slot, g.c_rows);
    }
#pragma unroll
    for (int nb = 0; nb < NBX; ++nb) {
#pragma unroll
      for (int run = 0; run < 4; ++run) {
        const int64_t n = n0 + wn0 + nb * 32 + run * 8 + lhi * 4;
        if (n >= g.N) continue;  // N is a multiple of 8, so a run is all in or all out
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = acc[mb][nb][run * 4 + j];
        if (g.flags & MOE_GEMM_SAVE_PREACT) {
          T pre[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) pre[j] = from_f32<T>(v[j]);
          *reinterpret_cast<uint2*>(static_cast<T*>(g.preact) + static_cast<int64_t>(p) * g.ld_preact + n) =
              *reinterpret_cast<const uint2*>(pre);
        }
        if constexpr (GLU) {
          const float o0 = apply_act<ACT>(v[0]) * v[1];
          const float o1 = apply_act<ACT>(v[2]) * v[3];
          const int64_t c = n / 2;
          if (g.flags & MOE_GEMM_SCATTER_ADD) {
            float* dst = static_cast<float*>(g.c) + crow * g.ldc + c;
            unsafeAtomicAdd(dst, wgt * o0);
            unsafeAtomicAdd(dst + 1, wgt * o1);
          } else {
            T o[2] = {from_f32<T>(o0), from_f32<T>(o1)};
            *reinterpret_cast<uint32_t*>(static_cast<T*>(g.c) + crow * g.ldc + c) =
                *reinterpret_cast<const uint32_t*>(o);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = apply_act<ACT>(v[j]);
          if (g.flags & MOE_GEMM_SCATTER_ADD) {
            float* dst = static_cast<float*>(g.c) + crow * g.ldc + n;
#pragma unroll
            for (int j = 0; j < 4; ++j) unsafeAtomicAdd(dst + j, wgt * v[j]);
          } else {
            T o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = from_f32<T>(v[j]);
            *reinterpret_cast<uint2*>(static_cast<T*>(g.c) + crow * g.ldc + n) =
                *reinterpret_cast<const uint2*>(o);
          }
        }
      }
    }
  }
}

// Epilogue through LDS: the accumulators of PASS_ROWS (64 or 32) token rows of a
// wavefront are rounded, written to a private LDS region (row stride padded by 8 bytes, which
// keeps the 32 rows written by one instruction on different banks), read back
// row-wise and stored with 16 bytes per lane, so one store instruction covers
// whole contiguous row pieces instead of 64 different cache lines.  Handles the
// plain and the row-scatter store, the pre-activation copy and every activation;
// the atomic scatter-add and outputs that cannot take 16-byte stores use
// store_tile().  `epi` is this wavefront's region of epi_wave_bytes<NBX, PASS_ROWS>() bytes;
// the caller has made sure that no wavefront still reads the main-loop tiles.
template <int NBX, int PASS_ROWS = 64>
constexpr int epi_wave_bytes() {
  return PASS_ROWS * (NBX * 64 + 8);
}

template <typename T>
__host__ __device__ inline bool lds_epilogue_ok(const MGemmArgs& g) {
  if (g.flags & MOE_GEMM_GLU_BWD)  // dh, s*glu(h) and h rows in 16-byte pieces
    return g.N % 8 == 0 && g.ldc % 8 == 0 && g.ld_preact % 8 == 0 && g.ldh % 8 == 0 &&
           !(reinterpret_cast<uintptr_t>(g.c) & 15) && !(reinterpret_cast<uintptr_t>(g.preact) & 15) &&
           !(reinterpret_cast<uintptr_t>(g.h) & 15);
  if (g.flags & MOE_GEMM_SCATTER_ADD) return false;
  // store_tile_lds() has no pre-activation store for the identity epilogue (the entry
  // point copies c instead where the two coincide)
  if ((g.flags & MOE_GEMM_SAVE_PREACT) && g.epilogue == MOE_ACT_NONE) return false;
  const int64_t width = act_is_glu(g.epilogue) ? g.N / 2 : g.N;
  if (width % 8 != 0 || g.ldc % 8 != 0 || (reinterpret_cast<uintptr_t>(g.c) & 15)) return false;
  if ((g.flags & MOE_GEMM_SAVE_PREACT) &&
      (g.ld_preact % 8 != 0 || (reinterpret_cast<uintptr_t>(g.preact) & 15)))
    return false;
  return true;
}

template <typename T, int ACT, int MB, int NBX, int PASS_ROWS = 64>
__device__ __forceinline__ void store_tile_lds(const MGemmArgs& g, f32x16 (&acc)[MB][NBX],
                                               char* epi, int row0, int end, int64_t n0, int wm0,
                                               int wn0, int lane) {
  constexpr bool GLU = act_is_glu(ACT);
  constexpr int ROW_BYTES = NBX * 64 + 8;
  constexpr int MBH = PASS_ROWS / 32 < MB ? PASS_ROWS / 32 : MB;  // row blocks staged at a time
  constexpr int HALVES = MB / MBH;
  const int l32 = lane & 31, lhi = lane >> 5;

  // row-wise read-back and store of `cols` columns (16 bytes = 8 columns per lane)
  auto flush = [&](int half, int cols, T* base, int64_t ld, int64_t col0, int64_t width,
                   bool scatter) {
    const int lanes_per_row = cols / 8;           // 4, 8 or 16
    const int rows_per_inst = 64 / lanes_per_row;
    const int lr = lane / lanes_per_row, lc = lane % lanes_per_row;
    for (int it = 0; it < MBH * 32 / rows_per_inst; ++it) {
      const int r = it * rows_per_inst + lr;
      const char* src = epi + r * ROW_BYTES + lc * 16;
      const uint2 v0 = *reinterpret_cast<const uint2*>(src);
      const uint2 v1 = *reinterpret_cast<const uint2*>(src + 8);
      const int p = row0 + wm0 + half * (MBH * 32) + r;
      const int64_t col = col0 + lc * 8;
      if (p < end && col < width) {
        int64_t crow = p;
        if (scatter) crow = clamp_index(load_index(g.indices, g.idx_bytes, p), g.c_rows);
        *reinterpret_cast<uint4*>(base + crow * ld + col) = make_uint4(v0.x, v0.y, v1.x, v1.y);
      }
    }
  };

#pragma unroll
  for (int half = 0; half < HALVES; ++half) {
    if (ACT != MOE_ACT_NONE && (g.flags & MOE_GEMM_SAVE_PREACT)) {
#pragma unroll
      for (int mbh = 0; mbh < MBH; ++mbh)
#pragma unroll
        for (int nb = 0; nb < NBX; ++nb)
#pragma unroll
          for (int run = 0; run < 4; ++run) {
            T v[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = from_f32<T>(acc[half * MBH + mbh][nb][run * 4 + j]);
            *reinterpret_cast<uint2*>(epi + (mbh * 32 + l32) * ROW_BYTES +
                                      (nb * 32 + run * 8 + lhi * 4) * 2) =
                *reinterpret_cast<const uint2*>(v);
          }
      flush(half, NBX * 32, static_cast<T*>(g.preact), g.ld_preact, n0 + wn0, g.N, false);
    }
#pragma unroll
    for (int mbh = 0; mbh < MBH; ++mbh)
#pragma unroll
      for (int nb = 0; nb < NBX; ++nb)
#pragma unroll
        for (int run = 0; run < 4; ++run) {
          const f32x16& a = acc[half * MBH + mbh][nb];
          char* dst = epi + (mbh * 32 + l32) * ROW_BYTES;
          if constexpr (GLU) {
            T o[2] = {from_f32<T>(apply_act<ACT>(a[run * 4 + 0]) * a[run * 4 + 1]),
                      from_f32<T>(apply_act<ACT>(a[run * 4 + 2]) * a[run * 4 + 3])};
            *reinterpret_cast<uint32_t*>(dst + (nb * 16 + run * 4 + lhi * 2) * 2) =
                *reinterpret_cast<const uint32_t*>(o);
          } else {
            T o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = from_f32<T>(apply_act<ACT>(a[run * 4 + j]));
            *reinterpret_cast<uint2*>(dst + (nb * 32 + run * 8 + lhi * 4) * 2) =
                *reinterpret_cast<const uint2*>(o);
          }
        }
    if constexpr (GLU)
      flush(half, NBX * 16, static_cast<T*>(g.c), g.ldc, (n0 + wn0) / 2, g.N / 2,
            g.flags & MOE_GEMM_SCATTER_C);
    else
      flush(half, NBX * 32, static_cast<T*>(g.c), g.ldc, n0 + wn0, g.N,
            g.flags & MOE_GEMM_SCATTER_C);
    // keep the passes apart: overlapped by the scheduler, the rounded rows, index loads
    // and addresses of all of them would be live at once, next to the accumulators
    __builtin_amdgcn_sched_barrier(0);
  }
}

// Epilogue through LDS for the 16 x 16 x 32 accumulator layout: a lane owns token row
// (lane & 15) of each 16-row block and, per 16-column block, the four consecutive columns
// 4 * (lane >> 4) + {0..3} (so a gate/up pair is again two neighbouring registers).  Passes
// of 32 token rows through `epi` (epi_wave_bytes<NB16 / 2, 32>() bytes), otherwise as
// store_tile_lds().
template <typename T, int ACT, int MB16, int NB16>
__device__ __forceinline__ void store_tile_lds16(const MGemmArgs& g, f32x4 (&acc)[MB16][NB16],
                                                 char* epi, int row0, int end, int64_t n0,
                                                 int wm0, int wn0, int lane) {
  constexpr bool GLU = act_is_glu(ACT);
  constexpr int ROW_BYTES = NB16 * 32 + 8;
  constexpr int PASSES = MB16 / 2;
  const int l16 = lane & 15, lg = lane >> 4;

  auto flush = [&](int pass, int cols, T* base, int64_t ld, int64_t col0, int64_t width,
                   bool scatter) {
    const int lanes_per_row = cols / 8;           // 4 or 8
    const int rows_per_inst = 64 / lanes_per_row;
    const int lr = lane / lanes_per_row, lc = lane % lanes_per_row;
    for (int it = 0; it < 32 / rows_per_inst; ++it) {
      const int r = it * rows_per_inst + lr;
      const char* src = epi + r * ROW_BYTES + lc * 16;
      const uint2 v0 = *reinterpret_cast<const uint2*>(src);
      const uint2 v1 = *reinterpret_cast<const uint2*>(src + 8);
      const int p = row0 + wm0 + pass * 32 + r;
      const int64_t col = col0 + lc * 8;
      if (p < end && col < width) {
        int64_t crow = p;
        if (scatter) crow = clamp_index(load_index(g.indices, g.idx_bytes, p), g.c_rows);
        *reinterpret_cast<uint4*>(base + crow * ld + col) = make_uint4(v0.x, v0.y, v1.x, v1.y);
      }
    }
  };

#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    if (ACT != MOE_ACT_NONE && (g.flags & MOE_GEMM_SAVE_PREACT)) {
#pragma unroll
      for (int mbh = 0; mbh < 2; ++mbh)
#pragma unroll
        for (int nb = 0; nb < NB16; ++nb) {
          T v[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = from_f32<T>(acc[pass * 2 + mbh][nb][j]);
          *reinterpret_cast<uint2*>(epi + (mbh * 16 + l16) * ROW_BYTES + (nb * 16 + lg * 4) * 2) =
              *reinterpret_cast<const uint2*>(v);
        }
      flush(pass, NB16 * 16, static_cast<T*>(g.preact), g.ld_preact, n0 + wn0, g.N, false);
    }
#pragma unroll
    for (int mbh = 0; mbh < 2; ++mbh)
#pragma unroll
      for (int nb = 0; nb < NB16; ++nb) {
        const f32x4& a = acc[pass * 2 + mbh][nb];
        char* dst = epi + (mbh * 16 + l16) * ROW_BYTES;
        if constexpr (GLU) {
          T o[2] = {from_f32<T>(apply_act<ACT>(a[0]) * a[1]), from_f32<T>(apply_act<ACT>(a[2]) * a[3])};
          *reinterpret_cast<uint32_t*>(dst + (nb * 8 + lg * 2) * 2) =
              *reinterpret_cast<const uint32_t*>(o);
        } else {
          T o[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = from_f32<T>(apply_act<ACT>(a[j]));
          *reinterpret_cast<uint2*>(dst + (nb * 16 + lg * 4) * 2) = *reinterpret_cast<const uint2*>(o);
        }
      }
    if constexpr (GLU)
      flush(pass, NB16 * 8, static_cast<T*>(g.c), g.ldc, (n0 + wn0) / 2, g.N / 2,
            g.flags & MOE_GEMM_SCATTER_C);
    else
      flush(pass, NB16 * 16, static_cast<T*>(g.c), g.ldc, n0 + wn0, g.N,
            g.flags & MOE_GEMM_SCATTER_C);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// Epilogue of the fused GLU backward (MOE_GEMM_GLU_BWD): the accumulators hold
// G[p, j] = d loss / d glu(h)[p, j] / s_p for the wavefront's 16 x 16 blocks.  With
// (gate, up) = h[p, 2j], h[p, 2j+1], a = act(gate), y = a * up:
//     dh[p, 2j] = s_p G up act'(gate),  dh[p, 2j+1] = s_p G a,  ys[p, j] = s_p y,
//     dscale[p] += sum_j G y            (scales and dscale are indexed by position p)
// Two phases, because the h values that hide their own load latency do not fit next to
// the accumulators: G is rounded to T and parked in `region` (WM rows of 64 columns, pitch
// glu_bwd_pitch; the workgroup's whole LDS is free, so every wavefront has its own region),
// then the wavefront walks its rows eight at a time with eight lanes a row (8 columns of
// G, 16 of h and dh each): loads, stores and the h prefetch of half the tile at once.
constexpr int glu_bwd_pitch = 64 * 2 + 8;
template <typename T, int ACT, int MB16, int NB16>
__device__ __forceinline__ void store_tile_glu_bwd16(const MGemmArgs& g, f32x4 (&acc)[MB16][NB16],
                                                     char* region, int row0, int end, int64_t n0,
                                                     int wm0, int wn0, int lane) {
  static_assert(act_is_glu(ACT) && NB16 == 4, "GLU activations, 64-column wave tiles");
  constexpr int PITCH = glu_bwd_pitch;
  {
    const int l16 = lane & 15, lg = lane >> 4;
#pragma unroll
    for (int mb = 0; mb < MB16; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB16; ++nb) {
        T v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = from_f32<T>(acc[mb][nb][j]);
        *reinterpret_cast<uint2*>(region + (mb * 16 + l16) * PITCH + (nb * 16 + lg * 4) * 2) =
            *reinterpret_cast<const uint2*>(v);
      }
  }
  __builtin_amdgcn_sched_barrier(0);
  const T* h = static_cast<const T*>(g.h);
  T* dh = static_cast<T*>(g.c);
  T* ys = static_cast<T*>(g.preact);
  const int lr = lane >> 3, lc = lane & 7;
  int64_t col = n0 + wn0 + lc * 8;
  const bool col_ok = col < g.N;   // N is a multiple of 8: a lane's eight columns are all in or out
  col = col_ok ? col : g.N - 8;
  constexpr int STEPS = MB16 * 2;  // 8 rows a step
  constexpr int CH = 8;            // steps whose h values are in flight together
#pragma unroll
  for (int c0 = 0; c0 < STEPS; c0 += CH) {
    uint4 ha[CH], hb[CH];
    float sv[CH];
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int p = row0 + wm0 + (c0 + i) * 8 + lr;
      const int pc = p < end ? p : end - 1;
      const T* hp = h + static_cast<int64_t>(pc) * g.ldh + 2 * col;
      ha[i] = *reinterpret_cast<const uint4*>(hp);
      hb[i] = *reinterpret_cast<const uint4*>(hp + 8);
      sv[i] = g.scales != nullptr ? to_f32(static_cast<const T*>(g.scales)[pc]) : 1.0f;
    }
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int r = (c0 + i) * 8 + lr;
      const int p = row0 + wm0 + r;
      const char* src = region + r * PITCH + lc * 16;
      uint2 gv[2] = {*reinterpret_cast<const uint2*>(src), *reinterpret_cast<const uint2*>(src + 8)};
      const T* gp = reinterpret_cast<const T*>(gv);
      uint4 hh[2] = {ha[i], hb[i]};
      const T* hp = reinterpret_cast<const T*>(hh);
      const float s = sv[i];
      T dv[16], yt[8];
      float dot = 0.0f;
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        const float G = to_f32(gp[v]);
        const float gate = to_f32(hp[2 * v]), up = to_f32(hp[2 * v + 1]);
        const float a = apply_act<ACT>(gate);
        const float y = a * up;
        dv[2 * v] = from_f32<T>(s * G * up * apply_act_grad<ACT>(gate));
        dv[2 * v + 1] = from_f32<T>(s * G * a);
        yt[v] = from_f32<T>(s * y);
        dot += G * y;
      }
      if (p < end && col_ok) {
        T* dp = dh + static_cast<int64_t>(p) * g.ldc + 2 * col;
        *reinterpret_cast<uint4*>(dp) = *reinterpret_cast<const uint4*>(dv);
        *reinterpret_cast<uint4*>(dp + 8) = *reinterpret_cast<const uint4*>(dv + 8);
        *reinterpret_cast<uint4*>(ys + static_cast<int64_t>(p) * g.ld_preact + col) =
            *reinterpret_cast<const uint4*>(yt);
      }
      if (g.dscale != nullptr) {
        if (!col_ok) dot = 0.0f;
        dot += __shfl_xor(dot, 1, 64);
        dot += __shfl_xor(dot, 2, 64);
        dot += __shfl_xor(dot, 4, 64);
        if (lc == 0 && p < end) unsafeAtomicAdd(g.dscale + p, dot);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

}  // namespace mfma
}  // namespace moe
