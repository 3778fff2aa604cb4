// M-grouped GEMM in fp32 on the matrix cores (v_mfma_f32_32x32x2_f32: exact fp32 products,
// fp32 accumulation, 256 FLOP a clock and compute unit).  Same operation and flags as the
// 16-bit kernel of gemm_mfma.hip (reference m_grouped_gemm.py:33-267: fused row gather on the
// token load, row scatter / weighted scatter-add on the store, activation or GLU epilogue
// of epilogue_split.py:4-44, saved pre-activation), for the reference's fp32 runs.
//
// Shape of the kernel
//   * workgroup = 8 wavefronts (2 along rows x 4 along columns), one BM x 256 output tile,
//     K consumed 32 at a time (128-byte rows, as the 16-bit tiles) from two LDS stages that
//     are filled through registers while the stage before is multiplied;
//   * operands swapped as in the 16-bit kernels (weights first, tokens second), so a lane owns
//     one token row and runs of four consecutive columns;
//   * a lane fetches 16 bytes = four k values of its row from a K-contiguous tile and feeds
//     them to four MFMAs; which k a lane half supplies to which MFMA is the same for both
//     operands, which is all the contraction needs;
//   * an N-contiguous weight tile [32][256] is read with four 4-byte loads per column block:
//     the 32 lanes of a half read 128 consecutive bytes, and the two halves (k and k + 4)
//     are kept in different banks by moving every other group of four k rows by 128 bytes.
#include "gemm_mfma.h"

namespace moe {
namespace {

using namespace mfma;

constexpr int BKF = 32;  // K step in elements

// Byte offset of element (k, n) of an N-contiguous tile of COLS columns; nbyte = 4 n.
template <int COLS = BN>
__device__ __forceinline__ int nmajor_f32_off(int k, int nbyte) {
  return k * (COLS * 4) + (nbyte ^ (((k >> 2) & 1) << 7));
}

// v or nothing, component by component (a select between two float4 objects goes through memory)
__device__ __forceinline__ float4 keep_if(bool keep, float4 v) {
  return make_float4(keep ? v.x : 0.0f, keep ? v.y : 0.0f, keep ? v.z : 0.0f, keep ? v.w : 0.0f);
}

template <int ACT, int MB>
__device__ __forceinline__ void store_tile_f32(const MGemmArgs& g, f32x16 (&acc)[MB][NB], int row0,
                                               int end, int64_t n0, int wm0, int wn0, int l32,
                                               int lhi) {
  constexpr bool GLU = act_is_glu(ACT);
  float* c = static_cast<float*>(g.c);
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
      if (g.scales != nullptr) wgt = static_cast<const float*>(g.scales)[clamp_index(slot, g.P)];
    } else {
      crow = clamp_index(slot, g.c_rows);
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int run = 0; run < 4; ++run) {
        const int64_t n = n0 + wn0 + nb * 32 + run * 8 + lhi * 4;
        if (n >= g.N) continue;  // N is a multiple of 4: a run is all in or all out
        float4 v = make_float4(acc[mb][nb][run * 4], acc[mb][nb][run * 4 + 1],
                               acc[mb][nb][run * 4 + 2], acc[mb][nb][run * 4 + 3]);
        if (g.flags & MOE_GEMM_SAVE_PREACT)
          *reinterpret_cast<float4*>(static_cast<float*>(g.preact) +
                                     static_cast<int64_t>(p) * g.ld_preact + n) = v;
        if constexpr (GLU) {
          const float o0 = apply_act<ACT>(v.x) * v.y;
          const float o1 = apply_act<ACT>(v.z) * v.w;
          float* dst = c + crow * g.ldc + n / 2;
          if (g.flags & MOE_GEMM_SCATTER_ADD) {
            unsafeAtomicAdd(dst, wgt * o0);
            unsafeAtomicAdd(dst + 1, wgt * o1);
          } else {
            *reinterpret_cast<float2*>(dst) = make_float2(o0, o1);
          }
        } else {
          v = make_float4(apply_act<ACT>(v.x), apply_act<ACT>(v.y), apply_act<ACT>(v.z),
                          apply_act<ACT>(v.w));
          float* dst = c + crow * g.ldc + n;
          if (g.flags & MOE_GEMM_SCATTER_ADD) {
            unsafeAtomicAdd(dst, wgt * v.x);
            unsafeAtomicAdd(dst + 1, wgt * v.y);
            unsafeAtomicAdd(dst + 2, wgt * v.z);
            unsafeAtomicAdd(dst + 3, wgt * v.w);
          } else {
            *reinterpret_cast<float4*>(dst) = v;
          }
        }
      }
    }
  }
}

// WL: 0 = weight N-contiguous (ldw_n == 1), 1 = weight K-contiguous (ldw_k == 1)
template <int BM, int WL, int ACT>
__global__ __launch_bounds__(kThreads) void m_grouped_f32_kernel(MGemmArgs g, Sched s) {
  constexpr int WM = BM / WAVES_M;
  constexpr int MB = WM / 32;
  constexpr int A_CHUNKS = BM * 8 / kThreads;  // 16-byte chunks of the token tile per lane
  constexpr int W_CHUNKS = BN * 8 / kThreads;
  constexpr int A_BYTES = BM * BKF * 4, W_BYTES = BN * BKF * 4;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  __shared__ int sh_tile[4];
  auto a_lds = [&](int stage) { return smem + stage * (A_BYTES + W_BYTES); };
  auto w_lds = [&](int stage) { return smem + stage * (A_BYTES + W_BYTES) + A_BYTES; };

  // Workgroup ids id, id + 8, .. run on one XCD; each XCD is handed whole blocks of GM x GN
  // neighbouring tiles, so the tiles in flight on it share panels in its L2.
  int mt, nt;
  {
    const int ch = s.GM * s.GN;
    const int id = blockIdx.x;
    const int xcd = id % kNumXcd, j = id / kNumXcd;
    const int blk = (j / ch) * kNumXcd + xcd, within = j % ch;
    const int blk_m = blk / s.nblk_n, blk_n = blk - blk_m * s.nblk_n;
    mt = blk_m * s.GM + within % s.GM;
    nt = blk_n * s.GN + within / s.GM;
    if (nt >= s.NT) return;
  }
  if (threadIdx.x < 64) find_tile<BM>(g.group_indices, g.E, static_cast<int>(g.P), mt, sh_tile);
  __syncthreads();
  const int expert = sh_tile[0];
  if (expert < 0) return;
  const int row0 = sh_tile[1], end = sh_tile[2];
  const int64_t n0 = static_cast<int64_t>(nt) * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;

  // ---- global -> register staging -------------------------------------------------------
  const float* a_ptr[A_CHUNKS];
  int a_off[A_CHUNKS];
  const int a_kc = tid & 7;  // chunk (4 elements) along K
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    const int r = (tid >> 3) + i * (kThreads / 8);
    int p = row0 + r;
    p = p < end ? p : end - 1;  // rows past the group re-read its last row; masked at the store
    int64_t arow = p;
    if (g.flags & MOE_GEMM_GATHER_A) arow = g.by_topk.div(load_index32(g.indices, g.idx_bytes, p));
    arow = clamp_index(arow, g.a_rows);
    a_ptr[i] = static_cast<const float*>(g.a) + arow * g.lda + a_kc * 4;
    a_off[i] = kmajor_off(r, a_kc);
  }
  const float* w_ptr[W_CHUNKS];
  int w_off[W_CHUNKS];
  const float* wbase = static_cast<const float*>(g.w) + static_cast<int64_t>(expert) * g.ldw_e;
  int w_kc;  // K offset (elements) of this lane's first chunk inside a K step
  constexpr int W_KSTEP = kThreads / 64;  // k rows between a lane's chunks (N-contiguous tile)
  if constexpr (WL == 0) {
    const int nc = tid & 63;  // chunk along N
    w_kc = tid >> 6;
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int k = w_kc + i * W_KSTEP;
      const int64_t n = n0 + nc * 4;
      w_ptr[i] = wbase + static_cast<int64_t>(k) * g.ldw_k + (n < g.N ? n : 0);
      w_off[i] = nmajor_f32_off(k, nc * 16);
    }
  } else {
    w_kc = (tid & 7) * 4;
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int r = (tid >> 3) + i * (kThreads / 8);
      int64_t n = n0 + r;
      n = n < g.N ? n : g.N - 1;
      w_ptr[i] = wbase + n * g.ldw_n + w_kc;
      w_off[i] = kmajor_off(r, tid & 7);
    }
  }

  float4 a_reg[A_CHUNKS], w_reg[W_CHUNKS];

  // Columns past N and rows past the group only feed outputs that are never stored, so their
  // loads are merely kept in bounds.  The contraction tail (K not a multiple of 32, last
  // step) must read as zero on both operands: those chunks are loaded from the start of the
  // row and cleared by a value select (K is a multiple of 4: a chunk is all in or all out).
  auto load_global = [&](int64_t k0, auto tail_tag) {
    constexpr bool TAIL = decltype(tail_tag)::value;
    const bool a_in = !TAIL || (k0 + a_kc * 4 < g.K);
    const int64_t a_k = a_in ? k0 : -static_cast<int64_t>(a_kc) * 4;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      float4 v = *reinterpret_cast<const float4*>(a_ptr[i] + a_k);
      a_reg[i] = keep_if(!TAIL || a_in, v);
    }
    if constexpr (WL == 0) {
#pragma unroll
      for (int i = 0; i < W_CHUNKS; ++i) {
        const bool in = !TAIL || (k0 + w_kc + i * W_KSTEP < g.K);
        const int64_t kk = in ? k0 : -static_cast<int64_t>(w_kc + i * W_KSTEP);
        float4 v = *reinterpret_cast<const float4*>(w_ptr[i] + kk * g.ldw_k);
        w_reg[i] = keep_if(!TAIL || in, v);
      }
    } else {
      const bool w_in = !TAIL || (k0 + w_kc < g.K);
      const int64_t w_k = w_in ? k0 : -static_cast<int64_t>(w_kc);
#pragma unroll
      for (int i = 0; i < W_CHUNKS; ++i) {
        float4 v = *reinterpret_cast<const float4*>(w_ptr[i] + w_k);
        w_reg[i] = keep_if(!TAIL || w_in, v);
      }
    }
  };
  auto store_lds = [&](int stage) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) *reinterpret_cast<float4*>(a_lds(stage) + a_off[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) *reinterpret_cast<float4*>(w_lds(stage) + w_off[i]) = w_reg[i];
  };

  const int l32 = lane & 31, lhi = lane >> 5;

  f32x16 acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.0f;

  const int KT = static_cast<int>((g.K + BKF - 1) / BKF);
  const bool k_tail = (g.K % BKF) != 0;
  using no_tail = std::integral_constant<bool, false>;
  using with_tail = std::integral_constant<bool, true>;

  auto compute = [&](int stage) {
    const char* at = a_lds(stage);
    const char* wt = w_lds(stage);
#pragma unroll
    for (int kk = 0; kk < BKF / 8; ++kk) {
      // a lane holds k = 8 kk + 4 lhi + {0..3} of its row / column
      float4 tf[MB], wf[NB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        tf[mb] = *reinterpret_cast<const float4*>(at + kmajor_off(wm0 + mb * 32 + l32, kk * 2 + lhi));
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        if constexpr (WL == 0) {
          const int k = kk * 8 + 4 * lhi;
          const int nbyte = (wn0 + nb * 32 + l32) * 4;
          wf[nb].x = *reinterpret_cast<const float*>(wt + nmajor_f32_off(k, nbyte));
          wf[nb].y = *reinterpret_cast<const float*>(wt + nmajor_f32_off(k + 1, nbyte));
          wf[nb].z = *reinterpret_cast<const float*>(wt + nmajor_f32_off(k + 2, nbyte));
          wf[nb].w = *reinterpret_cast<const float*>(wt + nmajor_f32_off(k + 3, nbyte));
        } else {
          wf[nb] = *reinterpret_cast<const float4*>(wt + kmajor_off(wn0 + nb * 32 + l32, kk * 2 + lhi));
        }
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[nb].x, tf[mb].x, acc[mb][nb], 0, 0, 0);
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[nb].y, tf[mb].y, acc[mb][nb], 0, 0, 0);
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[nb].z, tf[mb].z, acc[mb][nb], 0, 0, 0);
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf[nb].w, tf[mb].w, acc[mb][nb], 0, 0, 0);
        }
    }
  };

  if (KT == 1 && k_tail) load_global(0, with_tail{}); else load_global(0, no_tail{});
  store_lds(0);
  __syncthreads();
  // steady state: the next K step's global loads are in flight while this one is multiplied
  // out of LDS; the last (possibly partial) step is peeled
  for (int kt = 0; kt < KT - 2; ++kt) {
    load_global(static_cast<int64_t>(kt + 1) * BKF, no_tail{});
    compute(kt & 1);
    store_lds((kt & 1) ^ 1);
    __syncthreads();
  }
  if (KT >= 2) {
    const int kt = KT - 2;
    if (k_tail) load_global(static_cast<int64_t>(kt + 1) * BKF, with_tail{});
    else load_global(static_cast<int64_t>(kt + 1) * BKF, no_tail{});
    compute(kt & 1);
    store_lds((kt & 1) ^ 1);
    __syncthreads();
  }
  compute((KT - 1) & 1);

  store_tile_f32<ACT, MB>(g, acc, row0, end, n0, wm0, wn0, l32, lhi);
}

template <int BM, int WL>
int launch_act(const MGemmArgs& g, hipStream_t stream) {
  Sched s = make_sched(g, BM);
  if (s.wgs > 0x7fffffff) return fail(MOE_ERR_UNSUPPORTED, "grid too large");
  const size_t lds = 2 * (BM * BKF * 4 + BN * BKF * 4);
  const dim3 grid(static_cast<unsigned>(s.wgs));
  MOE_DISPATCH_ACT(g.epilogue, ACT, {
    auto kernel = m_grouped_f32_kernel<BM, WL, ACT>;
    const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds);
    if (rc != MOE_OK) return rc;
    kernel<<<grid, kThreads, lds, stream>>>(g, s);
  });
  return check_launch("m_grouped_gemm (fp32 MFMA kernel)");
}


// K-grouped GEMM in fp32 (the weight gradients; reference k_grouped_gemm.py:9-120):
// out[e] = A[rows of e]^T B[rows of e], rows optionally fetched by id.  Both operands are
// contracted over their rows, so both tiles are [32 positions][columns] as they lie in
// memory and are read like the N-contiguous weight tile above.  One workgroup per
// (expert, BA x 256 output tile) walks the expert's positions 32 at a time; B supplies the
// first MFMA operand, so a lane owns one row of out and runs of four consecutive columns.
template <int BA>
__global__ __launch_bounds__(kThreads) void k_grouped_f32_kernel(KGemmArgs g) {
  constexpr int WA = BA / WAVES_M;  // out rows (columns of A) per wavefront
  constexpr int MB = WA / 32;
  constexpr int A_CHUNKS = BA * 8 / kThreads, B_CHUNKS = BN * 8 / kThreads;
  constexpr int A_ROW_CHUNKS = BA / 4;            // 16-byte chunks in a tile row of A
  constexpr int A_KSTEP = kThreads / A_ROW_CHUNKS;  // positions between a lane's chunks
  constexpr int B_KSTEP = kThreads / (BN / 4);
  constexpr int A_BYTES = BKF * BA * 4, B_BYTES = BKF * BN * 4;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  auto a_lds = [&](int stage) { return smem + stage * (A_BYTES + B_BYTES); };
  auto b_lds = [&](int stage) { return smem + stage * (A_BYTES + B_BYTES) + A_BYTES; };

  const int e = blockIdx.z;
  int lo = g.group_indices[e], hi = g.group_indices[e + 1];
  lo = lo < 0 ? 0 : lo;
  hi = hi > g.P ? static_cast<int>(g.P) : hi;
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BA;  // over Ka
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * BN;  // over Nb

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm0 = (wave / WAVES_N) * WA, wn0 = (wave % WAVES_N) * WN;
  const int l32 = lane & 31, lhi = lane >> 5;

  const float* A = static_cast<const float*>(g.a);
  const float* B = static_cast<const float*>(g.b);
  const int a_cc = tid % A_ROW_CHUNKS, a_k = tid / A_ROW_CHUNKS;
  const int b_cc = tid % (BN / 4), b_k = tid / (BN / 4);
  // columns past the matrix only feed outputs that are never stored: kept in bounds
  const int64_t a_col = m0 + a_cc * 4 < g.Ka ? m0 + a_cc * 4 : 0;
  const int64_t b_col = n0 + b_cc * 4 < g.Nb ? n0 + b_cc * 4 : 0;

  float4 a_reg[A_CHUNKS], b_reg[B_CHUNKS];

  // positions past the end of the group must contribute nothing: zero on both operands
  auto row_of = [&](int p, bool gathered, int64_t rows) {
    int64_t r = p;
    if (gathered) r = g.by_topk.div(load_index32(g.indices, g.idx_bytes, p));
    return clamp_index(r, rows);
  };
  auto load_global = [&](int p0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      const int p = p0 + a_k + i * A_KSTEP;
      const bool in = p < hi;
      const int64_t r = row_of(in ? p : lo, g.flags & MOE_KGEMM_GATHER_A, g.a_rows);
      const float4 v = *reinterpret_cast<const float4*>(A + r * g.lda + a_col);
      a_reg[i] = keep_if(in, v);
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
      const int p = p0 + b_k + i * B_KSTEP;
      const bool in = p < hi;
      const int64_t r = row_of(in ? p : lo, g.flags & MOE_KGEMM_GATHER_B, g.b_rows);
      const float4 v = *reinterpret_cast<const float4*>(B + r * g.ldb + b_col);
      b_reg[i] = keep_if(in, v);
    }
  };
  auto store_lds = [&](int stage) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i)
      *reinterpret_cast<float4*>(a_lds(stage) + nmajor_f32_off<BA>(a_k + i * A_KSTEP, a_cc * 16)) = a_reg[i];
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i)
      *reinterpret_cast<float4*>(b_lds(stage) + nmajor_f32_off<BN>(b_k + i * B_KSTEP, b_cc * 16)) = b_reg[i];
  };

  f32x16 acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.0f;

  auto compute = [&](int stage) {
    const char* at = a_lds(stage);
    const char* bt = b_lds(stage);
#pragma unroll
    for (int kk = 0; kk < BKF / 8; ++kk) {
      const int k = kk * 8 + 4 * lhi;  // this lane's four positions
      float af[MB][4], bf[NB][4];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          af[mb][i] = *reinterpret_cast<const float*>(at + nmajor_f32_off<BA>(k + i, (wm0 + mb * 32 + l32) * 4));
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          bf[nb][i] = *reinterpret_cast<const float*>(bt + nmajor_f32_off<BN>(k + i, (wn0 + nb * 32 + l32) * 4));
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[nb][i], af[mb][i], acc[mb][nb], 0, 0, 0);
    }
  };

  const int KT = hi > lo ? (hi - lo + BKF - 1) / BKF : 0;
  if (KT > 0) {
    load_global(lo);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < KT - 1; ++kt) {
      load_global(lo + (kt + 1) * BKF);
      compute(kt & 1);
      store_lds((kt & 1) ^ 1);
      __syncthreads();
    }
    compute((KT - 1) & 1);
  }

  float* out = static_cast<float*>(g.out) + static_cast<int64_t>(e) * g.Ka * g.Nb;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int64_t m = m0 + wm0 + mb * 32 + l32;
    if (m >= g.Ka) continue;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int run = 0; run < 4; ++run) {
        const int64_t n = n0 + wn0 + nb * 32 + run * 8 + lhi * 4;
        if (n >= g.Nb) continue;  // Nb is a multiple of 4
        *reinterpret_cast<float4*>(out + m * g.Nb + n) =
            make_float4(acc[mb][nb][run * 4], acc[mb][nb][run * 4 + 1], acc[mb][nb][run * 4 + 2],
                        acc[mb][nb][run * 4 + 3]);
      }
  }
}

template <int BA>
int launch_k(const KGemmArgs& g, hipStream_t stream) {
  const int64_t ty = (g.Ka + BA - 1) / BA, tx = (g.Nb + BN - 1) / BN;
  if (ty > 65535 || g.E > 65535) return fail(MOE_ERR_UNSUPPORTED, "grid too large");
  const size_t lds = 2 * (BKF * BA * 4 + BKF * BN * 4);
  auto kernel = k_grouped_f32_kernel<BA>;
  const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds);
  if (rc != MOE_OK) return rc;
  const dim3 grid(static_cast<unsigned>(tx), static_cast<unsigned>(ty), static_cast<unsigned>(g.E));
  kernel<<<grid, kThreads, lds, stream>>>(g);
  return check_launch("k_grouped_gemm (fp32 MFMA kernel)");
}

}  // namespace

bool m_grouped_f32_mfma_supported(const MGemmArgs& g) {
  if (g.dtype != MOE_DTYPE_F32 || g.ksplit > 1 || (g.flags & MOE_GEMM_GLU_BWD)) return false;
  if (g.K % 4 != 0 || g.N % 4 != 0 || g.K == 0) return false;
  if (g.lda % 4 != 0 || !aligned16(g.a) || !aligned16(g.w) || g.ldw_e % 4 != 0) return false;
  const bool nmajor = g.ldw_n == 1 && g.ldw_k % 4 == 0;
  const bool kmajor = g.ldw_k == 1 && g.ldw_n % 4 == 0;
  if (!nmajor && !kmajor) return false;
  // 16-byte stores (8 after a GLU); the scatter-add goes through single-word atomics
  if (!(g.flags & MOE_GEMM_SCATTER_ADD)) {
    const int64_t align = act_is_glu(g.epilogue) ? 2 : 4;
    if (g.ldc % align != 0 || (reinterpret_cast<uintptr_t>(g.c) & (4 * align - 1))) return false;
  }
  if ((g.flags & MOE_GEMM_SAVE_PREACT) && (g.ld_preact % 4 != 0 || !aligned16(g.preact))) return false;
  return true;
}

int launch_m_grouped_f32_mfma(const MGemmArgs& g, hipStream_t stream) {
  const bool use_nmajor = g.ldw_n == 1 && g.ldw_k % 4 == 0;
  // 256-row blocks when groups are large, unless 128-row blocks fill the device's rounds of
  // workgroups markedly better (rounds x rows a block is the time of the launch)
  const int64_t nt = (g.N + BN - 1) / BN, cus = num_cus();
  if (cus <= 0) return MOE_ERR_HIP;
  const int64_t cost256 = (((g.P + 255) / 256 + g.E) * nt + cus - 1) / cus * 256;
  const int64_t cost128 = (((g.P + 127) / 128 + g.E) * nt + cus - 1) / cus * 128;
  const bool big = g.P / g.E >= 256 && 10 * cost128 >= 9 * cost256;
  if (use_nmajor) return big ? launch_act<256, 0>(g, stream) : launch_act<128, 0>(g, stream);
  return big ? launch_act<256, 1>(g, stream) : launch_act<128, 1>(g, stream);
}

bool k_grouped_f32_mfma_supported(const KGemmArgs& g) {
  if (g.dtype != MOE_DTYPE_F32) return false;
  if (g.flags & (MOE_KGEMM_A_KMAJOR | MOE_KGEMM_B_KMAJOR)) return false;
  if (g.Ka % 4 != 0 || g.Nb % 4 != 0 || g.lda % 4 != 0 || g.ldb % 4 != 0) return false;
  return aligned16(g.a) && aligned16(g.b) && aligned16(g.out);
}

int launch_k_grouped_f32_mfma(const KGemmArgs& g, hipStream_t stream) {
  // 256 x 256 tiles when they fill the device, else 128 x 256
  const int64_t tiles256 = ((g.Ka + 255) / 256) * ((g.Nb + BN - 1) / BN) * g.E;
  const int cus = num_cus();
  if (cus <= 0) return MOE_ERR_HIP;
  return tiles256 >= cus ? launch_k<256>(g, stream) : launch_k<128>(g, stream);
}

}  // namespace moe
