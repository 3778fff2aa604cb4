// M-grouped GEMM on gfx950 matrix cores (bf16 / fp16 in, fp32 accumulate).
// Replaces the reference's persistent Triton kernel (m_grouped_gemm.py:33-267):
// same math, same fused row gather on the token load (:104-109), row scatter on
// the store (:168-172) and activation / GLU epilogue (epilogue_split.py:4-44,
// activation.py:24-36), plus the weighted scatter-add combine and the saved
// pre-activation that the backward pass needs.
//
// Shape of the kernel
//   * workgroup = 8 wavefronts (2 along rows x 4 along columns), one BM x 256
//     output tile, K consumed 64 at a time from two LDS stages;
//   * v_mfma_f32_32x32x16 with the operands swapped (weights as the first
//     operand, tokens as the second): a lane then owns one token row and runs
//     of four consecutive output columns, so a gate/up column pair of the
//     interleaved GLU layout sits in one lane and stores are 8-byte vectors;
//   * token tile [BM][64] and K-contiguous weight tile [256][64] are read from
//     LDS with ds_read_b128 under a 16-byte XOR swizzle; an N-contiguous weight
//     tile [64][256] is read with ds_read_b64_tr_b16, the LDS transpose load;
//   * tile -> (expert, row block) is resolved on the device from group_indices
//     by a wavefront scan, so ragged groups need no host synchronisation; the
//     grid is the static bound cdiv(P, BM) + E row blocks;
//   * workgroup ids are dealt round-robin to the 8 XCDs by the hardware; the id
//     is remapped so that each XCD walks blocks of GM x GN neighbouring tiles and
//     re-uses their token / weight panels from its own L2.
#include "gemm_mfma.h"

namespace moe {
namespace {

using namespace mfma;

// WL: 0 = weight N-contiguous (ldw_n == 1), 1 = weight K-contiguous (ldw_k == 1)
template <typename T, int BM, int WL, int ACT>
__global__ __launch_bounds__(kThreads) void m_grouped_mfma_kernel(MGemmArgs g, Sched s) {
  constexpr int WM = BM / WAVES_M;  // token rows per wavefront
  constexpr int MB = WM / 32;       // row blocks per wavefront
  constexpr int A_CHUNKS = BM * 8 / kThreads;  // 16-byte chunks of the token tile per lane
  constexpr int W_CHUNKS = BN * 8 / kThreads;
  constexpr int A_BYTES = BM * BK * 2, W_BYTES = BN * BK * 2;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  __shared__ int sh_tile[4];
  auto a_lds = [&](int stage) { return smem + stage * (A_BYTES + W_BYTES); };
  auto w_lds = [&](int stage) { return smem + stage * (A_BYTES + W_BYTES) + A_BYTES; };

  // ---- which tile -------------------------------------------------------------
  // Workgroup ids id, id+8, id+16.. run on one XCD.  Each XCD is handed whole
  // blocks of GM x GN neighbouring tiles (rows fastest), blocks dealt round-robin
  // over the XCDs, so the tiles in flight on an XCD share token and weight panels
  // in its L2 and the empty tail of the static grid is spread over all XCDs.
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

  // ---- global -> register staging addresses -------------------------------------
  const char* a_ptr[A_CHUNKS];
  int a_off[A_CHUNKS];
  const int a_kc = tid & 7;  // chunk (8 elements) along K
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    const int r = (tid >> 3) + i * (kThreads / 8);
    int p = row0 + r;
    p = p < end ? p : end - 1;  // rows past the group re-read its last row; masked at the store
    int64_t arow = p;
    if (g.flags & MOE_GEMM_GATHER_A) arow = g.by_topk.div(load_index32(g.indices, g.idx_bytes, p));
    arow = clamp_index(arow, g.a_rows);
    a_ptr[i] = static_cast<const char*>(g.a) + (arow * g.lda + a_kc * 8) * 2;
    a_off[i] = kmajor_off(r, a_kc);
  }
  const char* w_ptr[W_CHUNKS];
  int w_off[W_CHUNKS];
  const char* wbase = static_cast<const char*>(g.w) + static_cast<int64_t>(expert) * g.ldw_e * 2;
  int w_kc;  // K offset (elements) of this lane's chunks inside a K step
  if constexpr (WL == 0) {
    const int nc = tid & 31;  // chunk along N
    w_kc = tid >> 5;          // k row, + 16 per chunk
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int k = w_kc + i * (kThreads / 32);
      const int64_t n = n0 + nc * 8;
      w_ptr[i] = wbase + (static_cast<int64_t>(k) * g.ldw_k + (n < g.N ? n : 0)) * 2;
      w_off[i] = nmajor_off(k, nc * 16);
    }
  } else {
    w_kc = (tid & 7) * 8;
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) {
      const int r = (tid >> 3) + i * (kThreads / 8);
      int64_t n = n0 + r;
      n = n < g.N ? n : g.N - 1;
      w_ptr[i] = wbase + (n * g.ldw_n + w_kc) * 2;
      w_off[i] = kmajor_off(r, tid & 7);
    }
  }

  uint4 a_reg[A_CHUNKS], w_reg[W_CHUNKS];

  // Columns past N and rows past the group only feed outputs that are never
  // stored, so their loads are merely kept in bounds.  Only the contraction tail
  // (K not a multiple of 64, last step) must read as zero on both operands: those
  // chunks are loaded from offset 0 of the row and cleared by a value select.
  auto load_global = [&](int64_t k0, auto tail_tag) {
    constexpr bool TAIL = decltype(tail_tag)::value;
    const bool a_in = !TAIL || (k0 + a_kc * 8 < g.K);
    const int64_t a_k = a_in ? k0 * 2 : -static_cast<int64_t>(a_kc) * 16;
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
      uint4 v = *reinterpret_cast<const uint4*>(a_ptr[i] + a_k);
      if (TAIL && !a_in) v = make_uint4(0, 0, 0, 0);
      a_reg[i] = v;
    }
    if constexpr (WL == 0) {
#pragma unroll
      for (int i = 0; i < W_CHUNKS; ++i) {
        const bool in = !TAIL || (k0 + w_kc + i * (kThreads / 32) < g.K);
        const int64_t kk = in ? k0 : -static_cast<int64_t>(w_kc + i * (kThreads / 32));
        uint4 v = *reinterpret_cast<const uint4*>(w_ptr[i] + kk * g.ldw_k * 2);
        if (TAIL && !in) v = make_uint4(0, 0, 0, 0);
        w_reg[i] = v;
      }
    } else {
      const bool w_in = !TAIL || (k0 + w_kc < g.K);
      const int64_t w_k = w_in ? k0 * 2 : -static_cast<int64_t>(w_kc) * 2;
#pragma unroll
      for (int i = 0; i < W_CHUNKS; ++i) {
        uint4 v = *reinterpret_cast<const uint4*>(w_ptr[i] + w_k);
        if (TAIL && !w_in) v = make_uint4(0, 0, 0, 0);
        w_reg[i] = v;
      }
    }
  };
  auto store_lds = [&](int stage) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) *reinterpret_cast<uint4*>(a_lds(stage) + a_off[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < W_CHUNKS; ++i) *reinterpret_cast<uint4*>(w_lds(stage) + w_off[i]) = w_reg[i];
  };

  // ---- LDS -> register fragment addresses ----------------------------------------
  const int l32 = lane & 31, lhi = lane >> 5;
  int t_frag_row[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) t_frag_row[mb] = wm0 + mb * 32 + l32;
  // transpose-load geometry: 16-lane group gq, k row inside the 4-row quad, column quad
  const int tr_g = lane >> 4, tr_i = (lane >> 2) & 3, tr_q = lane & 3;
  const int tr_n = wn0 + 16 * (tr_g & 1) + 4 * tr_q;  // + nb * 32
  const int tr_k = 8 * (tr_g >> 1) + tr_i;            // + kk * 16 (+ 4 for the second half)

  f32x16 acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.0f;

  const int KT = static_cast<int>((g.K + BK - 1) / BK);
  const bool k_tail = (g.K % BK) != 0;
  using no_tail = std::integral_constant<bool, false>;
  using with_tail = std::integral_constant<bool, true>;

  auto compute = [&](int stage) {
    const char* at = a_lds(stage);
    const char* wt = w_lds(stage);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      s16x8 tf[MB], wf[NB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        tf[mb] = *reinterpret_cast<const s16x8*>(at + kmajor_off(t_frag_row[mb], kk * 2 + lhi));
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        if constexpr (WL == 0) {
          const int k = kk * 16 + tr_k;
          const int nbyte = (tr_n + nb * 32) * 2;
          s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (lds_s16x4*)(wt + nmajor_off(k, nbyte)));
          s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (lds_s16x4*)(wt + nmajor_off(k + 4, nbyte)));
          wf[nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
          wf[nb] = *reinterpret_cast<const s16x8*>(
              wt + kmajor_off(wn0 + nb * 32 + l32, kk * 2 + lhi));
        }
      }
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = mfma32<T>(wf[nb], tf[mb], acc[mb][nb]);
    }
  };

  if (KT == 1 && k_tail) load_global(0, with_tail{}); else load_global(0, no_tail{});
  store_lds(0);
  __syncthreads();
  // steady state: the next K step's global loads are in flight while this one is
  // multiplied out of LDS; the last (possibly partial) step is peeled
  for (int kt = 0; kt < KT - 2; ++kt) {
    load_global(static_cast<int64_t>(kt + 1) * BK, no_tail{});
    compute(kt & 1);
    store_lds((kt & 1) ^ 1);
    __syncthreads();
  }
  if (KT >= 2) {
    const int kt = KT - 2;
    if (k_tail) load_global(static_cast<int64_t>(kt + 1) * BK, with_tail{});
    else load_global(static_cast<int64_t>(kt + 1) * BK, no_tail{});
    compute(kt & 1);
    store_lds((kt & 1) ^ 1);
    __syncthreads();
  }
  compute((KT - 1) & 1);

  if (lds_epilogue_ok<T>(g)) {
    __syncthreads();  // the main-loop tiles are dead: the epilogue regions alias them
    store_tile_lds<T, ACT, MB, NB>(g, acc, smem + wave * epi_wave_bytes<NB>(), row0, end, n0, wm0,
                                   wn0, lane);
  } else {
    store_tile<T, ACT, MB>(g, acc, row0, end, n0, wm0, wn0, l32, lhi);
  }
}

template <typename T, int BM, int WL>
int launch_act(const MGemmArgs& g, hipStream_t stream) {
  Sched s = make_sched(g, BM);
  if (s.wgs > 0x7fffffff) return fail(MOE_ERR_UNSUPPORTED, "grid too large");
  const size_t lds = 2 * (BM * BK * 2 + BN * BK * 2);
  const dim3 grid(static_cast<unsigned>(s.wgs));
  MOE_DISPATCH_ACT(g.epilogue, ACT, {
    auto kernel = m_grouped_mfma_kernel<T, BM, WL, ACT>;
    const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds);
    if (rc != MOE_OK) return rc;
    kernel<<<grid, kThreads, lds, stream>>>(g, s);
  });
  return check_launch("m_grouped_gemm (MFMA kernel)");
}

}  // namespace

bool m_grouped_mfma_supported(const MGemmArgs& g) {
  if (g.dtype != MOE_DTYPE_BF16 && g.dtype != MOE_DTYPE_F16) return false;
  if (g.K % 8 != 0 || g.N % 8 != 0 || g.K == 0) return false;
  if (g.lda % 8 != 0 || !aligned16(g.a) || !aligned16(g.w)) return false;
  if (g.ldw_e % 8 != 0) return false;
  const bool nmajor = g.ldw_n == 1 && g.ldw_k % 8 == 0;
  const bool kmajor = g.ldw_k == 1 && g.ldw_n % 8 == 0;
  if (!nmajor && !kmajor) return false;
  // vector stores of 4 (2 after GLU) elements
  const bool glu = act_is_glu(g.epilogue);
  if (g.flags & MOE_GEMM_SCATTER_ADD) {
    if (g.ldc % 2 != 0 || (reinterpret_cast<uintptr_t>(g.c) & 7)) return false;
  } else {
    const int64_t align = glu ? 2 : 4;
    if (g.ldc % align != 0 || (reinterpret_cast<uintptr_t>(g.c) & (2 * align - 1))) return false;
  }
  if ((g.flags & MOE_GEMM_SAVE_PREACT) &&
      (g.ld_preact % 4 != 0 || (reinterpret_cast<uintptr_t>(g.preact) & 7)))
    return false;
  return true;
}

int launch_m_grouped_mfma(const MGemmArgs& g, hipStream_t stream) {
  // whole K steps and an output that can leave through LDS in 16-byte pieces: the kernel
  // that copies global memory straight into LDS (the atomic scatter-add and oddly
  // aligned outputs stay here)
  if (m_grouped_mfma_dma_supported(g)) return launch_m_grouped_mfma_dma(g, stream);
  const bool use_nmajor = g.ldw_n == 1 && g.ldw_k % 8 == 0;
  // rows per expert decide the row-block height: 256 when groups are large
  const int64_t rows_per_expert = g.P / g.E;
  const bool big = rows_per_expert >= 512;
  if (g.dtype == MOE_DTYPE_BF16) {
    if (use_nmajor) return big ? launch_act<bf16_t, 256, 0>(g, stream) : launch_act<bf16_t, 128, 0>(g, stream);
    return big ? launch_act<bf16_t, 256, 1>(g, stream) : launch_act<bf16_t, 128, 1>(g, stream);
  } else {
    if (use_nmajor) return big ? launch_act<f16_t, 256, 0>(g, stream) : launch_act<f16_t, 128, 0>(g, stream);
    return big ? launch_act<f16_t, 256, 1>(g, stream) : launch_act<f16_t, 128, 1>(g, stream);
  }
}

}  // namespace moe

