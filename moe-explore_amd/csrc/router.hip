// Fused router: logits = x @ W_r, fp32 softmax, top-k selection, renormalisation and
// the cast of the scores, in one pass over x (reference router.py:17-35 topk_router and
// :37-54 ernie_router, which run a matmul, a softmax, a top-k, a gather, a sum, a
// division and a cast as separate kernels), plus the gradient of the scores with
// respect to the logits for the backward pass.
//
// The logits GEMM is skinny (N = number of experts) and bound by reading x once, so the
// kernel is organised around memory-level parallelism rather than MFMA occupancy:
//   * a workgroup owns 32 tokens; its wavefronts split K, and every wavefront streams
//     its K slice of the 32 token rows straight from global memory into MFMA operand
//     registers (lane = token row, 16 bytes of K), several K steps in flight;
//   * the router weight is first transposed into a K-contiguous copy in the caller's
//     workspace (a few hundred KiB at most, L2 resident), so the weight operand is
//     loaded the same way and the K loop has neither LDS traffic nor barriers;
//   * the partial logits of the wavefronts are added in LDS in a fixed order
//     (deterministic sums), then eight lanes per token run softmax and top-k.
// 16-bit inputs use v_mfma_f32_32x32x16 (bf16 / f16); fp32 weights (the Ernie router
// and fp32 layers) use v_mfma_f32_32x32x2_f32 on fp32 operands.
#include "common.h"

#include <type_traits>

namespace moe {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kBlock = 32;    // tokens per MFMA row block; a workgroup owns MBW of them
constexpr int kLpt = 8;       // lanes per token in the selection phase
constexpr int kMaxTopk = 16;
constexpr int kChunk = 256;       // experts a wavefront accumulates (8 blocks of 32)
constexpr int kMaxExperts = 512;   // two chunks, handled by different wavefronts (with four the
                                   // selection phase, 8 lanes a token, takes longer than ATen's kernels)

struct RouterArgs {
  const void* x;
  int64_t ldx;
  const void* wt;      // transposed weight [E][dpad] in the compute type, zero past d
  int64_t dpad;
  const float* bias;   // Ernie: added to the probabilities for selection only
  void* scores;        // [T, topk] in the dtype of x
  int64_t* idx;        // [T, topk]
  float* logits_out;   // [T, E] or NULL
  int64_t T, d;
  int E, topk, flags;
};

// ---- weight transpose ----------------------------------------------------------
// wt[e][k] = w[k][e] converted to CT, zero for d <= k < dpad.
template <typename TW, typename CT>
__global__ __launch_bounds__(256) void router_transpose_kernel(const TW* __restrict__ w,
                                                               int64_t ldw_k, int64_t ldw_e,
                                                               CT* __restrict__ wt, int64_t d,
                                                               int64_t dpad, int E) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  const int64_t k0 = static_cast<int64_t>(blockIdx.x) * 32;
  const int e0 = blockIdx.y * 32;
  for (int r = ty; r < 32; r += 8) {  // read: rows k, columns e
    const int64_t k = k0 + r;
    const int e = e0 + tx;
    tile[r][tx] = (k < d && e < E) ? to_f32(w[k * ldw_k + e * ldw_e]) : 0.0f;
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) {  // write: rows e, columns k
    const int e = e0 + r;
    const int64_t k = k0 + tx;
    if (e < E && k < dpad) wt[static_cast<int64_t>(e) * dpad + k] = from_f32<CT>(tile[tx][r]);
  }
}

// ---- fused forward ---------------------------------------------------------------
template <typename TX>
__device__ __forceinline__ f32x16 mfma16(uint4 a, uint4 b, f32x16 acc) {
  if constexpr (__is_same(TX, bf16_t))
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}

// Four consecutive elements of x as fp32 (fp32 compute path).
template <typename TX>
__device__ __forceinline__ float4 load4_as_f32(const TX* p) {
  if constexpr (sizeof(TX) == 4) {
    return *reinterpret_cast<const float4*>(p);
  } else {
    const uint2 raw = *reinterpret_cast<const uint2*>(p);
    const TX* h = reinterpret_cast<const TX*>(&raw);
    return make_float4(to_f32(h[0]), to_f32(h[1]), to_f32(h[2]), to_f32(h[3]));
  }
}

// F32: operands and MFMA in fp32 (wt is float); otherwise wt has the type of x.
// NB: 32-expert blocks a wavefront accumulates.  EC: chunks of NB * 32 experts; with more
// than one, wavefront w works on chunk w % EC and the wavefronts of a chunk split K (more
// than 256 experts: NB = 8, EC = 2).  MBW: 32-token blocks of a workgroup (every weight
// fragment is used MBW times; 2 for 129-256 experts and many tokens, else 1).  U: K steps whose loads are issued
// together.  LPT: lanes that share a token in the selection phase (8, or 16 with eight
// wavefronts and more than 64 experts, where the selection is most of the kernel).  Dynamic LDS: the logits of the workgroup's tokens, kBlock * MBW * (EC * NB * 32 + 1)
// floats.
template <typename TX, bool F32, int NB, int MBW, int U, int EC = 1, int LPT = kLpt>
__global__ __launch_bounds__(512) void router_fwd_kernel(RouterArgs g) {
  constexpr int KSTEP = F32 ? 8 : 16;  // K consumed per step: a 16-byte load per lane and operand
  constexpr int EP = EC * NB * 32;
  constexpr int PITCH = EP + 1;
  constexpr int kTokens = kBlock * MBW;
  extern __shared__ float logits[];
  __shared__ int sel_s[kBlock][kMaxTopk];  // per token of the block being selected
  __shared__ float val_s[kBlock][kMaxTopk];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nwaves = (blockDim.x >> 6) / EC;  // wavefronts that split K for one chunk of experts
  const int chunk = EC == 1 ? 0 : wave % EC;
  const int kwave = EC == 1 ? wave : wave / EC;
  const int l32 = lane & 31, lhi = lane >> 5;
  const int64_t t0 = static_cast<int64_t>(blockIdx.x) * kTokens;

  f32x16 acc[MBW][NB];
#pragma unroll
  for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.0f;

  // K steps [s_begin, s_end) of this wavefront
  const int steps = static_cast<int>(g.dpad / KSTEP);
  const int per_wave = (steps + nwaves - 1) / nwaves;
  const int s_begin = kwave * per_wave;
  const int s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;

  const TX* xrow[MBW];
#pragma unroll
  for (int mb = 0; mb < MBW; ++mb) {
    int64_t trow = t0 + mb * kBlock + l32;
    trow = trow < g.T ? trow : g.T - 1;
    xrow[mb] = static_cast<const TX*>(g.x) + trow * g.ldx;
  }
  using CT = typename std::conditional<F32, float, TX>::type;
  const CT* wrow[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    int e = chunk * (NB * 32) + nb * 32 + l32;
    e = e < g.E ? e : g.E - 1;
    wrow[nb] = static_cast<const CT*>(g.wt) + static_cast<int64_t>(e) * g.dpad;
  }
  const int koff = (KSTEP / 2) * lhi;  // this lane's half of a K step

  // `GUARD`: the step may reach past d (only the last step of the row can)
  auto run = [&](int s, auto count, auto guard) __attribute__((always_inline)) {
    constexpr int N = decltype(count)::value;
    constexpr bool GUARD = decltype(guard)::value;
    uint4 xa[N][MBW], wb[N][NB];
#pragma unroll
    for (int u = 0; u < N; ++u) {
      const int64_t k = static_cast<int64_t>(s + u) * KSTEP + koff;
#pragma unroll
      for (int mb = 0; mb < MBW; ++mb) {
        if constexpr (F32) {
          float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
          if (!GUARD || k < g.d) v = load4_as_f32<TX>(xrow[mb] + k);
          xa[u][mb] = __builtin_bit_cast(uint4, v);
        } else {
          xa[u][mb] = make_uint4(0, 0, 0, 0);
          if (!GUARD || k < g.d) xa[u][mb] = *reinterpret_cast<const uint4*>(xrow[mb] + k);
        }
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) wb[u][nb] = *reinterpret_cast<const uint4*>(wrow[nb] + k);
    }
#pragma unroll
    for (int u = 0; u < N; ++u) {
#pragma unroll
      for (int mb = 0; mb < MBW; ++mb) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          if constexpr (F32) {
            const float4 a = __builtin_bit_cast(float4, wb[u][nb]);
            const float4 b = __builtin_bit_cast(float4, xa[u][mb]);
            acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc[mb][nb], 0, 0, 0);
            acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc[mb][nb], 0, 0, 0);
            acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc[mb][nb], 0, 0, 0);
            acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc[mb][nb], 0, 0, 0);
          } else {
            acc[mb][nb] = mfma16<TX>(wb[u][nb], xa[u][mb], acc[mb][nb]);
          }
        }
      }
    }
  };
  const int s_whole = static_cast<int>(g.d / KSTEP);  // steps that lie inside the row
  const int s_safe = s_end < s_whole ? s_end : s_whole;
  int s = s_begin;
  for (; s + U <= s_safe; s += U) run(s, std::integral_constant<int, U>{}, std::false_type{});
  for (; s < s_safe; ++s) run(s, std::integral_constant<int, 1>{}, std::false_type{});
  for (; s < s_end; ++s) run(s, std::integral_constant<int, 1>{}, std::true_type{});

  // ---- add the partial logits of the wavefronts, in wavefront order -----------------
  // accumulator element run*4 + j of block nb: token l32, expert nb*32 + run*8 + lhi*4 + j
  // (the wavefronts of different chunks write different columns)
  for (int w = 0; w < nwaves; ++w) {
    if (kwave == w) {
#pragma unroll
      for (int mb = 0; mb < MBW; ++mb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float* p = &logits[(mb * kBlock + l32) * PITCH + chunk * (NB * 32) + nb * 32 + r * 8 + lhi * 4 + j];
              *p = (w == 0 ? 0.0f : *p) + acc[mb][nb][r * 4 + j];
            }
    }
    __syncthreads();
  }

  // ---- softmax, top-k, renormalisation: LPT lanes per token ---------------------------
  if (tid >= kBlock * LPT) return;
  const int q = tid % LPT;
#pragma unroll 1
  for (int mb = 0; mb < MBW; ++mb) {
  const int tt = mb * kBlock + tid / LPT;
  const int64_t t = t0 + tt;
  float* row = &logits[tt * PITCH];
  const int E = g.E, topk = g.topk;
  const bool ernie = g.flags & MOE_ROUTER_ERNIE;
  const bool softmax_first = ernie || (g.flags & MOE_ROUTER_SOFTMAX_FIRST);
  const bool normalize = ernie || (g.flags & MOE_ROUTER_NORMALIZE);

  auto group_max = [&](float v) __attribute__((always_inline)) {
#pragma unroll
    for (int o = 1; o < LPT; o <<= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
  };
  auto group_sum = [&](float v) __attribute__((always_inline)) {
#pragma unroll
    for (int o = 1; o < LPT; o <<= 1) v += __shfl_xor(v, o, 64);
    return v;
  };

  int* sel = sel_s[tid / LPT];
  float* val = val_s[tid / LPT];
  constexpr int EL = EP / LPT;  // experts a lane
  if constexpr (EL <= 16) {
    // A lane keeps its experts' values in registers: the rounds of the top-k then compare
    // registers (a scan through LDS with a test and a read per expert and round was most of
    // the kernel from 64 experts on).
    // the reference's logits are a matmul result in the dtype of x (router.py:22); the
    // Ernie router keeps them in fp32 (:44)
    float p[EL], key[EL];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < EL; ++i) {
      const int e = q + LPT * i;
      float v = -INFINITY;
      if (e < E) {
        v = row[e];
        if (!ernie && sizeof(TX) == 2) v = to_f32(from_f32<TX>(v));
        if (g.logits_out != nullptr && t < g.T) g.logits_out[t * E + e] = v;
      }
      p[i] = v;
      mx = fmaxf(mx, v);
    }
    mx = group_max(mx);
    if (softmax_first) {
      float z = 0.0f;
#pragma unroll
      for (int i = 0; i < EL; ++i) {
        p[i] = q + LPT * i < E ? expf(p[i] - mx) : 0.0f;
        z += p[i];
      }
      z = group_sum(z);
#pragma unroll
      for (int i = 0; i < EL; ++i) p[i] = p[i] / z;
    }
    // selection keys, and a bit per expert of this lane that can still win: set for the experts
    // below E, cleared when one is taken (a key itself may be -inf: a masked logit with the
    // top-k first; it is then chosen after every finite one, lowest id first, as torch.topk does)
    uint32_t open = 0;
#pragma unroll
    for (int i = 0; i < EL; ++i) {
      const int e = q + LPT * i;
      key[i] = e < E ? (ernie ? p[i] + g.bias[e] : p[i]) : -INFINITY;
      open |= e < E ? (1u << i) : 0u;
    }
    // top-k: each round, every lane offers its best remaining expert (ties: lowest id)
#pragma unroll 1
    for (int j = 0; j < topk; ++j) {
      float best = -INFINITY, best_v = 0.0f;
      int best_e = -1;
#pragma unroll
      for (int i = 0; i < EL; ++i) {
        const bool take = ((open >> i) & 1u) && (best_e < 0 || key[i] > best);
        best_v = take ? p[i] : best_v;
        best_e = take ? q + LPT * i : best_e;
        best = take ? key[i] : best;
      }
#pragma unroll
      for (int o = 1; o < LPT; o <<= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const float ov = __shfl_xor(best_v, o, 64);
        const int oe = __shfl_xor(best_e, o, 64);
        const bool take = oe >= 0 && (best_e < 0 || ob > best || (ob == best && oe < best_e));
        best = take ? ob : best;
        best_v = take ? ov : best_v;
        best_e = take ? oe : best_e;
      }
      best_e = best_e < 0 ? 0 : best_e;  // only if topk > E, which the entry point rejects
#pragma unroll
      for (int i = 0; i < EL; ++i) open &= best_e == q + LPT * i ? ~(1u << i) : ~0u;
      if (q == 0) {
        sel[j] = best_e;
        val[j] = best_v;
      }
    }
  } else {
    // the reference's logits are a matmul result in the dtype of x (router.py:22); the
    // Ernie router keeps them in fp32 (:44)
    float mx = -INFINITY;
    for (int e = q; e < E; e += LPT) {
      float v = row[e];
      if (!ernie && sizeof(TX) == 2) v = to_f32(from_f32<TX>(v));
      row[e] = v;
      if (g.logits_out != nullptr && t < g.T) g.logits_out[t * E + e] = v;
      mx = fmaxf(mx, v);
    }
    mx = group_max(mx);
    if (softmax_first) {
      float z = 0.0f;
      for (int e = q; e < E; e += LPT) {
        const float p = expf(row[e] - mx);
        row[e] = p;
        z += p;
      }
      z = group_sum(z);
      for (int e = q; e < E; e += LPT) row[e] = row[e] / z;
    }

    // top-k: each round, every lane offers its best remaining expert (ties: lowest id)
    constexpr int TW = (EP + 32 * LPT - 1) / (32 * LPT);
    uint32_t taken[TW];  // word c, bit b: expert q + LPT * (32 c + b)
#pragma unroll
    for (int c = 0; c < TW; ++c) taken[c] = 0;
#pragma unroll 1
    for (int j = 0; j < topk; ++j) {
      float best = 0.0f;
      int best_e = -1;
#pragma unroll
      for (int c = 0; c < TW; ++c) {
        const uint32_t tk = taken[c];
#pragma unroll 1
        for (int b = 0, e = q + LPT * 32 * c; b < 32 && e < E; ++b, e += LPT) {
          if (tk & (1u << b)) continue;
          const float key = ernie ? row[e] + g.bias[e] : row[e];
          if (best_e < 0 || key > best) {
            best = key;
            best_e = e;
          }
        }
      }
#pragma unroll
      for (int o = 1; o < LPT; o <<= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const int oe = __shfl_xor(best_e, o, 64);
        const bool take = oe >= 0 && (best_e < 0 || ob > best || (ob == best && oe < best_e));
        best = take ? ob : best;
        best_e = take ? oe : best_e;
      }
      best_e = best_e < 0 ? 0 : best_e;  // only if topk > E, which the entry point rejects
      if (best_e % LPT == q) {
        const int i = best_e / LPT;
#pragma unroll
        for (int c = 0; c < TW; ++c)
          if ((i >> 5) == c) taken[c] |= 1u << (i & 31);
      }
      if (q == 0) {
        sel[j] = best_e;
        val[j] = row[best_e];
      }
    }
  }
  // (the lanes of a token sit in one wavefront: LDS writes above are visible below)
  float scale = 1.0f, shift = 0.0f;
  if (!softmax_first) {  // softmax over the selected logits (router.py:28-29)
    float m2 = -INFINITY, z = 0.0f;
#pragma unroll 1
    for (int j = 0; j < topk; ++j) m2 = fmaxf(m2, val[j]);
#pragma unroll 1
    for (int j = 0; j < topk; ++j) z += expf(val[j] - m2);
    shift = m2;
    scale = z;
  }
  auto score = [&](int j) __attribute__((always_inline)) {
    return softmax_first ? val[j] : expf(val[j] - shift) / scale;
  };
  float sum = 1.0f;
  if (normalize) {
    sum = 0.0f;
#pragma unroll 1
    for (int j = 0; j < topk; ++j) sum += score(j);
    if (ernie) sum = fmaxf(sum, 1e-12f);  // router.py:52
  }
  if (t < g.T) {
    TX* so = static_cast<TX*>(g.scores) + t * topk;
    int64_t* io = g.idx + t * topk;
#pragma unroll 1
    for (int j = q; j < topk; j += LPT) {
      const float v = normalize ? score(j) / sum : score(j);
      so[j] = from_f32<TX>(v);
      io[j] = sel[j];
    }
  }
  }  // token blocks
}

// ---- gradient of the scores with respect to the logits ------------------------------
// One wavefront handles 8 tokens, 8 lanes each.  TG: dtype of dscores; TO: of dlogits.
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void router_bwd_kernel(const float* __restrict__ logits,
                                                         const int64_t* __restrict__ idx,
                                                         const TG* __restrict__ dscores,
                                                         TO* __restrict__ dlogits, int64_t T, int E,
                                                         int topk, int flags) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * (256 / kLpt) + threadIdx.x / kLpt;
  const int q = threadIdx.x % kLpt;
  if (t >= T) return;  // whole groups of kLpt lanes leave together
  const bool ernie = flags & MOE_ROUTER_ERNIE;
  const bool softmax_first = ernie || (flags & MOE_ROUTER_SOFTMAX_FIRST);
  const bool normalize = ernie || (flags & MOE_ROUTER_NORMALIZE);
  const float* row = logits + t * E;
  auto group_sum = [&](float v) __attribute__((always_inline)) {
#pragma unroll
    for (int o = 1; o < kLpt; o <<= 1) v += __shfl_xor(v, o, 64);
    return v;
  };
  auto group_max = [&](float v) __attribute__((always_inline)) {
#pragma unroll
    for (int o = 1; o < kLpt; o <<= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
  };
  // every lane holds the topk selected entries (topk <= 16)
  int sel[kMaxTopk];
  float raw[kMaxTopk], gs[kMaxTopk];
  float mx = -INFINITY, z = 1.0f;
  if (softmax_first) {
    for (int e = q; e < E; e += kLpt) mx = fmaxf(mx, row[e]);
    mx = group_max(mx);
    z = 0.0f;
    for (int e = q; e < E; e += kLpt) z += expf(row[e] - mx);
    z = group_sum(z);
  }
#pragma unroll
  for (int j = 0; j < kMaxTopk; ++j) {
    sel[j] = -1;
    raw[j] = 0.0f;
    gs[j] = 0.0f;
    if (j < topk) {
      int e = static_cast<int>(idx[t * topk + j]);
      e = e < 0 ? 0 : (e >= E ? E - 1 : e);
      sel[j] = e;
      gs[j] = to_f32(dscores[t * topk + j]);
      raw[j] = softmax_first ? expf(row[e] - mx) / z : row[e];
    }
  }
  if (!softmax_first) {  // raw = softmax over the selected logits
    float m2 = -INFINITY, z2 = 0.0f;
#pragma unroll
    for (int j = 0; j < kMaxTopk; ++j)
      if (j < topk) m2 = fmaxf(m2, raw[j]);
#pragma unroll
    for (int j = 0; j < kMaxTopk; ++j)
      if (j < topk) {
        raw[j] = expf(raw[j] - m2);
        z2 += raw[j];
      }
#pragma unroll
    for (int j = 0; j < kMaxTopk; ++j) raw[j] = raw[j] / z2;
  }
  // through the renormalisation: out_j = raw_j / S  ->  draw_j = (g_j - sum_l g_l out_l) / S
  if (normalize) {
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < kMaxTopk; ++j) sum += raw[j];
    const bool clamped = ernie && sum < 1e-12f;
    const float S = clamped ? 1e-12f : sum;
    float dot = 0.0f;
#pragma unroll
    for (int j = 0; j < kMaxTopk; ++j) dot += gs[j] * raw[j] / S;
    if (clamped) dot = 0.0f;  // the clamp passes no gradient to the sum
#pragma unroll
    for (int j = 0; j < kMaxTopk; ++j) gs[j] = (gs[j] - dot) / S;
  }
  // through the softmax: dlogit_e = y_e (dy_e - sum_l dy_l y_l), y the softmax output
  float c = 0.0f;
#pragma unroll
  for (int j = 0; j < kMaxTopk; ++j) c += gs[j] * raw[j];
  TO* out = dlogits + t * E;
  if (softmax_first) {
#pragma unroll 1
    for (int e = q; e < E; e += kLpt) {
      const float p = expf(row[e] - mx) / z;
      float dy = 0.0f;
#pragma unroll
      for (int j = 0; j < kMaxTopk; ++j) dy += sel[j] == e ? gs[j] : 0.0f;
      out[e] = from_f32<TO>(p * (dy - c));
    }
  } else {
#pragma unroll 1
    for (int e = q; e < E; e += kLpt) {
      float v = 0.0f;
#pragma unroll
      for (int j = 0; j < kMaxTopk; ++j) v += sel[j] == e ? raw[j] * (gs[j] - c) : 0.0f;
      out[e] = from_f32<TO>(v);
    }
  }
}

// The same gradient for up to 8 * EL experts (EL = 8 or 16), softmax before the top-k: a lane keeps its
// EL logits and then its probabilities in registers (the general kernel reads the row three times and
// calls expf three times an element), and the gradients of the selected scores reach their experts
// through a row of LDS instead of a compare per (element, selected entry).
template <typename TG, typename TO, int EL>
__global__ __launch_bounds__(256) void router_bwd_small_kernel(const float* __restrict__ logits,
                                                               const int64_t* __restrict__ idx,
                                                               const TG* __restrict__ dscores,
                                                               TO* __restrict__ dlogits, int64_t T, int E,
                                                               int topk, int flags) {
  constexpr int TB = 256 / kLpt;  // tokens a workgroup
  __shared__ float dy_s[TB][EL * kLpt + 1];
  const int tt = threadIdx.x / kLpt, q = threadIdx.x % kLpt;
  const int64_t t = static_cast<int64_t>(blockIdx.x) * TB + tt;
  if (t >= T) return;  // whole groups of kLpt lanes leave together; no workgroup barrier below
  const bool ernie = flags & MOE_ROUTER_ERNIE;
  const bool normalize = ernie || (flags & MOE_ROUTER_NORMALIZE);
  const float* row = logits + t * E;
  auto group_sum = [&](float v) __attribute__((always_inline)) {
#pragma unroll
    for (int o = 1; o < kLpt; o <<= 1) v += __shfl_xor(v, o, 64);
    return v;
  };
  auto group_max = [&](float v) __attribute__((always_inline)) {
#pragma unroll
    for (int o = 1; o < kLpt; o <<= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
  };
  float p[EL];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < EL; ++i) {
    const int e = q + kLpt * i;
    p[i] = e < E ? row[e] : -INFINITY;
    mx = fmaxf(mx, p[i]);
    dy_s[tt][e] = 0.0f;
  }
  mx = group_max(mx);
  float z = 0.0f;
#pragma unroll
  for (int i = 0; i < EL; ++i) {
    p[i] = q + kLpt * i < E ? expf(p[i] - mx) : 0.0f;
    z += p[i];
  }
  z = group_sum(z);
  const float rz = 1.0f / z;
#pragma unroll
  for (int i = 0; i < EL; ++i) p[i] *= rz;
  // selected entries: lane q holds entries q and q + kLpt (topk <= 16)
  int sel[2];
  float raw[2], gs[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int j = q + kLpt * h;
    sel[h] = -1;
    raw[h] = 0.0f;
    gs[h] = 0.0f;
    if (j < topk) {
      int e = static_cast<int>(idx[t * topk + j]);
      e = e < 0 ? 0 : (e >= E ? E - 1 : e);
      sel[h] = e;
      gs[h] = to_f32(dscores[t * topk + j]);
      raw[h] = expf(row[e] - mx) * rz;
    }
  }
  // through the renormalisation: out_j = raw_j / S  ->  draw_j = (g_j - sum_l g_l out_l) / S
  if (normalize) {
    const float sum = group_sum(raw[0] + raw[1]);
    const bool clamped = ernie && sum < 1e-12f;
    const float S = clamped ? 1e-12f : sum;
    float dot = group_sum((gs[0] * raw[0] + gs[1] * raw[1]) / S);
    if (clamped) dot = 0.0f;  // the clamp passes no gradient to the sum
    gs[0] = sel[0] >= 0 ? (gs[0] - dot) / S : 0.0f;
    gs[1] = sel[1] >= 0 ? (gs[1] - dot) / S : 0.0f;
  }
  // through the softmax: dlogit_e = y_e (dy_e - sum_l dy_l y_l), y the softmax output
  const float c = group_sum(gs[0] * raw[0] + gs[1] * raw[1]);
  // (the lanes of a token sit in one wavefront: the zeros above are in place; the selected
  // experts of a token are distinct)
  if (sel[0] >= 0) dy_s[tt][sel[0]] = gs[0];
  if (sel[1] >= 0) dy_s[tt][sel[1]] = gs[1];
  TO* out = dlogits + t * E;
#pragma unroll
  for (int i = 0; i < EL; ++i) {
    const int e = q + kLpt * i;
    if (e < E) out[e] = from_f32<TO>(p[i] * (dy_s[tt][e] - c));
  }
}

int64_t padded_k(int64_t d, bool f32) {
  const int64_t step = f32 ? 8 : 16;
  return (d + step - 1) / step * step;
}

template <typename TX, bool F32>
int launch_fwd(const RouterArgs& g, hipStream_t stream) {
  // One 32-token block per workgroup: more blocks would reuse every weight fragment
  // (read from L2) but leave fewer wavefronts to keep loads in flight, and measured
  // 40-70 % slower at 8192-16384 tokens.  Eight wavefronts split K unless there are
  // workgroups in plenty.
  const int nb = (g.E + 31) / 32;
  const int64_t wgs = (g.T + kBlock - 1) / kBlock;
  const dim3 grid(static_cast<unsigned>(wgs));
  const dim3 block(64 * (wgs >= 2048 && g.E <= kChunk ? 4 : 8));
  auto lds_bytes = [](int experts) { return static_cast<size_t>(kBlock) * (experts + 1) * sizeof(float); };
  if (nb <= 1) router_fwd_kernel<TX, F32, 1, 1, 16><<<grid, block, lds_bytes(32), stream>>>(g);
  else if (nb <= 2) router_fwd_kernel<TX, F32, 2, 1, 8><<<grid, block, lds_bytes(64), stream>>>(g);
  else if (nb <= 4 && block.x == 512 && wgs > num_cus()) {
    // 65-128 experts, more than one round of 32-token workgroups (and fewer than the 2048 from
    // which four wavefronts a workgroup do better): 64 tokens a workgroup, every weight fragment
    // serving two token blocks (E = 128, d = 2048: T = 16384 88 -> 70 us, T = 32000 166 -> 133 us)
    const dim3 grid2(static_cast<unsigned>((g.T + 2 * kBlock - 1) / (2 * kBlock)));
    router_fwd_kernel<TX, F32, 4, 2, 4, 1, 16><<<grid2, block, 2 * lds_bytes(128), stream>>>(g);
  }
  else if (nb <= 4 && block.x == 512) router_fwd_kernel<TX, F32, 4, 1, 4, 1, 16><<<grid, block, lds_bytes(128), stream>>>(g);
  else if (nb <= 4) router_fwd_kernel<TX, F32, 4, 1, 4><<<grid, block, lds_bytes(128), stream>>>(g);
  else if (nb <= 8 && wgs > num_cus()) {
    // 129-256 experts and more 32-token blocks than compute units: 64 tokens a workgroup, two
    // groups of four wavefronts with 128 experts each, so that every weight fragment (the
    // 2 MiB weight is re-read from L2 by every workgroup) serves two token blocks
    // (d = 4096, E = 256: T = 16384 220 -> 167 us, T = 32768 440 -> 335 us; with one round of
    // workgroups or less the 32-token form is faster, 115 against 156 us at T = 8192)
    auto kernel = router_fwd_kernel<TX, F32, 4, 2, 4, 2, 16>;
    const size_t lds = 2 * lds_bytes(256);
    const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds);
    if (rc != MOE_OK) return rc;
    kernel<<<dim3(static_cast<unsigned>((g.T + 2 * kBlock - 1) / (2 * kBlock))), dim3(512), lds, stream>>>(g);
  }
  else if (nb <= 8 && block.x == 512) router_fwd_kernel<TX, F32, 8, 1, 2, 1, 16><<<grid, block, lds_bytes(256), stream>>>(g);
  else if (nb <= 8) router_fwd_kernel<TX, F32, 8, 1, 2><<<grid, block, lds_bytes(256), stream>>>(g);
  else {
    // more than 256 experts: two chunks of 256, eight wavefronts; the logits of the 32
    // tokens need more than the 64 KiB of LDS a kernel gets without asking
    auto launch = [&](auto kernel, int experts) -> int {
      const size_t lds = lds_bytes(experts);
      const int rc = allow_dynamic_lds(reinterpret_cast<const void*>(kernel), lds);
      if (rc != MOE_OK) return rc;
      kernel<<<grid, block, lds, stream>>>(g);
      return MOE_OK;
    };
    const int rc = launch(router_fwd_kernel<TX, F32, 8, 1, 2, 2, 16>, 512);
    if (rc != MOE_OK) return rc;
  }
  return check_launch("router (fused logits, softmax, top-k)");
}

}  // namespace
}  // namespace moe

using namespace moe;

extern "C" {

size_t moe_router_workspace_bytes(int64_t d, int E, int x_dtype, int w_dtype) {
  const bool f32 = x_dtype == MOE_DTYPE_F32 || w_dtype == MOE_DTYPE_F32;
  if (d <= 0 || E <= 0) return 0;
  return static_cast<size_t>(E) * static_cast<size_t>(padded_k(d, f32)) * (f32 ? 4 : 2);
}

int moe_router_topk(const void* x, int64_t ldx, const void* w, int64_t ldw_k, int64_t ldw_e,
                    const float* bias, void* scores, int64_t* topk_indices, float* logits_out,
                    int64_t T, int64_t d, int E, int topk, int flags, int x_dtype, int w_dtype,
                    void* workspace, size_t workspace_bytes, moe_stream_t stream_) {
  clear_error();
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  MOE_REQUIRE(T >= 0 && d > 0 && E > 0, "router: T=%lld d=%lld E=%d", (long long)T, (long long)d, E);
  MOE_REQUIRE(topk >= 1 && topk <= E, "router: topk=%d with %d experts", topk, E);
  MOE_REQUIRE(dtype_bytes(x_dtype) != 0 && dtype_bytes(w_dtype) != 0, "router: unknown dtype");
  MOE_REQUIRE((flags & ~(MOE_ROUTER_SOFTMAX_FIRST | MOE_ROUTER_NORMALIZE | MOE_ROUTER_ERNIE)) == 0,
              "router: unknown flags %d", flags);
  MOE_REQUIRE(!(flags & MOE_ROUTER_ERNIE) || bias != nullptr, "router: the Ernie router needs a bias");
  if (T == 0) return MOE_OK;
  MOE_REQUIRE(x && w && scores && topk_indices && workspace, "router: null pointer");
  const bool f32 = x_dtype == MOE_DTYPE_F32 || w_dtype == MOE_DTYPE_F32;
  if (!f32 && x_dtype != w_dtype)
    return fail(MOE_ERR_UNSUPPORTED, "router: x and the router weight differ in 16-bit dtype");
  if (E > kMaxExperts || topk > kMaxTopk)
    return fail(MOE_ERR_UNSUPPORTED, "router: at most %d experts and top-%d", kMaxExperts, kMaxTopk);
  // 16-byte operand loads (8 bytes for 16-bit x on the fp32 path)
  const int xe = dtype_bytes(x_dtype);
  const int vec = f32 ? 4 : 8;
  if (d % vec != 0 || ldx % vec != 0 || (reinterpret_cast<uintptr_t>(x) % (vec * xe)) != 0)
    return fail(MOE_ERR_UNSUPPORTED, "router: d, the row stride of x and its address must be "
                                     "multiples of %d elements", vec);
  MOE_REQUIRE(ldx >= d, "router: ldx=%lld < d=%lld", (long long)ldx, (long long)d);
  MOE_REQUIRE(aligned16(workspace) && workspace_bytes >= moe_router_workspace_bytes(d, E, x_dtype, w_dtype),
              "router: workspace of %zu bytes, 16-byte aligned, needed", moe_router_workspace_bytes(d, E, x_dtype, w_dtype));

  RouterArgs g;
  g.x = x; g.ldx = ldx; g.wt = workspace; g.dpad = padded_k(d, f32); g.bias = bias;
  g.scores = scores; g.idx = topk_indices; g.logits_out = logits_out;
  g.T = T; g.d = d; g.E = E; g.topk = topk; g.flags = flags;

  const dim3 tgrid(static_cast<unsigned>((g.dpad + 31) / 32), static_cast<unsigned>((E + 31) / 32));
  if (f32) {
    float* wt = static_cast<float*>(workspace);
    MOE_DISPATCH_DTYPE(w_dtype, TW, router_transpose_kernel<TW, float><<<tgrid, 256, 0, stream>>>(
        static_cast<const TW*>(w), ldw_k, ldw_e, wt, d, g.dpad, E));
  } else if (x_dtype == MOE_DTYPE_BF16) {
    router_transpose_kernel<bf16_t, bf16_t><<<tgrid, 256, 0, stream>>>(
        static_cast<const bf16_t*>(w), ldw_k, ldw_e, static_cast<bf16_t*>(workspace), d, g.dpad, E);
  } else {
    router_transpose_kernel<f16_t, f16_t><<<tgrid, 256, 0, stream>>>(
        static_cast<const f16_t*>(w), ldw_k, ldw_e, static_cast<f16_t*>(workspace), d, g.dpad, E);
  }
  int st = check_launch("router (weight transpose)");
  if (st != MOE_OK) return st;

  if (f32) {
    MOE_DISPATCH_DTYPE(x_dtype, TX, return (launch_fwd<TX, true>(g, stream)));
  }
  if (x_dtype == MOE_DTYPE_BF16) return launch_fwd<bf16_t, false>(g, stream);
  return launch_fwd<f16_t, false>(g, stream);
}

int moe_router_bwd(const float* logits, const int64_t* topk_indices, const void* dscores,
                   void* dlogits, int64_t T, int E, int topk, int flags, int g_dtype, int out_dtype,
                   moe_stream_t stream_) {
  clear_error();
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  MOE_REQUIRE(T >= 0 && E > 0 && topk >= 1 && topk <= E, "router_bwd: T=%lld E=%d topk=%d",
              (long long)T, E, topk);
  MOE_REQUIRE((flags & ~(MOE_ROUTER_SOFTMAX_FIRST | MOE_ROUTER_NORMALIZE | MOE_ROUTER_ERNIE)) == 0,
              "router_bwd: unknown flags %d", flags);
  if (topk > kMaxTopk) return fail(MOE_ERR_UNSUPPORTED, "router_bwd: at most top-%d", kMaxTopk);
  if (T == 0) return MOE_OK;
  MOE_REQUIRE(logits && topk_indices && dscores && dlogits, "router_bwd: null pointer");
  const dim3 grid(static_cast<unsigned>((T + 256 / kLpt - 1) / (256 / kLpt)));
  const bool softmax_first = flags & (MOE_ROUTER_ERNIE | MOE_ROUTER_SOFTMAX_FIRST);
  if (softmax_first && E <= 16 * kLpt) {
    MOE_DISPATCH_DTYPE(g_dtype, TG, {
      MOE_DISPATCH_DTYPE(out_dtype, TO, {
        if (E <= 8 * kLpt)
          router_bwd_small_kernel<TG, TO, 8><<<grid, 256, 0, stream>>>(
              logits, topk_indices, static_cast<const TG*>(dscores), static_cast<TO*>(dlogits), T, E, topk, flags);
        else
          router_bwd_small_kernel<TG, TO, 16><<<grid, 256, 0, stream>>>(
              logits, topk_indices, static_cast<const TG*>(dscores), static_cast<TO*>(dlogits), T, E, topk, flags);
      });
    });
    return check_launch("router_bwd");
  }
  MOE_DISPATCH_DTYPE(g_dtype, TG, {
    MOE_DISPATCH_DTYPE(out_dtype, TO, router_bwd_kernel<TG, TO><<<grid, 256, 0, stream>>>(
        logits, topk_indices, static_cast<const TG*>(dscores), static_cast<TO*>(dlogits), T, E, topk,
        flags));
  });
  return check_launch("router_bwd");
}

}  // extern "C"
