// fp8 (OCP e4m3) inference variant of the M-grouped GEMM, and the per-row dynamic
// quantiser that feeds it.  The reference has no fp8 path; semantics:
//     scale[r] = max(amax |x[r, :]|, 1e-12) / 448      q[r, :] = e4m3(x[r, :] / scale[r])
//     row = epilogue( (qa[arow] . qw[e][n, :]) * a_scale[arow] * w_scale[e, n] )
// with the weights stored [E, N, K] (K contiguous) and one fp32 scale per output
// channel.
//
// The GEMM kernel is the direct-to-LDS kernel of gemm_mfma_dma.hip with one-byte
// elements: both LDS tiles are K-contiguous rows of 128 bytes (128 fp8 values per
// K step; two token stages, three weight stages), read with ds_read_b128, and multiplied with
// v_mfma_scale_f32_32x32x64_f8f6f4 (unit block scales), the gfx950 instruction
// that runs fp8 at twice the bf16 rate.  Both operands take their K values from
// LDS in the same order, so the product does not depend on how the instruction
// numbers K inside a lane.  The two scales are applied to the fp32 accumulators
// before the shared epilogue (activation / GLU, row scatter, LDS-staged stores).
#include "gemm_mfma.h"

namespace moe {
namespace {

using namespace mfma;

typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr int BKQ = 128;  // fp8 values (= bytes) of K per step

template <typename T>
struct type_tag {
  using type = T;
};

// ---------------------------------------------------------------------------- quantiser
// Generic form: one wavefront per row, two passes over the row (amax, then convert).
template <typename T>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const T* __restrict__ x, int64_t ldx,
                                                            uint8_t* __restrict__ q, int64_t ldq,
                                                            float* __restrict__ scale,
                                                            int64_t rows, int64_t cols) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) >> 6;
  const int64_t waves = static_cast<int64_t>(gridDim.x) * 4;
  for (int64_t r = wave; r < rows; r += waves) {
    const T* row = x + r * ldx;
    float amax = 0.0f;
    for (int64_t c = lane; c < cols; c += 64) amax = fmaxf(amax, fabsf(to_f32(row[c])));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const float s = fmaxf(amax, 1e-12f) / 448.0f;
    if (lane == 0) scale[r] = s;
    uint8_t* qrow = q + r * ldq;
    // four values per lane per step: one packed 32-bit store
    const int64_t cols4 = cols & ~static_cast<int64_t>(3);
    for (int64_t c = lane * 4; c < cols4; c += 256) {
      int w = 0;
      w = __builtin_amdgcn_cvt_pk_fp8_f32(to_f32(row[c]) / s, to_f32(row[c + 1]) / s, w, false);
      w = __builtin_amdgcn_cvt_pk_fp8_f32(to_f32(row[c + 2]) / s, to_f32(row[c + 3]) / s, w, true);
      if ((reinterpret_cast<uintptr_t>(qrow + c) & 3) == 0) {
        *reinterpret_cast<int*>(qrow + c) = w;
      } else {
        for (int j = 0; j < 4; ++j) qrow[c + j] = static_cast<uint8_t>(w >> (8 * j));
      }
    }
    for (int64_t c = cols4 + lane; c < cols; c += 64) {
      int w = __builtin_amdgcn_cvt_pk_fp8_f32(to_f32(row[c]) / s, 0.0f, 0, false);
      qrow[c] = static_cast<uint8_t>(w);
    }
  }
}

// One workgroup per row, the row read ONCE: every lane keeps up to CH 16-byte pieces
// (8 two-byte values each) in registers across the amax reduction, then converts them.
// For two-byte types, cols % 8 == 0 and 16-byte aligned rows (cols <= 2048 * CH).
// Bytes moved per row: 2 * cols read + cols written, against 4 * cols + cols above.
template <typename T, int CH>
__global__ __launch_bounds__(256) void quantize_rows_once_kernel(const T* __restrict__ x,
                                                                 int64_t ldx,
                                                                 uint8_t* __restrict__ q,
                                                                 int64_t ldq,
                                                                 float* __restrict__ scale,
                                                                 int64_t rows, int64_t cols) {
  __shared__ float part[4];
  const int tid = threadIdx.x;
  const int64_t pieces = cols / 8;
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const uint4* row = reinterpret_cast<const uint4*>(x + r * ldx);
    uint4 v[CH];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int64_t pc = tid + 256 * i;
      v[i] = pc < pieces ? row[pc] : make_uint4(0, 0, 0, 0);
      const T* e = reinterpret_cast<const T*>(&v[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(to_f32(e[j])));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if ((tid & 63) == 0) part[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
    __syncthreads();  // part is written again for the next row
    const float s = fmaxf(amax, 1e-12f) / 448.0f;
    if (tid == 0) scale[r] = s;
    uint2* qrow = reinterpret_cast<uint2*>(q + r * ldq);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
      const int64_t pc = tid + 256 * i;
      if (pc >= pieces) continue;
      const T* e = reinterpret_cast<const T*>(&v[i]);
      int w0 = 0, w1 = 0;
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(to_f32(e[0]) / s, to_f32(e[1]) / s, w0, false);
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(to_f32(e[2]) / s, to_f32(e[3]) / s, w0, true);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(to_f32(e[4]) / s, to_f32(e[5]) / s, w1, false);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(to_f32(e[6]) / s, to_f32(e[7]) / s, w1, true);
      qrow[pc] = make_uint2(static_cast<unsigned>(w0), static_cast<unsigned>(w1));
    }
  }
}

// ---------------------------------------------------------------------------- GEMM
struct Fp8Args {
  MGemmArgs g;  // a, w: fp8 bytes; lda, ldw_*: in elements (= bytes); dtype = output type
  const float* a_scale;
  const float* w_scale;
  int w_tiled;  // weights stored as the LDS images of their (column tile, K step) blocks
};

__device__ __forceinline__ void copy16_to_lds(const void* src, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_addr), "v"(src)
               : "memory");
}
__device__ __forceinline__ void wait_copies_and_barrier() {
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// As above, but the YOUNGEST copies of this wavefront (issued last; they complete in
// order) may stay in flight: they fill a stage that is not read before the next barrier.
template <int YOUNGEST>
__device__ __forceinline__ void wait_copies_keep_youngest_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(YOUNGEST) : "memory");
}

template <typename T, int BM, int ACT>
__global__ __launch_bounds__(kThreads) void m_grouped_fp8_kernel(Fp8Args fa, Sched s) {
  MGemmArgs g = fa.g;
  constexpr int WM = BM / WAVES_M;
  constexpr int MB = WM / 32;
  constexpr int A_INSTR = BM / 64, W_INSTR = BN / 64;
  constexpr int A_BYTES = BM * 128, W_BYTES = BN * 128;
  // LDS: two token stages, then three weight stages.  Weights are copied two K steps
  // ahead, tokens one: with few rows per expert the kernel only streams weights, and
  // the bytes a CU keeps in flight bound the HBM bandwidth it can draw.
  constexpr int W_BASE = 2 * A_BYTES;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  // tile descriptor: lives in the third weight stage, which is first written after
  // every wavefront has passed the first barrier of the main loop
  int* const sh_tile = reinterpret_cast<int*>(smem + W_BASE + 2 * W_BYTES);

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
  // a K part of a tile is scheduled like a column tile of its own
  const int real_nt = s.NT / s.ksplit;
  const int kpart = nt / real_nt;
  nt -= kpart * real_nt;
  const int KT = static_cast<int>(g.K / BKQ) / s.ksplit;  // K steps of this part
  const int64_t kt0 = static_cast<int64_t>(kpart) * KT;
  g.c = static_cast<char*>(g.c) + static_cast<int64_t>(kpart) * g.c_split_stride * sizeof(T);
  if (threadIdx.x < 64) find_tile<BM>(g.group_indices, g.E, static_cast<int>(g.P), mt, sh_tile);
  __syncthreads();
  const int expert = sh_tile[0];
  if (expert < 0) return;
  const int row0 = sh_tile[1], end = sh_tile[2];
  const int64_t n0 = static_cast<int64_t>(nt) * BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
  const int l32 = lane & 31, lhi = lane >> 5;

  const char* a_src[A_INSTR];
#pragma unroll
  for (int i = 0; i < A_INSTR; ++i) {
    const int r = 8 * (8 * i + wave) + (lane >> 3);
    const int c = (lane & 7) ^ ((r >> 1) & 7);
    int p = row0 + r;
    p = p < end ? p : end - 1;
    int64_t arow = p;
    if (g.flags & MOE_GEMM_GATHER_A) arow = g.by_topk.div(load_index32(g.indices, g.idx_bytes, p));
    arow = clamp_index(arow, g.a_rows);
    a_src[i] = static_cast<const char*>(g.a) + arow * g.lda + c * 16 + kt0 * BKQ;
  }
  const char* w_src[W_INSTR];
  int64_t w_kstep;  // bytes from one K step to the next
  if (fa.w_tiled) {
    // tile-major weights: the 32 KiB of column tile nt, K step kt are stored contiguously,
    // in the order (and with the swizzle) of the LDS tile, so a step is one linear copy
    // and the whole tile one sequential stream
    const int64_t tile = static_cast<int64_t>(expert) * real_nt + nt;
    const char* wbase = static_cast<const char*>(g.w) + (tile * (g.K / BKQ) + kt0) * W_BYTES;
#pragma unroll
    for (int i = 0; i < W_INSTR; ++i) w_src[i] = wbase + (8 * i + wave) * 1024 + lane * 16;
    w_kstep = W_BYTES;
  } else {
    const char* wbase = static_cast<const char*>(g.w) + static_cast<int64_t>(expert) * g.ldw_e;
#pragma unroll
    for (int i = 0; i < W_INSTR; ++i) {
      const int r = 8 * (8 * i + wave) + (lane >> 3);
      const int c = (lane & 7) ^ ((r >> 1) & 7);
      int64_t n = n0 + r;
      n = n < g.N ? n : g.N - 1;
      w_src[i] = wbase + n * g.ldw_n + c * 16 + kt0 * BKQ;
    }
    w_kstep = BKQ;
  }
  const unsigned lds0 =
      __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<size_t>((lds_void*)smem))) +
      wave * 1024;
  auto issue_token_copies = [&](int stage, int kt) {
    const unsigned base = lds0 + stage * A_BYTES;
#pragma unroll
    for (int i = 0; i < A_INSTR; ++i)
      copy16_to_lds(a_src[i] + static_cast<int64_t>(kt) * BKQ, base + i * 8192);
  };
  auto issue_weight_copies = [&](int wstage, int kt) {
    const unsigned base = lds0 + W_BASE + wstage * W_BYTES;
#pragma unroll
    for (int i = 0; i < W_INSTR; ++i)
      copy16_to_lds(w_src[i] + kt * w_kstep, base + i * 8192);
  };

  // a lane's fragment of a 32-row block for sub-step kk: 32 bytes = chunks 4kk + 2lhi, +1
  auto read32 = [&](const char* tile, int row, int kk) -> i32x8 {
    const i32x4 lo = *reinterpret_cast<const i32x4*>(tile + kmajor_off(row, kk * 4 + lhi * 2));
    const i32x4 hi = *reinterpret_cast<const i32x4*>(tile + kmajor_off(row, kk * 4 + lhi * 2 + 1));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  f32x16 acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.0f;

  // Fragments are 32 bytes per lane and block, so a full second set would not fit
  // in the register file next to the accumulators.  The token fragments roll: once
  // the MFMAs of row block mb are issued, its registers take the fragment of the
  // next sub-step; only the weight fragments (used by every row block) are kept
  // twice.  `next` = false on the very last sub-step.
  i32x8 tf[MB], wfa[NB], wfb[NB];
  auto substep = [&](i32x8 (&wf_cur)[NB], i32x8 (&wf_next)[NB], int next_stage, int next_wstage,
                     int next_kk, auto next_tag) {
    constexpr bool next = decltype(next_tag)::value;
    const char* at = smem + next_stage * A_BYTES;
    const char* wt = smem + W_BASE + next_wstage * W_BYTES;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        acc[mb][nb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
            wf_cur[nb], tf[mb], acc[mb][nb], 0 /* A: e4m3 */, 0 /* B: e4m3 */, 0, 127, 0, 127);
      if constexpr (next) {
        if (mb < NB) wf_next[mb] = read32(wt, wn0 + mb * 32 + l32, next_kk);
        tf[mb] = read32(at, wm0 + mb * 32 + l32, next_kk);
      }
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      __builtin_amdgcn_sched_group_barrier(0x008, NB, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  issue_token_copies(0, 0);
  issue_weight_copies(0, 0);
  if (KT > 1) {
    issue_weight_copies(1, 1);
    wait_copies_keep_youngest_and_barrier<W_INSTR>();
  } else {
    wait_copies_and_barrier();
  }
  {
    const char* at = smem;
    const char* wt = smem + W_BASE;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) wfa[nb] = read32(wt, wn0 + nb * 32 + l32, 0);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) tf[mb] = read32(at, wm0 + mb * 32 + l32, 0);
  }
  using yes = std::integral_constant<bool, true>;
  using no = std::integral_constant<bool, false>;
  int wcur = 0;  // weight stage of step kt: kt % 3
  for (int kt = 0; kt < KT - 1; ++kt) {
    const int stage = kt & 1;
    const int wnext = wcur == 2 ? 0 : wcur + 1;
    const int wahead = wnext == 2 ? 0 : wnext + 1;
    const bool ahead = kt + 2 < KT;
    issue_token_copies(stage ^ 1, kt + 1);
    __builtin_amdgcn_sched_barrier(0);
    substep(wfa, wfb, stage, wcur, 1, yes{});
    if (ahead) issue_weight_copies(wahead, kt + 2);
    // the token copies of step kt+1 and the weight copies of step kt+1 (issued a step
    // earlier) must have landed; the weight copies of step kt+2 may still fly
    if (ahead) wait_copies_keep_youngest_and_barrier<W_INSTR>();
    else wait_copies_and_barrier();
    substep(wfb, wfa, stage ^ 1, wnext, 0, yes{});
    wcur = wnext;
  }
  substep(wfa, wfb, (KT - 1) & 1, wcur, 1, yes{});
  substep(wfb, wfa, 0, 0, 0, no{});

  // ---- dequantise: acc * a_scale[row] * w_scale[e, n] -----------------------------------
  const float* wsc = fa.w_scale + static_cast<int64_t>(expert) * g.N;
  float as[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    int p = row0 + wm0 + mb * 32 + l32;
    p = p < end ? p : end - 1;
    int64_t arow = p;
    if (g.flags & MOE_GEMM_GATHER_A) arow = g.by_topk.div(load_index32(g.indices, g.idx_bytes, p));
    as[mb] = fa.a_scale[clamp_index(arow, g.a_rows)];
  }
  // One run of four channel scales at a time (and a scheduling barrier after it): with all
  // eight float4 loads hoisted next to the 128 accumulators the 256-row kernel spilled 31-40
  // registers a lane to scratch, 80 KiB written and read back per tile.
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int run = 0; run < 4; ++run) {
      int64_t n = n0 + wn0 + nb * 32 + run * 8 + lhi * 4;
      n = n + 3 < g.N ? n : g.N - 4;  // N is a multiple of 8; columns past N are not stored
      const float4 ws = *reinterpret_cast<const float4*>(wsc + n);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        acc[mb][nb][run * 4 + 0] *= as[mb] * ws.x;
        acc[mb][nb][run * 4 + 1] *= as[mb] * ws.y;
        acc[mb][nb][run * 4 + 2] *= as[mb] * ws.z;
        acc[mb][nb][run * 4 + 3] *= as[mb] * ws.w;
      }
      __builtin_amdgcn_sched_barrier(0);
    }

  if (lds_epilogue_ok<T>(g)) {
    __syncthreads();
    store_tile_lds<T, ACT, MB, NB>(g, acc, smem + wave * epi_wave_bytes<NB>(), row0, end, n0, wm0,
                                   wn0, lane);
  } else {
    store_tile<T, ACT, MB>(g, acc, row0, end, n0, wm0, wn0, l32, lhi);
  }
}

template <typename T, int BM>
int launch_fp8(const Fp8Args& fa, hipStream_t stream) {
  const MGemmArgs& g = fa.g;
  Sched s = make_sched(g, BM);
  if (s.wgs > 0x7fffffff) return fail(MOE_ERR_UNSUPPORTED, "grid too large");
  const size_t lds = 2 * (BM * 128) + 3 * (BN * 128);  // 2 token + 3 weight stages
  const dim3 grid(static_cast<unsigned>(s.wgs));
  MOE_DISPATCH_ACT(g.epilogue, ACT, {
    auto kernel = m_grouped_fp8_kernel<T, BM, ACT>;
    static bool configured = false;
    if (!configured) {
      hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(lds));
      if (err != hipSuccess)
        return fail(MOE_ERR_HIP, "hipFuncSetAttribute(%zu bytes of LDS): %s", lds,
                    hipGetErrorString(err));
      configured = true;
    }
    kernel<<<grid, kThreads, lds, stream>>>(fa, s);
  });
  return check_launch("m_grouped_gemm_fp8");
}

}  // namespace
}  // namespace moe

using namespace moe;

extern "C" int moe_quantize_rows_fp8(const void* x, int64_t ldx, void* q, int64_t ldq, float* scale,
                                     int64_t rows, int64_t cols, int dtype, moe_stream_t stream_) {
  clear_error();
  MOE_REQUIRE(rows >= 0 && cols >= 0, "negative size");
  MOE_REQUIRE(dtype_bytes(dtype) != 0, "unknown dtype %d", dtype);
  if (rows == 0) return MOE_OK;
  MOE_REQUIRE(x && q && scale, "null pointer");
  MOE_REQUIRE(ldx >= cols && ldq >= cols, "row stride smaller than cols");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  // rows that fit the register file of a workgroup are read once
  const bool once = dtype != MOE_DTYPE_F32 && cols % 8 == 0 && cols <= 2048 * 8 && ldx % 8 == 0 &&
                    ldq % 8 == 0 && aligned16(x) && (reinterpret_cast<uintptr_t>(q) & 7) == 0;
  if (once) {
    const unsigned blocks = static_cast<unsigned>(rows < 65536 ? rows : 65536);
    auto launch = [&](auto tag) {
      using T = typename decltype(tag)::type;
      const T* xp = static_cast<const T*>(x);
      uint8_t* qp = static_cast<uint8_t*>(q);
      if (cols <= 2048 * 2)
        quantize_rows_once_kernel<T, 2><<<blocks, 256, 0, stream>>>(xp, ldx, qp, ldq, scale, rows, cols);
      else if (cols <= 2048 * 4)
        quantize_rows_once_kernel<T, 4><<<blocks, 256, 0, stream>>>(xp, ldx, qp, ldq, scale, rows, cols);
      else
        quantize_rows_once_kernel<T, 8><<<blocks, 256, 0, stream>>>(xp, ldx, qp, ldq, scale, rows, cols);
    };
    if (dtype == MOE_DTYPE_BF16) launch(type_tag<bf16_t>{});
    else launch(type_tag<f16_t>{});
    return check_launch("quantize_rows_fp8");
  }
  int64_t blocks = (rows + 3) / 4;
  if (blocks > 65536) blocks = 65536;
  MOE_DISPATCH_DTYPE(dtype, T, {
    quantize_rows_kernel<T><<<static_cast<unsigned>(blocks), 256, 0, stream>>>(
        static_cast<const T*>(x), ldx, static_cast<uint8_t*>(q), ldq, scale, rows, cols);
  });
  return check_launch("quantize_rows_fp8");
}

extern "C" int moe_m_grouped_gemm_fp8(const void* a, const float* a_scale, int64_t a_rows,
                                      int64_t lda, const void* w, const float* w_scale, void* c,
                                      int64_t c_rows, int64_t ldc, const int32_t* group_indices,
                                      const void* indices, int idx_bytes, const void* scales, int E,
                                      int64_t K, int64_t N, int topk, int flags, int epilogue,
                                      int out_dtype, int ksplit, int64_t c_split_stride,
                                      moe_stream_t stream) {
  clear_error();
  MOE_REQUIRE(out_dtype == MOE_DTYPE_BF16 || out_dtype == MOE_DTYPE_F16,
              "fp8 GEMM output must be bf16 or f16");
  MOE_REQUIRE(epilogue >= MOE_ACT_NONE && epilogue <= MOE_ACT_GEGLU, "unknown epilogue %d", epilogue);
  MOE_REQUIRE(E >= 1 && K >= 0 && N >= 0 && topk >= 1, "bad sizes");
  MOE_REQUIRE(a_rows >= 0 && c_rows >= 0, "negative row count");
  MOE_REQUIRE((flags & ~(3 | MOE_FP8_W_TILED)) == 0,
              "fp8 GEMM takes GATHER_A, SCATTER_C and FP8_W_TILED only (flags 0x%x)", flags);
  const int w_tiled = (flags & MOE_FP8_W_TILED) ? 1 : 0;
  flags &= ~MOE_FP8_W_TILED;
  const bool gather = flags & MOE_GEMM_GATHER_A, scatter = flags & MOE_GEMM_SCATTER_C;
  MOE_REQUIRE(!act_is_glu(epilogue) || N % 2 == 0, "a GLU epilogue needs an even N");
  MOE_REQUIRE(group_indices != nullptr, "group_indices is null");
  if (gather || scatter) {
    MOE_REQUIRE(indices != nullptr, "gather/scatter needs indices");
    MOE_REQUIRE(idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8, got %d", idx_bytes);
  }
  const int64_t P = gather ? c_rows : a_rows;
  MOE_REQUIRE(P <= 0x7fffffff, "too many rows");
  if (P == 0 || N == 0) return MOE_OK;
  MOE_REQUIRE(a && a_scale && w && w_scale && c, "null operand");
  MOE_REQUIRE(a_rows > 0 && c_rows > 0, "empty operand with non-empty groups");
  const int64_t width = act_is_glu(epilogue) ? N / 2 : N;
  MOE_REQUIRE(lda >= K && ldc >= width, "row stride smaller than the row");
  MOE_REQUIRE(ksplit >= 1 && ksplit <= 8, "ksplit must be in [1,8], got %d", ksplit);
  if (ksplit > 1) {
    // partial sums over K parts can only be added afterwards where the epilogue is linear
    if (epilogue != MOE_ACT_NONE || K % (BKQ * ksplit) != 0)
      return fail(MOE_ERR_UNSUPPORTED, "split K needs no activation and K %% (128*ksplit) == 0");
    MOE_REQUIRE(c_split_stride >= (c_rows - 1) * ldc + N, "c_split_stride smaller than one copy of c");
  }
  if (K == 0 || K % BKQ != 0 || N % 8 != 0 || lda % 16 != 0 || !aligned16(a) || !aligned16(w) ||
      (reinterpret_cast<uintptr_t>(w_scale) & 15) || ldc % 4 != 0 ||
      (reinterpret_cast<uintptr_t>(c) & 7))
    return fail(MOE_ERR_UNSUPPORTED,
                "fp8 GEMM needs K %% 128 == 0, N %% 8 == 0, lda %% 16 == 0 and 16-byte aligned "
                "operands (K=%lld N=%lld lda=%lld)",
                (long long)K, (long long)N, (long long)lda);
  Fp8Args fa;
  fa.g = MGemmArgs{a,       a_rows, lda,     w,      N * K,         1,       K,         c,
                   c_rows,  ldc,    nullptr, 0,      group_indices, indices, idx_bytes, scales,
                   E,       K,      N,       topk,   flags,         epilogue, out_dtype, P,
                   FastDiv(static_cast<uint32_t>(topk)), ksplit, ksplit > 1 ? c_split_stride : 0};
  fa.a_scale = a_scale;
  fa.w_scale = w_scale;
  fa.w_tiled = w_tiled;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool big = P / E >= 512;
  if (out_dtype == MOE_DTYPE_BF16)
    return big ? launch_fp8<bf16_t, 256>(fa, s) : launch_fp8<bf16_t, 128>(fa, s);
  return big ? launch_fp8<f16_t, 256>(fa, s) : launch_fp8<f16_t, 128>(fa, s);
}
