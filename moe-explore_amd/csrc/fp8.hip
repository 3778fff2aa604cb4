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

// One 1 KiB copy instruction: lane i's 16 bytes at base + offset go to LDS address M0 + 16 i.
__device__ __forceinline__ void copy16_to_lds(const void* base, uint32_t offset, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr), "v"(offset), "s"(base)
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


// One work item: `tpw` adjacent column tiles of one row block, computed as ONE stream of K
// steps (token addresses stay, weight addresses move on), so that the copies of the next
// tile's first steps fly while the finished accumulators are stored.  A gate/up tile of
// config 4 has only 32 K steps: what a work item pays once (tile lookup, index fetch, the
// latency of the first copies, the store) weighs twice what it does in the 16-bit kernel.
// 2 x 4 wavefronts, a wavefront tile of BM/2 x 64 = MB x 2 blocks of 32 x 32; a K step of 128
// is four units (K half x token-row half) of MB MFMAs; the fragments of the next unit are read
// while a unit is multiplied, and the weight fragments of a K half serve both of its units.
template <typename T, int BM, int ACT>
__device__ __forceinline__ void fp8_work_item(const Fp8Args& fa, const Sched s, const int id,
                                              NextDraw& next) {
  MGemmArgs g = fa.g;
  constexpr int NWAVES = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M;
  constexpr int MB = WM / 32;   // 32-row blocks of a wavefront
  constexpr int HB = MB / 2;    // token blocks of one unit
  static_assert(NWAVES == 8 && NB == 2 && HB >= 1, "2 x 4 wavefronts of BM/2 x 64");
  constexpr int A_INSTR = BM / 8 / NWAVES;  // 1 KiB copy instructions per wavefront, token tile
  constexpr int W_INSTR = 32 / NWAVES;
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
  const int kpart = s.by_real_nt.div(nt);
  nt -= kpart * s.real_nt;
  const int KT = static_cast<int>(g.K / BKQ) / s.ksplit;  // K steps of this part
  const int kt0 = kpart * KT;
  g.c = static_cast<char*>(g.c) + static_cast<int64_t>(kpart) * g.c_split_stride * sizeof(T);
  if (threadIdx.x < 64) find_tile<BM>(g.group_indices, g.E, static_cast<int>(g.P), mt, sh_tile);
  __syncthreads();
  const int expert = __builtin_amdgcn_readfirstlane(sh_tile[0]);
  if (expert < 0) return;
  const int row0 = sh_tile[1], end = sh_tile[2];
  // column tiles nt0 .. nt0 + ntiles - 1 of this row block
  const int nt0 = nt * s.tpw;
  const int col_tiles = static_cast<int>((g.N + BN - 1) / BN);
  const int ntiles = col_tiles - nt0 < s.tpw ? col_tiles - nt0 : s.tpw;

  // (opaque: what depends only on the thread id would otherwise be computed once for all the
  // work items of the workgroup and held in registers across them, next to the accumulators)
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
  const int l32 = lane & 31, lhi = lane >> 5;

  // ---- global source of every copy instruction: a wave-uniform base + 32-bit byte offset ----
  // token tile: instruction i of wavefront w fills rows 8*(8i + w) .. +7, lane -> (row, chunk).
  // Rows that are not gathered are addressed from the first row of the block, so only a
  // gathered token matrix has to stay below 4 GiB (checked on the host).
  const bool gather = g.flags & MOE_GEMM_GATHER_A;
  const char* const abase = static_cast<const char*>(g.a) + (gather ? 0 : static_cast<int64_t>(row0) * g.lda);
  uint32_t a_src[A_INSTR];
  float a_scale[MB];  // activation scale of this lane's row in every row block of the wavefront
#pragma unroll
  for (int i = 0; i < A_INSTR; ++i) {
    const int r = 8 * (NWAVES * i + wave) + (lane >> 3);
    const int c = (lane & 7) ^ ((r >> 1) & 7);
    int p = row0 + r;
    p = p < end ? p : end - 1;
    int64_t arow = p;
    if (gather) arow = g.by_topk.div(load_index32(g.indices, g.idx_bytes, p));
    arow = clamp_index(arow, g.a_rows);
    a_src[i] = static_cast<uint32_t>((arow - (gather ? 0 : row0)) * g.lda + c * 16);
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    int p = row0 + wm0 + mb * 32 + l32;
    p = p < end ? p : end - 1;
    int64_t arow = p;
    if (gather) arow = g.by_topk.div(load_index32(g.indices, g.idx_bytes, p));
    a_scale[mb] = fa.a_scale[clamp_index(arow, g.a_rows)];
  }
  uint32_t w_src[W_INSTR];
  const char* wbase;  // weights of this expert (tile-major: of its current column tile)
  uint32_t w_step;    // bytes from one K step to the next
  auto set_w_src = [&](int tile) __attribute__((always_inline)) {  // weight sources of column tile nt0 + tile
    if (fa.w_tiled) {
      // tile-major weights: the 32 KiB of a column tile and K step are stored contiguously,
      // in the order (and with the swizzle) of the LDS tile, so a step is one linear copy
      // and the whole tile one sequential stream
      const int64_t t = static_cast<int64_t>(expert) * col_tiles + nt0 + tile;
      wbase = static_cast<const char*>(g.w) + t * (g.K / BKQ) * W_BYTES;
    } else {
      const int64_t n0 = static_cast<int64_t>(nt0 + tile) * BN;
#pragma unroll
      for (int i = 0; i < W_INSTR; ++i) {
        const int r = 8 * (NWAVES * i + wave) + (lane >> 3);
        const int c = (lane & 7) ^ ((r >> 1) & 7);
        int64_t n = n0 + r;
        n = n < g.N ? n : g.N - 1;
        w_src[i] = static_cast<uint32_t>(n * g.ldw_n + c * 16);
      }
    }
  };
  if (fa.w_tiled) {
#pragma unroll
    for (int i = 0; i < W_INSTR; ++i) w_src[i] = (NWAVES * i + wave) * 1024 + lane * 16;
    w_step = W_BYTES;
  } else {
    wbase = static_cast<const char*>(g.w) + static_cast<int64_t>(expert) * g.ldw_e;
    w_step = BKQ;
  }
  set_w_src(0);
  const unsigned lds0 =
      __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<size_t>((lds_void*)smem))) +
      wave * 1024;

  // Copy instructions [first, last) of a tile; the main loop spreads them over the units of a
  // K step so that they do not queue up in front of the MFMAs.  A copy instruction whose eight
  // token rows all lie past the end of the group is not issued: those LDS rows keep stale data
  // and only feed rows that are never stored.
  const int rows_here = __builtin_amdgcn_readfirstlane(end - row0);
  auto issue_token_copies = [&](int stage, int kt, int first, int last) __attribute__((always_inline)) {
    const unsigned base = lds0 + stage * A_BYTES;
#pragma unroll
    for (int i = 0; i < A_INSTR; ++i)
      if (i >= first && i < last && 8 * (NWAVES * i + wave) < rows_here)
        copy16_to_lds(abase, a_src[i] + static_cast<uint32_t>(kt0 + kt) * BKQ, base + i * (NWAVES * 1024));
  };
  auto issue_weight_copies = [&](int wstage, int kt, int first, int last) __attribute__((always_inline)) {
    const unsigned base = lds0 + W_BASE + wstage * W_BYTES;
#pragma unroll
    for (int i = 0; i < W_INSTR; ++i)
      if (i >= first && i < last)
        copy16_to_lds(wbase, w_src[i] + static_cast<uint32_t>(kt0 + kt) * w_step, base + i * (NWAVES * 1024));
  };

  // 32-row blocks of this wavefront that hold rows of the group: the K loop is compiled for
  // 0, MB/4, MB/2 and MB blocks and a wavefront runs the smallest that covers its own (every
  // variant copies and synchronises alike).  The last row block of a group is mostly empty.
  int live = (end - row0 - wm0 + 31) / 32;
  live = live < 0 ? 0 : (live > MB ? MB : live);
  live = __builtin_amdgcn_readfirstlane(live);

  // a lane's fragment of a 32-row block for K half kh: 32 bytes = chunks 4 kh + 2 lhi, +1
  auto read32 = [&](const char* tile, int row, int kh) __attribute__((always_inline)) -> i32x8 {
    const i32x4 lo = *reinterpret_cast<const i32x4*>(tile + kmajor_off(row, kh * 4 + lhi * 2));
    const i32x4 hi = *reinterpret_cast<const i32x4*>(tile + kmajor_off(row, kh * 4 + lhi * 2 + 1));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  // unit u of a K step = K half (u >> 1), token-row half (u & 1)
  auto read_unit_t = [&](int stage, int u, i32x8 (&tf)[HB], auto blocks) __attribute__((always_inline)) {
    constexpr int LC = decltype(blocks)::value;
    const char* at = smem + stage * A_BYTES;
    const int kh = u >> 1, rh = u & 1;
#pragma unroll
    for (int mb = 0; mb < HB; ++mb)
      if (rh * HB + mb < LC) tf[mb] = read32(at, wm0 + (rh * HB + mb) * 32 + l32, kh);
  };
  // column block `nb` of K half kh: block 0 before the unit of token-row half 0, block 1 at its
  // start (a wavefront with at most HB live blocks has no other unit)
  auto read_unit_w = [&](int wstage, int kh, int nb, i32x8 (&wf)[NB], auto blocks) __attribute__((always_inline)) {
    constexpr int LC = decltype(blocks)::value;
    if (LC == 0) return;
    wf[nb] = read32(smem + W_BASE + wstage * W_BYTES, wn0 + nb * 32 + l32, kh);
  };

  f32x16 acc[MB][NB];
  auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.0f;
  };
  zero_acc();
  auto multiply_unit = [&](int rh, i32x8 (&tf)[HB], i32x8 (&wf)[NB], auto blocks) __attribute__((always_inline)) {
    constexpr int LC = decltype(blocks)::value;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int mb = 0; mb < HB; ++mb) {
        if (rh == 0 && mb < LC)
          acc[mb][nb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
              wf[nb], tf[mb], acc[mb][nb], 0 /* A: e4m3 */, 0 /* B: e4m3 */, 0, 127, 0, 127);
        if (rh == 1 && HB + mb < LC)
          acc[HB + mb][nb] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
              wf[nb], tf[mb], acc[HB + mb][nb], 0, 0, 0, 127, 0, 127);
      }
    }
  };
  // A unit reads 2 * (HB + 1) pieces of 16 bytes a lane for its HB * 2 MFMAs.  The empty asm
  // statements tie the unit's accumulators to this point: an MFMA has no side effect, and the
  // compiler otherwise sinks all sixteen of a K step below the (conditional) copy blocks, to
  // the end of the step, with every fragment of the step live at once.
  auto interleave_unit = [&](int rh, auto blocks) __attribute__((always_inline)) {
    constexpr int LC = decltype(blocks)::value;
#pragma unroll
    for (int i = 0; i < HB * NB; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // two LDS reads
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mb = 0; mb < HB; ++mb)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        if (rh == 0 && mb < LC) asm volatile("" : "+v"(acc[mb][nb]));
        if (rh == 1 && HB + mb < LC) asm volatile("" : "+v"(acc[HB + mb][nb]));
      }
  };

  i32x8 tfA[HB], tfB[HB], wfP[NB], wfQ[NB];
  // The accumulators of column tile `tile` leave through LDS regions that no copy in flight
  // writes: wavefronts 0..3 through the token stage `a_free` (BM = 256; a spare region for
  // BM = 128, whose token stages are too small), the others through the weight stage `w_free`.
  constexpr int EPI_BYTES = epi_wave_bytes<NB, 32>();
  constexpr int SPARE_BASE = W_BASE + 3 * W_BYTES;
  const int row0_wg = row0, end_wg = end, lane_wg = lane;
  auto store_acc = [&](int tile, int a_free, int w_free) __attribute__((always_inline)) {
    const int64_t n0 = static_cast<int64_t>(nt0 + tile) * BN;
    // (opaque copies: the rows are the same for every tile of the work item, and the compiler
    // would otherwise keep the store's row addresses in registers across the K loop)
    int row0 = row0_wg, end = end_wg, lane = lane_wg;
    asm volatile("" : "+s"(row0), "+s"(end), "+v"(lane));
    const int l32 = lane & 31, lhi = lane >> 5;
    // dequantise: acc * a_scale[row] * w_scale[e, n], one run of four channel scales at a time
    // (all eight float4 loads hoisted next to the 128 accumulators spilled 31-40 registers)
    const float* wsc = fa.w_scale + static_cast<int64_t>(expert) * g.N;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int run = 0; run < 4; ++run) {
        int64_t n = n0 + wn0 + nb * 32 + run * 8 + lhi * 4;
        n = n + 3 < g.N ? n : g.N - 4;  // N is a multiple of 8; columns past N are not stored
        const float4 ws = *reinterpret_cast<const float4*>(wsc + n);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          acc[mb][nb][run * 4 + 0] *= a_scale[mb] * ws.x;
          acc[mb][nb][run * 4 + 1] *= a_scale[mb] * ws.y;
          acc[mb][nb][run * 4 + 2] *= a_scale[mb] * ws.z;
          acc[mb][nb][run * 4 + 3] *= a_scale[mb] * ws.w;
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    if (lds_epilogue_ok<T>(g)) {
      char* epi;
      if (wave < NWAVES / 2)
        epi = smem + (BM == 256 ? a_free * A_BYTES : SPARE_BASE) + wave * EPI_BYTES;
      else
        epi = smem + W_BASE + w_free * W_BYTES + (wave - NWAVES / 2) * EPI_BYTES;
      store_tile_lds<T, ACT, MB, NB, 32>(g, acc, epi, row0, end, n0, wm0, wn0, lane);
    } else {
      store_tile<T, ACT, MB>(g, acc, row0, end, n0, wm0, wn0, l32, lhi);
    }
  };
  auto main_loop = [&](auto blocks) __attribute__((always_inline)) {
    const int S = ntiles * KT;   // K steps of this work item; step gs is step gs % KT of tile gs / KT
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
      interleave_unit(0, blocks);
      if (more) {
        issue_token_copies(stage ^ 1, kt_a, AH, A_INSTR);
        advance_a();
      }
      __builtin_amdgcn_sched_barrier(0);
      read_unit_w(wcur, 1, 0, wfQ, blocks);
      read_unit_t(stage, 2, tfA, blocks);
      multiply_unit(1, tfB, wfP, blocks);
      interleave_unit(1, blocks);
      if (ahead) issue_weight_copies(wahead, kt_w, 0, WH);
      __builtin_amdgcn_sched_barrier(0);
      read_unit_w(wcur, 1, 1, wfQ, blocks);
      read_unit_t(stage, 3, tfB, blocks);
      multiply_unit(0, tfA, wfQ, blocks);
      interleave_unit(0, blocks);
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
      interleave_unit(1, blocks);
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
  if (live == 0) main_loop(std::integral_constant<int, 0>{});
  else if (MB >= 4 && live <= MB / 4) main_loop(std::integral_constant<int, (MB >= 4 ? MB / 4 : MB / 2)>{});
  else if (live <= MB / 2) main_loop(std::integral_constant<int, MB / 2>{});
  else main_loop(std::integral_constant<int, MB>{});
}

// One resident workgroup per compute unit draws work item ids from the tile queues of the
// launch stream (gemm_mfma.h describes them: id 8j + q belongs to queue q, a workgroup
// draws from the queue of its XCD first, word 8 counts the workgroups that are done and the
// last one clears the set); without a queue set (a launch that is being captured) workgroup b
// takes ids b, b + gridDim.x, ...
struct Fp8KernelArgs {
  Fp8Args fa;
  Sched s;
  unsigned* queue;
};
typedef __attribute__((address_space(4))) const Fp8KernelArgs* fp8_kernarg_ptr;

template <typename T, int BM, int ACT>
__global__ __launch_bounds__(kThreads) void m_grouped_fp8_kernel(Fp8KernelArgs ka) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // (beside the tile descriptor that fp8_work_item keeps in the third weight stage)
  int* const sh_next = reinterpret_cast<int*>(smem + 2 * (BM * 128) + 2 * (BN * 128)) + 8;
  // hardware register XCC_ID: the XCD this workgroup runs on
  const int home = __builtin_amdgcn_s_getreg((31 << 11) | 20) & (kNumXcd - 1);
  int tried = 0;  // queues found empty so far, the home queue first
  NextDraw next{nullptr, 0u, false};
  int64_t static_id = blockIdx.x;
  for (;;) {
    // The arguments are read from the kernel argument segment again for every work item: held
    // in scalar registers across them they crowd out what the K loop keeps there.
    fp8_kernarg_ptr kp = (fp8_kernarg_ptr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(kp));
    const Fp8KernelArgs* const args = (const Fp8KernelArgs*)kp;
    __syncthreads();  // every wavefront is done with the LDS of the work item before
    if (threadIdx.x == 0 && args->queue == nullptr) {
      *sh_next = static_id < args->s.wgs ? static_cast<int>(static_id) : -1;
      static_id += gridDim.x;
    } else if (threadIdx.x == 0) {
      // (draw_work_item() of gemm_mfma.h written out: called as a function this kernel measured 2 %
      // slower at T = 1024 and 8192, the scalar registers of its K loop falling differently)
      unsigned* const queue = args->queue;
      const int total = static_cast<int>(args->s.wgs);
      int id = -1;
      while (tried < kNumXcd) {
        const int q = (home + tried) & (kNumXcd - 1);
        // (a draw made during the last store went to this same queue)
        const unsigned got = next.drawn ? next.value : atomicAdd(&queue[q], 1u);
        next.drawn = false;
        const int64_t cand = static_cast<int64_t>(got) * kNumXcd + q;
        if (cand < total) {
          id = static_cast<int>(cand);
          break;
        }
        ++tried;
        // (a dry queue stays dry: one look at all counters passes over the other dry ones)
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
      *sh_next = id;
      next.slot = tried < kNumXcd ? &queue[(home + tried) & (kNumXcd - 1)] : nullptr;
    }
    __syncthreads();
    const int id = __builtin_amdgcn_readfirstlane(*sh_next);
    if (id < 0) break;
    fp8_work_item<T, BM, ACT>(args->fa, args->s, id, next);
  }
  // (every workgroup ends here: each queue runs dry after s.wgs / 8 draws)
  if (threadIdx.x == 0 && ka.queue != nullptr) {
    unsigned* const queue = ka.queue;
    __threadfence();
    if (atomicAdd(&queue[kNumXcd], 1u) == gridDim.x - 1) {
      for (int q = 0; q <= kNumXcd; ++q) atomicExch(&queue[q], 0u);
    }
  }
}

template <auto Kernel>
int launch_fp8_kernel(const Fp8Args& fa, const Sched& s, size_t lds, hipStream_t stream) {
  int rc = allow_dynamic_lds(reinterpret_cast<const void*>(Kernel), lds);
  if (rc != MOE_OK) return rc;
  int cus = 0;
  unsigned* queue = nullptr;
  rc = tile_queue_set_of(stream, &queue, &cus);
  if (rc != MOE_OK) return rc;
  Fp8KernelArgs ka;
  ka.fa = fa;
  ka.s = s;
  ka.queue = queue;
  // (a multiple of the XCD count, so that ids taken in strides of the grid stay on their XCD)
  unsigned wgs = static_cast<unsigned>(cus) / kNumXcd * kNumXcd;
  if (wgs == 0) wgs = static_cast<unsigned>(cus);
  if (s.wgs < wgs) wgs = static_cast<unsigned>(s.wgs);
  Kernel<<<dim3(wgs), kThreads, lds, stream>>>(ka);
  return MOE_OK;
}

template <typename T, int BM>
int launch_fp8(const Fp8Args& fa, hipStream_t stream) {
  const MGemmArgs& g = fa.g;
  // two column tiles a work item where that still leaves several rounds of work items
  const int64_t tiles = ((g.P + BM - 1) / BM + g.E / 2) * ((g.N + BN - 1) / BN) * (g.ksplit < 1 ? 1 : g.ksplit);
  Sched s = make_sched(g, BM, tiles >= 2048 ? 2 : 1);
  if (s.wgs > 0x7fffffff) return fail(MOE_ERR_UNSUPPORTED, "grid too large");
  // 2 token + 3 weight stages; BM = 128 adds room for the store staging of half the wavefronts
  const size_t lds = 2 * (BM * 128) + 3 * (BN * 128) + (BM == 256 ? 0 : 4 * epi_wave_bytes<NB, 32>());
  MOE_DISPATCH_ACT(g.epilogue, ACT, {
    const int rc = launch_fp8_kernel<m_grouped_fp8_kernel<T, BM, ACT>>(fa, s, lds, stream);
    if (rc != MOE_OK) return rc;
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
  // copy sources are a wave-uniform base and a 32-bit byte offset per lane: from the token matrix
  // when its rows are gathered (from the first row of a block otherwise), from the weights of one
  // expert (of one column tile when they are tile-major)
  {
    const int64_t limit = int64_t(1) << 32;
    const int64_t a_span = (gather ? a_rows : 256) * lda + K;
    const int64_t w_span = w_tiled ? (K / BKQ + 1) * (BN * BKQ) : N * K;
    if (a_span >= limit || w_span >= limit)
      return fail(MOE_ERR_UNSUPPORTED, "fp8 GEMM: a gathered token matrix and the weights of one expert "
                  "must stay below 4 GiB (%lld and %lld bytes)", (long long)a_span, (long long)w_span);
  }
  Fp8Args fa;
  fa.g = MGemmArgs{a,       a_rows, lda,     w,      N * K,         1,       K,         c,
                   c_rows,  ldc,    nullptr, 0,      group_indices, indices, idx_bytes, scales,
                   E,       K,      N,       topk,   flags,         epilogue, out_dtype, P,
                   FastDiv(static_cast<uint32_t>(topk)), ksplit, ksplit > 1 ? c_split_stride : 0};
  fa.a_scale = a_scale;
  fa.w_scale = w_scale;
  fa.w_tiled = w_tiled;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // (as in the 16-bit kernel: a group of ~256 rows is one full 256-row block and a short one
  // rather than two or three 128-row blocks that each stream the weight panel; T=1024 of
  // config 4 0.64 -> 0.58 ms)
  const bool big = P / E >= 256;
  if (out_dtype == MOE_DTYPE_BF16)
    return big ? launch_fp8<bf16_t, 256>(fa, s) : launch_fp8<bf16_t, 128>(fa, s);
  return big ? launch_fp8<f16_t, 256>(fa, s) : launch_fp8<f16_t, 128>(fa, s);
}
