// Row-wise, HBM-bound passes of the MoE layer: row gather / row scatter
// (reference triton_kernels/row_gather_scatter.py:10-116), the top-k weighted
// combine (functional/scale_and_reduce.py:3-5), the fp32 -> dtype cast that
// finishes the fused scatter-add combine, and the activation gradient.
// Every kernel moves 16 bytes per lane when pointers, strides and widths allow
// and falls back to single elements otherwise.
#include "common.h"

namespace moe {
namespace {

constexpr int kThreads = 256;

inline unsigned grid_for(int64_t items, int per_block = kThreads) {
  int64_t b = (items + per_block - 1) / per_block;
  if (b < 1) b = 1;
  if (b > 0x7fffffff) b = 0x7fffffff;
  return static_cast<unsigned>(b);
}

// ---- gather / scatter --------------------------------------------------------
// VEC = bytes moved per lane per step (16, or the element size).
template <int VEC, bool SCATTER>
__global__ __launch_bounds__(kThreads) void row_move_kernel(
    const char* __restrict__ src, int64_t src_rows, int64_t src_stride_b,
    const void* __restrict__ idx, int idx_bytes, int idx_div, char* __restrict__ dst,
    int64_t dst_rows, int64_t dst_stride_b, int64_t rows, int64_t row_bytes) {
  const int64_t vec_per_row = row_bytes / VEC;
  const int64_t total = rows * vec_per_row;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * kThreads) {
    const int64_t r = i / vec_per_row;
    const int64_t c = (i - r * vec_per_row) * VEC;
    int64_t v = load_index(idx, idx_bytes, r);
    int64_t sr, dr;
    if (SCATTER) {
      sr = r;
      dr = clamp_index(v, dst_rows);
    } else {
      sr = clamp_index(v / idx_div, src_rows);
      dr = r;
    }
    const char* s = src + sr * src_stride_b + c;
    char* d = dst + dr * dst_stride_b + c;
    if constexpr (VEC == 16) {
      *reinterpret_cast<uint4*>(d) = *reinterpret_cast<const uint4*>(s);
    } else if constexpr (VEC == 4) {
      *reinterpret_cast<uint32_t*>(d) = *reinterpret_cast<const uint32_t*>(s);
    } else {
      *reinterpret_cast<uint16_t*>(d) = *reinterpret_cast<const uint16_t*>(s);
    }
  }
}

template <bool SCATTER>
int launch_row_move(const void* src, int64_t src_rows, int64_t src_stride, const void* idx,
                    int idx_bytes, int idx_div, void* dst, int64_t dst_rows, int64_t dst_stride,
                    int64_t rows, int64_t cols, int elt_bytes, hipStream_t stream) {
  if (rows == 0 || cols == 0) return MOE_OK;
  const int64_t row_bytes = cols * elt_bytes;
  const int64_t ssb = src_stride * elt_bytes, dsb = dst_stride * elt_bytes;
  const bool vec16 = aligned16(src) && aligned16(dst) && row_bytes % 16 == 0 && ssb % 16 == 0 &&
                     dsb % 16 == 0;
  const char* s = static_cast<const char*>(src);
  char* d = static_cast<char*>(dst);
  if (vec16) {
    unsigned g = grid_for(rows * (row_bytes / 16));
    row_move_kernel<16, SCATTER><<<g, kThreads, 0, stream>>>(s, src_rows, ssb, idx, idx_bytes,
                                                            idx_div, d, dst_rows, dsb, rows,
                                                            row_bytes);
  } else if (elt_bytes == 4) {
    unsigned g = grid_for(rows * cols);
    row_move_kernel<4, SCATTER><<<g, kThreads, 0, stream>>>(s, src_rows, ssb, idx, idx_bytes,
                                                           idx_div, d, dst_rows, dsb, rows,
                                                           row_bytes);
  } else {
    unsigned g = grid_for(rows * cols);
    row_move_kernel<2, SCATTER><<<g, kThreads, 0, stream>>>(s, src_rows, ssb, idx, idx_bytes,
                                                           idx_div, d, dst_rows, dsb, rows,
                                                           row_bytes);
  }
  return check_launch(SCATTER ? "row_scatter" : "row_gather");
}

// Lanes that share a row (log2) and the grid of a kernel whose workgroups walk rows.
inline int row_lanes_log2(int64_t pieces) {
  int l = 0;
  while ((1 << l) < kThreads && (int64_t(1) << l) < pieces) ++l;
  return l;
}
inline unsigned row_grid(int64_t rows, int lanes_log2) {
  const int64_t rows_per_pass = kThreads >> lanes_log2;
  const int64_t blocks = (rows + rows_per_pass - 1) / rows_per_pass;
  const int64_t cap = 256 * 32;  // a few workgroups a CU in flight, the rest by the stride loop
  return static_cast<unsigned>(blocks < 1 ? 1 : (blocks < cap ? blocks : cap));
}

// ---- top-k weighted combine --------------------------------------------------
// One lane produces EPT consecutive output columns of one token; 2^lanes_log2 lanes (the power
// of two that covers a row's pieces, at most the workgroup) share a token and a workgroup walks
// tokens, so that token and column of a lane come from shifts and masks instead of a 64-bit
// division per piece (3-4 % at 4096 x 4096 and 8192 x 2048 outputs).
template <typename T, int EPT>
__global__ __launch_bounds__(kThreads) void scale_and_reduce_kernel(
    const T* __restrict__ in, int64_t in_stride, const T* __restrict__ scales,
    T* __restrict__ out, int64_t out_stride, int64_t T_tokens, int topk, int64_t n, int nsplit,
    int64_t split_stride, int lanes_log2) {
  const int per_row = static_cast<int>((n + EPT - 1) / EPT);
  const int lanes = 1 << lanes_log2;
  const int rows_per_pass = kThreads >> lanes_log2;
  const int first_c = threadIdx.x & (lanes - 1);
  for (int64_t t = static_cast<int64_t>(blockIdx.x) * rows_per_pass + (threadIdx.x >> lanes_log2);
       t < T_tokens; t += static_cast<int64_t>(gridDim.x) * rows_per_pass)
  for (int piece = first_c; piece < per_row; piece += lanes) {
    const int64_t c0 = static_cast<int64_t>(piece) * EPT;
    float acc[EPT];
#pragma unroll
    for (int e = 0; e < EPT; ++e) acc[e] = 0.0f;
    for (int j = 0; j < topk; ++j) {
      const int64_t s = t * topk + j;
      const float w = scales != nullptr ? to_f32(scales[s]) : 1.0f;
      for (int sp = 0; sp < nsplit; ++sp) {
        const T* row = in + sp * split_stride + s * in_stride + c0;
        if constexpr (EPT * sizeof(T) == 16) {
          uint4 raw = *reinterpret_cast<const uint4*>(row);
          const T* v = reinterpret_cast<const T*>(&raw);
#pragma unroll
          for (int e = 0; e < EPT; ++e) acc[e] += w * to_f32(v[e]);
        } else {
#pragma unroll
          for (int e = 0; e < EPT; ++e)
            if (c0 + e < n) acc[e] += w * to_f32(row[e]);
        }
      }
    }
    T* o = out + t * out_stride + c0;
    if constexpr (EPT * sizeof(T) == 16) {
      uint4 raw;
      T* v = reinterpret_cast<T*>(&raw);
#pragma unroll
      for (int e = 0; e < EPT; ++e) v[e] = from_f32<T>(acc[e]);
      *reinterpret_cast<uint4*>(o) = raw;
    } else {
#pragma unroll
      for (int e = 0; e < EPT; ++e)
        if (c0 + e < n) o[e] = from_f32<T>(acc[e]);
    }
  }
}

// ---- fp32 -> dtype ------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kThreads) void cast_from_f32_kernel(const float* __restrict__ src,
                                                                 int64_t src_stride,
                                                                 T* __restrict__ dst,
                                                                 int64_t dst_stride, int64_t rows,
                                                                 int64_t cols, bool vec4) {
  if (vec4) {
    const int64_t per_row = cols / 4;
    const int64_t total = rows * per_row;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
      const int64_t r = i / per_row;
      const int64_t c = (i - r * per_row) * 4;
      float4 v = *reinterpret_cast<const float4*>(src + r * src_stride + c);
      T o[4] = {from_f32<T>(v.x), from_f32<T>(v.y), from_f32<T>(v.z), from_f32<T>(v.w)};
      T* d = dst + r * dst_stride + c;
      if constexpr (sizeof(T) == 2) {
        *reinterpret_cast<uint2*>(d) = *reinterpret_cast<const uint2*>(o);
      } else {
        *reinterpret_cast<uint4*>(d) = *reinterpret_cast<const uint4*>(o);
      }
    }
  } else {
    const int64_t total = rows * cols;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x; i < total;
         i += static_cast<int64_t>(gridDim.x) * kThreads) {
      const int64_t r = i / cols;
      const int64_t c = i - r * cols;
      dst[r * dst_stride + c] = from_f32<T>(src[r * src_stride + c]);
    }
  }
}

// ---- activation gradient -------------------------------------------------------
// One wavefront per row; the row-wise dot product for dscale is reduced across
// the wavefront with DPP-free shuffles.  VEC output columns per lane and iteration:
// 4 (8- and 16-byte accesses; 16-bit types with aligned rows) or 1.
template <typename T, int ACT, int VEC>
__global__ __launch_bounds__(kThreads) void act_bwd_kernel(
    const T* __restrict__ h, int64_t ldh, const T* __restrict__ dy, int64_t lddy,
    T* __restrict__ dh, int64_t lddh, const T* __restrict__ row_scale,
    const void* __restrict__ indices, int idx_bytes, T* __restrict__ y_scaled, int64_t ldy,
    float* __restrict__ dscale, int64_t R, int64_t N) {
  constexpr bool GLU = act_is_glu(ACT);
  constexpr int HV = GLU ? 2 * VEC : VEC;  // elements of h (and dh) per lane and iteration
  const int lane = threadIdx.x % 64;
  const int64_t wave = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / 64;
  const int64_t waves = static_cast<int64_t>(gridDim.x) * kThreads / 64;
  const int64_t No = GLU ? N / 2 : N;
  for (int64_t p = wave; p < R; p += waves) {
    int64_t s = p;
    if (indices != nullptr) s = clamp_index(load_index(indices, idx_bytes, p), R);
    const float w = row_scale != nullptr ? to_f32(row_scale[s]) : 1.0f;
    const T* hrow = h + p * ldh;
    const T* dyrow = dy + p * lddy;
    T* dhrow = dh + p * lddh;
    float dot = 0.0f;
    for (int64_t j = static_cast<int64_t>(lane) * VEC; j < No; j += 64 * VEC) {
      T gv[VEC], hv[HV], dv[HV], yv[VEC];
      if constexpr (VEC == 4) {
        static_assert(sizeof(T) == 2, "vector path: 16-bit types");
        *reinterpret_cast<uint2*>(gv) = *reinterpret_cast<const uint2*>(dyrow + j);
        if constexpr (GLU) *reinterpret_cast<uint4*>(hv) = *reinterpret_cast<const uint4*>(hrow + 2 * j);
        else *reinterpret_cast<uint2*>(hv) = *reinterpret_cast<const uint2*>(hrow + j);
      } else {
        gv[0] = dyrow[j];
        if constexpr (GLU) {
          hv[0] = hrow[2 * j];
          hv[1] = hrow[2 * j + 1];
        } else {
          hv[0] = hrow[j];
        }
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float g = to_f32(gv[v]);
        float y;
        if constexpr (GLU) {
          const float gate = to_f32(hv[2 * v]);
          const float up = to_f32(hv[2 * v + 1]);
          const float a = apply_act<ACT>(gate);
          y = a * up;
          dv[2 * v] = from_f32<T>(w * g * up * apply_act_grad<ACT>(gate));
          dv[2 * v + 1] = from_f32<T>(w * g * a);
        } else {
          const float x = to_f32(hv[v]);
          y = apply_act<ACT>(x);
          dv[v] = from_f32<T>(w * g * apply_act_grad<ACT>(x));
        }
        dot += g * y;
        yv[v] = from_f32<T>(w * y);
      }
      if constexpr (VEC == 4) {
        if constexpr (GLU) *reinterpret_cast<uint4*>(dhrow + 2 * j) = *reinterpret_cast<const uint4*>(dv);
        else *reinterpret_cast<uint2*>(dhrow + j) = *reinterpret_cast<const uint2*>(dv);
        if (y_scaled != nullptr)
          *reinterpret_cast<uint2*>(y_scaled + p * ldy + j) = *reinterpret_cast<const uint2*>(yv);
      } else {
        if constexpr (GLU) {
          dhrow[2 * j] = dv[0];
          dhrow[2 * j + 1] = dv[1];
        } else {
          dhrow[j] = dv[0];
        }
        if (y_scaled != nullptr) y_scaled[p * ldy + j] = yv[0];
      }
    }
    if (dscale != nullptr) {
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
      if (lane == 0) dscale[s] = dot;
    }
  }
}

}  // namespace
}  // namespace moe

using namespace moe;

extern "C" int moe_row_gather(const void* src, int64_t src_rows, int64_t src_stride,
                              const void* idx, int idx_bytes, int idx_div, void* dst,
                              int64_t dst_stride, int64_t rows_out, int64_t cols, int elt_bytes,
                              moe_stream_t stream) {
  clear_error();
  MOE_REQUIRE(elt_bytes == 2 || elt_bytes == 4, "elt_bytes must be 2 or 4, got %d", elt_bytes);
  MOE_REQUIRE(idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8, got %d", idx_bytes);
  MOE_REQUIRE(idx_div >= 1, "idx_div must be >= 1, got %d", idx_div);
  MOE_REQUIRE(rows_out >= 0 && cols >= 0 && src_rows >= 0, "negative size");
  if (rows_out == 0 || cols == 0) return MOE_OK;
  MOE_REQUIRE(src_rows > 0, "gather from an empty source");
  MOE_REQUIRE(src && idx && dst, "null pointer");
  MOE_REQUIRE(src_stride >= cols && dst_stride >= cols, "row stride smaller than cols");
  return launch_row_move<false>(src, src_rows, src_stride, idx, idx_bytes, idx_div, dst, rows_out,
                                dst_stride, rows_out, cols, elt_bytes,
                                static_cast<hipStream_t>(stream));
}

extern "C" int moe_row_scatter(const void* src, int64_t src_stride, const void* idx, int idx_bytes,
                               void* dst, int64_t dst_rows, int64_t dst_stride, int64_t rows,
                               int64_t cols, int elt_bytes, moe_stream_t stream) {
  clear_error();
  MOE_REQUIRE(elt_bytes == 2 || elt_bytes == 4, "elt_bytes must be 2 or 4, got %d", elt_bytes);
  MOE_REQUIRE(idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8, got %d", idx_bytes);
  MOE_REQUIRE(rows >= 0 && cols >= 0 && dst_rows >= 0, "negative size");
  if (rows == 0 || cols == 0) return MOE_OK;
  MOE_REQUIRE(dst_rows > 0, "scatter into an empty destination");
  MOE_REQUIRE(src && idx && dst, "null pointer");
  MOE_REQUIRE(src_stride >= cols && dst_stride >= cols, "row stride smaller than cols");
  return launch_row_move<true>(src, rows, src_stride, idx, idx_bytes, 1, dst, dst_rows, dst_stride,
                               rows, cols, elt_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int moe_scale_and_reduce(const void* in, int64_t in_stride, const void* scales,
                                    void* out, int64_t out_stride, int64_t T, int topk, int64_t n,
                                    int dtype, int nsplit, int64_t split_stride,
                                    moe_stream_t stream_) {
  clear_error();
  MOE_REQUIRE(T >= 0 && n >= 0 && topk >= 1, "bad sizes T=%lld topk=%d n=%lld", (long long)T, topk,
              (long long)n);
  if (T == 0 || n == 0) return MOE_OK;
  MOE_REQUIRE(in && out, "null pointer");
  MOE_REQUIRE(in_stride >= n && out_stride >= n, "row stride smaller than n");
  MOE_REQUIRE(nsplit >= 1, "nsplit must be >= 1, got %d", nsplit);
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  MOE_DISPATCH_DTYPE(dtype, TT, {
    constexpr int V = 16 / sizeof(TT);
    const bool vec = aligned16(in) && aligned16(out) && n % V == 0 && in_stride % V == 0 &&
                     out_stride % V == 0 && (nsplit == 1 || split_stride % V == 0);
    if (vec) {
      const int ll = row_lanes_log2(n / V);
      scale_and_reduce_kernel<TT, V><<<row_grid(T, ll), kThreads, 0, stream>>>(
          static_cast<const TT*>(in), in_stride, static_cast<const TT*>(scales),
          static_cast<TT*>(out), out_stride, T, topk, n, nsplit, split_stride, ll);
    } else {
      const int ll = row_lanes_log2(n);
      scale_and_reduce_kernel<TT, 1><<<row_grid(T, ll), kThreads, 0, stream>>>(
          static_cast<const TT*>(in), in_stride, static_cast<const TT*>(scales),
          static_cast<TT*>(out), out_stride, T, topk, n, nsplit, split_stride, ll);
    }
  });
  return check_launch("scale_and_reduce");
}

extern "C" int moe_cast_from_f32(const float* src, int64_t src_stride, void* dst,
                                 int64_t dst_stride, int64_t rows, int64_t cols, int dtype,
                                 moe_stream_t stream_) {
  clear_error();
  MOE_REQUIRE(rows >= 0 && cols >= 0, "negative size");
  if (rows == 0 || cols == 0) return MOE_OK;
  MOE_REQUIRE(src && dst, "null pointer");
  MOE_REQUIRE(src_stride >= cols && dst_stride >= cols, "row stride smaller than cols");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  MOE_DISPATCH_DTYPE(dtype, TT, {
    const bool vec4 = aligned16(src) && aligned16(dst) && cols % 4 == 0 && src_stride % 4 == 0 &&
                      dst_stride % 4 == 0;
    const int64_t items = vec4 ? rows * (cols / 4) : rows * cols;
    cast_from_f32_kernel<TT><<<grid_for(items), kThreads, 0, stream>>>(
        src, src_stride, static_cast<TT*>(dst), dst_stride, rows, cols, vec4);
  });
  return check_launch("cast_from_f32");
}

extern "C" int moe_act_bwd(const void* h, int64_t ldh, const void* dy, int64_t lddy, void* dh,
                           int64_t lddh, const void* row_scale, const void* indices,
                           int idx_bytes, void* y_scaled, int64_t ldy, float* dscale, int64_t R,
                           int64_t N, int act, int dtype, moe_stream_t stream_) {
  clear_error();
  MOE_REQUIRE(R >= 0 && N >= 0, "negative size");
  MOE_REQUIRE(indices == nullptr || idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8");
  if (R == 0 || N == 0) return MOE_OK;
  MOE_REQUIRE(h && dy && dh, "null pointer");
  if (act == MOE_ACT_SWIGLU || act == MOE_ACT_GEGLU) MOE_REQUIRE(N % 2 == 0, "GLU needs even N");
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const unsigned grid = grid_for(R, kThreads / 64);
  // four output columns a lane: 16-bit types, rows that keep every 8- and 16-byte access aligned
  const int64_t No = (act == MOE_ACT_SWIGLU || act == MOE_ACT_GEGLU) ? N / 2 : N;
  const bool vec4 = dtype != MOE_DTYPE_F32 && No % 4 == 0 && ldh % 8 == 0 && lddh % 8 == 0 &&
                    lddy % 4 == 0 && (y_scaled == nullptr || ldy % 4 == 0) && aligned16(h) &&
                    aligned16(dh) && aligned16(dy) && aligned16(y_scaled);
  if (dtype == MOE_DTYPE_F32) {
    MOE_DISPATCH_ACT(act, ACT, {
      act_bwd_kernel<float, ACT, 1><<<grid, kThreads, 0, stream>>>(
          static_cast<const float*>(h), ldh, static_cast<const float*>(dy), lddy,
          static_cast<float*>(dh), lddh, static_cast<const float*>(row_scale), indices, idx_bytes,
          static_cast<float*>(y_scaled), ldy, dscale, R, N);
    });
    return check_launch("act_bwd");
  }
#define MOE_ACT_BWD_LAUNCH(TT, VEC)                                                              \
  MOE_DISPATCH_ACT(act, ACT, {                                                                   \
    act_bwd_kernel<TT, ACT, VEC><<<grid, kThreads, 0, stream>>>(                                 \
        static_cast<const TT*>(h), ldh, static_cast<const TT*>(dy), lddy, static_cast<TT*>(dh),  \
        lddh, static_cast<const TT*>(row_scale), indices, idx_bytes, static_cast<TT*>(y_scaled), \
        ldy, dscale, R, N);                                                                      \
  })
  if (dtype == MOE_DTYPE_BF16) {
    if (vec4) { MOE_ACT_BWD_LAUNCH(bf16_t, 4); } else { MOE_ACT_BWD_LAUNCH(bf16_t, 1); }
  } else if (dtype == MOE_DTYPE_F16) {
    if (vec4) { MOE_ACT_BWD_LAUNCH(f16_t, 4); } else { MOE_ACT_BWD_LAUNCH(f16_t, 1); }
  } else {
    return fail(MOE_ERR_INVALID_ARG, "unknown dtype %d", dtype);
  }
#undef MOE_ACT_BWD_LAUNCH
  return check_launch("act_bwd");
}
