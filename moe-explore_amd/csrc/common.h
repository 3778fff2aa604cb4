// Shared host/device helpers of libmoe_hip: status handling, element types,
// index loads and the activation functions used by every epilogue.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/moe_hip.h"

namespace moe {

// ---- status -----------------------------------------------------------------
// Records the message for moe_last_error_string() and returns `code`.
int fail(int code, const char* fmt, ...);
void clear_error();

#define MOE_REQUIRE(cond, ...)                                   \
  do {                                                           \
    if (!(cond)) return ::moe::fail(MOE_ERR_INVALID_ARG, __VA_ARGS__); \
  } while (0)

// Checks the launch that was just issued; does not synchronise.
// compute units of the current device (cached); -1 with the error set on failure
int num_cus();

// Lets `kernel` be launched with `bytes` of dynamic LDS (more than the 64 KiB a kernel gets
// without asking); set once per kernel and device.  Always called with the same size for a kernel.
int allow_dynamic_lds(const void* kernel, size_t bytes);

inline int check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return fail(MOE_ERR_HIP, "%s: %s", what, hipGetErrorString(err));
  return MOE_OK;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- element types ----------------------------------------------------------
typedef __bf16 bf16_t;
typedef _Float16 f16_t;

template <typename T>
__device__ __forceinline__ float to_f32(T v) {
  return static_cast<float>(v);
}
template <typename T>
__device__ __forceinline__ T from_f32(float v) {
  return static_cast<T>(v);  // round-to-nearest-even for f16 and bf16
}

// Index arrays come as int32 or int64; positions and slot ids fit in int64.
__device__ __forceinline__ int64_t load_index(const void* idx, int idx_bytes, int64_t i) {
  return idx_bytes == 8 ? static_cast<const int64_t*>(idx)[i]
                        : static_cast<int64_t>(static_cast<const int32_t*>(idx)[i]);
}

// Low 32 bits of an index: slot ids and positions are below 2^31, so this reads
// int32 and (little-endian) int64 arrays alike with one 4-byte load.
__device__ __forceinline__ int32_t load_index32(const void* idx, int idx_bytes, int64_t i) {
  return *reinterpret_cast<const int32_t*>(static_cast<const char*>(idx) + i * idx_bytes);
}

// Division of a value below 2^31 by a divisor fixed at launch (slot id -> token id
// is `slot / topk`): one 32x32->64 multiply and a shift instead of an integer
// division in the kernel.  mul = floor(2^(31+shift) / d) + 1 with 2^shift >= d.
struct FastDiv {
  uint32_t mul, shift;
  FastDiv() : mul(0x80000001u), shift(0) {}
  explicit FastDiv(uint32_t d) {
    shift = 0;
    while ((1u << shift) < d) ++shift;
    mul = static_cast<uint32_t>((1ull << (31 + shift)) / d) + 1u;
  }
  __host__ __device__ __forceinline__ int32_t div(int32_t n) const {
    const uint32_t u = n < 0 ? 0u : static_cast<uint32_t>(n);
    return static_cast<int32_t>((static_cast<uint64_t>(u) * mul) >> (31 + shift));
  }
};

__device__ __forceinline__ int64_t clamp_index(int64_t v, int64_t n) {
  return v < 0 ? 0 : (v >= n ? n - 1 : v);
}

// ---- activations (fp32, as the reference's epilogues compute them) ----------
// (v_rcp_f32, 1 ulp, instead of an IEEE division: the division's nine instructions were a third
// of the arithmetic of a SwiGLU epilogue, which is bound by arithmetic in the fused backward)
__device__ __forceinline__ float act_sigmoid(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}
__device__ __forceinline__ float act_silu(float x) { return x * act_sigmoid(x); }
// Phi(x) = (1 + erf(x / sqrt 2)) / 2 through the rational approximation 7.1.26 of Abramowitz
// and Stegun (|error of erf| < 1.5e-7, fp32 rounding level): an exponential, a reciprocal and
// five FMAs where the library's erff takes some forty instructions, which the GeGLU epilogue
// pays for every output element.  The negative side returns erfc / 2 directly (no 1 - 1).
__device__ __forceinline__ float act_norm_cdf(float x) {
  const float z = fabsf(x) * 0.70710678118654752440f;
  const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.0f));
  float p = fmaf(1.061405429f, t, -1.453152027f);
  p = fmaf(p, t, 1.421413741f);
  p = fmaf(p, t, -0.284496736f);
  p = fmaf(p, t, 0.254829592f);
  const float half_erfc = 0.5f * p * t * __expf(-z * z);
  return x < 0.0f ? half_erfc : 1.0f - half_erfc;
}
__device__ __forceinline__ float act_gelu(float x) { return x * act_norm_cdf(x); }
__device__ __forceinline__ float act_approx_gelu(float x) {
  const float c = 0.79788456080286535588f;  // sqrt(2/pi)
  // 0.5 * (1 + tanh u) = sigmoid(2u)
  return x * act_sigmoid(2.0f * c * (x + 0.044715f * x * x * x));
}
// derivatives
__device__ __forceinline__ float act_silu_grad(float x) {
  float s = act_sigmoid(x);
  return s * (1.0f + x * (1.0f - s));
}
__device__ __forceinline__ float act_gelu_grad(float x) {
  const float inv_sqrt_2pi = 0.39894228040143267794f;
  return act_norm_cdf(x) + x * inv_sqrt_2pi * __expf(-0.5f * x * x);
}
__device__ __forceinline__ float act_approx_gelu_grad(float x) {
  const float c = 0.79788456080286535588f;
  float u = c * (x + 0.044715f * x * x * x);
  float sg = act_sigmoid(2.0f * u);  // (1 + tanh u) / 2, so 1 - tanh^2 u = 4 sg (1 - sg)
  float du = c * (1.0f + 3.0f * 0.044715f * x * x);
  return sg + 2.0f * x * sg * (1.0f - sg) * du;
}

// Elementwise activation selected at compile time (non-GLU codes), or the gate
// function of a GLU code.
template <int ACT>
__device__ __forceinline__ float apply_act(float x) {
  if constexpr (ACT == MOE_ACT_SILU || ACT == MOE_ACT_SWIGLU) return act_silu(x);
  else if constexpr (ACT == MOE_ACT_GELU || ACT == MOE_ACT_GEGLU) return act_gelu(x);
  else if constexpr (ACT == MOE_ACT_APPROX_GELU) return act_approx_gelu(x);
  else return x;
}
template <int ACT>
__device__ __forceinline__ float apply_act_grad(float x) {
  if constexpr (ACT == MOE_ACT_SILU || ACT == MOE_ACT_SWIGLU) return act_silu_grad(x);
  else if constexpr (ACT == MOE_ACT_GELU || ACT == MOE_ACT_GEGLU) return act_gelu_grad(x);
  else if constexpr (ACT == MOE_ACT_APPROX_GELU) return act_approx_gelu_grad(x);
  else return 1.0f;
}
constexpr bool act_is_glu(int act) { return act == MOE_ACT_SWIGLU || act == MOE_ACT_GEGLU; }

inline int dtype_bytes(int dtype) {
  return dtype == MOE_DTYPE_F32 ? 4 : ((dtype == MOE_DTYPE_F16 || dtype == MOE_DTYPE_BF16) ? 2 : 0);
}

// Dispatch helpers ------------------------------------------------------------
#define MOE_DISPATCH_DTYPE(dtype, T, ...)                                    \
  switch (dtype) {                                                           \
    case MOE_DTYPE_F32: { using T = float; __VA_ARGS__; break; }             \
    case MOE_DTYPE_F16: { using T = ::moe::f16_t; __VA_ARGS__; break; }      \
    case MOE_DTYPE_BF16: { using T = ::moe::bf16_t; __VA_ARGS__; break; }    \
    default: return ::moe::fail(MOE_ERR_INVALID_ARG, "unknown dtype %d", dtype); \
  }

#define MOE_DISPATCH_ACT(act, ACT, ...)                                              \
  switch (act) {                                                                     \
    case MOE_ACT_NONE: { constexpr int ACT = MOE_ACT_NONE; __VA_ARGS__; break; }     \
    case MOE_ACT_SILU: { constexpr int ACT = MOE_ACT_SILU; __VA_ARGS__; break; }     \
    case MOE_ACT_GELU: { constexpr int ACT = MOE_ACT_GELU; __VA_ARGS__; break; }     \
    case MOE_ACT_APPROX_GELU: { constexpr int ACT = MOE_ACT_APPROX_GELU; __VA_ARGS__; break; } \
    case MOE_ACT_SWIGLU: { constexpr int ACT = MOE_ACT_SWIGLU; __VA_ARGS__; break; } \
    case MOE_ACT_GEGLU: { constexpr int ACT = MOE_ACT_GEGLU; __VA_ARGS__; break; }   \
    default: return ::moe::fail(MOE_ERR_INVALID_ARG, "unknown epilogue %d", act);    \
  }

}  // namespace moe
