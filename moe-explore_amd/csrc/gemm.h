// Argument records shared by the grouped-GEMM entry points and their kernels.
#pragma once
#include "common.h"

namespace moe {

struct MGemmArgs {
  const void* a;
  int64_t a_rows, lda;
  const void* w;
  int64_t ldw_e, ldw_k, ldw_n;
  void* c;
  int64_t c_rows, ldc;
  void* preact;
  int64_t ld_preact;
  const int32_t* group_indices;
  const void* indices;
  int idx_bytes;
  const void* scales;
  int E;
  int64_t K, N;
  int topk, flags, epilogue, dtype;
  int64_t P;  // number of expert-sorted positions; bounds group_indices
  FastDiv by_topk;
  int ksplit;               // K is cut into ksplit equal parts ...
  int64_t c_split_stride;   // ... part i stores to c + i * c_split_stride elements
  // MOE_GEMM_GLU_BWD (direct-to-LDS kernel only): the product is the gradient G of a GLU
  // output and never stored; the epilogue turns it into the gradient of the saved
  // pre-activation h: c = dh [P, 2N], preact = s * glu(h) [P, N], scales = s by position,
  // dscale[p] += <G, glu(h)> (fp32 atomics; zeroed by the caller), epilogue = the GLU.
  const void* h = nullptr;
  int64_t ldh = 0;
  float* dscale = nullptr;
};
constexpr int MOE_GEMM_GLU_BWD = 16;  // internal flag, set by moe_m_grouped_gemm_glu_bwd only

struct KGemmArgs {
  const void* a;
  int64_t a_rows, lda;
  const void* b;
  int64_t b_rows, ldb;
  void* out;
  const int32_t* group_indices;
  const void* indices;
  int idx_bytes;
  int E;
  int64_t Ka, Nb;
  int topk, flags, dtype;
  int64_t P;
  FastDiv by_topk;
};

int launch_m_grouped_generic(const MGemmArgs& g, hipStream_t stream);
int launch_k_grouped_generic(const KGemmArgs& g, hipStream_t stream);

// MFMA paths; `*_supported` is the host-side shape/alignment gate.
bool m_grouped_mfma_supported(const MGemmArgs& g);
int launch_m_grouped_mfma(const MGemmArgs& g, hipStream_t stream);
bool m_grouped_mfma_dma_supported(const MGemmArgs& g);  // K % 64 == 0, 16-byte stores, < 4 GiB spans
int launch_m_grouped_mfma_dma(const MGemmArgs& g, hipStream_t stream);
// fp32 on the matrix cores (exact products): K, N and strides multiples of 4, 16-byte aligned
bool m_grouped_f32_mfma_supported(const MGemmArgs& g);
int launch_m_grouped_f32_mfma(const MGemmArgs& g, hipStream_t stream);
bool k_grouped_f32_mfma_supported(const KGemmArgs& g);
int launch_k_grouped_f32_mfma(const KGemmArgs& g, hipStream_t stream);
bool k_grouped_mfma_supported(const KGemmArgs& g);
int launch_k_grouped_mfma(const KGemmArgs& g, hipStream_t stream);
// The tile-queue set of `stream` on the current device (16 words of a __device__ array that
// the persistent GEMM kernels draw work item ids from; nullptr while the stream is being
// captured: ids are then taken in strides of the grid) and the device's compute-unit count.
int tile_queue_set_of(hipStream_t stream, unsigned** queue, int* cus);
int launch_row_gather_kmajor(const void* src, int64_t src_rows, int64_t src_stride, const void* idx,
                             int idx_bytes, int idx_div, const int32_t* group_indices, int E,
                             int64_t P, void* dst, int64_t ld_dst, int64_t features, int dtype,
                             hipStream_t stream);

}  // namespace moe
