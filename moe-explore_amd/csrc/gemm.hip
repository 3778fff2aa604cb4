// Entry points of the grouped GEMMs: argument checks and the choice between the
// MFMA kernels and the scalar-FMA kernel.
#include "gemm.h"

using namespace moe;

extern "C" int moe_m_grouped_gemm(const void* a, int64_t a_rows, int64_t lda, const void* w,
                                  int64_t ldw_e, int64_t ldw_k, int64_t ldw_n, void* c,
                                  int64_t c_rows, int64_t ldc, void* preact, int64_t ld_preact,
                                  const int32_t* group_indices, const void* indices,
                                  int idx_bytes, const void* scales, int E, int64_t K, int64_t N,
                                  int topk, int flags, int epilogue, int dtype, int ksplit,
                                  int64_t c_split_stride, moe_stream_t stream) {
  clear_error();
  MOE_REQUIRE(dtype_bytes(dtype) != 0, "unknown dtype %d", dtype);
  MOE_REQUIRE(epilogue >= MOE_ACT_NONE && epilogue <= MOE_ACT_GEGLU, "unknown epilogue %d",
              epilogue);
  MOE_REQUIRE(E >= 1 && K >= 0 && N >= 0 && topk >= 1, "bad sizes E=%d K=%lld N=%lld topk=%d", E,
              (long long)K, (long long)N, topk);
  MOE_REQUIRE(a_rows >= 0 && c_rows >= 0, "negative row count");
  MOE_REQUIRE((flags & ~15) == 0, "unknown flag bits 0x%x", flags);
  MOE_REQUIRE(ksplit >= 1, "ksplit must be >= 1, got %d", ksplit);
  const bool gather = flags & MOE_GEMM_GATHER_A, scatter = flags & MOE_GEMM_SCATTER_C,
             scatter_add = flags & MOE_GEMM_SCATTER_ADD, save = flags & MOE_GEMM_SAVE_PREACT;
  MOE_REQUIRE(!(scatter && scatter_add), "SCATTER_C and SCATTER_ADD exclude each other");
  MOE_REQUIRE(!(gather && scatter_add), "GATHER_A with SCATTER_ADD is not supported");
  const bool glu = act_is_glu(epilogue);
  MOE_REQUIRE(!glu || N % 2 == 0, "a GLU epilogue needs an even N, got %lld", (long long)N);
  MOE_REQUIRE(group_indices != nullptr, "group_indices is null");
  const int64_t P = gather ? c_rows : a_rows;
  MOE_REQUIRE(P <= 0x7fffffff, "too many rows");
  if (gather || scatter || scatter_add) {
    // (an empty batch has an empty index array, whose pointer may be null)
    MOE_REQUIRE(indices != nullptr || P == 0, "gather/scatter needs indices");
    MOE_REQUIRE(idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8, got %d", idx_bytes);
  }
  if (P == 0 || N == 0) return MOE_OK;
  MOE_REQUIRE(a != nullptr && w != nullptr && c != nullptr, "null operand");
  MOE_REQUIRE(a_rows > 0 && c_rows > 0, "empty operand with non-empty groups");
  MOE_REQUIRE(!save || preact != nullptr, "SAVE_PREACT needs preact");
  const int64_t width = glu ? N / 2 : N;
  MOE_REQUIRE(lda >= K && ldc >= width, "row stride smaller than the row");
  MOE_REQUIRE(!save || ld_preact >= N, "preact row stride smaller than N");

  MGemmArgs g{a,     a_rows,        lda,     w,         ldw_e,  ldw_k, ldw_n, c,
              c_rows, ldc,          preact,  ld_preact, group_indices, indices, idx_bytes,
              scales, E,            K,       N,         topk,   flags, epilogue, dtype, P,
              FastDiv(static_cast<uint32_t>(topk)), ksplit, c_split_stride};
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (ksplit > 1) {
    // split K: only the direct-to-LDS MFMA kernel, and only where partial sums can be
    // added afterwards (no epilogue, plain or row-scatter store)
    MOE_REQUIRE(ksplit <= 8, "ksplit must be in [1,8], got %d", ksplit);
    if (epilogue != MOE_ACT_NONE || save || scatter_add ||
        !m_grouped_mfma_supported(g) || K % (64 * ksplit) != 0)
      return fail(MOE_ERR_UNSUPPORTED, "split K needs the MFMA kernel, no epilogue and K %% (64*ksplit) == 0");
    MOE_REQUIRE(c_split_stride >= (c_rows - 1) * ldc + N, "c_split_stride smaller than one copy of c");
    return launch_m_grouped_mfma_dma(g, s);
  }
  // Without an activation the saved pre-activation IS the output (same rows: it is kept
  // in sorted order, which excludes the scatter modes).  The kernels then store c only
  // and the copy is made here; their epilogues carry no second store for this case.
  const bool copy_preact = save && epilogue == MOE_ACT_NONE && !scatter && !scatter_add;
  if (copy_preact) g.flags &= ~MOE_GEMM_SAVE_PREACT;
  int rc;
  if (m_grouped_mfma_supported(g)) rc = launch_m_grouped_mfma(g, s);
  else if (m_grouped_f32_mfma_supported(g)) rc = launch_m_grouped_f32_mfma(g, s);
  else rc = launch_m_grouped_generic(g, s);
  if (rc != MOE_OK || !copy_preact) return rc;
  const size_t esz = dtype_bytes(dtype);
  hipError_t err = hipMemcpy2DAsync(preact, static_cast<size_t>(ld_preact) * esz, c,
                                    static_cast<size_t>(ldc) * esz, static_cast<size_t>(N) * esz,
                                    static_cast<size_t>(P), hipMemcpyDeviceToDevice, s);
  if (err != hipSuccess)
    return fail(MOE_ERR_HIP, "copy of the output into preact: %s", hipGetErrorString(err));
  return MOE_OK;
}

extern "C" int moe_m_grouped_gemm_glu_bwd(const void* a, int64_t a_rows, int64_t lda, const void* w,
                                          int64_t ldw_e, int64_t ldw_k, int64_t ldw_n,
                                          const void* h, int64_t ldh, void* dh, int64_t lddh,
                                          void* y_scaled, int64_t ldys, float* dscale,
                                          const int32_t* group_indices, const void* indices,
                                          int idx_bytes, const void* scales, int64_t P, int E,
                                          int64_t K, int64_t N, int topk, int flags, int act,
                                          int dtype, moe_stream_t stream) {
  clear_error();
  MOE_REQUIRE(dtype == MOE_DTYPE_BF16 || dtype == MOE_DTYPE_F16, "16-bit dtypes only, got %d", dtype);
  MOE_REQUIRE(act == MOE_ACT_SWIGLU || act == MOE_ACT_GEGLU, "a GLU activation is needed, got %d", act);
  MOE_REQUIRE(E >= 1 && K >= 0 && N >= 0 && topk >= 1 && P >= 0 && a_rows >= 0,
              "bad sizes E=%d K=%lld N=%lld topk=%d P=%lld", E, (long long)K, (long long)N, topk,
              (long long)P);
  MOE_REQUIRE((flags & ~MOE_GEMM_GATHER_A) == 0, "only MOE_GEMM_GATHER_A is allowed, got 0x%x", flags);
  MOE_REQUIRE(group_indices != nullptr, "group_indices is null");
  MOE_REQUIRE(indices == nullptr || idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8");
  MOE_REQUIRE(!(flags & MOE_GEMM_GATHER_A) || indices != nullptr || P == 0, "GATHER_A needs indices");
  MOE_REQUIRE(P <= 0x7fffffff, "too many rows");
  if (P == 0 || N == 0) return MOE_OK;
  MOE_REQUIRE(a && w && h && dh && y_scaled, "null operand");
  MOE_REQUIRE(a_rows > 0, "empty operand with non-empty groups");
  MOE_REQUIRE(lda >= K && ldh >= 2 * N && lddh >= 2 * N && ldys >= N, "row stride smaller than the row");
  MGemmArgs g{a,      a_rows, lda,      w,    ldw_e,         ldw_k,   ldw_n,     dh,
              P,      lddh,   y_scaled, ldys, group_indices, indices, idx_bytes, scales,
              E,      K,      N,        topk, flags | MOE_GEMM_GLU_BWD, act, dtype, P,
              FastDiv(static_cast<uint32_t>(topk)), 1, 0};
  g.h = h;
  g.ldh = ldh;
  g.dscale = dscale;
  if (!m_grouped_mfma_supported(g) || !m_grouped_mfma_dma_supported(g) ||
      !(g.ldw_k == 1 && g.ldw_n % 8 == 0))
    return fail(MOE_ERR_UNSUPPORTED, "fused GLU backward: needs the direct-to-LDS MFMA kernel with "
                                     "K-contiguous weights (K %% 64 == 0, aligned rows)");
  return launch_m_grouped_mfma_dma(g, static_cast<hipStream_t>(stream));
}

extern "C" int moe_k_grouped_gemm(const void* a, int64_t a_rows, int64_t lda, const void* b,
                                  int64_t b_rows, int64_t ldb, void* out,
                                  const int32_t* group_indices, const void* indices,
                                  int idx_bytes, int E, int64_t Ka, int64_t Nb, int topk,
                                  int flags, int dtype, moe_stream_t stream) {
  clear_error();
  MOE_REQUIRE(dtype_bytes(dtype) != 0, "unknown dtype %d", dtype);
  MOE_REQUIRE(E >= 1 && Ka >= 0 && Nb >= 0 && topk >= 1, "bad sizes");
  MOE_REQUIRE(a_rows >= 0 && b_rows >= 0, "negative row count");
  MOE_REQUIRE((flags & ~15) == 0, "unknown flag bits 0x%x", flags);
  const bool ga = flags & MOE_KGEMM_GATHER_A, gb = flags & MOE_KGEMM_GATHER_B;
  const bool ka = flags & MOE_KGEMM_A_KMAJOR, kb = flags & MOE_KGEMM_B_KMAJOR;
  MOE_REQUIRE(!(ga && gb), "only one operand can be gathered");
  MOE_REQUIRE(!(ka && kb) && !((ka || kb) && (ga || gb)),
              "at most one operand is K-major, and then nothing is gathered");
  MOE_REQUIRE(group_indices != nullptr, "group_indices is null");
  if (ga || gb) {
    // (an empty batch has an empty index array, whose pointer may be null)
    MOE_REQUIRE(indices != nullptr || (ga ? b_rows : a_rows) == 0, "gather needs indices");
    MOE_REQUIRE(idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8, got %d", idx_bytes);
  }
  if (Ka == 0 || Nb == 0) return MOE_OK;
  MOE_REQUIRE(out != nullptr, "out is null");
  // (a K-major operand is [features, columns]: its "rows" argument counts columns)
  const int64_t P = (ga || ka) ? b_rows : a_rows;
  MOE_REQUIRE(P <= 0x7fffffff, "too many rows");
  MOE_REQUIRE(P == 0 || (a != nullptr && b != nullptr && a_rows > 0 && b_rows > 0),
              "null or empty operand");
  if (ka || kb) {
    const int64_t need = moe_kmajor_columns(P, E);
    MOE_REQUIRE((ka ? a_rows : b_rows) >= need && (ka ? lda : ldb) >= need,
                "a K-major operand of %lld positions and %d experts has %lld columns",
                (long long)P, E, (long long)need);
    MOE_REQUIRE(ka ? ldb >= Nb : lda >= Ka, "row stride smaller than the row");
  } else {
    MOE_REQUIRE(lda >= Ka && ldb >= Nb, "row stride smaller than the row");
  }
  KGemmArgs g{a, a_rows, lda, b, b_rows, ldb, out, group_indices, indices, idx_bytes,
              E, Ka,     Nb,  topk, flags, dtype, P, FastDiv(static_cast<uint32_t>(topk))};
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (k_grouped_mfma_supported(g)) return launch_k_grouped_mfma(g, s);
  if (k_grouped_f32_mfma_supported(g)) return launch_k_grouped_f32_mfma(g, s);
  if (ka || kb)
    return fail(MOE_ERR_UNSUPPORTED, "K-major operands need the MFMA kernel (16-bit dtype, widths and "
                                     "strides multiples of 8, 16-byte aligned pointers)");
  return launch_k_grouped_generic(g, s);
}

extern "C" int64_t moe_kmajor_columns(int64_t P, int E) {
  if (P < 0 || E < 1) return 0;
  return 64 * (P / 64 + E + 1);
}

extern "C" int moe_row_gather_kmajor(const void* src, int64_t src_rows, int64_t src_stride,
                                     const void* idx, int idx_bytes, int idx_div,
                                     const int32_t* group_indices, int E, int64_t P, void* dst,
                                     int64_t ld_dst, int64_t features, int dtype,
                                     moe_stream_t stream) {
  clear_error();
  MOE_REQUIRE(dtype == MOE_DTYPE_BF16 || dtype == MOE_DTYPE_F16, "16-bit dtypes only, got %d", dtype);
  MOE_REQUIRE(idx_bytes == 4 || idx_bytes == 8, "idx_bytes must be 4 or 8, got %d", idx_bytes);
  MOE_REQUIRE(idx_div >= 1 && E >= 1 && P >= 0 && P <= 0x7fffffff && features >= 0 && src_rows >= 0,
              "bad sizes");
  MOE_REQUIRE(group_indices != nullptr, "group_indices is null");
  if (P == 0 || features == 0) return MOE_OK;
  MOE_REQUIRE(src && idx && dst && src_rows > 0, "null or empty operand");
  MOE_REQUIRE(ld_dst >= moe_kmajor_columns(P, E), "dst rows are shorter than moe_kmajor_columns(P, E)");
  if (features % 8 != 0 || src_stride % 8 != 0 || ld_dst % 8 != 0 || !aligned16(src) || !aligned16(dst))
    return fail(MOE_ERR_UNSUPPORTED, "row_gather_kmajor moves 16 bytes at a time: widths and strides "
                                     "must be multiples of 8 elements, pointers 16-byte aligned");
  return launch_row_gather_kmajor(src, src_rows, src_stride, idx, idx_bytes, idx_div, group_indices, E, P,
                                  dst, ld_dst, features, dtype, static_cast<hipStream_t>(stream));
}
