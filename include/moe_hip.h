/*
 * moe_hip.h -- C ABI of libmoe_hip.so: the MoE-layer hot path of moe-explore
 * as hand-written HIP kernels for gfx950 (MI355X).
 *
 * Conventions for every entry point:
 *   - plain C types only; device buffers are raw pointers owned by the caller
 *     and must stay alive until `stream` has passed the call;
 *   - returns 0 on success, a negative MOE_ERR_* code otherwise (the text of
 *     the last error of the calling thread is moe_last_error_string());
 *   - never allocates device memory, never synchronises the stream, never
 *     reads device data on the host (ragged group sizes are resolved on the
 *     device, as in m_grouped_gemm.py:226-227 of the reference);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *
 * Index vocabulary (reference expert_permute.py:19-41, m_grouped_gemm.py:104-109):
 *   T tokens, topk experts per token, R = T*topk routed rows; a flat slot id
 *   s = t*topk + j; p a position in expert-sorted order; indices[p] = s;
 *   group_indices[e]..group_indices[e+1] is expert e's range of positions.
 */
#ifndef MOE_HIP_H
#define MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* moe_stream_t;

/* every entry point is exported; everything else in the library is hidden */
#if defined(__GNUC__)
#define MOE_API __attribute__((visibility("default")))
#else
#define MOE_API
#endif

/* status codes */
#define MOE_OK 0
#define MOE_ERR_INVALID_ARG (-1) /* null pointer, negative size, bad enum     */
#define MOE_ERR_UNSUPPORTED (-2) /* legal but not implemented for these args  */
#define MOE_ERR_WORKSPACE (-3)   /* workspace missing or too small            */
#define MOE_ERR_HIP (-4)         /* a HIP runtime call or launch failed       */

/* element types */
#define MOE_DTYPE_F32 0
#define MOE_DTYPE_F16 1
#define MOE_DTYPE_BF16 2

/* epilogues of the grouped GEMM; names follow triton_kernels/activation.py:38-45 */
#define MOE_ACT_NONE 0
#define MOE_ACT_SILU 1
#define MOE_ACT_GELU 2        /* exact, erf */
#define MOE_ACT_APPROX_GELU 3 /* tanh form  */
#define MOE_ACT_SWIGLU 4      /* gate = even columns, up = odd columns */
#define MOE_ACT_GEGLU 5

/* flags of moe_m_grouped_gemm */
#define MOE_GEMM_GATHER_A 1        /* A row of position p is a[indices[p] / topk]      */
#define MOE_GEMM_SCATTER_C 2       /* C row of position p is stored at c[indices[p]]   */
#define MOE_GEMM_SCATTER_ADD 4     /* c32[indices[p] / topk] += w * row, fp32 atomics;
                                      w = scales[indices[p]] or 1 when scales is NULL  */
#define MOE_GEMM_SAVE_PREACT 8     /* also store the pre-activation rows to `preact`   */

/* flags of moe_k_grouped_gemm */
#define MOE_KGEMM_GATHER_A 1 /* A row of position p is a[indices[p] / topk] */
#define MOE_KGEMM_GATHER_B 2 /* B row of position p is b[indices[p] / topk] */
#define MOE_KGEMM_A_KMAJOR 4 /* a is [Ka, columns], written by moe_row_gather_kmajor */
#define MOE_KGEMM_B_KMAJOR 8 /* b is [Nb, columns], written by moe_row_gather_kmajor */

/* Library version: major*10000 + minor*100 + patch. */
MOE_API int moe_version(void);

/* Text of the last error returned to the calling thread ("" if none). */
MOE_API const char* moe_last_error_string(void);

/*
 * Routing preprocessing: replaces get_token_indices (expert_permute.py:19-41).
 *   expert_ids  [R] expert id of every flat slot, int32 or int64 (idx_bytes 4|8)
 *   indices_out [R] int64: slot ids in expert-sorted order, ascending slot id
 *                   inside an expert (the stable sort of expert_ids)
 *   group_indices_out [E+1] int32: 0 followed by the inclusive prefix sum of the
 *                   per-expert counts (zero_prefix=True form, :31-34)
 *   inclusive_out [E] int64 or NULL: the inclusive prefix sum alone
 *                   (zero_prefix=False form, :36)
 * Ids outside [0,E) are a caller error; they are counted into no expert and
 * their slots are not written to indices_out.
 * Workspace: moe_route_workspace_bytes(R, E) bytes, 16-byte aligned.
 */
MOE_API size_t moe_route_workspace_bytes(int64_t R, int E);
MOE_API int moe_route_preprocess(const void* expert_ids, int idx_bytes, int64_t R, int E,
                         int64_t* indices_out, int32_t* group_indices_out,
                         int64_t* inclusive_out, void* workspace, size_t workspace_bytes,
                         moe_stream_t stream);

/*
 * moe_route_preprocess without a workspace and without any allocation.  No counterpart in
 * the reference: it exists for callers that cannot allocate device memory -- code under HIP
 * graph capture, serving loops with a fixed memory plan, harnesses that forbid hipMalloc --
 * and so cannot provide the workspace either.  Same results as moe_route_preprocess, bit for
 * bit.  The per-chunk counts live in a buffer of moe_route_noalloc_max_bytes() bytes (4 MiB)
 * that is part of the library image on every device: calls with
 * moe_route_workspace_bytes(R, E) above that (ceil(R / 512) * E > 2^20) return
 * MOE_ERR_WORKSPACE.  All calls on one device share that buffer, and nothing in it has to be
 * cleared between calls.  Eager calls cannot race on it: calls on one stream are ordered, and a
 * call on another stream than the call before makes its stream wait (hipStreamWaitEvent) for that
 * call's launches, so calls from several streams run one after the other.  Under graph capture
 * nothing is waited for or recorded and the captured launches keep using that one buffer:
 * replays of a graph that holds this call must not overlap each other or an eager call on the
 * same device (replays launched into one stream are ordered and safe).  The first call on a
 * device looks up the buffer's address and creates the event; it is refused with MOE_ERR_HIP
 * while its stream is being captured: make one call (R = 0 will do) before the capture begins.
 */
MOE_API size_t moe_route_noalloc_max_bytes(void);
MOE_API int moe_route_preprocess_noalloc(const void* expert_ids, int idx_bytes, int64_t R, int E,
                                 int64_t* indices_out, int32_t* group_indices_out,
                                 int64_t* inclusive_out, moe_stream_t stream);

/*
 * Row gather / row scatter: replace row_gather and row_scatter
 * (triton_kernels/row_gather_scatter.py:36-58, :91-116).
 *   gather : dst[r, :] = src[idx[r] / idx_div, :]   r < rows_out, indices may repeat
 *   scatter: dst[idx[r], :] = src[r, :]             r < rows, idx a permutation
 * Rows are `cols` elements of elt_bytes (2 or 4) bytes; row strides in elements,
 * unit column stride.  idx is int32 or int64 (idx_bytes); idx_div >= 1 lets the
 * caller pass slot ids and gather by token (expert_permute.py:51).
 * Indices are clamped into [0, src_rows) / [0, dst_rows) instead of faulting.
 */
MOE_API int moe_row_gather(const void* src, int64_t src_rows, int64_t src_stride, const void* idx,
                   int idx_bytes, int idx_div, void* dst, int64_t dst_stride, int64_t rows_out,
                   int64_t cols, int elt_bytes, moe_stream_t stream);
MOE_API int moe_row_scatter(const void* src, int64_t src_stride, const void* idx, int idx_bytes,
                    void* dst, int64_t dst_rows, int64_t dst_stride, int64_t rows,
                    int64_t cols, int elt_bytes, moe_stream_t stream);

/*
 * Top-k weighted combine: replaces scale_and_reduce
 * (functional/scale_and_reduce.py:3-5):
 *   out[t, :] = sum_j scales[t*topk + j] * in[t*topk + j, :], summed in fp32.
 * in [T*topk, n] and out [T, n] in `dtype`, scales [T*topk] in `dtype`; a NULL
 * scales sums the topk rows unweighted (the dX reduction of the backward pass).
 * nsplit > 1 also adds the nsplit partial copies of `in` that a split-K grouped GEMM
 * left split_stride elements apart.
 */
MOE_API int moe_scale_and_reduce(const void* in, int64_t in_stride, const void* scales, void* out,
                         int64_t out_stride, int64_t T, int topk, int64_t n, int dtype,
                         int nsplit, int64_t split_stride, moe_stream_t stream);

/*
 * fp32 -> dtype conversion of a [rows, cols] matrix; finishes the fused
 * scatter-add combine, whose accumulator is fp32.
 */
MOE_API int moe_cast_from_f32(const float* src, int64_t src_stride, void* dst, int64_t dst_stride,
                      int64_t rows, int64_t cols, int dtype, moe_stream_t stream);

/*
 * M-grouped GEMM: replaces m_grouped_gemm (triton_kernels/m_grouped_gemm.py:332-393)
 * and its kernels (:33-267), epilogues (activation.py:5-45, epilogue_split.py:4-44).
 * For every expert e and position p in [group_indices[e], group_indices[e+1]):
 *     row = epilogue( a[arow(p), :] @ w[e] )          fp32 accumulate
 *   arow(p) = indices[p] / topk with MOE_GEMM_GATHER_A, else p
 *   row is stored at c[p], at c[indices[p]] (MOE_GEMM_SCATTER_C), or added into the
 *   fp32 matrix c at row indices[p] / topk scaled by scales[indices[p]]
 *   (MOE_GEMM_SCATTER_ADD: the down projection fused with the top-k combine of
 *   functional/topk_moe.py:36-54; c must be zeroed by the caller).
 *   a       [a_rows, K], row stride lda elements, unit column stride
 *   w       [E, K, N], element strides (ldw_e, ldw_k, ldw_n); a transposed view
 *           (ldw_k == 1) is how the backward pass multiplies by w[e]^T
 *   c       `dtype`, or float with MOE_GEMM_SCATTER_ADD; width N, or N/2 after a
 *           GLU epilogue; row stride ldc
 *   preact  with MOE_GEMM_SAVE_PREACT: [c_rows, N] in `dtype`, row stride ld_preact,
 *           receives the rows before the epilogue (saved for the backward pass)
 *   indices int32/int64 (idx_bytes) or NULL; scales [R] in `dtype` or NULL
 *   a_rows, c_rows: row counts of a and c, used to clamp positions and indices
 *   ksplit, c_split_stride: ksplit > 1 cuts K into ksplit equal parts that run as
 *           separate tiles (more, shorter tiles when the output has few of them);
 *           part i stores its partial product to c + i * c_split_stride elements and
 *           the caller adds the parts (moe_scale_and_reduce does).  MFMA kernel only,
 *           no epilogue; MOE_ERR_UNSUPPORTED otherwise.  Pass 1 and 0 for no split.
 * fp32 runs on fp32 MFMAs (exact products) when K, N and the strides are multiples of 4 and
 * the pointers 16-byte aligned.  Shapes the MFMA kernels do not cover (16-bit: K, N or strides
 * not multiples of 8; unaligned pointers) run on a scalar-FMA kernel with the same semantics.
 */
MOE_API int moe_m_grouped_gemm(const void* a, int64_t a_rows, int64_t lda, const void* w,
                       int64_t ldw_e, int64_t ldw_k, int64_t ldw_n, void* c, int64_t c_rows,
                       int64_t ldc, void* preact, int64_t ld_preact,
                       const int32_t* group_indices, const void* indices, int idx_bytes,
                       const void* scales, int E, int64_t K, int64_t N, int topk, int flags,
                       int epilogue, int dtype, int ksplit, int64_t c_split_stride,
                       moe_stream_t stream);

/*
 * K-grouped GEMM (expert weight gradients; no counterpart in the reference,
 * which is forward-only).  For every expert e:
 *     out[e] = sum over p in [group_indices[e], group_indices[e+1]) of
 *              a[arow(p), :]^T (outer) b[brow(p), :]          fp32 accumulate
 *   a [*, Ka], b [*, Nb] in `dtype` (row strides lda, ldb); out [E, Ka, Nb] in
 *   `dtype`, contiguous.  Experts with no rows get zeros.
 * MOE_KGEMM_A_KMAJOR / MOE_KGEMM_B_KMAJOR (one of them, no gather flags): that operand is
 * given feature-major, [Ka or Nb, columns] with row stride lda / ldb and a_rows / b_rows
 * counting its columns (>= moe_kmajor_columns(P, E)), in the layout moe_row_gather_kmajor
 * writes.  The weight gradients' small operand is a set of gathered token rows that has
 * to be materialised anyway; feature-major, the kernel reads it from LDS with plain
 * 16-byte loads instead of transpose loads (16-bit dtypes, MFMA kernel only:
 * MOE_ERR_UNSUPPORTED otherwise).
 *
 * moe_row_gather_kmajor: dst[f, qs(e) + (p - lo(e))] = src[idx[p] / idx_div, f] for every
 * position p of expert e (lo(e) = group_indices[e]), where qs(e) = 64 * (lo(e) / 64 + e):
 * every expert's segment starts on a multiple of 64 columns and is followed by zeros up to
 * the next multiple of 64.  dst is [features, ld_dst] with ld_dst >= moe_kmajor_columns(P, E)
 * = 64 * (P / 64 + E + 1); columns outside the segments and their zero fill are not written.
 * No counterpart in the reference (forward-only).
 */
MOE_API int64_t moe_kmajor_columns(int64_t P, int E);
MOE_API int moe_row_gather_kmajor(const void* src, int64_t src_rows, int64_t src_stride,
                          const void* idx, int idx_bytes, int idx_div,
                          const int32_t* group_indices, int E, int64_t P, void* dst,
                          int64_t ld_dst, int64_t features, int dtype, moe_stream_t stream);
MOE_API int moe_k_grouped_gemm(const void* a, int64_t a_rows, int64_t lda, const void* b,
                       int64_t b_rows, int64_t ldb, void* out,
                       const int32_t* group_indices, const void* indices, int idx_bytes,
                       int E, int64_t Ka, int64_t Nb, int topk, int flags, int dtype,
                       moe_stream_t stream);

/*
 * Gradient of the expert activation (no counterpart in the reference).
 *   h  [R, N]   saved pre-activation rows (N = 2*ff for GLU, gate/up interleaved)
 *   dy [R, No]  gradient of the activation output (No = N/2 for GLU, else N)
 *   dh [R, N]   = dy * act'(h)                            (written)
 *   row_scale [R] or NULL: dh row p is additionally multiplied by
 *           row_scale[idx(p)] (the routing weight of the row; idx(p) = indices[p]
 *           when indices is given, else p)
 *   y_scaled [R, No] or NULL: receives row_scale * act(h), the operand of the
 *           down-projection weight gradient
 *   dscale [R] fp32 or NULL: dscale[idx(p)] = <dy[p], act(h[p])>, the gradient of
 *           the routing weight
 * MOE_ACT_NONE is the identity (act' = 1): experts without an activation
 * (MLPParams.activation = None, params.py:11-15) still need the row scaling,
 * row_scale * h and dscale.
 */
MOE_API int moe_act_bwd(const void* h, int64_t ldh, const void* dy, int64_t lddy, void* dh,
                int64_t lddh, const void* row_scale, const void* indices, int idx_bytes,
                void* y_scaled, int64_t ldy, float* dscale, int64_t R, int64_t N, int act,
                int dtype, moe_stream_t stream);

/*
 * Fused GLU backward (no counterpart in the reference, which is forward-only): the grouped
 * product G[p, :] = a[arow(p), :] @ w[e(p)] (as moe_m_grouped_gemm with flags
 * MOE_GEMM_GATHER_A or 0; here the gradient of the GLU output, dOut @ W2[e]^T, scale left
 * out) is not stored; with (gate, up) = h[p, 2j], h[p, 2j+1], y = act(gate) * up and
 * s = scales[p] (1 without scales; here the routing weights are given by POSITION, i.e.
 * already permuted, so that the epilogue needs no index lookup):
 *     dh[p, 2j] = s G[p, j] up act'(gate)      dh[p, 2j+1] = s G[p, j] act(gate)
 *     y_scaled[p, j] = s y                     dscale[p] += sum_j G[p, j] y
 * i.e. moe_m_grouped_gemm followed by moe_act_bwd in one launch.  h [P, 2N], dh [P, 2N],
 * y_scaled [P, N], scales [P] and dscale [P] are in sorted position order; dscale (fp32, or
 * NULL) is accumulated with atomics and must be zeroed by the caller.  act is
 * MOE_ACT_SWIGLU or MOE_ACT_GEGLU.
 * MOE_ERR_UNSUPPORTED unless the direct-to-LDS MFMA kernel can take the call: 16-bit dtype,
 * K-contiguous weights (ldw_k == 1), K a multiple of 64, N of 8, 16-byte aligned rows; the
 * caller then runs the two calls separately.
 */
MOE_API int moe_m_grouped_gemm_glu_bwd(const void* a, int64_t a_rows, int64_t lda, const void* w,
                               int64_t ldw_e, int64_t ldw_k, int64_t ldw_n, const void* h,
                               int64_t ldh, void* dh, int64_t lddh, void* y_scaled, int64_t ldys,
                               float* dscale, const int32_t* group_indices, const void* indices,
                               int idx_bytes, const void* scales, int64_t P, int E, int64_t K,
                               int64_t N, int topk, int flags, int act, int dtype,
                               moe_stream_t stream);

/*
 * fp8 inference variant (no counterpart in the reference).
 * moe_quantize_rows_fp8: per-row dynamic quantisation to OCP e4m3:
 *     scale[r] = max(amax |x[r, :]|, tiny) / 448,  q[r, :] = e4m3(x[r, :] / scale[r])
 * moe_m_grouped_gemm_fp8: as moe_m_grouped_gemm with
 *     a  [a_rows, K] e4m3 with a_scale [a_rows] fp32 (per row)
 *     w  [E, N, K] e4m3, K contiguous, with w_scale [E, N] fp32 (per output channel)
 *     row = epilogue( (a @ w[e]^T) * a_scale[arow] * w_scale[e, :] ), c in out_dtype.
 * flags: MOE_GEMM_GATHER_A, MOE_GEMM_SCATTER_C and MOE_FP8_W_TILED.  With the last one w is
 * tile-major, [E][ceil(N/256)][K/128] blocks of 32 KiB, block (e, nt, kt) holding rows
 * n = 256*nt .. +255 (zeros past N) and bytes k = 128*kt .. +127 of w[e] as
 *     block[128*r + 16*(c ^ ((r >> 1) & 7)) + b] = w[e][256*nt + r][128*kt + 16*c + b]
 * (r < 256, c < 8, b < 16): the image of the kernel's LDS tile, so that a K step is one
 * linear 32 KiB read and a column tile one sequential stream from HBM.
 * ksplit, c_split_stride: as for moe_m_grouped_gemm (K cut into parts that store to their
 * own copy of c; only without an activation, K % (128 * ksplit) == 0).
 * MOE_ERR_UNSUPPORTED for K not a multiple of 128, N not a multiple of 8, rows that are not
 * 16-byte aligned, and for a gathered token matrix (a_rows * lda bytes) or the weights of one
 * expert (N * K bytes) of 4 GiB or more: the kernel addresses both with 32-bit offsets.
 */
#define MOE_FP8_W_TILED 4
MOE_API int moe_quantize_rows_fp8(const void* x, int64_t ldx, void* q, int64_t ldq, float* scale,
                          int64_t rows, int64_t cols, int dtype, moe_stream_t stream);
MOE_API int moe_m_grouped_gemm_fp8(const void* a, const float* a_scale, int64_t a_rows, int64_t lda,
                           const void* w, const float* w_scale, void* c, int64_t c_rows,
                           int64_t ldc, const int32_t* group_indices, const void* indices,
                           int idx_bytes, const void* scales, int E, int64_t K, int64_t N,
                           int topk, int flags, int epilogue, int out_dtype, int ksplit,
                           int64_t c_split_stride, moe_stream_t stream);

/*
 * Fused router: replaces topk_router (router.py:17-35) and ernie_router (router.py:37-54),
 * which the reference runs as a matmul, a softmax, a top-k, a sum, a division and a cast.
 *   logits = x @ w            x [T, d] (row stride ldx), w [d, E] (strides ldw_k, ldw_e)
 *   top-k router: logits are rounded to the dtype of x (:22).
 *     MOE_ROUTER_SOFTMAX_FIRST set: p = softmax_fp32(logits), the topk largest p are the
 *       scores (:23-26); else the topk largest logits, scores = softmax_fp32 over them (:28-29)
 *     MOE_ROUTER_NORMALIZE: scores /= sum(scores) (:31-32)
 *   MOE_ROUTER_ERNIE: fp32 logits and softmax, selection by p + bias[e], scores = p of the
 *     selected experts / max(sum, 1e-12) (:44-52); w must be fp32 (:42).
 *   scores [T, topk] in the dtype of x; topk_indices [T, topk] int64, in descending order of
 *   the selection key, ties to the lower expert id (the reference asks for sorted=False, so
 *   the order inside a token is unspecified there); logits_out [T, E] fp32 or NULL: the
 *   logits the scores were computed from, which moe_router_bwd takes.
 * x and w have the same 16-bit dtype (MFMA on 16-bit operands, fp32 accumulation), or w is
 * fp32 or both are (fp32 operands).  MOE_ERR_UNSUPPORTED for more than 512 experts,
 * top-k above 16, or x rows that cannot be read 16 bytes at a time.
 * Workspace: moe_router_workspace_bytes(d, E, x_dtype, w_dtype) bytes, 16-byte aligned (a
 * K-contiguous copy of w that the call writes first).
 *
 * moe_router_bwd: dlogits [T, E] (out_dtype) = gradient of sum(scores * dscores) with respect
 * to the logits, for the selection in topk_indices; dscores [T, topk] in g_dtype.  No
 * counterpart in the reference, which is forward-only.
 */
#define MOE_ROUTER_SOFTMAX_FIRST 1
#define MOE_ROUTER_NORMALIZE 2
#define MOE_ROUTER_ERNIE 4
MOE_API size_t moe_router_workspace_bytes(int64_t d, int E, int x_dtype, int w_dtype);
MOE_API int moe_router_topk(const void* x, int64_t ldx, const void* w, int64_t ldw_k, int64_t ldw_e,
                    const float* bias, void* scores, int64_t* topk_indices, float* logits_out,
                    int64_t T, int64_t d, int E, int topk, int flags, int x_dtype, int w_dtype,
                    void* workspace, size_t workspace_bytes, moe_stream_t stream);
MOE_API int moe_router_bwd(const float* logits, const int64_t* topk_indices, const void* dscores,
                   void* dlogits, int64_t T, int E, int topk, int flags, int g_dtype,
                   int out_dtype, moe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_HIP_H */
