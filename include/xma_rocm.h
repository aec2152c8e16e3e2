/*
 * xma_rocm.h - C ABI of libxma_rocm.so: the MI355X (gfx950) kernels behind
 * KernelBackend.rocm for XMA's MoE layer and continuous_count.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller (PyTorch's caching
 *     allocator in the Python host); the library allocates nothing.  What it keeps between calls: per-device
 *     constants looked up once (compute units, a kernel's raised LDS limit, the address of xma_rocm_route_static's
 *     scratch) and one process-wide switch, xma_rocm_route_set_rank_method;
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued on it and
 *     no entry point synchronises;
 *   - return value 0 = enqueued, negative = XMA_ROCM_E* (argument errors are
 *     detected before anything is launched; launch errors come from
 *     hipGetLastError right after the launch); xma_rocm_last_error() gives the
 *     message of the calling thread's last failure;
 *   - `dtype` is XMA_ROCM_BF16, XMA_ROCM_F16 or XMA_ROCM_F32 (fp32 accumulation in all);
 *   - leading dimensions (ld*) and expert strides are in ELEMENTS;
 *   - "grouped" order = position n in the expert-sorted list; "scattered" order
 *     = row sorted_scattered_idxs[n] of the flattened (T, k) selection.
 *
 * Citations are to the reference tree (xma/...), which each entry point replaces.
 */
#ifndef XMA_ROCM_H
#define XMA_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XMA_ROCM_ABI_VERSION 1

/* the library is built with hidden visibility; only these entry points are exported */
#define XMA_API __attribute__((visibility("default")))

#define XMA_ROCM_OK 0
#define XMA_ROCM_EINVAL (-1)       /* bad argument (null pointer, size, alignment) */
#define XMA_ROCM_EUNSUPPORTED (-2) /* shape or dtype the kernels do not cover */
#define XMA_ROCM_EWORKSPACE (-3)   /* workspace smaller than *_workspace_bytes */
#define XMA_ROCM_ELAUNCH (-4)      /* HIP reported an error at launch */

#define XMA_ROCM_BF16 0
#define XMA_ROCM_F16 1
#define XMA_ROCM_F32 2 /* exact fp32 kernels (v_mfma_f32_32x32x2_f32): parity runs and the fp32 points of the reference's test grid */

/* epilogues of xma_rocm_scatter2scatter */
#define XMA_ROCM_EPI_STORE 0      /* out = acc (optionally * row_scale) */
#define XMA_ROCM_EPI_SWIGLU 1     /* up-projection: out = z (pre-activation, may be NULL), aux = swiglu_packed(z) */
#define XMA_ROCM_EPI_SWIGLU_BWD 2 /* down-projection dX: aux = saved z, out = dz = swiglu_packed'(z) * (acc * row_scale) */

XMA_API int xma_rocm_abi_version(void);
XMA_API const char *xma_rocm_last_error(void);

/*
 * Histogram of ids in [0, bins): counts[b] += #{i : ids[i] == b}.  ids outside
 * the range are ignored.  Like the reference kernel the result is ACCUMULATED
 * into `counts`, which the caller zero-fills first.  `workspace` may be NULL;
 * with at least xma_rocm_continuous_count_workspace_bytes(n, bins) bytes large
 * inputs take a two-pass path (per-workgroup partial histograms, then one
 * reduction) instead of thousands of same-address device atomics.
 * Replaces _continuous_count_cuda, xma/functional/continuous_count/cuda_implementation.py:171-197
 * (called from xma/functional/continuous_count/__init__.py:43-45).
 */
XMA_API size_t xma_rocm_continuous_count_workspace_bytes(int64_t n, int32_t bins);
XMA_API int xma_rocm_continuous_count(const void *ids, int ids_are_int64, int64_t n, uint32_t *counts, int32_t bins,
                                      void *workspace, size_t workspace_bytes, void *stream);

/*
 * The same histogram with counts OVERWRITTEN instead of added to, so that the caller need not clear them (one launch
 * less per call): counts[b] = #{i : ids[i] == b}, b < bins <= 8192, ids outside the range ignored, n == 0 gives zeros.
 * Inputs of more than 4096 ids need xma_rocm_continuous_count_set_workspace_bytes(n, bins) bytes of workspace.
 * Same reference interface as xma_rocm_continuous_count (there the caller's torch.zeros, cuda_implementation.py callers
 * at xma/functional/continuous_count/__init__.py:41-45, is a launch of its own).
 */
XMA_API size_t xma_rocm_continuous_count_set_workspace_bytes(int64_t n, int32_t bins);
XMA_API int xma_rocm_continuous_count_set(const void *ids, int ids_are_int64, int64_t n, uint32_t *counts, int32_t bins,
                                  void *workspace, size_t workspace_bytes, void *stream);

/*
 * Routing in one op: counts, inclusive/exclusive expert offsets and the STABLE
 * expert-major permutation of the flattened top-k selection.
 * Replaces `selected_experts.flatten().sort()` + continuous_count + cumsum,
 * xma/layers/moe/__init__.py:210-217.
 *   ids                    (n,)  int32|int64 expert id of each (token, slot)
 *   counts                 (E,)  uint32, overwritten
 *   offsets_inclusive      (E,)  int64, cumsum(counts)
 *   offsets_exclusive      (E,)  int64, may be NULL
 *   sorted_expert_idxs     (n,)  same dtype as ids, may be NULL
 *   sorted_scattered_idxs  (n,)  int64
 * ids must lie in [0, E); E <= 2048.
 */
XMA_API size_t xma_rocm_route_workspace_bytes(int64_t n, int32_t num_experts);
/*
 * How the scatter kernel of xma_rocm_route finds the stable rank of an id among equal ids of its wave (process-wide,
 * takes effect with the next call): 0 (default) = value returned by an LDS atomic add, which gfx950 applies in lane
 * order; 1 = log2(E) wave ballots per 64 ids, which relies on no ordering property of the hardware.  Results are bit-identical; the switch exists so that the claim can be tested on any machine.
 */
XMA_API int xma_rocm_route_set_rank_method(int method);
XMA_API int xma_rocm_route(const void *ids, int ids_are_int64, int64_t n, int32_t num_experts, uint32_t *counts,
                   int64_t *offsets_inclusive, int64_t *offsets_exclusive, void *sorted_expert_idxs,
                   int64_t *sorted_scattered_idxs, void *workspace, size_t workspace_bytes, void *stream);

/*
 * xma_rocm_route without a workspace argument and without any allocation.  It has no counterpart in the reference; it
 * is for callers that cannot allocate device memory around the call (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  Same arguments, results and kernels as xma_rocm_route; the per-unit
 * histograms live in a device array that is part of the library image (1 MiB per GPU, held until the process ends).
 * Limit: ceil(n / 4096) * num_experts <= xma_rocm_route_static_max_units_times_experts() (= 262144; e.g. 4 Mi ids
 * over 256 experts); larger problems return XMA_ROCM_EWORKSPACE and must use xma_rocm_route.  All calls on one GPU
 * share that array: calls that overlap on one GPU (two streams, two threads) race and must be serialised by the caller.
 * The first call on a device looks up the array's address and raises a kernel's LDS limit, which are not stream
 * operations: make one ordinary call per device before capturing this entry point in a graph.
 */
XMA_API size_t xma_rocm_route_static_max_units_times_experts(void);
XMA_API int xma_rocm_route_static(const void *ids, int ids_are_int64, int64_t n, int32_t num_experts, uint32_t *counts,
                          int64_t *offsets_inclusive, int64_t *offsets_exclusive, void *sorted_expert_idxs,
                          int64_t *sorted_scattered_idxs, void *stream);

/*
 * Grouped GEMM with fused row gather / scatter: for every expert e and every
 * grouped position n in [offsets[e-1], offsets[e]):
 *     acc[n, :] = X[src(n), :K] @ B_e            B_e = W[e]^T  if !w_is_kn   (W[e] is (N, K), K contiguous)
 *                                                B_e = W[e]    if  w_is_kn   (W[e] is (K, N), N contiguous)
 *     src(n)  = n                         if x_grouped else sorted_scattered_idxs[n] / fan_out
 *     dst(n)  = n                         if y_grouped else sorted_scattered_idxs[n]
 * followed by the epilogue (XMA_ROCM_EPI_*).  row_scale (may be NULL) is a
 * vector indexed in scattered order (the flattened (T, k) router weights); a 16-bit scale is fetched as the aligned
 * 4-byte word around it, so the vector's allocation must extend to an even number of elements (a vector that starts
 * off a 4-byte boundary is accepted and takes a slower kernel).
 * Replaces scatter2scatter, xma/layers/moe/triton_implementation/scatter_kernel.py:137-183
 * (kernel :58-134), the separate activation pass xma/layers/moe/__init__.py:226
 * and its autograd backward, and the coefficient pass of `group`
 * (xma/layers/moe/triton_implementation/__init__.py:134-140).
 * Requirements: K % 8 == 0, N % 8 == 0, ld* % 8 == 0, 16-byte aligned bases.
 *   EPI_STORE       out (M, N)
 *   EPI_SWIGLU      out (M, N) = z or NULL;  aux (M, N/2) = h
 *   EPI_SWIGLU_BWD  aux (M, 2N) = z (read, grouped order);  out (M, 2N) = dz;  requires y_grouped
 * workspace (may be NULL): xma_rocm_scatter2scatter_workspace_bytes(M, N, K, E) bytes of scratch, 0 for launches of
 * many rounds of tiles.  With it the tiles of the last, partial round (the workgroups that would run while most
 * compute units idle) are split along K over the idle units and summed by a second kernel, in a fixed order: the
 * result does not depend on timing.  Without it every tile is computed by one workgroup.
 */
XMA_API size_t xma_rocm_scatter2scatter_workspace_bytes(int64_t M, int32_t N, int32_t K, int32_t num_experts);
XMA_API int xma_rocm_scatter2scatter(const void *X, int64_t ldx, const void *W, int64_t w_expert_stride, int64_t ldw,
                             int w_is_kn, const int64_t *sorted_scattered_idxs, const int64_t *expert_offsets,
                             void *out, int64_t ldo, void *aux, int64_t ldaux, const void *row_scale, int64_t M,
                             int32_t N, int32_t K, int32_t num_experts, int32_t fan_out, int x_grouped,
                             int y_grouped, int epilogue, int dtype, void *workspace,
                             size_t workspace_bytes, void *stream);

/*
 * xma_rocm_scatter2scatter with the experts' bias: acc[n, :] = bias[e(n), :N] + X[src(n), :K] @ B_e, the bias being the
 * first term of the fp32 sum (one rounding, like a linear layer with a bias), then the epilogue; a row scale multiplies
 * the biased row.  bias (E, N) with `bias_expert_stride` elements between experts (a multiple of 8), 16-byte aligned,
 * NULL = no bias; STORE and SWIGLU epilogues.  Covers the bias of Experts that the reference applies on its torch path
 * only, F.linear(x[e], weight[e], bias[e]) in xma/layers/moe/__init__.py:96-100 (its Triton path asserts there is none,
 * :53 and :75).
 */
XMA_API int xma_rocm_scatter2scatter_bias(const void *X, int64_t ldx, const void *W, int64_t w_expert_stride, int64_t ldw,
                                  int w_is_kn, const int64_t *sorted_scattered_idxs, const int64_t *expert_offsets,
                                  void *out, int64_t ldo, void *aux, int64_t ldaux, const void *row_scale,
                                  const void *bias, int64_t bias_expert_stride, int64_t M, int32_t N, int32_t K,
                                  int32_t num_experts, int32_t fan_out, int x_grouped, int y_grouped, int epilogue,
                                  int dtype, void *workspace, size_t workspace_bytes, void *stream);

/*
 * Gradient of the experts' bias: out[e, :N] = sum over the grouped rows n of expert e of A[src(n), :N] * scale, with
 * src(n) = n (sorted_scattered_idxs == NULL) or sorted_scattered_idxs[n] / fan_out, scale = row_scale[idx[n]] or 1.
 * fp32 sums in a fixed order; experts without rows get zeros; every element of out (E, N; row stride ldo) is written.
 * Replaces what autograd derives for the bias of F.linear in the reference's torch path
 * (xma/layers/moe/__init__.py:96-100).  N and the leading dimensions even, 8-byte aligned bases.
 */
XMA_API int xma_rocm_expert_column_sums(const void *A, int64_t lda, const int64_t *sorted_scattered_idxs, int32_t fan_out,
                                const void *row_scale, const int64_t *expert_offsets, void *out, int64_t ldo, int32_t N,
                                int32_t num_experts, int dtype, void *stream);

/*
 * dX of the down-projection with the SwiGLU backward in the epilogue (xma_rocm_scatter2scatter with
 * XMA_ROCM_EPI_SWIGLU_BWD, x_grouped = 0, y_grouped = 1) and one more output:
 *     dz (M, 2N)          = swiglu_packed'(z) * ((dY[idx[n] / fan_out] * row_scale[idx[n]]) @ B_e)
 *     scaled_act (M, N)   = swiglu_packed(z) * row_scale[idx[n]]        (grouped order)
 * scaled_act is the X operand of the down-projection's weight gradient when dY is taken unscaled through the index:
 * sum_n (w_n dy_n)^T h_n = sum_n dy_n^T (w_n h_n).  It replaces the scaled, grouped copy of dY that the reference
 * builds for that GEMM (`group` with coeff, xma/layers/moe/triton_implementation/__init__.py:134-140): k times fewer
 * bytes are written when H > N, and h need not be kept for the backward.  bf16 / fp16; row_scale and scaled_act required;
 * W[e] is (K, N) with N contiguous (the parameter of the down-projection as stored, B_e = W[e]).
 */
XMA_API int xma_rocm_down_projection_dx_swiglu(const void *dY, int64_t lddy, const void *W, int64_t w_expert_stride,
                                               int64_t ldw, const int64_t *sorted_scattered_idxs,
                                               const int64_t *expert_offsets, const void *z, int64_t ldz, void *dz,
                                               int64_t lddz, void *scaled_act, int64_t ld_scaled_act,
                                               const void *row_scale, int64_t M, int32_t N, int32_t K, int32_t num_experts,
                                               int32_t fan_out, int dtype, void *workspace, size_t workspace_bytes,
                                               void *stream);

/*
 * xma_rocm_scatter2scatter_bias / xma_rocm_down_projection_dx_swiglu for the few-token regime: the same arguments
 * (aux2 = the scaled activations of the latter, or NULL), the same results up to the order of the fp32 sums, bf16 / fp16
 * only.  With a handful of rows per expert the product is a stream over the weights.  W[e] as (N, K), up to 2 rows per
 * expert on average (and 64 in all), K at least 2048: vector FMAs, a wave reads two rows of W with its lanes along K.
 * Everything else: a small MFMA tile (32 rows of the expert x 128 output columns and four workgroups per compute unit,
 * or 128 rows and two from 24 rows per expert on average), cut along K where N alone gives too few workgroups.
 * Whatever does not finish in one kernel sums through the workspace (xma_rocm_scatter2scatter_few_rows_workspace_bytes
 * bytes for the same M, N, K, num_experts, w_is_kn and epilogue; 0 = none needed, pass NULL) to a small kernel that
 * applies the bias and the epilogue with the arithmetic of the MFMA kernels.  Limits: M and E at most 65535, N * ldw
 * below 2^31 - 128 elements for W as (N, K) (32-bit byte offsets inside an expert).
 * Correct for any M, but an expert's rows are walked 4 (vector kernel), 32 or 128 (small tile) at a time, each pass
 * streaming its weights again: meant for launches of a few rows per expert (the torch ops of this package take it up to
 * 96 on average, 48 with the SwiGLU backward, and 16384 in all).  No counterpart in the reference (its kernel is the
 * same for every size).
 */
XMA_API size_t xma_rocm_scatter2scatter_few_rows_workspace_bytes(int64_t M, int32_t N, int32_t K, int32_t num_experts,
                                                         int w_is_kn, int epilogue);
XMA_API int xma_rocm_scatter2scatter_few_rows(const void *X, int64_t ldx, const void *W, int64_t w_expert_stride, int64_t ldw,
                                      int w_is_kn, const int64_t *sorted_scattered_idxs,
                                      const int64_t *expert_offsets, void *out, int64_t ldo, void *aux, int64_t ldaux,
                                      void *aux2, int64_t ldaux2, const void *row_scale, const void *bias,
                                      int64_t bias_expert_stride, int64_t M, int32_t N, int32_t K, int32_t num_experts,
                                      int32_t fan_out, int x_grouped, int y_grouped, int epilogue, int dtype,
                                      void *workspace, size_t workspace_bytes, void *stream);

/*
 * Weight gradient of a grouped linear: for every expert e
 *     DW[e] (N_out, K_in) = sum_{n in expert e} DY[dsrc(n), :N_out]^T  X[xsrc(n), :K_in]
 *     dsrc(n) = n if dy_grouped else sorted_scattered_idxs[n] / dy_fan_out   (then scaled by dy_scale[idx[n]] if given)
 *     xsrc(n) = n if x_grouped  else sorted_scattered_idxs[n] / x_fan_out
 * Every element of DW is written exactly once (zeros for experts with no
 * rows), fp32 accumulation over the expert's whole row range, no atomics.
 * Replaces group_bwd_W, xma/layers/moe/triton_implementation/group_backward_kernel.py:102-128
 * (kernel :21-99), the zeros_like fill (triton_implementation/__init__.py:49,142)
 * and the `group` gather copies that feed it (:46-47, :134-140).
 * DW has the storage layout of the parameter, (E, N_out, K_in) row-major.
 */
XMA_API int xma_rocm_group_bwd_W(const void *DY, int64_t lddy, int dy_grouped, int32_t dy_fan_out, const void *dy_scale,
                         const void *X, int64_t ldx, int x_grouped, int32_t x_fan_out,
                         const int64_t *sorted_scattered_idxs, const int64_t *expert_offsets, void *DW,
                         int64_t dw_expert_stride, int64_t lddw, int32_t N_out, int32_t K_in, int32_t num_experts,
                         int dtype, void *stream);

/*
 * xma_rocm_group_bwd_W for the few-token regime (same arguments and limits plus M, same result up to the order of the
 * fp32 sums; bf16 / fp16 only; a scaled row of DY is rounded to the operand type before it is multiplied, as a scaled
 * grouped copy would hold it).  M = rows in all (the length of the grouped order), which picks the shape of a
 * workgroup's tile of DW[e]: 64 x 256 up to 24 rows per expert on average, 128 x 128 beyond or when M <= 0 (not known).
 * The expert's rows are the K dimension of the tile's MFMAs, 32 at a time: with a handful of rows per expert the launch
 * runs at the rate of a fill of DW, where xma_rocm_group_bwd_W spends a prologue, one K step and an epilogue per
 * 256 x 256 tile.  Correct for any number of rows; more rows are more passes over two small operand tiles, so it leads
 * until the loads outweigh the stores (the torch ops take it up to 128 rows per expert on average).  No counterpart in
 * the reference (its kernel is the same for every size).
 */
XMA_API int xma_rocm_group_bwd_W_few_rows(const void *DY, int64_t lddy, int dy_grouped, int32_t dy_fan_out,
                                  const void *dy_scale, const void *X, int64_t ldx, int x_grouped, int32_t x_fan_out,
                                  const int64_t *sorted_scattered_idxs, const int64_t *expert_offsets, void *DW,
                                  int64_t dw_expert_stride, int64_t lddw, int32_t N_out, int32_t K_in,
                                  int32_t num_experts, int64_t M, int dtype, void *stream);

/*
 * Gather copy: out[n, :] = A[idx[n] / fan_out, :] * (coeff ? coeff[idx[n]] : 1), n < M.
 * Replaces group, xma/layers/moe/triton_implementation/group_kernel.py:69-100.
 */
XMA_API int xma_rocm_group(const void *A, int64_t lda, const int64_t *idx, void *out, int64_t ldo, const void *coeff,
                   int64_t M, int32_t K, int32_t fan_out, int dtype, void *stream);

/*
 * Top-k combine: y[t, :] = sum_j (w ? w[t, j] : 1) * expert_out[t * k + j, :], fp32 accumulation.
 * Replaces the bmm of xma/layers/moe/triton_implementation/__init__.py:100-101
 * and, with w == NULL, the `.sum(-2)` reductions of :70 and :160.
 */
XMA_API int xma_rocm_combine(const void *expert_out, int64_t ld_in, const void *w, void *y, int64_t ldy, int64_t T,
                     int32_t k, int32_t H, int dtype, void *stream);

/*
 * Combine backward w.r.t. the router weights:
 *     d_w[t, j] = <expert_out[t * k + j, :], dy[t, :]>
 * Replaces the bmm of xma/layers/moe/triton_implementation/__init__.py:130-131.
 */
XMA_API int xma_rocm_combine_bwd(const void *expert_out, int64_t ld_in, const void *dy, int64_t lddy, void *d_w, int64_t T,
                         int32_t k, int32_t H, int dtype, void *stream);

/*
 * Stand-alone packed SwiGLU (gate = even columns, up = odd columns), fp32 math:
 *     y[r, c] = u * g * sigmoid(g),  g = x[r, 2c], u = x[r, 2c + 1]
 * and its closed-form backward.  Replaces xma/functional/swiglu/torch_implementation.py:21-30
 * and xma/functional/swiglu/triton_implementation/backward.py:14-23 for the packed layout.
 * Any cols_out >= 1 and any row pitch; rows whose starts are 16-byte aligned move as 16-byte accesses.
 */
XMA_API int xma_rocm_swiglu_packed_forward(const void *x, int64_t ldx, void *y, int64_t ldy, int64_t rows, int32_t cols_out,
                                   int dtype, void *stream);
XMA_API int xma_rocm_swiglu_packed_backward(const void *x, int64_t ldx, const void *dy, int64_t lddy, void *dx,
                                    int64_t lddx, int64_t rows, int32_t cols_out, int dtype, void *stream);

/*
 * Stand-alone SwiGLU on separate operands, y = up * gate * sigmoid(gate) over (rows, cols) with fp32 math, and its
 * backward d_gate = dy * up * (s + g s (1 - s)), d_up = dy * g * s with s = sigmoid(gate).  Replaces _Swiglu.run,
 * xma/functional/swiglu/__init__.py:39-63 (torch form: torch_implementation.py:9-18; backward:
 * triton_implementation/backward.py:14-23).  Any 2-D size and row pitch, bf16 / fp16 / fp32.
 */
XMA_API int xma_rocm_swiglu_forward(const void *gate, int64_t ld_gate, const void *up, int64_t ld_up, void *y, int64_t ldy,
                            int64_t rows, int32_t cols, int dtype, void *stream);
XMA_API int xma_rocm_swiglu_backward(const void *gate, int64_t ld_gate, const void *up, int64_t ld_up, const void *dy,
                             int64_t lddy, void *d_gate, int64_t ld_dgate, void *d_up, int64_t ld_dup, int64_t rows,
                             int32_t cols, int dtype, void *stream);

/*
 * Router behind the gate GEMM: for each of T rows of E expert logits, the k largest values in descending order
 * (equal values: lowest expert index first; NaN counts as the largest value), the fp32 softmax over those k values
 * cast to `dtype`, and their expert ids (int64 if ids_is_i64, else int32), all (T, k) row-major.
 * Replaces topk / max + softmax + type_as of xma/layers/moe/__init__.py:186-193 and :256-262 (three ATen launches
 * and an fp32 round trip).  E <= 2048, k <= min(E, 64); `ld` = row stride of the logits in elements.
 */
XMA_API int xma_rocm_router_topk(const void *logits, int64_t ld, int64_t T, int32_t E, int32_t k, int dtype, void *weights,
                         void *ids, int ids_is_i64, void *stream);
/*
 * Gate projection and router in one kernel: logits (T, E) = x (T, H) @ gate_weight (E, H)^T with fp32 accumulation,
 * rounded to `dtype` (what the stock linear layer returns), then everything xma_rocm_router_topk does, on those rounded
 * logits: weights (T, k), ids (T, k) (int32 for xma_rocm_route, or int64).  x is read from HBM once; the (T, E) logits
 * are written for the module's return value and the backward, never read back.
 * Replaces gate(x) + _get_topk + softmax + type_as, xma/layers/moe/__init__.py:182-195 and :256-262.
 * bf16 / fp16, H % 8 == 0, E <= 128, k <= min(E, 32): xma_rocm_router_gate_topk_supported says whether a shape is
 * covered (otherwise: a linear layer followed by xma_rocm_router_topk).
 */
XMA_API int xma_rocm_router_gate_topk_supported(int32_t H, int32_t E, int32_t k, int dtype);
XMA_API int xma_rocm_router_gate_topk(const void *x, int64_t ldx, const void *gate_weight, int64_t ldw, int64_t T, int32_t H,
                              int32_t E, int32_t k, int dtype, void *logits, int64_t ldl, void *weights, void *ids,
                              int ids_is_i64, void *stream);
/*
 * Backward of xma_rocm_router_topk: with w = softmax of the selected logits (fp32, recomputed),
 *     d_logits[t, ids[t, j]] = w_j * (d_weights[t, j] - sum_i w_i * d_weights[t, i]),  0 elsewhere.
 * Writes all T x E elements of d_logits (row stride ldd), so the caller need not clear it.  Replaces the autograd
 * chain of the same lines (type_as, softmax, float, topk backward with its zero fill and scatter).
 */
XMA_API int xma_rocm_router_topk_bwd(const void *logits, int64_t ld, int64_t T, int32_t E, int32_t k, int dtype, const void *ids,
                             int ids_is_i64, const void *d_weights, void *d_logits, int64_t ldd, void *stream);

/*
 * Measurement aid with no counterpart in the reference: `workgroups` workgroups of 4 waves each issue iters x 64
 * independent v_mfma_f32_32x32x16_bf16 on operands read once from `operands` (16 x 256 x 16 bytes: 8 A and 8 B fragments
 * per lane), nothing else in the loop.  2 * 32 * 32 * 16 * 64 * 4 * workgroups * iters FLOP per call; out receives
 * workgroups x 256 floats.  bench.py --workload mfma_peak times it with random and with all-zero operands: the rate the
 * matrix pipes sustain under the power limit, beside which the GEMM kernels' figures are read.
 */
XMA_API int xma_rocm_diag_mfma_stream(const void *operands, int32_t iters, float *out, int32_t workgroups, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* XMA_ROCM_H */
