/*
 * aops.h -- C ABI of the MI355X (gfx950) implementation of the
 * ascend910a_extras operator set.
 *
 * Every entry point takes raw DEVICE pointers and sizes, enqueues its kernels
 * on the HIP stream it is given (hipStream_t passed as void*; NULL = the
 * default stream) and returns without synchronising.  No entry point reads
 * device data on the host, so all of them can be captured into a HIP graph.
 * Return value: AOPS_OK (0) or a negative AOPS_ERR_* code; nothing is thrown
 * across this boundary.  All fp tensors are IEEE binary16 ("f16"), densely
 * packed and row-major in the shapes stated.  Every tensor and workspace
 * pointer must be 16-byte aligned (the kernels move 128 bits per lane); any
 * hipMalloc'ed buffer and any row of a tensor whose row length the operator
 * accepts is.
 *
 * Each declaration names the reference interface it replaces: the two-phase
 * aclnn*GetWorkspaceSize / aclnn* pair that csrc/ffi/ops.cpp of the reference
 * calls for that operator.
 */
#ifndef AOPS_H_
#define AOPS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AOPS_OK 0
#define AOPS_ERR_INVALID_ARGUMENT (-1) /* null pointer, negative size, size the kernels do not support */
#define AOPS_ERR_WORKSPACE (-2)        /* workspace missing or too small */
#define AOPS_ERR_LAUNCH (-3)           /* HIP reported an error at launch; see aops_last_hip_error() */
#define AOPS_ERR_SCRATCH_LIMIT (-4)    /* aops_paged_attention_noalloc_f16: problem beyond its fixed scratch */

/* Library version (major*10000 + minor*100 + patch). */
int aops_version(void);

/* Text for an AOPS_ERR_* code (static storage). */
const char* aops_strerror(int code);

/* hipError_t of the last failed launch on the calling thread (0 if none). */
int aops_last_hip_error(void);

/*
 * Fused residual add + RMSNorm.
 *   t = x + residual (fp32); residual_out = f16(t);
 *   y = f16(t * rsqrt(mean(t^2) + eps) * weight)
 * x, residual, y, residual_out: [num_tokens, hidden]; weight: [hidden].
 * hidden must be a multiple of 8.  y/residual_out must not alias the inputs.
 * Replaces aclnnAddRMSNormExGetWorkspaceSize + aclnnAddRMSNormEx
 * (reference csrc/ffi/ops.cpp:303-310).
 */
int aops_add_rms_norm_f16(const void* x, const void* residual, const void* weight, float epsilon,
                          void* y, void* residual_out, int64_t num_tokens, int64_t hidden,
                          void* stream);

/*
 * SwiGLU: y[t, j] = f16(silu(x[t, j]) * x[t, d + j]), x: [num_tokens, 2*d], y: [num_tokens, d].
 * d must be a multiple of 8.
 * Replaces aclnnSwiGluExGetWorkspaceSize + aclnnSwiGluEx (reference csrc/ffi/ops.cpp:138-145).
 */
int aops_swiglu_f16(const void* x, void* y, int64_t num_tokens, int64_t d, void* stream);

/*
 * Neox (rotate-half) rotary embedding on q and k.
 * q: [bs, num_heads, head_dim], k: [bs, num_kv_heads, head_dim], position_ids: int32 [bs],
 * cos_cache, sin_cache: [max_position, head_dim/2]; out_q/out_k like q/k.
 * head_dim must be a multiple of 16.  position_ids are not range-checked.
 * Replaces aclnnRopeExGetWorkspaceSize + aclnnRopeEx (reference csrc/ffi/ops.cpp:76-83).
 */
int aops_rope_neox_f16(const void* q, const void* k, const int32_t* position_ids,
                       const void* cos_cache, const void* sin_cache, void* out_q, void* out_k,
                       int64_t bs, int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                       void* stream);

/*
 * Scatter of new K (and optionally V) rows into the paged cache.
 * key, value: [num_tokens, row_elems] with row_elems = num_kv_heads*head_dim (multiple of 16);
 * key_cache, value_cache: [num_blocks, row_elems/16, block_size, 16];
 * slot_indices: int32 [num_tokens].  For token t with s = slot_indices[t]:
 *   cache[s / block_size, c, s % block_size, 0:16] = row[t, 16c : 16c+16]   for every c.
 * Slots outside [0, num_blocks*block_size) are skipped; if two tokens name the same slot, which
 * of them ends up in the cache is unspecified.  value and value_cache may both be
 * NULL (key only); if only one of them is NULL the value side is skipped.
 * Replaces aclnnReshapeAndCacheExGetWorkspaceSize + aclnnReshapeAndCacheEx
 * (reference csrc/ffi/ops.cpp:387-396).
 */
int aops_reshape_and_cache_f16(const void* key, const void* value, void* key_cache,
                               void* value_cache, const int32_t* slot_indices, int64_t num_tokens,
                               int64_t row_elems, int64_t num_blocks, int64_t block_size,
                               void* stream);

/*
 * Decode-step fusion of the two operators above: out_q = rope(q); the rotated k and the untouched v
 * of token b go straight to slot slot_indices[b] of the paged caches.  Bit for bit the result of
 * aops_rope_neox_f16 followed by aops_reshape_and_cache_f16 (rotary dimension == head_dim, one
 * position and one slot per token).  out_k may be NULL; if not, it also receives the rotated k.
 * q, out_q: [bs, num_heads, head_dim]; k, v, out_k: [bs, num_kv_heads, head_dim]; caches:
 * [num_blocks, num_kv_heads*head_dim/16, block_size, 16]; position_ids, slot_indices: int32 [bs].
 * Replaces the pair aclnnRopeEx -> aclnnReshapeAndCacheEx in the order the reference's decoder
 * layer runs them (reference csrc/ffi/graph.cpp:255-270; csrc/ffi/ops.cpp:76-83 and 387-396); the
 * reference has no fused operator.
 */
int aops_rope_reshape_and_cache_f16(const void* q, const void* k, const void* v,
                                    const int32_t* position_ids, const void* cos_cache,
                                    const void* sin_cache, void* out_q, void* out_k,
                                    void* key_cache, void* value_cache,
                                    const int32_t* slot_indices, int64_t bs, int64_t num_heads,
                                    int64_t num_kv_heads, int64_t head_dim, int64_t num_blocks,
                                    int64_t block_size, void* stream);

/*
 * The same with the per-head RMSNorm of q and k in front of the rotation (reference
 * csrc/ffi/graph.cpp:252-253: RMSNorm over head_dim without residual, weights [head_dim]):
 *   qn = f16( q * rsqrt(mean(q^2 over the head) + epsilon) * q_norm_weight ), likewise kn;
 *   out_q = rope(qn); rotated kn and v go to the caches.
 * head_dim: any multiple of 16.  Equal to the chain of the separate operators up to the
 * summation order of the mean (within the operators' tolerance, not bit for bit).
 */
int aops_qknorm_rope_reshape_and_cache_f16(
    const void* q, const void* k, const void* v, const void* q_norm_weight,
    const void* k_norm_weight, float epsilon, const int32_t* position_ids, const void* cos_cache,
    const void* sin_cache, void* out_q, void* out_k, void* key_cache, void* value_cache,
    const int32_t* slot_indices, int64_t bs, int64_t num_heads, int64_t num_kv_heads,
    int64_t head_dim, int64_t num_blocks, int64_t block_size, void* stream);

/*
 * Grouped (per-expert) matmul over expert-sorted rows.
 * x: [rows, k]; w: [num_experts, n, k] (each expert's weight stored N-major, K contiguous --
 * the logical [E, K, N] tensor with stride(1)==1, stride(2)==K); group_list: int64
 * [num_experts] cumulative row ends, read on the device; y: [rows, n].
 *   y[group_list[e-1] : group_list[e], :] = f16( x[...] (fp32 accumulate) @ w[e]^T )
 * Rows at or past group_list[num_experts-1] are not written.  k and n must be multiples of 64
 * (k at most 2^22).
 * Replaces aclnnGroupedMatMulExGetWorkspaceSize + aclnnGroupedMatMulEx
 * (reference csrc/ffi/ops.cpp:211-218).
 */
int aops_grouped_matmul_f16(const void* x, const void* w, const int64_t* group_list, void* y,
                            int64_t rows, int64_t k, int64_t num_experts, int64_t n,
                            void* stream);

/*
 * Two-phase form of aops_grouped_matmul_f16, the reference's own calling convention
 * (aclnnGroupedMatMulExGetWorkspaceSize, then aclnnGroupedMatMulEx with the workspace: reference
 * csrc/ffi/ops.cpp:211-218).  aops_grouped_matmul_workspace returns the bytes of device scratch the
 * call wants on the current device: non-zero only for one expert with few rows and a long k, which
 * then runs the k-split kernels of aops_matmul_nt_ws_f16 (rows at or past group_list[0] are not
 * written, as everywhere); 0 = no scratch, and aops_grouped_matmul_ws_f16 does exactly what
 * aops_grouped_matmul_f16 does.  A workspace that is wanted but missing or too small returns
 * AOPS_ERR_WORKSPACE.
 */
size_t aops_grouped_matmul_workspace(int64_t rows, int64_t k, int64_t num_experts, int64_t n);
int aops_grouped_matmul_ws_f16(const void* x, const void* w, const int64_t* group_list, void* y,
                               void* workspace, size_t workspace_bytes, int64_t rows, int64_t k,
                               int64_t num_experts, int64_t n, void* stream);

/*
 * aops_grouped_matmul_f16 with the kernel fixed by the caller instead of chosen from the problem
 * size: for tests (every kernel over every edge case) and tuning sweeps.  variant 1 = 320 x 256 tiles
 * with direct HBM -> LDS copies, one workgroup per tile; 2 = 320 x 128, 3 = 256 x 128, 4 = 128 x 128,
 * 5 = 64 x 64 register-staged tiles; 6 = the persistent 320 x 256 kernel (k % 128 == 0, k >= 256, else
 * variant 1); 7 = 256 x 128, 8 = 128 x 128 direct copies; 9 = 256 x 128 with three LDS stages.  Any
 * other value returns AOPS_ERR_INVALID_ARGUMENT.  With num_experts == 1, group_list may be NULL (one
 * group that holds every row).  Same results as aops_grouped_matmul_f16 within fp16 rounding.
 * No counterpart in the reference, whose kernel has one tile shape (reference
 * csrc/opdev/op_kernel/matmul_core.h:8-40).
 */
int aops_grouped_matmul_variant_f16(int variant, const void* x, const void* w,
                                    const int64_t* group_list, void* y, int64_t rows, int64_t k,
                                    int64_t num_experts, int64_t n, void* stream);

/*
 * aops_grouped_matmul_f16 for weights whose rows are padded: row r of expert e starts at element
 * (e * n + r) * ldw of w, ldw >= k a multiple of 8, and only its first k elements are read (in torch terms the
 * logical [E, K, N] tensor with stride(1) == 1, stride(2) == ldw, stride(0) == n * ldw).  Why a caller might pad:
 * with k * 2 bytes a power of two (k = 2048: 4 KiB) the 128-byte pieces that a weight tile takes from 256
 * consecutive rows fall into the same few memory channels; a pure read stream of that pattern runs at 4.8 TB/s
 * and at 7.0 TB/s with rows 4224 bytes apart (ldw = k + 64; aops_probe_read_stream shows both).  The grouped
 * matmul itself gains little from it (configs of 32768 routed rows, 128 experts, k = 2048: 2 %), because its
 * operand copies are bound by the number of cache lines in flight per CU, not by the weight stream alone; the
 * entry point exists so that this can be measured.  Runs the persistent 320 x 256 kernel for every problem
 * size: k must be a multiple of 128 from 256 on, n a multiple of 64.  Same bits as aops_grouped_matmul_f16
 * with that kernel on the unpadded weights.
 * No counterpart in the reference, whose binding insists on stride(2) == K (reference csrc/ffi/ops.cpp:171-172).
 */
int aops_grouped_matmul_ldw_f16(const void* x, const void* w, int64_t ldw, const int64_t* group_list, void* y,
                                int64_t rows, int64_t k, int64_t num_experts, int64_t n, void* stream);

/*
 * Dense NT matmul: y = f16( x (fp32 accumulate) @ w^T ), x: [m, k], w: [n, k], y: [m, n]; the
 * grouped matmul with one group that holds every row (no group_list needed).  k and n must be
 * multiples of 64.
 * Replaces matmul of the reference's legacy tree (reference _csrc/ffi.cpp:408-442,
 * benchmark/test_matmul.py).
 */
int aops_matmul_nt_f16(const void* x, const void* w, void* y, int64_t m, int64_t k, int64_t n,
                       void* stream);

/*
 * The same product for shapes with few rows and a long k (a decode-time down projection:
 * 256 x 14336 -> 4096), where whole-k output tiles would leave most CUs idle: the k range is
 * split over several workgroups per tile, the fp32 partial results go to `workspace` and a second
 * kernel adds them in a fixed order (deterministic) and writes y.
 * aops_matmul_nt_workspace returns the bytes of device scratch the call needs on the current
 * device, or 0 when splitting does not pay for the shape; aops_matmul_nt_ws_f16 then computes
 * exactly what aops_matmul_nt_f16 does and ignores the workspace.  A workspace that is required
 * but missing or too small returns AOPS_ERR_WORKSPACE.  The workspace may be freed or reused as
 * soon as the call's work on `stream` is done; calls on different streams need their own.
 * Same reference counterpart as aops_matmul_nt_f16 (the reference's two-phase
 * GetWorkspaceSize + launch convention, reference csrc/ffi/ops.cpp:211-218, kept visible).
 */
size_t aops_matmul_nt_workspace(int64_t m, int64_t k, int64_t n);
int aops_matmul_nt_ws_f16(const void* x, const void* w, void* y, void* workspace,
                          size_t workspace_bytes, int64_t m, int64_t k, int64_t n, void* stream);

/*
 * Grouped matmul of a gate_up projection with the SwiGLU activation fused into its epilogue:
 *   h = x[rows of expert e] (fp32 accumulate) @ w[e]^T          (never stored)
 *   y[r, c] = f16( silu(h[r, c]) * h[r, n/2 + c] ),  c < n/2
 * x, w, group_list as for aops_grouped_matmul_f16 (k and n multiples of 64); y: [rows, n/2].
 * Equal, within fp16 rounding, to aops_grouped_matmul_f16 followed by aops_swiglu_f16, without
 * the [rows, n] intermediate.  Large routed batches (48 rows per expert and more, k a multiple of
 * 128 from 256 on) run the persistent 320 x 256 kernel, which applies the activation to the fp32
 * accumulators; fewer rows per expert or another k run small tiles, which round h to fp16 first,
 * as the two-operator chain does.
 * Replaces the chain aclnnGroupedMatMulEx -> aclnnSwiGluEx of an expert MLP (reference
 * csrc/ffi/ops.cpp:211-218 and 138-145, chained as in benchmark/test_mlp.py:37-41); the reference
 * has no fused operator.
 */
int aops_grouped_matmul_swiglu_f16(const void* x, const void* w, const int64_t* group_list, void* y,
                                   int64_t rows, int64_t k, int64_t num_experts, int64_t n,
                                   void* stream);

/*
 * aops_grouped_matmul_swiglu_f16 with the row gather of a routed batch folded into the operand
 * copies: sorted row j is row row_idx[j] / idx_div of x (x: [x_rows, k]; row_idx: int32 [rows], e.g.
 * sorted_idx of aops_moe_sort_i32 with idx_div = top-k), so the expert-sorted copy of x is never
 * written.  y: [rows, n/2].  Same shape limits; x_rows * k must be below 2^32.
 */
int aops_grouped_matmul_swiglu_gather_f16(const void* x, const int32_t* row_idx, int64_t idx_div,
                                          int64_t x_rows, const void* w, const int64_t* group_list,
                                          void* y, int64_t rows, int64_t k, int64_t num_experts,
                                          int64_t n, void* stream);

/*
 * Routing glue of an expert MLP (no counterpart among the reference's operators: its caller does
 * these steps; the reference itself only shows the host-side construction of group_list,
 * benchmark/test_grouped_matmul.py:46-50).
 *
 * aops_moe_sort_i32: stable counting sort of n expert ids (the flattened [tokens, topk] routing).
 *   sorted_idx[j]   = index i of the id that lands at sorted position j (token = i / topk)
 *   inverse_idx[i]  = j (may be NULL)
 *   group_list[e]   = number of ids <= e, int64, the cumulative form aops_grouped_matmul_f16 reads
 * Ids outside [0, num_experts) sort behind every valid id, in their original order, and are not
 * counted in group_list.  num_experts <= 4095, n < 2^31.  aops_moe_sort_workspace() returns the
 * bytes of workspace needed (0 = unsupported size).
 *
 * aops_moe_gather_f16: out[j, :] = x[sorted_idx[j] / topk, :] for j < group_list[num_experts-1]
 *   (x: [n / topk, hidden], out: [n, hidden], hidden a multiple of 8; later rows are not written).
 *
 * aops_moe_combine_f16: out[t, :] = f16( sum_k weights[t, k] * y[inverse_idx[t*topk + k], :] ) over
 *   the k with a valid expert id, fp32 accumulation in the order of k
 *   (y: [tokens*topk, hidden]; weights: fp32 [tokens, topk]; expert_ids: int32 [tokens, topk]).
 */
size_t aops_moe_sort_workspace(int64_t n, int64_t num_experts);

int aops_moe_sort_i32(const int32_t* expert_ids, int64_t n, int64_t num_experts, int32_t* sorted_idx,
                      int32_t* inverse_idx, int64_t* group_list, void* workspace,
                      size_t workspace_bytes, void* stream);

int aops_moe_gather_f16(const void* x, const int32_t* sorted_idx, const int64_t* group_list, void* out,
                        int64_t n, int64_t topk, int64_t hidden, int64_t num_experts, void* stream);

int aops_moe_combine_f16(const void* y, const int32_t* inverse_idx, const float* weights,
                         const int32_t* expert_ids, void* out, int64_t tokens, int64_t topk,
                         int64_t hidden, int64_t num_experts, void* stream);

/*
 * Paged-attention decode (one query token per sequence).
 * q, o: [bs, num_heads, head_dim]; key_cache, value_cache:
 * [num_blocks, num_kv_heads*head_dim/16, block_size, 16]; block_tables: int32
 * [bs, max_blocks_per_seq]; context_lens: int32 [bs] (read on the device).
 *   o[b,h] = softmax_j( q[b,h] . K[j,g] / sqrt(head_dim) ) . V[j,g],  g = h / (num_heads/num_kv_heads)
 * The kernels split every sequence into fixed-size chunks of the KV cache and keep partial
 * results in `workspace`; aops_paged_attention_workspace() returns the bytes needed (the
 * counterpart of the reference's GetWorkspaceSize phase; 0 = shape not supported).  head_dim must
 * be a multiple of 16 up to 256; any whole number of query heads per kv head.  With block_size a
 * multiple of 16 the operator runs on the matrix cores; other page sizes take a generic, slower
 * kernel.  A sequence with context_len <= 0 gets zeros; a context_len beyond
 * max_blocks_per_seq*block_size is cut there.  Block-table entries outside [0, num_blocks) are
 * clamped into it (garbage in, garbage out, no fault).  The workspace size depends on the compute-unit
 * count of the current device: make the query and the call it sizes with the same device current
 * (the same holds for the other *_workspace queries of this header).
 * Replaces aclnnPagedAttentionExGetWorkspaceSize + aclnnPagedAttentionEx
 * (reference csrc/ffi/ops.cpp:454-461).
 */
size_t aops_paged_attention_workspace(int64_t bs, int64_t num_heads, int64_t num_kv_heads,
                                      int64_t head_dim, int64_t block_size,
                                      int64_t max_blocks_per_seq);

int aops_paged_attention_f16(const void* q, const void* key_cache, const void* value_cache,
                             const int32_t* block_tables, const int32_t* context_lens, void* o,
                             void* workspace, size_t workspace_bytes, int64_t bs,
                             int64_t num_heads, int64_t num_kv_heads, int64_t head_dim,
                             int64_t block_size, int64_t max_blocks_per_seq, int64_t num_blocks,
                             void* stream);

/*
 * aops_paged_attention_f16 for callers that cannot allocate device memory or pass a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference, whose binding allocates a workspace tensor per call
 * (reference csrc/ffi/ops.cpp:454-461).  Same arguments, kernels and results as
 * aops_paged_attention_f16, bit for bit, minus the workspace: the partial results of the split-KV
 * kernels live in a fixed array of AOPS_PA_NOALLOC_SCRATCH_BYTES inside the library's device image
 * (every GPU the library runs on holds its own copy until the process ends).  The call allocates
 * and frees nothing.  The first call on a device looks up that device's address of the array
 * (hipGetSymbolAddress, once per device); make it outside a graph capture.
 * A problem whose aops_paged_attention_workspace() exceeds AOPS_PA_NOALLOC_SCRATCH_BYTES returns
 * AOPS_ERR_SCRATCH_LIMIT and launches nothing.  All calls on one GPU share the one array, which keeps
 * the previous call's contents (nothing in it needs clearing: every value a call reads it has written
 * itself): calls that overlap on one GPU, on different streams or from different threads, race;
 * calls on one stream are ordered and safe.
 */
#define AOPS_PA_NOALLOC_SCRATCH_BYTES (32 * 1024 * 1024)

int aops_paged_attention_noalloc_f16(const void* q, const void* key_cache, const void* value_cache,
                                     const int32_t* block_tables, const int32_t* context_lens,
                                     void* o, int64_t bs, int64_t num_heads, int64_t num_kv_heads,
                                     int64_t head_dim, int64_t block_size,
                                     int64_t max_blocks_per_seq, int64_t num_blocks, void* stream);

/*
 * Measurement aid: launches a kernel that does nothing, `workgroups` workgroups of `threads` threads
 * (1..1024).  Its duration is the floor that any launch of that geometry pays for dispatch, ramp-up
 * and drain: what a latency-bound operator (a few MB of traffic) is up against besides HBM.
 * No counterpart in the reference.
 */
int aops_empty_launch(int64_t workgroups, int threads, void* stream);

/*
 * Measurement aid: a pure read stream with the access pattern of a GEMM operand copy.  buf is a
 * [rows, row_bytes] byte matrix (rows a multiple of 128); every workgroup owns 128 consecutive rows and
 * walks along them in steps of seg_bytes (128, 256, 512 or 1024, dividing row_bytes) per row.  With
 * seg_bytes = 128 and row_bytes = 2 * k this is how the weight tiles of the grouped matmul are fetched;
 * with row_bytes == seg_bytes every workgroup reads one contiguous block (a linear stream).  via_lds: 0 =
 * ordinary 128-bit loads into registers, 1 = global_load_lds_dwordx4 straight into LDS, the instruction the
 * persistent grouped-matmul kernel fetches its operands with.  sink: 4 bytes of device memory that are never
 * written for finite data.  Bandwidth = rows * row_bytes / duration.
 * No counterpart in the reference.
 */
int aops_probe_read_stream(const void* buf, int64_t rows, int64_t row_bytes, int64_t seg_bytes, int via_lds,
                           void* sink, void* stream);

/*
 * Measurement aid: the rate at which the matrix cores execute fp16 MFMAs of one shape (shape 32:
 * v_mfma_f32_32x32x16_f16, shape 16: v_mfma_f32_16x16x32_f16) on operands held in registers, with nothing else
 * going on.  One workgroup of eight waves per CU; every wave reads sixteen fragments (16 KiB of fp16 at
 * `operands`, device memory) once and then issues iters (a multiple of 8, at most 2^20) rounds of MFMAs worth
 * 8 x 16384 multiply-adds each, so a launch does CUs x 8 x iters x 8 x 32768 flop.  With all-zero operands the
 * result is the peak; with operands that differ from one instruction to the next it is what the power limit
 * leaves.  sink: 4 bytes of device memory (never written for finite operands).  No counterpart in the reference.
 */
int aops_probe_mfma_rate(int shape, const void* operands, int64_t iters, void* sink, void* stream);

/*
 * Measurement aid: the persistent 320 x 256 kernel of aops_grouped_matmul_f16 (k % 128 == 0, k >= 256)
 * with parts of its k loop switched off, to time what the rest costs by itself.  ldw = elements from one
 * weight row to the next (k: densely packed, as the operator takes them; more: padded rows, as
 * aops_grouped_matmul_ldw_f16 takes them).  parts_off: 9 = operand
 * copies and barriers only (no MFMAs, no LDS fragment reads), 11 = weight copies only, 13 = activation
 * copies only, 6 = MFMAs and fragment reads only (no copies), 14 = MFMAs only, 1 = everything but the MFMAs,
 * 8 = everything but the LDS fragment reads, 25 and 27 = 9 and 11 with the weight copies of a k tile taking
 * 256 bytes of every row of half the tile's rows instead of 128 bytes of every row (the same requests in
 * pieces twice as long); anything else returns AOPS_ERR_INVALID_ARGUMENT.  y is written with values that are wrong by construction.
 * No counterpart in the reference.
 */
int aops_grouped_matmul_probe_f16(int parts_off, const void* x, const void* w, int64_t ldw,
                                  const int64_t* group_list, void* y, int64_t rows, int64_t k, int64_t num_experts,
                                  int64_t n, void* stream);

/*
 * Device summary (CU count, LDS, L2, memory size, clocks) written as text into buf
 * (at most buf_len bytes including the terminator).  Returns the length written or a
 * negative code.  Replaces print_info (reference csrc/ffi/bind.cpp:26-51).
 */
int aops_device_info(int device, char* buf, size_t buf_len);

#ifdef __cplusplus
}
#endif

#endif /* AOPS_H_ */
