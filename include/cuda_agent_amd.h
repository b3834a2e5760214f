/*
 * C ABI of libcuda_agent_amd.so: hand-written gfx950 HIP kernels behind the launcher
 * interface of the CUDA-Agent workspace.
 *
 * Every operator is one `extern "C" void <op>_launcher(pointers..., sizes..., int config,
 * hipStream_t stream)`, the interface the reference workspace defines for its kernels
 * (agent_workdir/kernels/axpby.cu:12-20; template agent_workdir/SKILL.md:61-88) and binds from
 * kernels/<op>_binding.cpp (agent_workdir/kernels/axpby_binding.cpp:7-15,28-36):
 *
 *   - plain device pointers and int sizes only; no torch types;
 *   - asynchronous on the caller's stream, no synchronisation, no device-side allocation:
 *     outputs and scratch are allocated by the caller and passed in;
 *   - void return; an empty problem (a size <= 0) is a silent no-op (axpby.cu:21);
 *   - `config` selects a launch variant without recompiling (axpby.cu:22-41); a value with no
 *     meaning for an operator selects that operator's default.
 *
 * One addition: a launcher that is handed a shape it has no kernel for, a null or misaligned
 * pointer, or too small a workspace launches nothing and records a code that
 * cuda_agent_amd_last_status() returns (and clears) on the same host thread.
 *
 * hipStream_t is an opaque pointer; callers without the HIP headers may pass it as void*.
 */
#ifndef CUDA_AGENT_AMD_H
#define CUDA_AGENT_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __HIP_PLATFORM_AMD__
#include <hip/hip_runtime_api.h>
#else
typedef struct ihipStream_t* hipStream_t;
#endif

#ifdef __cplusplus
extern "C" {
#endif

enum {
    CUDA_AGENT_AMD_OK = 0,
    CUDA_AGENT_AMD_UNSUPPORTED_SHAPE = 1,
    CUDA_AGENT_AMD_BAD_ARGUMENT = 2,
    CUDA_AGENT_AMD_WORKSPACE_TOO_SMALL = 3,
    CUDA_AGENT_AMD_SCRATCH_LIMIT = 4, /* more scratch needed than the library's static array holds */
    CUDA_AGENT_AMD_RUNTIME_ERROR = 5  /* a HIP runtime call of a launcher's set-up failed */
};

/* Code of the calling thread's most recent rejected launch since the last query; resets to 0. */
int cuda_agent_amd_last_status(void);

/* out[i] = alpha*a[i] + b[i], fp32, i < size. Replaces axpby_launcher of
 * agent_workdir/kernels/axpby.cu:12-42 (same signature, stream type aside).
 * config: 1 -> 128 lanes per workgroup, 2 -> 512, otherwise 256. */
void axpby_launcher(float* out, const float* a, const float* b, float alpha, int size, int config,
                    hipStream_t stream);

/* Gated DeltaNet single-token decode step (workload configs 0 and 1 of the benchmark
 * definition; the launcher pattern is agent_workdir/kernels/axpby.cu:12-20).
 *   o      [batch, n_v_heads, dv] fp32, written
 *   state  [batch, n_v_heads, dk, dv] fp32, updated in place
 *   q, k   [batch, n_qk_heads, dk]; v [batch, n_v_heads, dv]; fp32 if qkv_dtype == 0,
 *          bf16 if qkv_dtype == 1
 *   g, beta [batch, n_v_heads] fp32 (g is the decay factor itself)
 * Value head h reads q/k head h / (n_v_heads / n_qk_heads). Supported: dk == dv == 128,
 * n_v_heads % n_qk_heads == 0. o and state must be 16-byte aligned.
 * config: 0 chooses the column tiling from batch*n_v_heads; 1, 2, 3 force 128, 64, 32 value
 * columns per workgroup. */
void gdn_decode_launcher(float* o, float* state, const void* q, const void* k, const void* v,
                         const float* g, const float* beta, int batch, int n_v_heads,
                         int n_qk_heads, int dk, int dv, int qkv_dtype, int config,
                         hipStream_t stream);

/* The same step with the step in front of it fused in (the caller of the path in Qwen3-Next-style
 * layers; same launcher pattern, agent_workdir/kernels/axpby.cu:12-20): q and k arrive
 * unnormalised and are scaled by rsqrt(sum x^2 + 1e-6) per head inside the kernel, and the gates
 * are computed from
 *   a, b [batch, n_v_heads] fp32 (per-request gate inputs), a_log, dt_bias [n_v_heads] fp32:
 *   g = exp(-exp(a_log[h]) * softplus(a + dt_bias[h])),  beta = sigmoid(b).
 * Everything else as gdn_decode_launcher. */
void gdn_decode_fused_launcher(float* o, float* state, const void* q, const void* k, const void* v,
                               const float* a, const float* b, const float* a_log,
                               const float* dt_bias, int batch, int n_v_heads, int n_qk_heads,
                               int dk, int dv, int qkv_dtype, int config, hipStream_t stream);

/* gdn_decode_fused_launcher with the step after it in the same kernel: the layer's gated RMS
 * normalisation of the read-out (same launcher pattern; caller-side neighbour):
 *   out [batch, n_v_heads, 128], in the storage type of q/k/v =
 *       norm_w * o * rsqrt(mean_j(o_j^2) + eps) * silu(z)
 *   o the step's fp32 read-out (not stored), z [batch, n_v_heads, 128] the output gate and
 *   norm_w [128] the norm's weight, both in the storage type of q/k/v.
 * Everything else as gdn_decode_fused_launcher. config: one value (0). */
void gdn_decode_fused_norm_launcher(void* out, float* state, const void* q, const void* k,
                                    const void* v, const float* a, const float* b,
                                    const float* a_log, const float* dt_bias, const void* z,
                                    const void* norm_w, float eps, int batch, int n_v_heads,
                                    int n_qk_heads, int dk, int dv, int qkv_dtype, int config,
                                    hipStream_t stream);

/* Short causal depthwise convolution, single-token update: the step before the GDN decode step
 * in a Qwen3-Next-style layer (launcher pattern agent_workdir/kernels/axpby.cu:12-20; not one of
 * the benchmark's workloads, the caller-side neighbour of gdn_decode_fused_launcher). Per request
 * b and channel c of the concatenated q|k|v projection:
 *   seq = [conv_state[b,c,0..L-1], x[b,c]];  conv_state[b,c,:] <- seq[1..L]   (in place)
 *   y   = bias[c] + sum_{j<K} weight[c,j] * seq[L+1-K+j];  out = y*sigmoid(y) or y
 *   channels [0,key_dim) -> q_out [batch,key_dim], [key_dim,2*key_dim) -> k_out [batch,key_dim],
 *   the rest -> v_out [batch,value_dim]
 *   conv_state [batch, 2*key_dim+value_dim, L], x [batch, 2*key_dim+value_dim],
 *   weight [2*key_dim+value_dim, K], bias [2*key_dim+value_dim] or NULL
 * dtype: storage type of every array, 0 = fp32, 1 = bf16 (arithmetic is fp32; the state is moved,
 * so it stays bit-exact). activation: 0 none, 1 SiLU. Supported: K = kernel_size in 2..4,
 * L = state_len = K-1 or K, key_dim and value_dim multiples of 8 (key_dim 0: one output, q_out
 * and k_out may be NULL), batch <= 65535, all pointers 16-byte aligned. config: one value (0). */
void causal_conv1d_update_launcher(void* q_out, void* k_out, void* v_out, void* conv_state,
                                   const void* x, const void* weight, const void* bias, int batch,
                                   int key_dim, int value_dim, int state_len, int kernel_size,
                                   int activation, int dtype, int config, hipStream_t stream);

/* Sparse-MLA decode attention (workload config 3 of the benchmark definition; launcher
 * pattern agent_workdir/kernels/axpby.cu:12-20). Per request every head attends to the rows
 * of that request's latent cache listed in idx:
 *   out[b,h,:] = softmax_k(q[b,h,:] . kv[b,idx[b,k],:] * sm_scale) @ kv[b,idx[b,k],:512]
 *   out  [batch, n_heads, 512], written: bf16 if out_dtype == 0 (the operator's output), fp32
 *        if out_dtype == 1 (the same values before the final rounding; lets a checker separate
 *        arithmetic error from the bf16 output rounding)
 *   q    [batch, n_heads, 576] bf16
 *   kv   [batch, n_kv_rows, 576] bf16
 *   idx  [batch, topk] int32; entries < 0 or >= n_kv_rows are padding and are skipped
 *   workspace: device scratch of sparse_mla_decode_workspace_bytes(...) bytes (partial
 *              outputs of the key splits), allocated by the caller
 * Supported: d_qk == 576, d_v == 512, n_heads in {32, 64} or a multiple of 128. All pointers
 * 16-byte aligned.
 * config: 0 chooses the number of key splits so that about one workgroup per CU is resident;
 * n > 0 forces n splits (raised if a split would exceed 2048 rows, lowered to the number of
 * 32-row tiles). 1000 + n: as n, on the kernel with one wavefront per 32 heads, which multiples of
 * 128 heads otherwise use only when a request's cache block is 4 GB or larger (the default kernel
 * for them addresses the block with 32-bit offsets). */
void sparse_mla_decode_launcher(void* out, const void* q, const void* kv, const int* idx,
                                void* workspace, size_t workspace_bytes, int batch, int n_heads,
                                int n_kv_rows, int topk, int d_qk, int d_v, float sm_scale,
                                int out_dtype, int config, hipStream_t stream);

/* The same attention over a paged latent cache, the layout a serving engine keeps (one pool of
 * fixed-size pages shared by all requests and a block table per request). Same launcher pattern
 * (agent_workdir/kernels/axpby.cu:12-20); the operator is the caller-side neighbour of the one
 * above, not a separate workload of the benchmark definition.
 *   kv_pool     [n_pages, page_size, 576] bf16; page_size a power of two,
 *               n_pages * page_size < 2^31
 *   block_table [batch, max_pages_per_request] int32, physical page of each logical page of a
 *               request, negative = not mapped; or NULL
 *   idx         [batch, topk] int32. With a block table: logical positions of the request;
 *               position p is row p % page_size of page block_table[b][p / page_size].
 *               With block_table == NULL: rows of the pool (page * page_size + row).
 *               Negative entries, positions beyond the block table, unmapped pages and rows
 *               beyond the pool are padding and are skipped.
 * Everything else (out, q, workspace and its size, sm_scale, out_dtype, config, supported
 * shapes) as for sparse_mla_decode_launcher. A pool of 4 GB or more is served by the kernel with
 * one wavefront per 32 heads. */
void sparse_mla_decode_paged_launcher(void* out, const void* q, const void* kv_pool,
                                      const int* block_table, const int* idx, void* workspace,
                                      size_t workspace_bytes, int batch, int n_heads, int n_pages,
                                      int page_size, int max_pages_per_request, int topk, int d_qk,
                                      int d_v, float sm_scale, int out_dtype, int config,
                                      hipStream_t stream);

/* Number of key splits the launcher will use for these sizes and this config. */
int sparse_mla_decode_num_splits(int batch, int n_heads, int topk, int config);

/* Bytes of workspace sparse_mla_decode_launcher needs for these sizes and this config. */
size_t sparse_mla_decode_workspace_bytes(int batch, int n_heads, int topk, int config);

/* sparse_mla_decode_launcher without a workspace argument. No counterpart in the reference workspace: it is for
 * callers that cannot allocate device memory (code under HIP graph capture, serving loops with a fixed memory
 * plan, harnesses that forbid hipMalloc). The partial outputs of the key splits go to a static device array of
 * the library (sparse_mla_decode_static_scratch_bytes() = 72 MiB per GPU, held from module load to process end);
 * the kernels and the result are those of sparse_mla_decode_launcher, bit for bit. A problem whose
 * sparse_mla_decode_workspace_bytes(...) exceeds that size is rejected (status 4) and nothing is launched.
 * All calls on one GPU share the array: calls that overlap in time on one GPU race, calls on one stream are safe.
 * The first call on a device looks up the array's address and must not be made under graph capture; no call
 * allocates or frees memory. */
size_t sparse_mla_decode_static_scratch_bytes(void);
void sparse_mla_decode_static_launcher(void* out, const void* q, const void* kv, const int* idx, int batch,
                                       int n_heads, int n_kv_rows, int topk, int d_qk, int d_v,
                                       float sm_scale, int out_dtype, int config, hipStream_t stream);

/* e4m3 storage form of the latent cache (caller-side neighbour of sparse_mla_decode_launcher; same launcher
 * pattern agent_workdir/kernels/axpby.cu:12-20). A row is 656 bytes: 512 e4m3 codes of the latent values,
 * 4 fp32 scales (scale i: values [128*i, 128*i+128), value = code * scale), then the 64 rope values as bf16.
 * mla_latent_quant_launcher writes such rows from bf16 rows kv [rows, 576]: scale = amax / 448 per block of
 * 128, or with config bit 32 the smallest power of two that is at least that. cache and kv 16-byte aligned. */
void mla_latent_quant_launcher(void* cache, const void* kv, long rows, int config, hipStream_t stream);

/* Workspace bytes of sparse_mla_decode_fp8_launcher: the workspace of sparse_mla_decode_launcher plus a
 * block [batch, topk, 576] bf16 of dequantised selected rows and its index list. */
size_t sparse_mla_decode_fp8_workspace_bytes(int batch, int n_heads, int topk, int config);

/* sparse_mla_decode_launcher over kv_fp8 [batch, n_kv_rows, 656] bytes in the form above. Each selected row is
 * dequantised as code * scale in fp32, rounded to nearest-even bf16, and attended as by
 * sparse_mla_decode_launcher: the result equals that launcher's on the dequantised cache bit for bit. With
 * n_heads a multiple of 128, config below 1000 and a cache below 4 GB per request the split kernel gathers the
 * 656-byte rows itself and dequantises every key tile in LDS; otherwise, or with 5000 added to config, the
 * selected rows are first dequantised into the workspace and the bf16 kernels run on that block (same bits).
 * Other arguments, limits and config as sparse_mla_decode_launcher. */
void sparse_mla_decode_fp8_launcher(void* out, const void* q, const void* kv_fp8, const int* idx,
                                    void* workspace, size_t workspace_bytes, int batch, int n_heads,
                                    int n_kv_rows, int topk, int d_qk, int d_v, float sm_scale,
                                    int out_dtype, int config, hipStream_t stream);

/* sparse_mla_decode_fp8_launcher over a paged cache: kv_pool_fp8 [n_pages, page_size, 656] bytes shared by all
 * requests; block_table, idx, page limits as sparse_mla_decode_paged_launcher; workspace as
 * sparse_mla_decode_fp8_launcher. */
void sparse_mla_decode_fp8_paged_launcher(void* out, const void* q, const void* kv_pool_fp8,
                                          const int* block_table, const int* idx, void* workspace,
                                          size_t workspace_bytes, int batch, int n_heads, int n_pages,
                                          int page_size, int max_pages_per_request, int topk, int d_qk,
                                          int d_v, float sm_scale, int out_dtype, int config,
                                          hipStream_t stream);

/* Index scores of the sparse-attention indexer, decode step (caller-side neighbour of the top-k
 * selection below; same launcher pattern agent_workdir/kernels/axpby.cu:12-20):
 *   scores[b, t] = sum_h w[b, h] * max(0, scale * q[b, h, :] . k_cache[b, t, :])  for t < lengths[b]
 *                  (all n_rows if lengths is NULL), -inf beyond
 *   scores [batch, n_rows] fp32; q [batch, n_heads, 128] bf16; k_cache [batch, n_rows, 128] bf16;
 *   w [batch, n_heads] fp32 (per-head weights, any normalisation already applied).
 * n_heads 32 or 64, head_dim 128; q, k_cache, w 16-byte aligned. config: one value (0). */
void mla_index_scores_launcher(float* scores, const void* q, const void* k_cache, const float* w,
                               const int* lengths, int batch, int n_heads, int n_rows, int head_dim,
                               float scale, int config, hipStream_t stream);

/* The same scores over a paged index-key cache: k_pool [n_pages, page_size, 128] bf16 shared by
 * all requests and block_table [batch, max_pages_per_request] int32 (negative = not mapped);
 * position t of request b is row t % page_size of page block_table[b][t / page_size]. scores
 * [batch, max_pages_per_request * page_size], -inf at positions >= lengths[b] and on unmapped pages:
 * logical positions, as sparse_mla_decode_paged_launcher takes them with a block table. page_size a
 * power of two; n_pages * page_size and max_pages_per_request * page_size below 2^31. */
void mla_index_scores_paged_launcher(float* scores, const void* q, const void* k_pool,
                                     const int* block_table, const float* w, const int* lengths,
                                     int batch, int n_heads, int n_pages, int page_size,
                                     int max_pages_per_request, int head_dim, float scale, int config,
                                     hipStream_t stream);

/* Index scores over e4m3 index keys (the storage form of the indexer's key cache: 128 one-byte
 * codes and one fp32 scale per position; caller-side neighbour, same launcher pattern
 * agent_workdir/kernels/axpby.cu:12-20):
 *   scores[b, t] = k_scale[b, t] * sum_h w[b, h] * max(0, scale * q[b, h, :] . k_cache[b, t, :])
 *   q [batch, n_heads, 128] and k_cache [batch, n_rows, 128] OCP e4m3 codes (bias 7, no infinities),
 *   k_scale [batch, n_rows] fp32 (key row = code * k_scale: what moe_quant_bf16_launcher writes for
 *   rows of 128 values), w [batch, n_heads] fp32 = head weight * the scale that head's q was
 *   quantised with. Masking, shapes and alignment as mla_index_scores_launcher. */
void mla_index_scores_fp8_launcher(float* scores, const void* q, const void* k_cache,
                                   const float* k_scale, const float* w, const int* lengths,
                                   int batch, int n_heads, int n_rows, int head_dim, float scale,
                                   int config, hipStream_t stream);

/* The same over a paged e4m3 key cache: k_pool [n_pages, page_size, 128] codes and k_scale_pool
 * [n_pages, page_size] fp32 shared by all requests; block table, scores and limits as
 * mla_index_scores_paged_launcher. */
void mla_index_scores_fp8_paged_launcher(float* scores, const void* q, const void* k_pool,
                                         const float* k_scale_pool, const int* block_table,
                                         const float* w, const int* lengths, int batch, int n_heads,
                                         int n_pages, int page_size, int max_pages_per_request,
                                         int head_dim, float scale, int config, hipStream_t stream);

/* Top-k selection of index scores, the step that produces idx for the two launchers above
 * (caller-side neighbour; same launcher pattern agent_workdir/kernels/axpby.cu:12-20):
 *   idx_out [batch, k] int32: per request the indices of the k largest scores among the first
 *           lengths[b] entries (all n if lengths is NULL) of scores [batch, n] fp32; ties go to
 *           the lower index; listed in ascending index order; -1 where fewer than k candidates
 *           exist (the attention skips them). NaN scores rank below every number.
 * Exact (integer work on the bit patterns of the scores). config: one value (0). */
void topk_select_launcher(int* idx_out, const float* scores, const int* lengths, int batch, int n,
                          int k, int config, hipStream_t stream);

/* ---- FP8 block-scaled MoE layer (workload configs 2 and 4 of the benchmark definition;
 * launcher pattern agent_workdir/kernels/axpby.cu:12-20). Expert weights are e4m3 with one fp32
 * scale per 128x128 block: w13_q [E, 2*inter, hidden] (rows 0..inter-1 gate, inter..2*inter-1
 * up), w13_s [E, 2*inter/128, hidden/128], w2_q [E, hidden, inter], w2_s [E, hidden/128,
 * inter/128]. Activations are quantised per row and 128-wide group:
 * scale = max(amax, 1e-12) * fp32(1/448), code = e4m3_rne(clamp(v/scale, -448, 448)).
 * The stages are exported one by one so that a checker can compare each against a reference;
 * moe_fp8_launcher runs them in sequence. ---- */

/* ids [tokens, top_k] int32: the top_k largest logits of each token, descending, ties to the
 * lower expert id; weights [tokens, top_k] fp32: sigmoid(logit) normalised over the top_k.
 * logits [tokens, n_experts] fp32. n_experts <= 512, top_k <= 64.
 * config bit 64 (also understood by moe_route_sort_launcher): every token gets one more slot after
 * its top_k, expert number n_experts with weight 1 (a shared expert stored behind the routed ones);
 * ids and weights are then [tokens, top_k + 1] and the sort covers n_experts + 1 experts. */
void moe_route_launcher(int* ids, float* weights, const float* logits, int tokens, int n_experts,
                        int top_k, int config, hipStream_t stream);

/* Router projection in front of the routing (caller-side neighbour, same launcher pattern):
 *   logits [tokens, n_experts] fp32 = x [tokens, hidden] . w [n_experts, hidden]^T
 * x fp32 (x_dtype 0) or bf16 (1), w fp32; both enter the fp32 matrix cores exactly, so the result
 * differs from an fp32 reference only by the order of the additions. hidden a multiple of 64;
 * x, w and workspace 16-byte aligned. For few tokens K is split over workgroups and the partial
 * sums are added in a fixed order from workspace: moe_router_logits_workspace_bytes(...) bytes
 * (0, and workspace may be NULL, when moe_router_logits_num_splits(...) is 1). */
int moe_router_logits_num_splits(int tokens, int hidden, int n_experts);
size_t moe_router_logits_workspace_bytes(int tokens, int hidden, int n_experts);
void moe_router_logits_launcher(float* logits, const void* x, const float* w, void* workspace,
                                size_t workspace_bytes, int tokens, int hidden, int n_experts,
                                int x_dtype, int config, hipStream_t stream);

/* The router weight as three bf16 planes [3, n_experts, hidden] whose sum is w exactly (the 24 significand
 * bits of an fp32 number cut 8 + 8 + 8); prepared once per weight for the launcher below. */
void moe_router_split_weight_launcher(void* planes, const float* w, int n_experts, int hidden,
                                      hipStream_t stream);

/* moe_router_logits_launcher for a bf16 x and the weight given as those planes: every product is exact in
 * fp32, so the logits differ from the fp32 launcher's by the order of the additions only, and the
 * projection runs on the bf16 matrix cores. Scratch (moe_router_logits_workspace_bytes), sizes and limits as
 * moe_router_logits_launcher; x and planes 16-byte aligned. */
void moe_router_logits_split_launcher(float* logits, const void* x, const void* planes, void* workspace,
                                      size_t workspace_bytes, int tokens, int hidden, int n_experts,
                                      int config, hipStream_t stream);

/* Group-limited routing with a selection bias, the router of DeepSeek-V3-style layers (caller-
 * side neighbour of moe_route_launcher; same launcher pattern):
 *   score = sigmoid(logit), choice = score + bias; a group (n_experts/n_group consecutive
 *   experts) is valued by the sum of its 2 largest choice values; only the topk_group best groups
 *   stay (ties to the lower group); ids = the top_k largest choice values among the experts that
 *   stay, descending, ties to the lower expert id; weights = score[ids], divided by their sum +
 *   1e-20 if normalise != 0, times routed_scaling_factor.
 * bias [n_experts] fp32 or NULL. n_experts <= 512 and a multiple of n_group, n_group <= 64,
 * topk_group <= n_group, top_k <= min(64, topk_group * n_experts / n_group). */
void moe_route_grouped_launcher(int* ids, float* weights, const float* logits, const float* bias,
                                int tokens, int n_experts, int top_k, int n_group, int topk_group,
                                int normalise, float routed_scaling_factor, int config,
                                hipStream_t stream);

/* Stable counting sort of the tokens*top_k (token, slot) pairs by expert id:
 * sorted_pairs[pos] = token*top_k + slot, pair_pos = its inverse, expert e owns positions
 * expert_offsets[e] .. expert_offsets[e+1]-1 (expert_offsets has n_experts+1 entries).
 * chunk_scratch: ceil(tokens/256)*n_experts ints of device scratch. */
void moe_sort_launcher(int* sorted_pairs, int* pair_pos, int* expert_offsets, int* chunk_scratch,
                       const int* ids, int tokens, int n_experts, int top_k, int config,
                       hipStream_t stream);

/* moe_route_launcher followed by the sort; same outputs. With tokens*top_k <= 1024 (the decode case) the sort is
 * one single-workgroup kernel behind the routing kernel; config 1 forces the chunked sort, config 2 a single
 * kernel that routes and sorts in one workgroup. */
void moe_route_sort_launcher(int* ids, float* weights, int* sorted_pairs, int* pair_pos,
                             int* expert_offsets, int* chunk_scratch, const float* logits, int tokens,
                             int n_experts, int top_k, int config, hipStream_t stream);

/* q [rows, cols] e4m3 codes and scales [rows, cols/128] fp32 from x [rows, cols] bf16. */
void moe_quant_bf16_launcher(void* q, float* scales, const void* x, int rows, int cols, int config,
                             hipStream_t stream);

/* The RMS norm in front of the layer fused with that quantiser (caller-side neighbour; same launcher
 * pattern): y = weight * bf16(x * rsqrt(mean(x^2) + eps)) rounded to bf16 (the two roundings of a bf16
 * norm layer), then q, scales = the quantisation above applied to y.
 *   x [rows, cols] bf16, weight [cols] bf16, y [rows, cols] bf16 or NULL (the normalised row, e.g. for
 *   the router projection), q [rows, cols] e4m3 codes, scales [rows, cols/128] fp32.
 * cols a multiple of 128, at most 8192; x, weight, y 16-byte and q 8-byte aligned. config bit 32:
 * power-of-two scales. */
void moe_rmsnorm_quant_launcher(void* q, float* scales, void* y, const void* x, const void* weight,
                                float eps, int rows, int cols, int config, hipStream_t stream);

/* Grouped gate/up GEMM with SiLU(gate)*up and requantisation fused:
 * h_q [tokens*top_k, inter] e4m3, h_s [tokens*top_k, inter/128] fp32, rows in sorted order.
 * config: 0 sizes the pass from the average pairs per expert; 1, 2, 4 force 16, 32, 64 pairs
 * per pass. */
void moe_gate_up_launcher(void* h_q, float* h_s, const void* x_q, const float* x_s,
                          const void* w13_q, const float* w13_s, const int* sorted_pairs,
                          const int* expert_offsets, int tokens, int hidden, int inter,
                          int n_experts, int top_k, int config, hipStream_t stream);

/* Grouped down GEMM: y [tokens*top_k, hidden] fp32, rows in sorted order. config as above. */
void moe_down_launcher(float* y, const void* h_q, const float* h_s, const void* w2_q,
                       const float* w2_s, const int* expert_offsets, int tokens, int hidden,
                       int inter, int n_experts, int top_k, int config, hipStream_t stream);

/* out[t, :] = sum_k weights[t, k] * y[pair_pos[t*top_k + k], :], k ascending, in fp32;
 * out is bf16 (out_dtype 0) or fp32 (out_dtype 1). */
void moe_combine_launcher(void* out, const float* y, const float* weights, const int* pair_pos,
                          int tokens, int hidden, int top_k, int out_dtype, int config,
                          hipStream_t stream);

/* Bytes of device scratch moe_fp8_launcher needs (routing tables, quantised activations,
 * intermediate h and y). */
size_t moe_fp8_workspace_bytes(int tokens, int hidden, int inter, int n_experts, int top_k);

/* Byte offsets, inside that workspace, of ids, weights, expert_offsets, sorted_pairs, pair_pos,
 * x_q, x_s, h_q, h_s, y, y_scale (in this order), for checkers that inspect the stages. Writes
 * min(n_offsets, 11) entries and returns the number of fields the layout has (11), so that a caller
 * built against another version of the list can tell.
 * y [tokens*top_k, hidden]: fp32 rows when the layer ran the weight-streaming GEMMs; when it ran the
 * LDS-tiled ones (moe_fp8_uses_tiled_gemms), fp16 rows in the first half of the buffer, to be
 * multiplied by y_scale [tokens*top_k, hidden/256] (one power of two per row and run of 256 columns). */
int moe_fp8_workspace_layout(size_t* offsets, int n_offsets, int tokens, int hidden, int inter,
                             int n_experts, int top_k);

/* 1 if moe_fp8_launcher runs these sizes and this config on the LDS-tiled GEMMs, 0 if on the
 * weight-streaming ones, -1 if it rejects them. */
int moe_fp8_uses_tiled_gemms(int tokens, int hidden, int inter, int n_experts, int top_k, int config);

/* The whole layer: out [tokens, hidden] (bf16 if out_dtype == 0, the operator's output type;
 * fp32 if 1, the same values before the final rounding) from x [tokens, hidden] bf16 and
 * logits [tokens, n_experts] fp32. workspace: moe_fp8_workspace_bytes(...) bytes, 256-byte
 * aligned. hidden and inter multiples of 128. config: 0 picks the GEMM form from the average number
 * of pairs per expert (above 32 and hidden % 256 == 0: LDS-tiled 256x256 GEMMs; otherwise the
 * weight-streaming form); 16 forces the tiled form; 1, 2, 4 (+8) force streaming as for
 * moe_gate_up_launcher. +32 (also understood by moe_quant_bf16_launcher and moe_gate_up_launcher):
 * every block scale is a power of two (UE8M0). w13_s and w2_s must then hold powers of two; x and
 * the intermediate are quantised with scale = the smallest power of two >= max(amax, 1e-12)/448,
 * and the tiled GEMMs apply the scales inside the MFMA.
 * +256 / +512: how the intermediate h = silu(g) * u is requantised. The e4m3 matrix core sums a
 * 128-block with about 16 significant bits, so about one code of h in a thousand would differ by one
 * step from an fp32 evaluation, and one step on an element near its group's maximum moves single
 * outputs by up to 3 % of their rms. The streaming gate/up GEMM therefore runs on the bf16 matrix core
 * (exact sums, same time: it is bound by the weight stream); +512 puts it on the e4m3 one. The tiled
 * gate/up GEMM by default stays on the e4m3 matrix core and recomputes, in its epilogue, the elements
 * in the two highest binades of their group's range (at least 128 of 448 code units) that lie within
 * the matrix core's error of a rounding boundary, together with the candidates for the maximum of
 * those groups, as plain dot products: codes of large elements as an fp32 evaluation gives them,
 * small ones (a code step of at most 8/448 of the group's maximum) as the matrix core rounds them.
 * +256: the tiled gate/up GEMM on the bf16 matrix core instead: every code exact, twice the
 * matrix-core time. +512: e4m3 matrix core, no repair. +1024 / +2048 / +3072: the band is half /
 * twice / four times as wide. +4096*s (s = 1..8): repair elements of at least 2^s code units. */
void moe_fp8_launcher(void* out, const void* x, const float* logits, const void* w13_q,
                      const float* w13_s, const void* w2_q, const float* w2_s, void* workspace,
                      size_t workspace_bytes, int tokens, int hidden, int inter, int n_experts,
                      int top_k, int out_dtype, int config, hipStream_t stream);

/* The same sum with one more fp32 row per token added last: y_shared [tokens, hidden] (the shared
 * expert's output) or NULL. */
void moe_combine_shared_launcher(void* out, const float* y, const float* weights,
                                 const int* pair_pos, const float* y_shared, int tokens, int hidden,
                                 int top_k, int out_dtype, int config, hipStream_t stream);

/* The layer with a shared expert (the caller-side neighbour of moe_fp8_launcher in
 * DeepSeek-V3-style layers; same launcher pattern): out = sum_k w[t,k] * expert_k(x[t]) +
 * shared(x[t]). The shared expert is one more block-scaled MLP, sw13_q [2*shared_inter, hidden],
 * sw13_s [2*shared_inter/128, hidden/128], sw2_q [hidden, shared_inter], sw2_s [hidden/128,
 * shared_inter/128], applied to every token with weight 1 on the activations quantised once for
 * both; its fp32 row is added after the routed experts' weighted sum. workspace:
 * moe_fp8_shared_workspace_bytes(...) bytes, 256-byte aligned; its first
 * moe_fp8_workspace_bytes(...) bytes have the layout moe_fp8_workspace_layout describes.
 * Everything else as moe_fp8_launcher. */
size_t moe_fp8_shared_workspace_bytes(int tokens, int hidden, int inter, int shared_inter,
                                      int n_experts, int top_k);
void moe_fp8_shared_launcher(void* out, const void* x, const float* logits, const void* w13_q,
                             const float* w13_s, const void* w2_q, const float* w2_s,
                             const void* sw13_q, const float* sw13_s, const void* sw2_q,
                             const float* sw2_s, void* workspace, size_t workspace_bytes, int tokens,
                             int hidden, int inter, int shared_inter, int n_experts, int top_k,
                             int out_dtype, int config, hipStream_t stream);

/* The same layer with the shared expert stored as expert number n_experts behind the routed ones
 * (w13_q [n_experts + 1, 2*inter, hidden], w13_s, w2_q, w2_s likewise; same inter): every token
 * takes it as one more slot with weight 1, so it runs inside the routed experts' launches rather
 * than as launches of its own that fill a fraction of the chip. Same sum as above. logits
 * [tokens, n_experts]. workspace: moe_fp8_workspace_bytes(tokens, hidden, inter, n_experts + 1,
 * top_k + 1) bytes, with the layout of that shape (rows of ids/weights have top_k + 1 entries, the
 * last one the shared expert). n_experts <= 511, top_k <= 63; config as moe_fp8_launcher. */
void moe_fp8_fused_shared_launcher(void* out, const void* x, const float* logits, const void* w13_q,
                                   const float* w13_s, const void* w2_q, const float* w2_s,
                                   void* workspace, size_t workspace_bytes, int tokens, int hidden,
                                   int inter, int n_experts, int top_k, int out_dtype, int config,
                                   hipStream_t stream);

/* Measuring aid of bench.py, no counterpart in the reference workspace: one workgroup per CU whose first four
 * wavefronts issue `iters` rounds of four e4m3 MFMAs (v_mfma_f32_32x32x64_f8f6f4; config 1: bf16,
 * v_mfma_f32_32x32x16_bf16) on the random operands given, while the other four stream stream_src (stream_bytes
 * of it, 0 for none) from memory until the MFMAs are done. result [n_cus][2] uint64, cleared by the caller:
 * ticks at 100 MHz of each workgroup's MFMA loop, and the bytes streamed meanwhile. operands: n_cus * 16384 bytes. */
void calibrate_mfma_launcher(const void* operands, const void* stream_src, size_t stream_bytes, void* result,
                             float* sink, int n_cus, int iters, int config, hipStream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* CUDA_AGENT_AMD_H */
