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
    CUDA_AGENT_AMD_WORKSPACE_TOO_SMALL = 3
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
 * 32-row tiles). */
void sparse_mla_decode_launcher(void* out, const void* q, const void* kv, const int* idx,
                                void* workspace, size_t workspace_bytes, int batch, int n_heads,
                                int n_kv_rows, int topk, int d_qk, int d_v, float sm_scale,
                                int out_dtype, int config, hipStream_t stream);

/* Number of key splits the launcher will use for these sizes and this config. */
int sparse_mla_decode_num_splits(int batch, int n_heads, int topk, int config);

/* Bytes of workspace sparse_mla_decode_launcher needs for these sizes and this config. */
size_t sparse_mla_decode_workspace_bytes(int batch, int n_heads, int topk, int config);

#ifdef __cplusplus
}
#endif

#endif /* CUDA_AGENT_AMD_H */
