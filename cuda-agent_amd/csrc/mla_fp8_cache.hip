// e4m3 storage form of the latent KV cache of sparse-MLA decode, and decode over it.
//
// A cache row in this form is 656 bytes instead of the 1152 of the bf16 row:
//   bytes [  0, 512)  e4m3 codes of the 512 latent values
//   bytes [512, 528)  4 fp32 scales; scale i belongs to values [128*i, 128*i + 128): value = code * scale
//   bytes [528, 656)  the 64 rope values as bf16, unchanged
// (the layout third-party sparse-attention decoders use for a quantised latent cache: 57 % of the bytes
// per cached token).
//
//   mla_latent_quant_launcher        bf16 rows [rows, 576] -> rows of 656 bytes (the cache write side)
//   sparse_mla_decode_fp8_launcher   decode over such a cache
//
// Decode has two forms with the same result, bit for bit what sparse_mla_decode_launcher gives on the
// dequantised cache (code * scale in fp32, rounded to nearest-even bf16).
//   * Head counts that are multiples of 128: the 8-wavefront kernel of sparse_mla.hip gathers the 656-byte
//     rows itself and converts every key tile in LDS (its FP8 instantiation); the selected rows cross HBM once
//     and nothing else is written.
//   * Otherwise, or with 5000 added to config, two steps: the kernel below gathers the selected rows of every
//     request and dequantises them into a compact per-request block [batch, topk, 576] in the workspace, with
//     an index list 0..topk-1 beside it (-1 where the caller's entry was padding); the decode kernels of
//     sparse_mla.hip then run on that block unchanged. The compact block is written and read back.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "launch_status.hpp"
#include "mla_addressing.hpp"
#include "moe_common.hpp"

extern "C" size_t sparse_mla_decode_workspace_bytes(int batch, int n_heads, int topk, int config);
extern "C" void sparse_mla_decode_launcher(void* out, const void* q, const void* kv, const int* idx,
                                           void* workspace, size_t workspace_bytes, int batch,
                                           int n_heads, int n_kv_rows, int topk, int d_qk, int d_v,
                                           float sm_scale, int out_dtype, int config, hipStream_t stream);
extern "C" int sparse_mla_decode_fp8_fused(void* out, const void* q, const void* kv_fp8, const int* idx,
                                           void* workspace, size_t workspace_bytes, int batch, int n_heads,
                                           int n_kv_rows, int topk, int d_qk, int d_v, float sm_scale,
                                           int out_dtype, int config, const int* block_table,
                                           int table_stride, int page_shift, int batch_rows,
                                           hipStream_t stream);

namespace {

constexpr int LATENT = 512;
constexpr int ROPE = 64;
constexpr int ROW_VALUES = LATENT + ROPE;          // 576
constexpr int ROW_BF16_BYTES = ROW_VALUES * 2;     // 1152
constexpr int SCALES_AT = LATENT;                  // byte offset of the 4 scales
constexpr int ROPE_AT = LATENT + 16;               // byte offset of the rope values
constexpr int ROW_FP8_BYTES = ROPE_AT + ROPE * 2;  // 656 = 41 chunks of 16 bytes
constexpr int ROW_FP8_CHUNKS = ROW_FP8_BYTES / 16;

typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

// ---- write side: one wavefront per row, 4 rows per workgroup ------------------------------------------
// lane l quantises latent values [8l, 8l+8) (16 lanes per 128-value block); lanes 0-7 also move the rope
__global__ __launch_bounds__(256) void mla_latent_quant_kernel(const __hip_bfloat16* __restrict__ kv,
                                                               uint8_t* __restrict__ cache, long rows,
                                                               bool pow2) {
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;  // (no barrier in this kernel)
    const __hip_bfloat16* src = kv + row * ROW_VALUES;
    uint8_t* dst = cache + row * ROW_FP8_BYTES;
    const uintx4 raw = *reinterpret_cast<const uintx4*>(src + 8 * lane);
    uintx4 rope = {0u, 0u, 0u, 0u};
    if (lane < 8) rope = *reinterpret_cast<const uintx4*>(src + LATENT + 8 * lane);
    float v[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float(raw[j] << 16);
        v[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
    }
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const float scale = moe::group_scale(amax, pow2);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = fminf(fmaxf(v[j] / scale, -moe::E4M3_MAX), moe::E4M3_MAX);
    uintx2 packed;
    int lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], lo, true);
    int hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], 0, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], hi, true);
    packed[0] = (unsigned)lo;
    packed[1] = (unsigned)hi;
    *reinterpret_cast<uintx2*>(dst + 8 * lane) = packed;
    if ((lane & 15) == 0) *reinterpret_cast<float*>(dst + SCALES_AT + 4 * (lane >> 4)) = scale;
    if (lane < 8) *reinterpret_cast<uintx4*>(dst + ROPE_AT + 16 * lane) = rope;
}

// ---- read side: gather + dequantise the selected rows -------------------------------------------------
constexpr int ROWS_PER_WAVE = 8;
constexpr int ROWS_PER_WG = 4 * ROWS_PER_WAVE;

// two e4m3 codes (one half of a dword) times a scale -> two bf16 in one dword (v_cvt_pk_bf16_f32 rounds to
// nearest even)
__device__ __forceinline__ unsigned dequant_pair(unsigned codes, bool upper, float scale) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const floatx2 f = upper ? __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, true)
                            : __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, false);
    const bf16x2 r = {(__bf16)(f[0] * scale), (__bf16)(f[1] * scale)};
    return __builtin_bit_cast(unsigned, r);
}

// grid: x = blocks of 32 selected rows, y = request. A wavefront takes 8 selected rows; per row lane l < 41
// fetches 16-byte chunk l: lanes 0-31 hold 16 codes each, lane 32 the four scales, lanes 33-40 the rope.
__global__ __launch_bounds__(256) void mla_latent_gather_kernel(const uint8_t* __restrict__ cache,
                                                                const int* __restrict__ idx,
                                                                __hip_bfloat16* __restrict__ rows_out,
                                                                int* __restrict__ idx_out, int n_kv_rows,
                                                                int topk, mla::KvAddressing kva) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int b = blockIdx.y;
    const int first = blockIdx.x * ROWS_PER_WG + wave * ROWS_PER_WAVE;
    if (first >= topk) return;  // (no barrier in this kernel)
    const uint8_t* cache_b = cache + (size_t)b * kva.batch_rows * ROW_FP8_BYTES;
    // rows of this wavefront's entries (block table, bounds), one per lane, then broadcast
    int my_key = -1;
    if (lane < ROWS_PER_WAVE && first + lane < topk)
        my_key = mla::resolve_key(idx[(size_t)b * topk + first + lane], b, kva, n_kv_rows);
    if (lane < ROWS_PER_WAVE && first + lane < topk) idx_out[(size_t)b * topk + first + lane] = my_key < 0 ? -1 : first + lane;

    uintx4 chunk[ROWS_PER_WAVE];
    int key[ROWS_PER_WAVE];
#pragma unroll
    for (int r = 0; r < ROWS_PER_WAVE; ++r) {
        key[r] = __builtin_amdgcn_readlane(my_key, r);
        // unconditional loads (padding entries read row 0, lanes past the row its last chunk; neither is used):
        // all eight requests of the wavefront are in flight together
        const int safe_row = key[r] < 0 ? 0 : key[r];
        const int safe_chunk = lane < ROW_FP8_CHUNKS ? lane : ROW_FP8_CHUNKS - 1;
        chunk[r] = __builtin_nontemporal_load(
            reinterpret_cast<const uintx4*>(cache_b + (size_t)safe_row * ROW_FP8_BYTES) + safe_chunk);
    }
#pragma unroll
    for (int r = 0; r < ROWS_PER_WAVE; ++r) {
        if (key[r] < 0) continue;  // padding: the decode kernel skips the row, whatever the block holds
        uint8_t* dst = reinterpret_cast<uint8_t*>(rows_out + ((size_t)b * topk + first + r) * ROW_VALUES);
        // the four scales sit in lane 32; lane l < 32 needs scale l / 8
        const float s0 = __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)chunk[r][0], 32));
        const float s1 = __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)chunk[r][1], 32));
        const float s2 = __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)chunk[r][2], 32));
        const float s3 = __uint_as_float((unsigned)__builtin_amdgcn_readlane((int)chunk[r][3], 32));
        if (lane < 32) {
            const int block = lane >> 3;
            const float scale = block == 0 ? s0 : block == 1 ? s1 : block == 2 ? s2 : s3;
            uintx4 lo, hi;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                lo[2 * j] = dequant_pair(chunk[r][j], false, scale);
                lo[2 * j + 1] = dequant_pair(chunk[r][j], true, scale);
                hi[2 * j] = dequant_pair(chunk[r][2 + j], false, scale);
                hi[2 * j + 1] = dequant_pair(chunk[r][2 + j], true, scale);
            }
            *reinterpret_cast<uintx4*>(dst + 32 * lane) = lo;
            *reinterpret_cast<uintx4*>(dst + 32 * lane + 16) = hi;
        } else if (lane >= 33 && lane < ROW_FP8_CHUNKS) {
            *reinterpret_cast<uintx4*>(dst + 2 * LATENT + 16 * (lane - 33)) = chunk[r];
        }
        __builtin_amdgcn_sched_barrier(0);  // one row at a time: the conversions of all rows at once need 236 registers
    }
}

size_t align16(size_t n) { return (n + 15) & ~(size_t)15; }

}  // namespace

// cache [rows, 656] bytes from kv [rows, 576] bf16: per row and block of 128 latent values one scale
// (amax / 448, or with config bit 32 the smallest power of two that is at least that) and 128 e4m3
// codes; the 64 rope values are copied. kv and cache 16-byte aligned.
extern "C" void mla_latent_quant_launcher(void* cache, const void* kv, long rows, int config,
                                          hipStream_t stream) {
    if (rows <= 0) return;
    if (rows > 0x7fffffffl * 4) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!cache || !kv || ((reinterpret_cast<uintptr_t>(cache) | reinterpret_cast<uintptr_t>(kv)) & 15u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    mla_latent_quant_kernel<<<(unsigned)((rows + 3) / 4), 256, 0, stream>>>(
        static_cast<const __hip_bfloat16*>(kv), static_cast<uint8_t*>(cache), rows,
        (config & moe::CONFIG_UE8M0) != 0);
}

// bytes of scratch sparse_mla_decode_fp8_launcher needs: the workspace of sparse_mla_decode_launcher, the
// compact block of dequantised rows and its index list
extern "C" size_t sparse_mla_decode_fp8_workspace_bytes(int batch, int n_heads, int topk, int config) {
    if (batch <= 0 || n_heads <= 0 || topk <= 0) return 0;
    if (config >= 5000) config -= 5000;
    return align16(sparse_mla_decode_workspace_bytes(batch, n_heads, topk, config)) +
           align16((size_t)batch * topk * ROW_BF16_BYTES) + align16((size_t)batch * topk * sizeof(int));
}

namespace {

void launch_decode_fp8(void* out, const void* q, const void* kv_fp8, const int* idx, void* workspace,
                       size_t workspace_bytes, int batch, int n_heads, int n_kv_rows, int topk, int d_qk,
                       int d_v, float sm_scale, int out_dtype, int config, const mla::KvAddressing& kva,
                       hipStream_t stream) {
    if (batch <= 0 || n_heads <= 0 || topk <= 0) return;
    if (d_qk != ROW_VALUES || d_v != LATENT || n_kv_rows <= 0 || batch > 65535) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!out || !q || !kv_fp8 || !idx || !workspace ||
        ((reinterpret_cast<uintptr_t>(kv_fp8) | reinterpret_cast<uintptr_t>(workspace)) & 15u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    if (workspace_bytes < sparse_mla_decode_fp8_workspace_bytes(batch, n_heads, topk, config)) {
        caa::set_status(CAA_WORKSPACE_TOO_SMALL);
        return;
    }
    // config 5000 + n: the two-step form (gather + dequantise into the workspace, then the bf16 kernels) with
    // config n; otherwise the 128-head kernel dequantises its tiles itself where the shape allows
    const bool two_step = config >= 5000;
    if (two_step) config -= 5000;
    const size_t base_bytes = align16(sparse_mla_decode_workspace_bytes(batch, n_heads, topk, config));
    if (!two_step &&
        sparse_mla_decode_fp8_fused(out, q, kv_fp8, idx, workspace, base_bytes, batch, n_heads, n_kv_rows, topk,
                                    d_qk, d_v, sm_scale, out_dtype, config, kva.block_table, kva.table_stride,
                                    kva.page_shift, kva.batch_rows, stream))
        return;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    __hip_bfloat16* rows = reinterpret_cast<__hip_bfloat16*>(ws + base_bytes);
    int* compact_idx = reinterpret_cast<int*>(ws + base_bytes + align16((size_t)batch * topk * ROW_BF16_BYTES));
    const dim3 grid((topk + ROWS_PER_WG - 1) / ROWS_PER_WG, batch);
    mla_latent_gather_kernel<<<grid, 256, 0, stream>>>(static_cast<const uint8_t*>(kv_fp8), idx, rows,
                                                       compact_idx, n_kv_rows, topk, kva);
    sparse_mla_decode_launcher(out, q, rows, compact_idx, workspace, base_bytes, batch, n_heads, topk, topk,
                               d_qk, d_v, sm_scale, out_dtype, config, stream);
}

}  // namespace

// sparse_mla_decode_launcher over a cache in the 656-byte form: kv_fp8 [batch, n_kv_rows, 656] bytes,
// 16-byte aligned; everything else as there (idx entries < 0 or >= n_kv_rows are padding). The result
// equals sparse_mla_decode_launcher on the dequantised cache bit for bit.
extern "C" void sparse_mla_decode_fp8_launcher(void* out, const void* q, const void* kv_fp8,
                                               const int* idx, void* workspace, size_t workspace_bytes,
                                               int batch, int n_heads, int n_kv_rows, int topk, int d_qk,
                                               int d_v, float sm_scale, int out_dtype, int config,
                                               hipStream_t stream) {
    const mla::KvAddressing kva{nullptr, 0, 0, n_kv_rows};
    launch_decode_fp8(out, q, kv_fp8, idx, workspace, workspace_bytes, batch, n_heads, n_kv_rows, topk, d_qk,
                      d_v, sm_scale, out_dtype, config, kva, stream);
}

// The same over a paged cache in the 656-byte form: kv_pool_fp8 [n_pages, page_size, 656] bytes shared by
// all requests; block_table, idx and limits as sparse_mla_decode_paged_launcher (with a block table idx holds
// logical positions, without one rows of the pool). The workspace is that of sparse_mla_decode_fp8_launcher.
extern "C" void sparse_mla_decode_fp8_paged_launcher(void* out, const void* q, const void* kv_pool_fp8,
                                                     const int* block_table, const int* idx,
                                                     void* workspace, size_t workspace_bytes, int batch,
                                                     int n_heads, int n_pages, int page_size,
                                                     int max_pages_per_request, int topk, int d_qk, int d_v,
                                                     float sm_scale, int out_dtype, int config,
                                                     hipStream_t stream) {
    if (batch <= 0 || n_heads <= 0 || topk <= 0) return;
    if (n_pages <= 0 || page_size <= 0 || (page_size & (page_size - 1)) != 0 ||
        (long long)n_pages * page_size > 0x7fffffffll ||
        (block_table != nullptr && max_pages_per_request <= 0)) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    const mla::KvAddressing kva{block_table, max_pages_per_request, page_shift, 0};
    launch_decode_fp8(out, q, kv_pool_fp8, idx, workspace, workspace_bytes, batch, n_heads,
                      n_pages * page_size, topk, d_qk, d_v, sm_scale, out_dtype, config, kva, stream);
}
