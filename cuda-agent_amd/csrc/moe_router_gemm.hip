// Router projection of a MoE layer: logits[t, e] = sum_h x[t, h] * w[e, h], fp32.
//
// x is the layer's bf16 (or fp32) input, w the fp32 router weight [n_experts, hidden]; both are
// taken to fp32 exactly and multiplied on the fp32 matrix cores (v_mfma_f32_32x32x2_f32), so the
// result differs from an fp32 reference only by the order of the additions: the routing that
// follows compares these logits with each other, and a lower-precision product would move
// experts across the top-k boundary.
//
// A wavefront owns a 32-token x 32-expert tile of the output. The MFMA pairs lane l's A value
// (token l % 32) with lane l's B value (expert l % 32) as one k of the dot product, and any
// assignment of k to (lane half, step) works as long as A and B agree. So for every 64 values of
// k lane (row, half) reads the 32 consecutive values [64c + 32*half, +32) of its row: whole
// 128-byte lines of w, 64-byte pieces of bf16 x, straight from global memory into the operand
// registers (at 64 cycles per MFMA the loads are a small fraction of the time and need no LDS
// staging). 4 wavefronts of a workgroup cover 64 tokens x 64 experts.
//
// Few tokens: K is cut into n_splits ranges (grid z) so that the weight matrix is streamed by
// many CUs; partial sums go to a caller-provided scratch and a second kernel adds them in
// ascending split order, so the result does not depend on timing.
//
// Split-weight form (moe_router_split_weight_launcher + moe_router_logits_split_launcher): an fp32
// weight is the exact sum of three bf16 numbers (its 24 significand bits cut into 8 + 8 + 8), and a
// product of two bf16 numbers is exact in fp32. With the weight stored once as those three planes the
// projection of a bf16 x runs on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16: 8 times the rate of
// the fp32 shape, three products per weight) and still differs from an fp32 reference by the order of the
// additions only. At that rate the operand loads are what matters: rows are fetched as whole lines and
// turned into the operand layout through a small LDS buffer private to the wavefront.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch_status.hpp"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int K_CHUNK = 64;

// 32 consecutive values of a row as fp32
__device__ __forceinline__ void load32(float (&dst)[32], const float* p) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const floatx4 v = reinterpret_cast<const floatx4*>(p)[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[4 * i + j] = v[j];
    }
}
__device__ __forceinline__ void load32(float (&dst)[32], const uint16_t* p) {  // bf16 bits
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u32x4 v = reinterpret_cast<const u32x4*>(p)[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            dst[8 * i + 2 * j] = __uint_as_float(v[j] << 16);
            dst[8 * i + 2 * j + 1] = __uint_as_float(v[j] & 0xffff0000u);
        }
    }
}

// grid: x = 64-token tiles, y = 64-expert tiles, z = K split. out is logits (n_splits == 1) or
// the partial sums [split][tokens][n_experts].
template <typename X>
__global__ __launch_bounds__(256) void moe_router_gemm_kernel(const X* __restrict__ x,
                                                              const float* __restrict__ w,
                                                              float* __restrict__ out, int tokens,
                                                              int hidden, int n_experts,
                                                              int chunks_per_split) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row = lane & 31;
    const int half = lane >> 5;
    const int t0 = blockIdx.x * 64 + (wave & 1) * 32;
    const int e0 = blockIdx.y * 64 + (wave >> 1) * 32;
    if (t0 >= tokens || e0 >= n_experts) return;  // (no barrier in this kernel)
    // rows beyond the end read the last valid row; their results are not stored
    const int t = t0 + row < tokens ? t0 + row : tokens - 1;
    const int e = e0 + row < n_experts ? e0 + row : n_experts - 1;
    const int chunk_begin = blockIdx.z * chunks_per_split;
    int chunk_end = chunk_begin + chunks_per_split;
    const int n_chunks = hidden / K_CHUNK;
    if (chunk_end > n_chunks) chunk_end = n_chunks;
    const X* xp = x + (size_t)t * hidden + 32 * half;
    const float* wp = w + (size_t)e * hidden + 32 * half;

    floatx16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // two register sets: the loads of chunk c+1 are in flight while the MFMAs of chunk c run
    float a0[32], b0[32], a1[32], b1[32];
    if (chunk_begin < chunk_end) {
        load32(a0, xp + (size_t)chunk_begin * K_CHUNK);
        load32(b0, wp + (size_t)chunk_begin * K_CHUNK);
    }
    for (int c = chunk_begin; c < chunk_end; c += 2) {
        // (past the end the last chunk is read again and not used)
        const int c1 = c + 1 < chunk_end ? c + 1 : c;
        load32(a1, xp + (size_t)c1 * K_CHUNK);
        load32(b1, wp + (size_t)c1 * K_CHUNK);
#pragma unroll
        for (int s = 0; s < 32; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[s], b0[s], acc, 0, 0, 0);
        if (c + 1 >= chunk_end) break;
        const int c2 = c + 2 < chunk_end ? c + 2 : c + 1;
        load32(a0, xp + (size_t)c2 * K_CHUNK);
        load32(b0, wp + (size_t)c2 * K_CHUNK);
#pragma unroll
        for (int s = 0; s < 32; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[s], b1[s], acc, 0, 0, 0);
    }
    // result register i of a lane: token 8*(i/4) + 4*half + i%4 of the tile, expert `row`
    float* dst = out + (size_t)blockIdx.z * tokens * n_experts;
    if (e0 + row < n_experts) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int tt = t0 + 8 * (i / 4) + 4 * half + (i % 4);
            if (tt < tokens) dst[(size_t)tt * n_experts + e0 + row] = acc[i];
        }
    }
}

// ---- split-weight form ---------------------------------------------------------------------------------

// w [n] fp32 -> planes [3][n] bf16 with hi + mid + lo == w exactly: hi = the upper 16 bits of w, mid the upper
// 16 bits of w - hi, lo = w - hi - mid (at most 8 significant bits are left, so it is a bf16 number)
__global__ __launch_bounds__(256) void moe_router_split_kernel(const float* __restrict__ w,
                                                               uint16_t* __restrict__ planes, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = w[i];
    const uint32_t hi = __float_as_uint(v) & 0xffff0000u;
    const float r1 = v - __uint_as_float(hi);
    const uint32_t mid = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(mid);
    planes[i] = (uint16_t)(hi >> 16);
    planes[n + i] = (uint16_t)(mid >> 16);
    planes[2 * n + i] = (uint16_t)(__float_as_uint(r2) >> 16);
}

// grid as moe_router_gemm_kernel. A wavefront owns 32 tokens x 32 experts; per 64 values of k it fetches
// four tiles of 32 rows x 128 bytes (x and the three weight planes), each with 4 load instructions of whole
// lines (lane l: 16-byte chunk l % 8 of row 8*j + l / 8), and passes them one after the other through its
// 4 KB LDS buffer (chunk c of row r at slot c ^ ((r >> 1) & 7)) into the operand layout: lane (row, half)
// holds values [32*half, +32) of its row, 8 per MFMA step. No barrier: the buffer is private and the LDS
// operations of a wavefront execute in order.
__global__ __launch_bounds__(256) void moe_router_gemm_split_kernel(const uint16_t* __restrict__ x,
                                                                    const uint16_t* __restrict__ planes,
                                                                    float* __restrict__ out, int tokens,
                                                                    int hidden, int n_experts,
                                                                    int chunks_per_split) {
    __shared__ u32x4 s_tile[4][32 * 8];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row = lane & 31;
    const int half = lane >> 5;
    const int t0 = blockIdx.x * 64 + (wave & 1) * 32;
    const int e0 = blockIdx.y * 64 + (wave >> 1) * 32;
    if (t0 >= tokens || e0 >= n_experts) return;  // (no barrier in this kernel)
    u32x4* tile = s_tile[wave];
    const int chunk_begin = blockIdx.z * chunks_per_split;
    int chunk_end = chunk_begin + chunks_per_split;
    const int n_chunks = hidden / K_CHUNK;
    if (chunk_end > n_chunks) chunk_end = n_chunks;
    const size_t plane = (size_t)n_experts * hidden;

    // fill side: rows 8*j + lane/8 of the tile, chunk lane%8 (rows beyond the end repeat the last valid one)
    const u32x4* src[4][4];  // [x, hi, mid, lo][instruction]
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = 8 * j + (lane >> 3);
        const int t = t0 + r < tokens ? t0 + r : tokens - 1;
        const int e = e0 + r < n_experts ? e0 + r : n_experts - 1;
        src[0][j] = reinterpret_cast<const u32x4*>(x + (size_t)t * hidden) + (lane & 7);
#pragma unroll
        for (int p = 0; p < 3; ++p)
            src[1 + p][j] = reinterpret_cast<const u32x4*>(planes + p * plane + (size_t)e * hidden) + (lane & 7);
    }
    u32x4 raw[4][4];
    auto load_chunk = [&](int c) {
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int j = 0; j < 4; ++j) raw[m][j] = src[m][j][(size_t)c * (K_CHUNK * 2 / 16)];
    };
    // operand of matrix m: through the buffer
    bf16x8 op[4][4];
    auto stage = [&](int m) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = 8 * j + (lane >> 3);
            tile[r * 8 + ((lane & 7) ^ ((r >> 1) & 7))] = raw[m][j];
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
            op[m][s] = __builtin_bit_cast(bf16x8, tile[row * 8 + ((4 * half + s) ^ ((row >> 1) & 7))]);
    };

    floatx16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (chunk_begin < chunk_end) load_chunk(chunk_begin);
    for (int c = chunk_begin; c < chunk_end; ++c) {
#pragma unroll
        for (int m = 0; m < 4; ++m) stage(m);
        if (c + 1 < chunk_end) load_chunk(c + 1);  // in flight under the MFMAs below
        // smallest terms first
#pragma unroll
        for (int p = 3; p >= 1; --p)
#pragma unroll
            for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(op[0][s], op[p][s], acc, 0, 0, 0);
    }
    float* dst = out + (size_t)blockIdx.z * tokens * n_experts;
    if (e0 + row < n_experts) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int tt = t0 + 8 * (i / 4) + 4 * half + (i % 4);
            if (tt < tokens) dst[(size_t)tt * n_experts + e0 + row] = acc[i];
        }
    }
}

// The same product for many tokens: a workgroup owns 128 tokens x 64 experts and shares its operand tiles
// through LDS (per 64 values of k: 128 rows of x and 3 x 64 rows of planes, 128 bytes each = 40 KB, two
// stages). Every lane fetches 10 chunks of 16 bytes per stage (whole lines: 8 lanes per row), stores them
// swizzled as above, and after ONE barrier per stage each wavefront (64 tokens x 32 experts) reads its two x
// tiles and three plane tiles in operand layout. The per-wavefront kernel above asks its CU's L1 for 170
// bytes per clock at the bf16 MFMA rate; this one for 52.
constexpr int BIG_TOKENS = 128;
constexpr int BIG_EXPERTS = 64;
constexpr int BIG_STAGE = (BIG_TOKENS + 3 * BIG_EXPERTS) * 8;  // 16-byte slots per stage (40 KB)

__global__ __launch_bounds__(256) void moe_router_gemm_split_tiled_kernel(const uint16_t* __restrict__ x,
                                                                          const uint16_t* __restrict__ planes,
                                                                          float* __restrict__ out, int tokens,
                                                                          int hidden, int n_experts) {
    __shared__ u32x4 s_stage[2][BIG_STAGE];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int row = lane & 31;
    const int half = lane >> 5;
    const int t0 = blockIdx.x * BIG_TOKENS;
    const int e0 = blockIdx.y * BIG_EXPERTS;
    const int n_chunks = hidden / K_CHUNK;
    const size_t plane = (size_t)n_experts * hidden;

    // fill side: slot tid + 256*i of the stage, i < 10; rows 0..127 are x, then 64 rows of each plane
    const u32x4* src[10];
    int dst[10];
#pragma unroll
    for (int i = 0; i < 10; ++i) {
        const int r = (tid + 256 * i) >> 3;  // row of the stage
        const int c = tid & 7;
        if (r < BIG_TOKENS) {
            const int t = t0 + r < tokens ? t0 + r : tokens - 1;
            src[i] = reinterpret_cast<const u32x4*>(x + (size_t)t * hidden) + c;
        } else {
            const int p = (r - BIG_TOKENS) / BIG_EXPERTS;
            const int er = (r - BIG_TOKENS) % BIG_EXPERTS;
            const int e = e0 + er < n_experts ? e0 + er : n_experts - 1;
            src[i] = reinterpret_cast<const u32x4*>(planes + p * plane + (size_t)e * hidden) + c;
        }
        dst[i] = r * 8 + (c ^ ((r >> 1) & 7));
    }
    u32x4 raw[10];
    auto load_chunk = [&](int c) {
#pragma unroll
        for (int i = 0; i < 10; ++i) raw[i] = src[i][(size_t)c * (K_CHUNK * 2 / 16)];
    };
    auto store_stage = [&](int st) {
#pragma unroll
        for (int i = 0; i < 10; ++i) s_stage[st][dst[i]] = raw[i];
    };
    // read side: wavefront (wave & 1) takes tokens [64*(wave&1), +64), (wave >> 1) experts [32*(wave>>1), +32)
    const int a_row0 = 64 * (wave & 1) + row;
    const int b_row0 = BIG_TOKENS + 32 * (wave >> 1) + row;
    auto operand = [&](int st, int r, int s) {
        return __builtin_bit_cast(bf16x8, s_stage[st][r * 8 + ((4 * half + s) ^ ((r >> 1) & 7))]);
    };

    floatx16 acc[2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
        acc[a] = floatx16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    load_chunk(0);
    store_stage(0);
    __syncthreads();
    for (int c = 0; c < n_chunks; ++c) {
        const int st = c & 1;
        if (c + 1 < n_chunks) load_chunk(c + 1);  // in flight under the MFMAs below
        bf16x8 a_op[2][4];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int s = 0; s < 4; ++s) a_op[a][s] = operand(st, a_row0 + 32 * a, s);
        // smallest terms first
#pragma unroll
        for (int p = 2; p >= 0; --p) {
            bf16x8 b_op[4];
#pragma unroll
            for (int s = 0; s < 4; ++s) b_op[s] = operand(st, b_row0 + BIG_EXPERTS * p, s);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_op[0][s], b_op[s], acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_op[1][s], b_op[s], acc[1], 0, 0, 0);
            }
        }
        if (c + 1 < n_chunks) store_stage(st ^ 1);  // (last read before the barrier that ended the previous pass)
        __syncthreads();
    }
    const int e = e0 + 32 * (wave >> 1) + row;
    if (e < n_experts) {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int tt = t0 + 64 * (wave & 1) + 32 * a + 8 * (i / 4) + 4 * half + (i % 4);
                if (tt < tokens) out[(size_t)tt * n_experts + e] = acc[a][i];
            }
    }
}

// logits = partial[0] + partial[1] + ... in that order
__global__ __launch_bounds__(256) void moe_router_reduce_kernel(const float* __restrict__ partial,
                                                                float* __restrict__ logits,
                                                                size_t count, int n_splits) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    // eight loads at a time are in flight; the additions stay in ascending split order
    float sum = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = s0 + j < n_splits ? partial[(size_t)(s0 + j) * count + i] : 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (s0 + j < n_splits) sum = (s0 + j == 0) ? v[j] : sum + v[j];
    }
    logits[i] = sum;
}

int pick_router_splits(int tokens, int hidden, int n_experts) {
    const long tiles = (long)((tokens + 63) / 64) * ((n_experts + 63) / 64);
    const int n_chunks = hidden / K_CHUNK;
    int splits = 1;
    // aim at about two workgroups per CU; every split keeps at least 2 chunks
    while (tiles * splits < 512 && splits * 2 * 2 <= n_chunks) splits *= 2;
    return splits;
}

}  // namespace

// K splits the launcher uses for these sizes (1 = no scratch needed)
extern "C" int moe_router_logits_num_splits(int tokens, int hidden, int n_experts) {
    if (tokens <= 0 || hidden <= 0 || n_experts <= 0 || hidden % K_CHUNK != 0) return 0;
    return pick_router_splits(tokens, hidden, n_experts);
}

// bytes of scratch moe_router_logits_launcher needs (0 when K is not split)
extern "C" size_t moe_router_logits_workspace_bytes(int tokens, int hidden, int n_experts) {
    const int splits = moe_router_logits_num_splits(tokens, hidden, n_experts);
    return splits <= 1 ? 0 : (size_t)splits * tokens * n_experts * sizeof(float);
}

// logits [tokens, n_experts] fp32 = x [tokens, hidden] (x_dtype 0 = fp32, 1 = bf16) times
// w [n_experts, hidden] fp32, transposed. hidden a multiple of 64; x and w 16-byte aligned.
// workspace: moe_router_logits_workspace_bytes(...) bytes of device scratch (may be null if 0).
extern "C" void moe_router_logits_launcher(float* logits, const void* x, const float* w,
                                           void* workspace, size_t workspace_bytes, int tokens,
                                           int hidden, int n_experts, int x_dtype, int config,
                                           hipStream_t stream) {
    (void)config;
    if (tokens <= 0 || n_experts <= 0) return;
    if (hidden <= 0 || hidden % K_CHUNK != 0 || (x_dtype != 0 && x_dtype != 1) ||
        (tokens + 63) / 64 > 0x7fffffff / 64 || (n_experts + 63) / 64 > 65535) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) |
                           reinterpret_cast<uintptr_t>(workspace);
    if (!logits || !x || !w || (bits & 15u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const int splits = pick_router_splits(tokens, hidden, n_experts);
    const size_t need = splits <= 1 ? 0 : (size_t)splits * tokens * n_experts * sizeof(float);
    if (need > 0 && (!workspace || workspace_bytes < need)) {
        caa::set_status(CAA_WORKSPACE_TOO_SMALL);
        return;
    }
    const int n_chunks = hidden / K_CHUNK;
    const int chunks_per_split = (n_chunks + splits - 1) / splits;
    float* out = splits > 1 ? static_cast<float*>(workspace) : logits;
    const dim3 grid((tokens + 63) / 64, (n_experts + 63) / 64, splits);
    if (x_dtype == 0) {
        moe_router_gemm_kernel<float><<<grid, 256, 0, stream>>>(
            static_cast<const float*>(x), w, out, tokens, hidden, n_experts, chunks_per_split);
    } else {
        moe_router_gemm_kernel<uint16_t><<<grid, 256, 0, stream>>>(
            static_cast<const uint16_t*>(x), w, out, tokens, hidden, n_experts, chunks_per_split);
    }
    if (splits > 1) {
        const size_t count = (size_t)tokens * n_experts;
        moe_router_reduce_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(
            static_cast<const float*>(workspace), logits, count, splits);
    }
}

// planes [3, n_experts, hidden] bf16 (written) from w [n_experts, hidden] fp32: the three bf16 numbers whose
// sum is the weight, for moe_router_logits_split_launcher. Done once per weight.
extern "C" void moe_router_split_weight_launcher(void* planes, const float* w, int n_experts, int hidden,
                                                 hipStream_t stream) {
    if (n_experts <= 0 || hidden <= 0) return;
    if (!planes || !w) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const size_t n = (size_t)n_experts * hidden;
    moe_router_split_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(w, static_cast<uint16_t*>(planes), n);
}

// moe_router_logits_launcher for a bf16 x and a weight given as the planes above: the same logits up to the
// order of the fp32 additions, on the bf16 matrix cores. Sizes, scratch (moe_router_logits_workspace_bytes)
// and limits as there; x and planes 16-byte aligned, hidden a multiple of 64.
extern "C" void moe_router_logits_split_launcher(float* logits, const void* x, const void* planes,
                                                 void* workspace, size_t workspace_bytes, int tokens,
                                                 int hidden, int n_experts, int config, hipStream_t stream) {
    if (tokens <= 0 || n_experts <= 0) return;
    if (hidden <= 0 || hidden % K_CHUNK != 0 || (tokens + 63) / 64 > 0x7fffffff / 64 ||
        (n_experts + 63) / 64 > 65535) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(planes) |
                           reinterpret_cast<uintptr_t>(workspace);
    if (!logits || !x || !planes || (bits & 15u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const int splits = pick_router_splits(tokens, hidden, n_experts);
    const size_t need = splits <= 1 ? 0 : (size_t)splits * tokens * n_experts * sizeof(float);
    if (need > 0 && (!workspace || workspace_bytes < need)) {
        caa::set_status(CAA_WORKSPACE_TOO_SMALL);
        return;
    }
    const int n_chunks = hidden / K_CHUNK;
    // enough 128 x 64 tiles to fill the chip: the workgroup-tiled kernel (config 1 forces the other one)
    if (splits == 1 && config != 1 &&
        (long)((tokens + BIG_TOKENS - 1) / BIG_TOKENS) * ((n_experts + BIG_EXPERTS - 1) / BIG_EXPERTS) >= 192) {
        const dim3 big_grid((tokens + BIG_TOKENS - 1) / BIG_TOKENS, (n_experts + BIG_EXPERTS - 1) / BIG_EXPERTS);
        moe_router_gemm_split_tiled_kernel<<<big_grid, 256, 0, stream>>>(
            static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(planes), logits, tokens, hidden,
            n_experts);
        return;
    }
    const int chunks_per_split = (n_chunks + splits - 1) / splits;
    float* out = splits > 1 ? static_cast<float*>(workspace) : logits;
    const dim3 grid((tokens + 63) / 64, (n_experts + 63) / 64, splits);
    moe_router_gemm_split_kernel<<<grid, 256, 0, stream>>>(static_cast<const uint16_t*>(x),
                                                           static_cast<const uint16_t*>(planes), out, tokens,
                                                           hidden, n_experts, chunks_per_split);
    if (splits > 1) {
        const size_t count = (size_t)tokens * n_experts;
        moe_router_reduce_kernel<<<(unsigned)((count + 255) / 256), 256, 0, stream>>>(
            static_cast<const float*>(workspace), logits, count, splits);
    }
}
