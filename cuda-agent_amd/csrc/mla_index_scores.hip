// Index scores of the sparse-attention indexer, decode step: the scores whose top-k are the rows
// sparse-MLA decode gathers. Per request b and cached position t:
//
//   score[b, t] = sum_h w[b, h] * max(0, scale * q[b, h, :] . k[b, t, :])       h over the index heads
//
// q [batch, n_heads, 128] and the index-key cache k [batch, n_rows, 128] are bf16, w [batch, n_heads]
// fp32 (the per-head weights, with whatever normalisation the layer applies already in them);
// positions at or beyond lengths[b] get -inf, so that a top-k over the row never selects them.
//
// The cache is read once (256 bytes per position) against 2 * n_heads * 128 flops per position: with
// 64 heads the step is bound by HBM, so the kernel is a stream. A wavefront owns tiles of 32
// positions: S = Q K^T on v_mfma_f32_32x32x16_bf16 with Q (heads x 128) resident in registers as the
// A operand and the 32 cache rows as the B operand. In the 32x32 shapes any assignment of k to (lane
// half, step) is valid as long as both operands use it, so lane (row, half) takes the contiguous 64
// values [64*half, +64) of its row. The rows are fetched with whole lines per load instruction and
// reach that layout through a small LDS buffer private to the wavefront (see the kernel); the next
// tile's loads are in flight while the current tile is multiplied. In the result a lane holds 16
// heads of one position per head tile: ReLU, weight and the sum over heads are in-lane, plus one
// exchange between the two lane halves.
//
// FP8 form (mla_index_scores_fp8_kernel): the index keys are stored as e4m3 codes (128 bytes per
// position) with one fp32 scale per position, q as e4m3 codes with its per-head scales already
// multiplied into w:
//
//   score[b, t] = k_scale[b, t] * sum_h w[b, h] * max(0, scale * q8[b, h, :] . k8[b, t, :])
//
// Half the bytes per position; the products run on v_mfma_f32_32x32x64_f8f6f4 (two steps per head
// tile), the data path (whole-line loads, wavefront-private LDS buffer, next tiles in flight) is the same.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch_status.hpp"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int intx8 __attribute__((ext_vector_type(8)));

constexpr int INDEX_DIM = 128;
constexpr int K_STEPS = INDEX_DIM / 16;   // MFMAs per head tile and position tile
constexpr int TILE_POS = 32;
constexpr int TILES_PER_WAVE = 4;
constexpr int WG_POS = 4 * TILES_PER_WAVE * TILE_POS;  // positions per workgroup of 4 wavefronts

// grid: x = blocks of WG_POS positions, y = request. HT = n_heads / 32.
template <int HT>
__global__ __launch_bounds__(256) void mla_index_scores_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ k_cache, const float* __restrict__ w,
    const int* __restrict__ lengths, float* __restrict__ scores, int n_rows, float scale,
    const int* __restrict__ block_table, int table_stride, int page_shift, int pool_rows) {
    // block_table == null: position t of request b is row b * n_rows + t of k_cache. Otherwise k_cache is
    // a pool of pages shared by all requests and position t is row t % page of page
    // block_table[b * table_stride + t / page]; positions of unmapped pages score -inf.
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row = lane & 31;
    const int half = lane >> 5;
    const int b = blockIdx.y;
    const int n_heads = 32 * HT;
    int valid = lengths != nullptr ? lengths[b] : n_rows;
    valid = valid < 0 ? 0 : (valid > n_rows ? n_rows : valid);
    const int first_tile = (blockIdx.x * 4 * TILES_PER_WAVE + wave * TILES_PER_WAVE) * TILE_POS;
    if (first_tile >= n_rows) return;  // (no barrier in this kernel)

    // Cache rows come in with whole lines per instruction (lane l of load j fetches 16-byte chunk
    // l % 16 of row 4*j + l / 16 of the tile) and are turned into the operand layout (lane = row)
    // through an 8 KB LDS buffer private to the wavefront: chunk c of row r sits at chunk slot
    // c ^ (r % 16), which makes the 16 lanes that a write or a read instruction serves per cycle hit
    // 16 different chunk slots. (Loading the operand layout directly asks the memory pipeline for 64
    // different lines per instruction and ran at 2.2 TB/s.)
    __shared__ u32x4 s_tile[4][TILE_POS * 16];
    u32x4* tile = s_tile[wave];
    const u32x4* kb = reinterpret_cast<const u32x4*>(k_cache) +
                      (block_table == nullptr ? (size_t)b * n_rows * 16 : 0);
    u32x4 raw[8];
    auto load_tile = [&](int t0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            int t = t0 + 4 * j + (lane >> 4);
            t = t < n_rows ? t : n_rows - 1;  // rows past the end repeat the last one; not stored
            size_t r = (size_t)t;
            if (block_table != nullptr) {
                const int page = block_table[(size_t)b * table_stride + (t >> page_shift)];
                const long long pr = ((long long)page << page_shift) + (t & ((1 << page_shift) - 1));
                r = (page >= 0 && pr < pool_rows) ? (size_t)pr : 0;  // unmapped: any row, masked below
            }
            raw[j] = __builtin_nontemporal_load(kb + r * 16 + (lane & 15));
        }
    };
    auto stage_tile = [&]() {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int r = 4 * j + (lane >> 4);
            tile[r * 16 + ((lane & 15) ^ (r & 15))] = raw[j];
        }
    };
    bf16x8 kf[K_STEPS];
    auto read_operand = [&]() {
#pragma unroll
        for (int s = 0; s < K_STEPS; ++s)
            kf[s] = __builtin_bit_cast(bf16x8, tile[row * 16 + ((8 * half + s) ^ (row & 15))]);
    };
    load_tile(first_tile);

    // Q operand: head 32*ht + row, values [64*half + 8*s, +8) of step s; and this lane's weights:
    // result register i of head tile ht is head 32*ht + 8*(i/4) + 4*half + i%4
    bf16x8 qf[HT][K_STEPS];
    floatx4 wf[HT][4];
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
        const bf16x8* src = reinterpret_cast<const bf16x8*>(
            q + ((size_t)b * n_heads + 32 * ht + row) * INDEX_DIM + 64 * half);
#pragma unroll
        for (int s = 0; s < K_STEPS; ++s) qf[ht][s] = src[s];
#pragma unroll
        for (int g = 0; g < 4; ++g)
            wf[ht][g] = *reinterpret_cast<const floatx4*>(w + (size_t)b * n_heads + 32 * ht + 8 * g + 4 * half);
    }

#pragma unroll
    for (int i = 0; i < TILES_PER_WAVE; ++i) {
        const int t0 = first_tile + i * TILE_POS;
        if (t0 >= n_rows) break;
        stage_tile();  // (LDS operations of a wavefront execute in order: no barrier, the buffer is private)
        if (i + 1 < TILES_PER_WAVE && t0 + TILE_POS < n_rows) load_tile(t0 + TILE_POS);
        read_operand();
        float total = 0.f;
#pragma unroll
        for (int ht = 0; ht < HT; ++ht) {
            floatx16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < K_STEPS; ++s)
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qf[ht][s], kf[s], acc, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 16; ++j) total = fmaf(wf[ht][j / 4][j % 4], fmaxf(scale * acc[j], 0.f), total);
        }
        total += __shfl_xor(total, 32);
        const int t = t0 + row;
        if (half == 0 && t < n_rows) {
            bool live = t < valid;
            if (live && block_table != nullptr) {
                const int page = block_table[(size_t)b * table_stride + (t >> page_shift)];
                live = page >= 0 && (((long long)page << page_shift) + (t & ((1 << page_shift) - 1))) < pool_rows;
            }
            scores[(size_t)b * n_rows + t] = live ? total : -INFINITY;
        }
    }
}

constexpr int FP8_TILES_PER_WAVE = 8;
constexpr int FP8_WG_POS = 4 * FP8_TILES_PER_WAVE * TILE_POS;  // positions per workgroup of 4 wavefronts

__device__ __forceinline__ intx8 join32(u32x4 lo, u32x4 hi) {
    return intx8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
}

// grid: x = blocks of FP8_WG_POS positions, y = request. HT = n_heads / 32. Addressing as in the
// kernel above; k_scale is indexed like the rows of k_cache.
template <int HT>
__global__ __launch_bounds__(256) void mla_index_scores_fp8_kernel(
    const uint8_t* __restrict__ q, const uint8_t* __restrict__ k_cache, const float* __restrict__ k_scale,
    const float* __restrict__ w, const int* __restrict__ lengths, float* __restrict__ scores, int n_rows,
    float scale, const int* __restrict__ block_table, int table_stride, int page_shift, int pool_rows) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row = lane & 31;
    const int half = lane >> 5;
    const int b = blockIdx.y;
    const int n_heads = 32 * HT;
    int valid = lengths != nullptr ? lengths[b] : n_rows;
    valid = valid < 0 ? 0 : (valid > n_rows ? n_rows : valid);
    const int first_tile = (blockIdx.x * 4 * FP8_TILES_PER_WAVE + wave * FP8_TILES_PER_WAVE) * TILE_POS;
    if (first_tile >= n_rows) return;  // (no barrier in this kernel)

    // A key row is one 128-byte line: lane l of load j fetches 16-byte chunk l % 8 of row 8*j + l / 8
    // of the tile (8 whole lines per instruction). In the 4 KB LDS buffer of the wavefront chunk c of
    // row r sits at chunk slot c ^ ((r >> 1) & 7): rows are 128 bytes, so among the 16 rows a read
    // instruction serves per cycle the 8 of equal parity share their banks and need 8 different slots.
    __shared__ u32x4 s_tile[4][TILE_POS * 8];
    u32x4* tile = s_tile[wave];
    const size_t request_row0 = block_table == nullptr ? (size_t)b * n_rows : 0;
    const u32x4* kb = reinterpret_cast<const u32x4*>(k_cache) + request_row0 * 8;
    const float* ksb = k_scale + request_row0;
    // position -> row of the cache block (any valid row for positions that are masked below)
    auto cache_row = [&](int t) -> size_t {
        t = t < n_rows ? t : n_rows - 1;
        if (block_table == nullptr) return (size_t)t;
        const int page = block_table[(size_t)b * table_stride + (t >> page_shift)];
        const long long pr = ((long long)page << page_shift) + (t & ((1 << page_shift) - 1));
        return (page >= 0 && pr < pool_rows) ? (size_t)pr : 0;
    };
    u32x4 raw[2][4];
    float ksc[2];
    auto load_tile = [&](int t0, int slot) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            raw[slot][j] = __builtin_nontemporal_load(kb + cache_row(t0 + 8 * j + (lane >> 3)) * 8 + (lane & 7));
        ksc[slot] = ksb[cache_row(t0 + row)];
    };
    auto stage_tile = [&](int slot) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int r = 8 * j + (lane >> 3);
            tile[r * 8 + ((lane & 7) ^ ((r >> 1) & 7))] = raw[slot][j];
        }
    };
    load_tile(first_tile, 0);
    if (first_tile + TILE_POS < n_rows) load_tile(first_tile + TILE_POS, 1);

    // Q operand: head 32*ht + row; step s takes bytes [64*half + 32*s, +32) of the head's 128 (any
    // assignment of k to (lane half, step) is valid as long as the key operand uses the same);
    // weights: result register i of head tile ht is head 32*ht + 8*(i/4) + 4*half + i%4
    intx8 qf[HT][2];
    floatx4 wf[HT][4];
#pragma unroll
    for (int ht = 0; ht < HT; ++ht) {
        const u32x4* src = reinterpret_cast<const u32x4*>(q + ((size_t)b * n_heads + 32 * ht + row) * INDEX_DIM + 64 * half);
#pragma unroll
        for (int s = 0; s < 2; ++s) qf[ht][s] = join32(src[2 * s], src[2 * s + 1]);
#pragma unroll
        for (int g = 0; g < 4; ++g)
            wf[ht][g] = *reinterpret_cast<const floatx4*>(w + (size_t)b * n_heads + 32 * ht + 8 * g + 4 * half);
    }

#pragma unroll
    for (int i = 0; i < FP8_TILES_PER_WAVE; ++i) {
        const int t0 = first_tile + i * TILE_POS;
        if (t0 >= n_rows) break;
        stage_tile(i & 1);  // (LDS operations of a wavefront execute in order: no barrier, the buffer is private)
        const float key_scale = ksc[i & 1];
        if (i + 2 < FP8_TILES_PER_WAVE && t0 + 2 * TILE_POS < n_rows) load_tile(t0 + 2 * TILE_POS, i & 1);
        intx8 kf[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int c = 4 * half + 2 * s;
            kf[s] = join32(tile[row * 8 + (c ^ ((row >> 1) & 7))], tile[row * 8 + ((c + 1) ^ ((row >> 1) & 7))]);
        }
        float total = 0.f;
#pragma unroll
        for (int ht = 0; ht < HT; ++ht) {
            floatx16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 2; ++s)
                acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(qf[ht][s], kf[s], acc, 0, 0, 0, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < 16; ++j) total = fmaf(wf[ht][j / 4][j % 4], fmaxf(scale * acc[j], 0.f), total);
        }
        total += __shfl_xor(total, 32);
        const int t = t0 + row;
        if (half == 0 && t < n_rows) {
            bool live = t < valid;
            if (live && block_table != nullptr) {
                const int page = block_table[(size_t)b * table_stride + (t >> page_shift)];
                live = page >= 0 && (((long long)page << page_shift) + (t & ((1 << page_shift) - 1))) < pool_rows;
            }
            scores[(size_t)b * n_rows + t] = live ? total * key_scale : -INFINITY;
        }
    }
}

}  // namespace

namespace {

void launch_index_scores(float* scores, const void* q, const void* k_cache, const float* w,
                         const int* lengths, int batch, int n_heads, int n_rows, int head_dim,
                         float scale, const int* block_table, int table_stride, int page_shift,
                         int pool_rows, hipStream_t stream) {
    if (batch <= 0 || n_rows <= 0) return;
    if ((n_heads != 32 && n_heads != 64) || head_dim != INDEX_DIM || batch > 65535) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_cache) |
                           reinterpret_cast<uintptr_t>(w);
    if (!scores || !q || !k_cache || !w || (bits & 15u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const dim3 grid((n_rows + WG_POS - 1) / WG_POS, batch);
    const __bf16* qb = static_cast<const __bf16*>(q);
    const __bf16* kb = static_cast<const __bf16*>(k_cache);
    if (n_heads == 32) {
        mla_index_scores_kernel<1><<<grid, 256, 0, stream>>>(qb, kb, w, lengths, scores, n_rows, scale,
                                                             block_table, table_stride, page_shift, pool_rows);
    } else {
        mla_index_scores_kernel<2><<<grid, 256, 0, stream>>>(qb, kb, w, lengths, scores, n_rows, scale,
                                                             block_table, table_stride, page_shift, pool_rows);
    }
}

}  // namespace

// scores [batch, n_rows] fp32, written: sum over heads of w * relu(scale * q . k) for positions below
//        lengths[b] (all, if lengths is null), -inf beyond
// q [batch, n_heads, 128] bf16; k_cache [batch, n_rows, 128] bf16; w [batch, n_heads] fp32;
// lengths [batch] int32 or null. n_heads 32 or 64; q, k_cache and w 16-byte aligned.
// config is accepted for the launcher pattern and has one value.
extern "C" void mla_index_scores_launcher(float* scores, const void* q, const void* k_cache,
                                          const float* w, const int* lengths, int batch,
                                          int n_heads, int n_rows, int head_dim, float scale,
                                          int config, hipStream_t stream) {
    (void)config;
    launch_index_scores(scores, q, k_cache, w, lengths, batch, n_heads, n_rows, head_dim, scale, nullptr,
                        0, 0, 0, stream);
}

// The same scores over a paged index-key cache: k_pool [n_pages, page_size, 128] bf16 shared by all
// requests, block_table [batch, max_pages_per_request] int32 (negative = not mapped). Position t of
// request b is row t % page_size of page block_table[b][t / page_size]; scores has
// max_pages_per_request * page_size columns, -inf at positions >= lengths[b] and at unmapped pages.
// page_size a power of two, n_pages * page_size < 2^31.
extern "C" void mla_index_scores_paged_launcher(float* scores, const void* q, const void* k_pool,
                                                const int* block_table, const float* w,
                                                const int* lengths, int batch, int n_heads,
                                                int n_pages, int page_size, int max_pages_per_request,
                                                int head_dim, float scale, int config,
                                                hipStream_t stream) {
    (void)config;
    if (batch <= 0) return;
    if (n_pages <= 0 || page_size <= 0 || (page_size & (page_size - 1)) != 0 || max_pages_per_request <= 0 ||
        (long long)n_pages * page_size > 0x7fffffffll ||
        (long long)max_pages_per_request * page_size > 0x7fffffffll) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!block_table) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    launch_index_scores(scores, q, k_pool, w, lengths, batch, n_heads, max_pages_per_request * page_size,
                        head_dim, scale, block_table, max_pages_per_request, page_shift,
                        n_pages * page_size, stream);
}

namespace {

void launch_index_scores_fp8(float* scores, const void* q, const void* k_cache, const float* k_scale,
                             const float* w, const int* lengths, int batch, int n_heads, int n_rows,
                             int head_dim, float scale, const int* block_table, int table_stride,
                             int page_shift, int pool_rows, hipStream_t stream) {
    if (batch <= 0 || n_rows <= 0) return;
    if ((n_heads != 32 && n_heads != 64) || head_dim != INDEX_DIM || batch > 65535) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_cache) |
                           reinterpret_cast<uintptr_t>(w);
    if (!scores || !q || !k_cache || !k_scale || !w || (bits & 15u) != 0 ||
        (reinterpret_cast<uintptr_t>(k_scale) & 3u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const dim3 grid((n_rows + FP8_WG_POS - 1) / FP8_WG_POS, batch);
    const uint8_t* qb = static_cast<const uint8_t*>(q);
    const uint8_t* kb = static_cast<const uint8_t*>(k_cache);
    if (n_heads == 32) {
        mla_index_scores_fp8_kernel<1><<<grid, 256, 0, stream>>>(qb, kb, k_scale, w, lengths, scores, n_rows,
                                                                 scale, block_table, table_stride, page_shift,
                                                                 pool_rows);
    } else {
        mla_index_scores_fp8_kernel<2><<<grid, 256, 0, stream>>>(qb, kb, k_scale, w, lengths, scores, n_rows,
                                                                 scale, block_table, table_stride, page_shift,
                                                                 pool_rows);
    }
}

}  // namespace

// The scores over e4m3 index keys (OCP e4m3: 4 exponent bits, bias 7, no infinities):
// scores [batch, n_rows] fp32 = k_scale[b, t] * sum_h w[b, h] * relu(scale * q[b, h] . k_cache[b, t])
// q       [batch, n_heads, 128] e4m3 codes; the scale each head's q was quantised with is expected
//         inside w (w = head weight * q scale)
// k_cache [batch, n_rows, 128] e4m3 codes, k_scale [batch, n_rows] fp32: key row = code * k_scale
//         (what moe_quant_bf16_launcher writes for rows of 128 values)
// w [batch, n_heads] fp32; lengths [batch] int32 or null. n_heads 32 or 64; q, k_cache, w 16-byte aligned.
extern "C" void mla_index_scores_fp8_launcher(float* scores, const void* q, const void* k_cache,
                                              const float* k_scale, const float* w, const int* lengths,
                                              int batch, int n_heads, int n_rows, int head_dim,
                                              float scale, int config, hipStream_t stream) {
    (void)config;
    launch_index_scores_fp8(scores, q, k_cache, k_scale, w, lengths, batch, n_heads, n_rows, head_dim, scale,
                            nullptr, 0, 0, 0, stream);
}

// The same over a paged e4m3 key cache: k_pool [n_pages, page_size, 128] codes and
// k_scale_pool [n_pages, page_size] fp32 shared by all requests, block_table as in
// mla_index_scores_paged_launcher.
extern "C" void mla_index_scores_fp8_paged_launcher(float* scores, const void* q, const void* k_pool,
                                                    const float* k_scale_pool, const int* block_table,
                                                    const float* w, const int* lengths, int batch,
                                                    int n_heads, int n_pages, int page_size,
                                                    int max_pages_per_request, int head_dim, float scale,
                                                    int config, hipStream_t stream) {
    (void)config;
    if (batch <= 0) return;
    if (n_pages <= 0 || page_size <= 0 || (page_size & (page_size - 1)) != 0 || max_pages_per_request <= 0 ||
        (long long)n_pages * page_size > 0x7fffffffll ||
        (long long)max_pages_per_request * page_size > 0x7fffffffll) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!block_table) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    launch_index_scores_fp8(scores, q, k_pool, k_scale_pool, w, lengths, batch, n_heads,
                            max_pages_per_request * page_size, head_dim, scale, block_table,
                            max_pages_per_request, page_shift, n_pages * page_size, stream);
}
