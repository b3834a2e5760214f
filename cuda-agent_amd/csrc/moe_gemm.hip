// Grouped FP8 GEMMs of the MoE layer, weight-streaming form.
//
//   gate/up:  gu[p, :] = sum_kb (x_q[tok(p), kb] . w13_q[e, :, kb]) * x_s[tok(p), kb] * w13_s[e, nb, kb]
//             h[p, j]  = silu(gu[p, j]) * gu[p, I + j]  -> quantised per 128 group to e4m3
//   down:     y[p, :]  = sum_kb (h_q[p, kb] . w2_q[e, :, kb]) * h_s[p, kb] * w2_s[e, nb, kb]
//
// for every sorted pair p of expert e (kb runs over 128-wide blocks of the reduction
// dimension). A workgroup owns one expert and one 128-row block of its weight matrix (for
// gate/up: 128 gate rows and the matching 128 up rows, so the activation can be fused) and
// streams those rows from HBM exactly once per pass over up to 16*NT pairs.
//
// One v_mfma_f32_16x16x128_f8f6f4 consumes a whole 128-block of K for 16 weight rows (A operand)
// and 16 pairs (B operand): its 16x16 fp32 result is the unscaled partial of that block and is
// folded into the accumulator with one multiply-add per value by the product of the two block
// scales. In the result layout a lane holds four consecutive weight rows of ONE pair, so the
// scale product is a per-lane scalar. The position of a byte inside a 128-block is immaterial to
// a dot product as long as both operands agree, so a lane's 32 operand bytes are bytes
// [16g, 16g+16) and [64+16g, 64+16g+16) of the block (g = lane/16): each 16-byte load
// instruction then covers 64 contiguous bytes of every row it touches.
//
// With few pairs per expert (decode) the kernel is a pure weight stream: every weight byte is
// read once, used by one MFMA per 16 pairs, and the accumulators stay in registers. With many
// pairs per expert it makes one pass per 16*NT pairs and re-reads the block from L2.
#include "launch_status.hpp"
#include "moe_common.hpp"

namespace {

using namespace moe;

typedef int intx8 __attribute__((ext_vector_type(8)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ intx8 join(intx4 lo, intx4 hi) {
    return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

__device__ __forceinline__ float silu(float x) { return x / (1.f + expf(-x)); }

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// 8 e4m3 codes (two dwords) -> 8 bf16, exactly (every e4m3 value is a bf16 value)
__device__ __forceinline__ bf16x8 e4m3x8_to_bf16(int lo, int hi) {
    const bf16x2 a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
    const bf16x2 b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
    const bf16x2 c = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
    const bf16x2 d = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
    return bf16x8{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

// A lane's 32 operand bytes of one 128-block as the operands of four v_mfma_f32_16x16x32_bf16 steps:
// step s takes bytes 8s..8s+7 of the lane (which 32 of the block's 128 elements a step covers is
// immaterial as long as both operands are cut the same way).
struct Bf16Block {
    bf16x8 step[4];
};
__device__ __forceinline__ Bf16Block to_bf16_block(intx8 v) {
    Bf16Block r;
#pragma unroll
    for (int s = 0; s < 4; ++s) r.step[s] = e4m3x8_to_bf16(v[2 * s], v[2 * s + 1]);
    return r;
}

// Unscaled dot products of one 128-block for 16 weight rows x 16 pairs.
// EXACT: on the bf16 matrix core, which adds the (exact) products without losing bits that matter (measured
// on gfx950: |error| <= 2^-25 of the sum of |products|, against 2^-16 for the e4m3 instruction), so that the
// requantised codes of h agree with an fp32 evaluation. Otherwise one e4m3 instruction.
__device__ __forceinline__ floatx4 block_dot_bf16(const Bf16Block& a, const Bf16Block& b) {
    floatx4 part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 4; ++s) part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.step[s], b.step[s], part, 0, 0, 0);
    return part;
}

// Epilogue of the streaming gate/up kernels: h = silu(gate) * up, e4m3 with one scale per pair over the
// workgroup's 128 columns. acc[nt][t]: tiles 0, 1 gate, 2, 3 up; a lane holds rows 4g..4g+3 of each 16-row
// tile for pair column `col`.
template <int NT>
__device__ __forceinline__ void gate_up_epilogue(const floatx4 (&acc)[NT][4], float (*s_amax)[NT * 16],
                                                 const int (&pos)[NT], int end, uint8_t* __restrict__ h_q,
                                                 float* __restrict__ h_s, int inter, int rb, int wave, int col,
                                                 int g, bool pow2) {
    floatx4 h[NT][2];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        float amax = 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float v = silu(acc[nt][i][r]) * acc[nt][2 + i][r];
                h[nt][i][r] = v;
                amax = fmaxf(amax, fabsf(v));
            }
        }
        amax = fmaxf(amax, __shfl_xor(amax, 16));
        amax = fmaxf(amax, __shfl_xor(amax, 32));
        if (g == 0) s_amax[wave][nt * 16 + col] = amax;
    }
    __syncthreads();
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int idx = nt * 16 + col;
        const float amax =
            fmaxf(fmaxf(s_amax[0][idx], s_amax[1][idx]), fmaxf(s_amax[2][idx], s_amax[3][idx]));
        const float scale = group_scale(amax, pow2);
        if (pos[nt] < end) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                float q[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    q[r] = fminf(fmaxf(h[nt][i][r] / scale, -E4M3_MAX), E4M3_MAX);
                }
                int packed = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
                packed = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], packed, true);
                *reinterpret_cast<int*>(h_q + (size_t)pos[nt] * inter + rb * GROUP + wave * 32 + i * 16 +
                                        4 * g) = packed;
            }
            if (wave == 0 && g == 0) h_s[(size_t)pos[nt] * (inter / GROUP) + rb] = scale;
        }
    }
}

// GATE_UP: 4 weight tiles per wavefront (2 gate + 2 up), output h_q/h_s.
// otherwise: 2 weight tiles per wavefront, output y.
template <bool GATE_UP, int NT, bool EXACT = false>
__global__ __launch_bounds__(256) void moe_stream_gemm_kernel(
    const uint8_t* __restrict__ w_q, const float* __restrict__ w_s, const uint8_t* __restrict__ a_q,
    const float* __restrict__ a_s, const int* __restrict__ sorted_pairs,
    const int* __restrict__ expert_offsets, uint8_t* __restrict__ h_q, float* __restrict__ h_s,
    float* __restrict__ y, int K, int n_rows, int inter, int top_k, bool pow2,
    bool last_first) {
    constexpr int TILES = GATE_UP ? 4 : 2;
    __shared__ float s_amax[4][NT * 16];

    // last_first: the last expert is the heaviest (a shared expert that every token uses): its
    // workgroups are dispatched first, so that its several passes do not become the launch's tail
    const int e = last_first ? (blockIdx.y == 0 ? (int)gridDim.y - 1 : (int)blockIdx.y - 1) : (int)blockIdx.y;
    const int rb = blockIdx.x;  // 128-row block of the output dimension
    const int begin = expert_offsets[e];
    const int end = expert_offsets[e + 1];
    if (end <= begin) return;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int col = lane & 15;
    const int g = lane >> 4;
    const int KB = K / GROUP;
    const int row_blocks = n_rows / GROUP;

    // weight row pointers of this lane's A operands, at byte 16*g of block 0
    const uint8_t* a_ptr[TILES];
    const float* ws_ptr[GATE_UP ? 2 : 1];
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        int row = rb * GROUP + wave * 32 + (t & 1) * 16 + col;
        if (GATE_UP && t >= 2) row += inter;
        a_ptr[t] = w_q + ((size_t)e * n_rows + row) * K + 16 * g;
    }
    ws_ptr[0] = w_s + ((size_t)e * row_blocks + rb) * KB;
    if (GATE_UP) ws_ptr[1] = w_s + ((size_t)e * row_blocks + inter / GROUP + rb) * KB;

    for (int pass_begin = begin; pass_begin < end; pass_begin += 16 * NT) {
        // activation rows of this lane's B operands
        const uint8_t* b_ptr[NT];
        const float* bs_ptr[NT];
        int pos[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            pos[nt] = pass_begin + 16 * nt + col;
            const int p = pos[nt] < end ? pos[nt] : end - 1;  // clamped rows are computed, not stored
            const int row = GATE_UP ? sorted_pairs[p] / top_k : p;
            b_ptr[nt] = a_q + (size_t)row * K + 16 * g;
            bs_ptr[nt] = a_s + (size_t)row * KB;
        }

        floatx4 acc[NT][TILES];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int t = 0; t < TILES; ++t) acc[nt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

        intx4 a_lo[2][TILES], a_hi[2][TILES], b_lo[2][NT], b_hi[2][NT];
        float b_scale[2][NT], w_scale[2][GATE_UP ? 2 : 1];
        auto load_block = [&](int kb, int buf) {
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                a_lo[buf][t] = __builtin_nontemporal_load(
                    reinterpret_cast<const intx4*>(a_ptr[t] + (size_t)kb * GROUP));
                a_hi[buf][t] = __builtin_nontemporal_load(
                    reinterpret_cast<const intx4*>(a_ptr[t] + (size_t)kb * GROUP + 64));
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                b_lo[buf][nt] = *reinterpret_cast<const intx4*>(b_ptr[nt] + (size_t)kb * GROUP);
                b_hi[buf][nt] = *reinterpret_cast<const intx4*>(b_ptr[nt] + (size_t)kb * GROUP + 64);
                b_scale[buf][nt] = bs_ptr[nt][kb];
            }
            w_scale[buf][0] = ws_ptr[0][kb];
            if (GATE_UP) w_scale[buf][1] = ws_ptr[1][kb];
        };
        auto compute_block = [&](int buf) {
            if constexpr (EXACT) {
                Bf16Block a[TILES];
#pragma unroll
                for (int t = 0; t < TILES; ++t) a[t] = to_bf16_block(join(a_lo[buf][t], a_hi[buf][t]));
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const Bf16Block b = to_bf16_block(join(b_lo[buf][nt], b_hi[buf][nt]));
#pragma unroll
                    for (int t = 0; t < TILES; ++t) {
                        const float s = b_scale[buf][nt] * w_scale[buf][GATE_UP ? (t >> 1) : 0];
                        acc[nt][t] += block_dot_bf16(a[t], b) * s;
                    }
                }
                return;
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const intx8 b = join(b_lo[buf][nt], b_hi[buf][nt]);
#pragma unroll
                for (int t = 0; t < TILES; ++t) {
                    const floatx4 part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        join(a_lo[buf][t], a_hi[buf][t]), b, floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0,
                        0, 0);
                    const float s = b_scale[buf][nt] * w_scale[buf][GATE_UP ? (t >> 1) : 0];
                    acc[nt][t] += part * s;
                }
            }
        };

        load_block(0, 0);
        for (int kb = 0; kb < KB; kb += 2) {
            if (kb + 1 < KB) load_block(kb + 1, 1);
            compute_block(0);
            if (kb + 1 < KB) {
                if (kb + 2 < KB) load_block(kb + 2, 0);
                compute_block(1);
            }
        }

        if constexpr (GATE_UP) {
            gate_up_epilogue<NT>(acc, s_amax, pos, end, h_q, h_s, inter, rb, wave, col, g, pow2);
            __syncthreads();  // s_amax is reused by the next pass
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (pos[nt] < end) {
#pragma unroll
                    for (int i = 0; i < 2; ++i) {
                        *reinterpret_cast<floatx4*>(y + (size_t)pos[nt] * n_rows + rb * GROUP +
                                                    wave * 32 + i * 16 + 4 * g) = acc[nt][i];
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Streaming form, LDS-staged (the decode path).
//
// Loading the MFMA operand directly makes every load instruction touch 64-byte half lines of 16
// different rows, and that access pattern was measured to saturate at 5.3 TB/s on this part,
// against 6.9 TB/s as soon as each instruction covers whole 128-byte lines. Here the weights
// (and the activations) are therefore brought in by global->LDS loads of 16 bytes per lane in
// which the 8 lanes of a row fetch one full 128-byte line, and the operands are then read from
// LDS in the MFMA layout. Every wavefront stages only the rows it consumes itself (4 tiles of 16
// weight rows, and its own copy of the 16*NT activation rows), so the K loop needs no
// workgroup barrier: a wavefront waits on its own load counter only. A ring of DEPTH stages of one
// 128-block each keeps DEPTH-1 blocks (~40 KB per block and workgroup) in flight.
//
// LDS slot of the 16-byte chunk c of row r in a 16x128-byte tile: r*8 + (c ^ (r & 7)); the 8
// lanes that read chunk g of rows 0..7 (or 8..15) then hit 8 different bank groups.
// A workgroup covers 256 output rows: 128 gate + 128 up rows (GATE_UP), or 256 rows of w2.
// ---------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_void_ptr;

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
    asm volatile("" ::: "memory");  // LDS reads below must not be moved above the wait
}

// 64 lanes x 16 bytes: global (base + per-lane byte offset) -> LDS (lds_base + lane*16).
// An asm statement, so the loads stay outside the compiler's bookkeeping of outstanding memory
// operations; their completion is awaited explicitly with wait_vmcnt<>().
__device__ __forceinline__ void dma16(const void* base, uint32_t lane_byte_offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_byte_offset), "s"(base), "s"(lds_base)
                 : "memory", "m0");
}
// The same load with the non-temporal hint, for weights that this launch reads exactly once (an expert whose
// pairs fit one pass): the stream then does not displace what the caches hold for others and runs 10 % faster
// (decode layer 1.65 -> 1.48 ms); weights that a later pass reads again keep the plain load (with the hint a
// 1024-token layer, two passes per expert, was 1.4 % slower).
__device__ __forceinline__ void dma16_stream(const void* base, uint32_t lane_byte_offset, uint32_t lds_base, bool once) {
    if (once) {
        asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     :
                     : "v"(lane_byte_offset), "s"(base), "s"(lds_base)
                     : "memory", "m0");
    } else {
        dma16(base, lane_byte_offset, lds_base);
    }
}
__device__ __forceinline__ void dma16_ptr(const void* lane_ptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(lane_ptr), "s"(lds_base)
                 : "memory", "m0");
}

template <bool GATE_UP, int NT, bool EXACT = false>
__global__ __launch_bounds__(256) void moe_stream_gemm_lds_kernel(
    const uint8_t* __restrict__ w_q, const float* __restrict__ w_s, const uint8_t* __restrict__ a_q,
    const float* __restrict__ a_s, const int* __restrict__ sorted_pairs,
    const int* __restrict__ expert_offsets, uint8_t* __restrict__ h_q, float* __restrict__ h_s,
    float* __restrict__ y, int K, int n_rows, int inter, int top_k, bool pow2,
    bool last_first) {
    constexpr int TILES = 4;
    constexpr int DEPTH = 3;
    constexpr int TILE_BYTES = 16 * GROUP;                       // 2 KB
    constexpr int STAGE_BYTES = (TILES + NT) * TILE_BYTES;       // per wavefront
    constexpr int PER_STAGE = 2 * (TILES + NT);                  // load instructions per stage
    constexpr int MAX_KB = 64;
    __shared__ __attribute__((aligned(16))) uint8_t s_ring[4 * DEPTH * STAGE_BYTES];
    __shared__ float s_bscale[MAX_KB][NT * 16];
    __shared__ float s_amax[4][NT * 16];

    // last_first: the last expert is the heaviest (a shared expert that every token uses): its
    // workgroups are dispatched first, so that its several passes do not become the launch's tail
    const int e = last_first ? (blockIdx.y == 0 ? (int)gridDim.y - 1 : (int)blockIdx.y - 1) : (int)blockIdx.y;
    const int rb = blockIdx.x;  // block of 256 output rows (GATE_UP: 128 gate + 128 up)
    const int begin = expert_offsets[e];
    const int end = expert_offsets[e + 1];
    if (end <= begin) return;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col = lane & 15;
    const int g = lane >> 4;
    const int KB = K / GROUP;
    const int row_blocks = n_rows / GROUP;

    // first weight row of each of this wavefront's tiles, and the scale rows they belong to
    const uint8_t* tile_base[TILES];
    const float* ws_ptr[2];
    if (GATE_UP) {
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const int row = (t >> 1) * inter + rb * GROUP + wave * 32 + (t & 1) * 16;
            tile_base[t] = w_q + ((size_t)e * n_rows + row) * K;
        }
        ws_ptr[0] = w_s + ((size_t)e * row_blocks + rb) * KB;
        ws_ptr[1] = w_s + ((size_t)e * row_blocks + inter / GROUP + rb) * KB;
    } else {
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const int row = rb * 256 + wave * 64 + t * 16;
            tile_base[t] = w_q + ((size_t)e * n_rows + row) * K;
        }
        // wavefronts 0,1 sit in the first 128-row block, 2,3 in the second
        ws_ptr[0] = w_s + ((size_t)e * row_blocks + rb * 2 + (wave >> 1)) * KB;
        ws_ptr[1] = ws_ptr[0];
    }

    // load side: lane j of instruction i fills slot i*64 + j = (row i*8 + j/8, position j%8),
    // i.e. fetches chunk (j%8) ^ (j/8) of that row
    const uint32_t ld_row = lane >> 3;
    const uint32_t ld_chunk = (lane & 7) ^ ld_row;
    const uint32_t ld_off = ld_row * (uint32_t)K + 16 * ld_chunk;  // + 8*K for the second instruction
    // read side: lane (col, g) takes chunks g and 4+g of row col
    const uint32_t rd_off = (col * 8 + (g ^ (col & 7))) * 16;

    const uint32_t ring_base = (uint32_t)(size_t)((lds_void_ptr)s_ring) + wave * (DEPTH * STAGE_BYTES);
    typedef const __attribute__((address_space(3))) intx4* lds_x4;
    const __attribute__((address_space(3))) uint8_t* ring_ptr =
        (const __attribute__((address_space(3))) uint8_t*)s_ring + wave * (DEPTH * STAGE_BYTES);

    const bool single_pass = end - begin <= 16 * NT;  // the weights of this workgroup are read once
    for (int pass_begin = begin; pass_begin < end; pass_begin += 16 * NT) {
        // activation rows: the one this lane loads (row ld_row / ld_row + 8 of tile nt) and the
        // one whose results it ends up holding (col)
        const uint8_t* b_ld[NT][2];
        int pos[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            pos[nt] = pass_begin + 16 * nt + col;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                int p = pass_begin + 16 * nt + i * 8 + (int)ld_row;
                p = p < end ? p : end - 1;  // clamped rows are computed, not stored
                const int row = GATE_UP ? sorted_pairs[p] / top_k : p;
                b_ld[nt][i] = a_q + (size_t)row * K + 16 * ld_chunk;
            }
        }
        __syncthreads();  // the previous pass is done with s_bscale / s_amax
        for (int i = threadIdx.x; i < KB * NT * 16; i += 256) {
            const int kb = i / (NT * 16);
            const int c = i - kb * (NT * 16);
            int p = pass_begin + c;
            p = p < end ? p : end - 1;
            const int row = GATE_UP ? sorted_pairs[p] / top_k : p;
            s_bscale[kb][c] = a_s[(size_t)row * KB + kb];
        }
        __syncthreads();
        wait_vmcnt<0>();  // nothing of the compiler's is in flight when the counted loads start

        auto issue_stage = [&](int kb) {
            const uint32_t stage = ring_base + (kb % DEPTH) * STAGE_BYTES;
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                dma16_stream(tile_base[t] + (size_t)kb * GROUP, ld_off, stage + t * TILE_BYTES, single_pass);
                dma16_stream(tile_base[t] + (size_t)kb * GROUP + (size_t)8 * K, ld_off, stage + t * TILE_BYTES + 1024,
                             single_pass);
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                dma16_ptr(b_ld[nt][0] + (size_t)kb * GROUP, stage + (TILES + nt) * TILE_BYTES);
                dma16_ptr(b_ld[nt][1] + (size_t)kb * GROUP, stage + (TILES + nt) * TILE_BYTES + 1024);
            }
        };

        floatx4 acc[NT][TILES];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int t = 0; t < TILES; ++t) acc[nt][t] = floatx4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
            if (d < KB) issue_stage(d);

        for (int kb = 0; kb < KB; ++kb) {
            if (kb + DEPTH - 1 < KB) {
                issue_stage(kb + DEPTH - 1);
                wait_vmcnt<(DEPTH - 1) * PER_STAGE>();
            } else if (kb + DEPTH - 2 < KB && DEPTH > 2) {
                wait_vmcnt<(DEPTH - 2) * PER_STAGE>();
            } else {
                wait_vmcnt<0>();
            }
            const __attribute__((address_space(3))) uint8_t* stage = ring_ptr + (kb % DEPTH) * STAGE_BYTES;
            const float ws0 = ws_ptr[0][kb];
            const float ws1 = ws_ptr[1][kb];
            intx8 a[TILES];
#pragma unroll
            for (int t = 0; t < TILES; ++t) {
                const intx4 lo = *(lds_x4)(stage + t * TILE_BYTES + rd_off);
                const intx4 hi = *(lds_x4)(stage + t * TILE_BYTES + (rd_off ^ 64));
                a[t] = join(lo, hi);
            }
            if constexpr (EXACT) {
                Bf16Block ab[TILES];
#pragma unroll
                for (int t = 0; t < TILES; ++t) ab[t] = to_bf16_block(a[t]);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const intx4 lo = *(lds_x4)(stage + (TILES + nt) * TILE_BYTES + rd_off);
                    const intx4 hi = *(lds_x4)(stage + (TILES + nt) * TILE_BYTES + (rd_off ^ 64));
                    const Bf16Block b = to_bf16_block(join(lo, hi));
                    const float bs = s_bscale[kb][nt * 16 + col];
#pragma unroll
                    for (int t = 0; t < TILES; ++t) {
                        acc[nt][t] += block_dot_bf16(ab[t], b) * (bs * ((t >> 1) ? ws1 : ws0));
                    }
                }
            } else {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const intx4 lo = *(lds_x4)(stage + (TILES + nt) * TILE_BYTES + rd_off);
                    const intx4 hi = *(lds_x4)(stage + (TILES + nt) * TILE_BYTES + (rd_off ^ 64));
                    const intx8 b = join(lo, hi);
                    const float bs = s_bscale[kb][nt * 16 + col];
#pragma unroll
                    for (int t = 0; t < TILES; ++t) {
                        const floatx4 part = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            a[t], b, floatx4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                        acc[nt][t] += part * (bs * ((t >> 1) ? ws1 : ws0));
                    }
                }
            }
            asm volatile("" ::: "memory");  // this stage's LDS reads stay above the next refill
        }

        if constexpr (GATE_UP) {
            gate_up_epilogue<NT>(acc, s_amax, pos, end, h_q, h_s, inter, rb, wave, col, g, pow2);
        } else {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                if (pos[nt] < end) {
#pragma unroll
                    for (int t = 0; t < TILES; ++t) {
                        *reinterpret_cast<floatx4*>(y + (size_t)pos[nt] * n_rows + rb * 256 + wave * 64 +
                                                    t * 16 + 4 * g) = acc[nt][t];
                    }
                }
            }
        }
    }
}

bool check_common(int hidden, int inter, int n_experts) {
    return hidden > 0 && inter > 0 && n_experts > 0 && hidden % GROUP == 0 && inter % GROUP == 0 &&
           n_experts <= 65535;
}

}  // namespace

// h_q [pairs, inter] e4m3 and h_s [pairs, inter/128] fp32 (rows in sorted order) from
// x_q [tokens, hidden] e4m3, x_s [tokens, hidden/128], w13_q [E, 2*inter, hidden] e4m3,
// w13_s [E, 2*inter/128, hidden/128].
// config: 0 sizes the pass from the average pairs per expert; 1, 2, 4 force 16, 32, 64 pairs per
// pass; adding 8 selects the kernel that loads MFMA operands directly instead of staging in LDS.
// The block products run on the bf16 matrix core (codes converted in registers; exact sums, so that the
// requantised h agrees with an fp32 evaluation); +512 (CONFIG_APPROX_REQUANT): on the e4m3 matrix core,
// whose sums carry about 16 bits.
extern "C" void moe_gate_up_launcher(void* h_q, float* h_s, const void* x_q, const float* x_s,
                                     const void* w13_q, const float* w13_s, const int* sorted_pairs,
                                     const int* expert_offsets, int tokens, int hidden, int inter,
                                     int n_experts, int top_k, int config, hipStream_t stream) {
    if (tokens <= 0) return;
    if (!check_common(hidden, inter, n_experts) || top_k <= 0) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!h_q || !h_s || !x_q || !x_s || !w13_q || !w13_s || !sorted_pairs || !expert_offsets ||
        ((reinterpret_cast<uintptr_t>(x_q) | reinterpret_cast<uintptr_t>(w13_q) |
          reinterpret_cast<uintptr_t>(h_q)) & 15u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const dim3 grid(inter / GROUP, n_experts);
    auto* hq = static_cast<uint8_t*>(h_q);
    const auto* xq = static_cast<const uint8_t*>(x_q);
    const auto* wq = static_cast<const uint8_t*>(w13_q);
    const bool pow2 = (config & CONFIG_UE8M0) != 0;
    const bool last_first = (config & CONFIG_LAST_EXPERT_FIRST) != 0;
    const bool exact = (config & CONFIG_APPROX_REQUANT) == 0;
    config &= ~(CONFIG_UE8M0 | CONFIG_LAST_EXPERT_FIRST | CONFIG_REQUANT_BITS);
    int nt = config & 7;
    if (nt != 1 && nt != 2 && nt != 4) {
        const long avg = (long)tokens * top_k / n_experts;  // pairs per expert if spread evenly
        nt = avg <= 16 ? 1 : avg <= 32 ? 2 : 4;
    }
    const bool lds_path = config < 8 && hidden / GROUP <= 64 && nt < 4;  // config 8+nt: direct-operand loads
#define MOE_GATE_UP_LAUNCH(KERNEL, NT_, EXACT_)                                                           \
    KERNEL<true, NT_, EXACT_><<<grid, 256, 0, stream>>>(wq, w13_s, xq, x_s, sorted_pairs, expert_offsets, \
                                                       hq, h_s, nullptr, hidden, 2 * inter, inter, top_k, \
                                                       pow2, last_first)
#define MOE_GATE_UP_CASE(NT_)                                                           \
    if (lds_path && exact) MOE_GATE_UP_LAUNCH(moe_stream_gemm_lds_kernel, NT_, true);   \
    else if (lds_path) MOE_GATE_UP_LAUNCH(moe_stream_gemm_lds_kernel, NT_, false);      \
    else if (exact) MOE_GATE_UP_LAUNCH(moe_stream_gemm_kernel, NT_, true);              \
    else MOE_GATE_UP_LAUNCH(moe_stream_gemm_kernel, NT_, false)
    switch (nt) {
        case 1: MOE_GATE_UP_CASE(1); break;
        case 2: MOE_GATE_UP_CASE(2); break;
        default:
            if (exact) MOE_GATE_UP_LAUNCH(moe_stream_gemm_kernel, 4, true);
            else MOE_GATE_UP_LAUNCH(moe_stream_gemm_kernel, 4, false);
            break;
    }
#undef MOE_GATE_UP_CASE
#undef MOE_GATE_UP_LAUNCH
}

// y [pairs, hidden] fp32 (rows in sorted order) from h_q/h_s and w2_q [E, hidden, inter] e4m3,
// w2_s [E, hidden/128, inter/128].
extern "C" void moe_down_launcher(float* y, const void* h_q, const float* h_s, const void* w2_q,
                                  const float* w2_s, const int* expert_offsets, int tokens, int hidden,
                                  int inter, int n_experts, int top_k, int config,
                                  hipStream_t stream) {
    if (tokens <= 0) return;
    if (!check_common(hidden, inter, n_experts) || top_k <= 0) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!y || !h_q || !h_s || !w2_q || !w2_s || !expert_offsets ||
        ((reinterpret_cast<uintptr_t>(h_q) | reinterpret_cast<uintptr_t>(w2_q) |
          reinterpret_cast<uintptr_t>(y)) & 15u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const dim3 grid(hidden / GROUP, n_experts);
    const auto* hq = static_cast<const uint8_t*>(h_q);
    const auto* wq = static_cast<const uint8_t*>(w2_q);
    const bool last_first = (config & CONFIG_LAST_EXPERT_FIRST) != 0;
    // (the down GEMM has no requantisation: nothing depends on the scale convention)
    config &= ~(CONFIG_UE8M0 | CONFIG_LAST_EXPERT_FIRST | CONFIG_REQUANT_BITS);
    int nt = config & 7;
    if (nt != 1 && nt != 2 && nt != 4) {
        const long avg = (long)tokens * top_k / n_experts;
        nt = avg <= 16 ? 1 : avg <= 32 ? 2 : 4;
    }
    const bool lds_path = config < 8 && hidden % 256 == 0 && inter / GROUP <= 64;
    const dim3 grid256(hidden / 256, n_experts);
    switch (nt) {
        case 1:
            if (lds_path) {
                moe_stream_gemm_lds_kernel<false, 1><<<grid256, 256, 0, stream>>>(
                    wq, w2_s, hq, h_s, nullptr, expert_offsets, nullptr, nullptr, y, inter, hidden,
                    inter, top_k, false, last_first);
            } else {
                moe_stream_gemm_kernel<false, 1><<<grid, 256, 0, stream>>>(
                    wq, w2_s, hq, h_s, nullptr, expert_offsets, nullptr, nullptr, y, inter, hidden,
                    inter, top_k, false, last_first);
            }
            break;
        case 2:
            if (lds_path) {
                moe_stream_gemm_lds_kernel<false, 2><<<grid256, 256, 0, stream>>>(
                    wq, w2_s, hq, h_s, nullptr, expert_offsets, nullptr, nullptr, y, inter, hidden,
                    inter, top_k, false, last_first);
            } else {
                moe_stream_gemm_kernel<false, 2><<<grid, 256, 0, stream>>>(
                    wq, w2_s, hq, h_s, nullptr, expert_offsets, nullptr, nullptr, y, inter, hidden,
                    inter, top_k, false, last_first);
            }
            break;
        default:
            moe_stream_gemm_kernel<false, 4><<<grid, 256, 0, stream>>>(
                wq, w2_s, hq, h_s, nullptr, expert_offsets, nullptr, nullptr, y, inter, hidden, inter,
                top_k, false, last_first);
            break;
    }
}
