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

// GATE_UP: 4 weight tiles per wavefront (2 gate + 2 up), output h_q/h_s.
// otherwise: 2 weight tiles per wavefront, output y.
template <bool GATE_UP, int NT>
__global__ __launch_bounds__(256) void moe_stream_gemm_kernel(
    const uint8_t* __restrict__ w_q, const float* __restrict__ w_s, const uint8_t* __restrict__ a_q,
    const float* __restrict__ a_s, const int* __restrict__ sorted_pairs,
    const int* __restrict__ expert_offsets, uint8_t* __restrict__ h_q, float* __restrict__ h_s,
    float* __restrict__ y, int K, int n_rows, int inter, int top_k) {
    constexpr int TILES = GATE_UP ? 4 : 2;
    __shared__ float s_amax[4][NT * 16];

    const int e = blockIdx.y;
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

        if (GATE_UP) {
            // h = silu(gate) * up, then e4m3 with one scale per pair over this block's 128 columns
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
                const float scale = fmaxf(amax, AMAX_FLOOR) * INV_E4M3_MAX;
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
                        *reinterpret_cast<int*>(h_q + (size_t)pos[nt] * inter + rb * GROUP + wave * 32 +
                                                i * 16 + 4 * g) = packed;
                    }
                    if (wave == 0 && g == 0) h_s[(size_t)pos[nt] * (inter / GROUP) + rb] = scale;
                }
            }
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

bool check_common(int hidden, int inter, int n_experts) {
    return hidden > 0 && inter > 0 && n_experts > 0 && hidden % GROUP == 0 && inter % GROUP == 0 &&
           n_experts <= 65535;
}

}  // namespace

// h_q [pairs, inter] e4m3 and h_s [pairs, inter/128] fp32 (rows in sorted order) from
// x_q [tokens, hidden] e4m3, x_s [tokens, hidden/128], w13_q [E, 2*inter, hidden] e4m3,
// w13_s [E, 2*inter/128, hidden/128].
// config: 0 sizes the pass from max_pairs_hint; 1, 2, 4 force 16, 32, 64 pairs per pass.
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
    int nt = config;
    if (nt != 1 && nt != 2 && nt != 4) {
        const long avg = (long)tokens * top_k / n_experts;  // pairs per expert if spread evenly
        nt = avg <= 16 ? 1 : avg <= 32 ? 2 : 4;
    }
    switch (nt) {
        case 1:
            moe_stream_gemm_kernel<true, 1><<<grid, 256, 0, stream>>>(
                wq, w13_s, xq, x_s, sorted_pairs, expert_offsets, hq, h_s, nullptr, hidden, 2 * inter,
                inter, top_k);
            break;
        case 2:
            moe_stream_gemm_kernel<true, 2><<<grid, 256, 0, stream>>>(
                wq, w13_s, xq, x_s, sorted_pairs, expert_offsets, hq, h_s, nullptr, hidden, 2 * inter,
                inter, top_k);
            break;
        default:
            moe_stream_gemm_kernel<true, 4><<<grid, 256, 0, stream>>>(
                wq, w13_s, xq, x_s, sorted_pairs, expert_offsets, hq, h_s, nullptr, hidden, 2 * inter,
                inter, top_k);
            break;
    }
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
    int nt = config;
    if (nt != 1 && nt != 2 && nt != 4) {
        const long avg = (long)tokens * top_k / n_experts;
        nt = avg <= 16 ? 1 : avg <= 32 ? 2 : 4;
    }
    switch (nt) {
        case 1:
            moe_stream_gemm_kernel<false, 1><<<grid, 256, 0, stream>>>(
                wq, w2_s, hq, h_s, nullptr, expert_offsets, nullptr, nullptr, y, inter, hidden, inter,
                top_k);
            break;
        case 2:
            moe_stream_gemm_kernel<false, 2><<<grid, 256, 0, stream>>>(
                wq, w2_s, hq, h_s, nullptr, expert_offsets, nullptr, nullptr, y, inter, hidden, inter,
                top_k);
            break;
        default:
            moe_stream_gemm_kernel<false, 4><<<grid, 256, 0, stream>>>(
                wq, w2_s, hq, h_s, nullptr, expert_offsets, nullptr, nullptr, y, inter, hidden, inter,
                top_k);
            break;
    }
}
