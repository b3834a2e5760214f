// Exact requantisation of h = silu(g) * u after the gate/up GEMM of the FP8 MoE layer.
//
// The e4m3 matrix core adds the products of a 128-block with about 16 significant bits, so the GEMM's g and u
// are off in the 5th digit. h is quantised right away (scale = group maximum / 448, codes by rounding), and a
// value that sits within that error of a rounding boundary gets the neighbouring code: one step, 6-12 % of the
// element. The gate/up epilogue therefore leaves one byte of marks per element (moe_common.hpp: MARK_NEAR, the
// scaled value may round either way; MARK_CANDIDATE, the element may be the group's maximum), and this pass
// recomputes exactly the marked pre-activations: fp32 products of the dequantised operands summed in fp64, i.e.
// the dot product itself to fp32 accuracy. One wavefront owns one (pair, 128-column group) of h:
//   1. candidates -> exact values -> exact group maximum -> the group's scale (h_s and its transposed copy);
//   2. marked elements -> exact value / exact scale -> code, stored over the GEMM's code.
// Unmarked elements keep the GEMM's code: the band that decides the marks covers the GEMM's error and the
// difference between the GEMM's scale and the exact one.
// The activation row of the pair is read once per wavefront; every recomputed element reads its gate row and
// its up row of the expert's weights (2 * K bytes) again.
#include "launch_status.hpp"
#include "moe_common.hpp"

namespace {

using namespace moe;

typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float silu(float x) { return x / (1.f + expf(-x)); }

// sum over 16 e4m3 pairs of a * b, in fp32 (the products are exact, the sum is rounded 15 times)
__device__ __forceinline__ float dot16(uintx4 a, uintx4 b) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const floatx2 a0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)a[j], false);
        const floatx2 a1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)a[j], true);
        const floatx2 b0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)b[j], false);
        const floatx2 b1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)b[j], true);
        s = fmaf(a0[0], b0[0], s);
        s = fmaf(a0[1], b0[1], s);
        s = fmaf(a1[0], b1[0], s);
        s = fmaf(a1[1], b1[1], s);
    }
    return s;
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) v += __shfl_xor(v, d);
    return v;
}

// MAXC: 16-byte chunks of a row per lane, K <= 1024 * MAXC
template <int MAXC>
__global__ __launch_bounds__(256) void moe_requant_fix_kernel(
    uint8_t* __restrict__ h_q, float* __restrict__ h_s, float* __restrict__ hs_t,
    const uint8_t* __restrict__ h_marks, const uint8_t* __restrict__ x_q, const float* __restrict__ x_s,
    const uint8_t* __restrict__ w13_q, const float* __restrict__ w13_s, const int* __restrict__ sorted_pairs,
    const int* __restrict__ expert_offsets, long n_units, int K, int inter, int n_experts, int top_k,
    int scale_stride, bool pow2) {
    const int lane = threadIdx.x & 63;
    const long unit = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= n_units) return;
    const int groups = inter / GROUP;
    const int pos = (int)(unit / groups);
    const int grp = (int)(unit - (long)pos * groups);

    // this lane's two marks: columns 2*lane and 2*lane + 1 of the group
    const uint32_t m2 = *reinterpret_cast<const uint16_t*>(h_marks + (size_t)pos * inter + grp * GROUP + 2 * lane);
    const unsigned long long cand[2] = {__builtin_amdgcn_ballot_w64((m2 & MARK_CANDIDATE) != 0),
                                        __builtin_amdgcn_ballot_w64((m2 & (MARK_CANDIDATE << 8)) != 0)};
    const unsigned long long near[2] = {__builtin_amdgcn_ballot_w64((m2 & MARK_NEAR) != 0),
                                        __builtin_amdgcn_ballot_w64((m2 & (MARK_NEAR << 8)) != 0)};
    if ((cand[0] | cand[1] | near[0] | near[1]) == 0) return;

    const int KB = K / GROUP;
    const int n_chunks = K / 16;
    const int token = sorted_pairs[pos] / top_k;
    int lo = 0, hi = n_experts;  // largest e with expert_offsets[e] <= pos
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (expert_offsets[mid] <= pos) lo = mid; else hi = mid;
    }
    const int e = lo;

    // the pair's activation row: chunk lane + 64*j, with the scale of its block of 128
    uintx4 xq[MAXC];
    float xs[MAXC];
#pragma unroll
    for (int j = 0; j < MAXC; ++j) {
        const int c = lane + 64 * j;
        xq[j] = uintx4{0u, 0u, 0u, 0u};
        xs[j] = 0.f;
        if (c < n_chunks) {
            xq[j] = *reinterpret_cast<const uintx4*>(x_q + (size_t)token * K + 16 * c);
            xs[j] = x_s[(size_t)token * KB + (c >> 3)];
        }
    }
    const size_t row_blocks = (size_t)2 * inter / GROUP;
    const float* ws_gate = w13_s + ((size_t)e * row_blocks + grp) * KB;
    const float* ws_up = w13_s + ((size_t)e * row_blocks + groups + grp) * KB;

    // h of column `col` of the group, exactly (every lane returns the same value)
    auto exact_h = [&](int col) {
        const uint8_t* gate_row = w13_q + ((size_t)e * 2 * inter + grp * GROUP + col) * K;
        const uint8_t* up_row = gate_row + (size_t)inter * K;
        uintx4 wg[MAXC], wu[MAXC];
        float sg[MAXC], su[MAXC];
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
            const int c = lane + 64 * j;
            wg[j] = wu[j] = uintx4{0u, 0u, 0u, 0u};
            sg[j] = su[j] = 0.f;
            if (c < n_chunks) {
                wg[j] = *reinterpret_cast<const uintx4*>(gate_row + 16 * c);
                wu[j] = *reinterpret_cast<const uintx4*>(up_row + 16 * c);
                sg[j] = ws_gate[c >> 3];
                su[j] = ws_up[c >> 3];
            }
        }
        double g = 0.0, u = 0.0;
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
            g += (double)(dot16(xq[j], wg[j]) * (xs[j] * sg[j]));
            u += (double)(dot16(xq[j], wu[j]) * (xs[j] * su[j]));
        }
        const float gf = (float)wave_sum(g);
        const float uf = (float)wave_sum(u);
        return silu(gf) * uf;
    };

    // 1. the group's scale from the exact maximum over the candidates
    float scale = h_s[(size_t)pos * groups + grp];
    if ((cand[0] | cand[1]) != 0) {
        float amax = 0.f;
#pragma unroll
        for (int odd = 0; odd < 2; ++odd) {
            for (unsigned long long m = cand[odd]; m != 0; m &= m - 1) {
                const int col = 2 * __builtin_ctzll(m) + odd;
                amax = fmaxf(amax, fabsf(exact_h(col)));
            }
        }
        scale = group_scale(amax, pow2);
        if (lane == 0) {
            h_s[(size_t)pos * groups + grp] = scale;
            if (hs_t != nullptr) hs_t[(size_t)grp * scale_stride + pos] = scale;
        }
    }
    // 2. the codes of the marked elements
#pragma unroll
    for (int odd = 0; odd < 2; ++odd) {
        for (unsigned long long m = near[odd]; m != 0; m &= m - 1) {
            const int col = 2 * __builtin_ctzll(m) + odd;
            const float v = fminf(fmaxf(exact_h(col) / scale, -E4M3_MAX), E4M3_MAX);
            const int code = __builtin_amdgcn_cvt_pk_fp8_f32(v, v, 0, false);
            if (lane == 0) h_q[(size_t)pos * inter + grp * GROUP + col] = (uint8_t)(code & 0xff);
        }
    }
}

}  // namespace

// Rewrites the marked codes of h_q [pairs, inter] and the scales h_s [pairs, inter/128] (and hs_t
// [inter/128][scale_stride], the transposed copy the tiled down GEMM reads; null if there is none) from exact
// pre-activations; h_marks [pairs, inter] as left by the gate/up stage. x_q, x_s, w13_q, w13_s, sorted_pairs,
// expert_offsets: the inputs of that stage. ue8m0: power-of-two scales. Internal to the library (called by
// the layer launchers between the gate/up and the down stage).
extern "C" void moe_requant_fix_launcher(void* h_q, float* h_s, float* hs_t, const void* h_marks,
                                         const void* x_q, const float* x_s, const void* w13_q,
                                         const float* w13_s, const int* sorted_pairs,
                                         const int* expert_offsets, int tokens, int hidden, int inter,
                                         int n_experts, int top_k, int scale_stride, int ue8m0,
                                         hipStream_t stream) {
    if (tokens <= 0) return;
    if (hidden <= 0 || inter <= 0 || hidden % GROUP != 0 || inter % GROUP != 0 || hidden > 16384 ||
        n_experts <= 0 || top_k <= 0) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!h_q || !h_s || !h_marks || !x_q || !x_s || !w13_q || !w13_s || !sorted_pairs || !expert_offsets ||
        ((reinterpret_cast<uintptr_t>(x_q) | reinterpret_cast<uintptr_t>(w13_q)) & 15u) ||
        (reinterpret_cast<uintptr_t>(h_marks) & 1u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const long n_units = (long)tokens * top_k * (inter / GROUP);
    const dim3 grid((unsigned)((n_units + 3) / 4));
#define MOE_FIX_LAUNCH(MAXC)                                                                              \
    moe_requant_fix_kernel<MAXC><<<grid, 256, 0, stream>>>(                                               \
        static_cast<uint8_t*>(h_q), h_s, hs_t, static_cast<const uint8_t*>(h_marks),                      \
        static_cast<const uint8_t*>(x_q), x_s, static_cast<const uint8_t*>(w13_q), w13_s, sorted_pairs,   \
        expert_offsets, n_units, hidden, inter, n_experts, top_k, scale_stride, ue8m0 != 0)
    if (hidden <= 1024) MOE_FIX_LAUNCH(1);
    else if (hidden <= 2048) MOE_FIX_LAUNCH(2);
    else if (hidden <= 4096) MOE_FIX_LAUNCH(4);
    else if (hidden <= 8192) MOE_FIX_LAUNCH(8);
    else MOE_FIX_LAUNCH(16);
#undef MOE_FIX_LAUNCH
}
