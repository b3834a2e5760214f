// Shared declarations of the FP8 block-scaled MoE kernels (route/sort, quantise, grouped GEMMs,
// combine). Each stage has its own extern "C" launcher; moe_fp8_launcher chains them.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace moe {

constexpr int GROUP = 128;            // quantisation group along K, and weight block edge
constexpr float E4M3_MAX = 448.f;
constexpr float INV_E4M3_MAX = (float)(1.0 / 448.0);  // scales are amax times this, rounded once
constexpr float AMAX_FLOOR = 1e-12f;  // an all-zero group gets the scale 1e-12 * fp32(1/448)
constexpr int SORT_CHUNK_TOKENS = 256;

// config bit of the layer, quantiser and gate/up launchers: block scales are powers of two (the UE8M0
// convention: 8 exponent bits, no mantissa). The caller's weight scales must then be powers of two; the
// activation scales become the smallest power of two >= amax / 448.
constexpr int CONFIG_UE8M0 = 32;

// config bit of the routing launchers: every token gets one more slot after its top_k, expert number
// n_experts with weight 1 (a shared expert stored as one more expert behind the routed ones); ids and
// weights then have top_k + 1 entries per token and the sort covers n_experts + 1 experts.
constexpr int CONFIG_SHARED_SLOT = 64;

// config bit of the streaming GEMM launchers (and of the layer's internal calls): the last expert holds far
// more pairs than the others (the shared expert above): dispatch its workgroups first.
constexpr int CONFIG_LAST_EXPERT_FIRST = 128;

#ifdef __HIPCC__
// scale of a 128-wide activation group with maximum magnitude amax
__device__ __forceinline__ float group_scale(float amax, bool pow2) {
    amax = fmaxf(amax, AMAX_FLOOR);
    if (!pow2) return amax * INV_E4M3_MAX;
    // amax = (1 + m) * 2^k and 448 = 1.75 * 2^8: the smallest power of two that is >= amax / 448 is
    // 2^(k-8) if m <= 0.75, else 2^(k-7). Exact: integer work on the bit pattern.
    const uint32_t u = __float_as_uint(amax);
    const uint32_t exponent = (u >> 23) - 8u + ((u & 0x7fffffu) > 0x600000u ? 1u : 0u);
    return __uint_as_float(exponent << 23);
}
#endif

// Device scratch of one forward pass, carved from the caller's workspace.
struct Workspace {
    int* ids;             // [T*k]  expert of every (token, slot) pair, slots by descending logit
    float* weights;       // [T*k]  routing weight of the pair
    int* chunk_hist;      // [chunks*E] pairs of each expert in each 256-token chunk, then their
                          //           exclusive prefix over chunks
    int* expert_offsets;  // [E+1]  first sorted position of every expert
    int* sorted_pairs;    // [T*k]  flat pair index at each sorted position
    int* pair_pos;        // [T*k]  sorted position of each flat pair index
    uint8_t* x_q;         // [T*H]  e4m3 activations
    float* x_s;           // [T*H/128]
    uint8_t* h_q;         // [T*k*I] e4m3 silu(g)*u, rows in sorted order
    float* h_s;           // [T*k*I/128]
    float* y;             // [T*k*H] expert outputs, rows in sorted order
    int* tile_start;      // [E+1]  first 256-pair tile of every expert (tiled path)
    float* xs_t;          // [H/128][scale_stride] activation scales by sorted position, transposed
    float* hs_t;          // [I/128][scale_stride] the same for h
    int scale_stride;     // pairs rounded up to 256, plus 256 of padding
    size_t bytes;
};

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline Workspace carve_workspace(void* base, int tokens, int hidden, int inter, int n_experts,
                                 int top_k) {
    Workspace w{};
    size_t off = 0;
    char* p = static_cast<char*>(base);
    auto take = [&](size_t bytes) {
        char* r = p ? p + off : nullptr;
        off += align_up(bytes, 256);
        return r;
    };
    const size_t pairs = (size_t)tokens * top_k;
    const size_t chunks = (tokens + SORT_CHUNK_TOKENS - 1) / SORT_CHUNK_TOKENS;
    w.ids = reinterpret_cast<int*>(take(pairs * 4));
    w.weights = reinterpret_cast<float*>(take(pairs * 4));
    w.chunk_hist = reinterpret_cast<int*>(take(chunks * n_experts * 4));
    w.expert_offsets = reinterpret_cast<int*>(take(((size_t)n_experts + 1) * 4));
    w.sorted_pairs = reinterpret_cast<int*>(take(pairs * 4));
    w.pair_pos = reinterpret_cast<int*>(take(pairs * 4));
    w.x_q = reinterpret_cast<uint8_t*>(take((size_t)tokens * hidden));
    w.x_s = reinterpret_cast<float*>(take((size_t)tokens * (hidden / GROUP) * 4));
    w.h_q = reinterpret_cast<uint8_t*>(take(pairs * inter));
    w.h_s = reinterpret_cast<float*>(take(pairs * (inter / GROUP) * 4));
    w.y = reinterpret_cast<float*>(take(pairs * hidden * 4));
    w.scale_stride = (int)(align_up(pairs, 256) + 256);
    w.tile_start = reinterpret_cast<int*>(take(((size_t)n_experts + 1) * 4));
    w.xs_t = reinterpret_cast<float*>(take((size_t)(hidden / GROUP) * w.scale_stride * 4));
    w.hs_t = reinterpret_cast<float*>(take((size_t)(inter / GROUP) * w.scale_stride * 4));
    w.bytes = off;
    return w;
}

}  // namespace moe
