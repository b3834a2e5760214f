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

// config bits of the layer and of the gate/up stage that decide how h = silu(g) * u is requantised.
// The e4m3 matrix core adds the products of a 128-block with about 16 significant bits, so its g and u carry
// an error in the 5th digit and about one code of h in a thousand lands on the other side of a rounding
// boundary (one code step, 6-12 % of that element; the group's scale moves in the 5th digit as well). One such
// step on an element near its group's maximum moves single outputs of the layer by up to 3 % of their rms.
//  * The streaming gate/up GEMM (few pairs per expert, bound by the weight stream) converts the codes to bf16
//    in registers and uses the bf16 matrix core, whose sums are exact to fp32 accuracy: its h agrees with an
//    fp32 evaluation. CONFIG_APPROX_REQUANT puts it on the e4m3 matrix core.
//  * The tiled gate/up GEMM (many pairs per expert, bound by the matrix core):
//      default: e4m3 matrix core, and the epilogue repairs the codes that matter. It marks every element whose
//        scaled magnitude reaches 2^s code units (s = bits 12-15; 0: default_requant_significance, which is 7 at
//        the sizes this form is meant for: 128 of 448, i.e. the two highest binades, where one code step is 16 or
//        32 units) and lies within the error band of a rounding boundary,
//        and recomputes those pre-activations, and the candidates for the maximum of their group of 128, as
//        plain dot products; the group's scale then comes from the exact maximum and the marked codes from
//        the exact values. Smaller elements keep the matrix core's code (a step of at most 8 units there).
//      CONFIG_EXACT_REQUANT: bf16 matrix core (twice the matrix-core time): every code as an fp32
//        evaluation gives it, as in the streaming form.
//      CONFIG_APPROX_REQUANT: e4m3 matrix core, codes as they come.
//    Bits 10-11 scale the width of the band: 0 the default, 1 half, 2 twice, 3 four times as wide.
constexpr int CONFIG_EXACT_REQUANT = 256;
constexpr int CONFIG_APPROX_REQUANT = 512;
constexpr int CONFIG_BAND_SHIFT = 10;
constexpr int CONFIG_BAND_MASK = 3 << CONFIG_BAND_SHIFT;
constexpr int CONFIG_SIGNIF_SHIFT = 12;
constexpr int CONFIG_SIGNIF_MASK = 15 << CONFIG_SIGNIF_SHIFT;
constexpr int CONFIG_REQUANT_BITS = CONFIG_EXACT_REQUANT | CONFIG_APPROX_REQUANT | CONFIG_BAND_MASK | CONFIG_SIGNIF_MASK;

// marks of one element of h
constexpr uint32_t MARK_NEAR = 1;       // the scaled value may round to either of two codes
constexpr uint32_t MARK_CANDIDATE = 2;  // the element may be the largest magnitude of its group

// Significance level s the layer uses when the config names none: elements of at least 2^s code units are
// repaired. One code step of an element moves an output by an amount that shrinks, relative to the output's rms,
// with the square root of the number of terms an output sums (inter * top_k): 2^7 at inter * top_k = 16384
// (a step of at most 8 units below it, which measured moves no output by more than 2e-3 of the rms there),
// half of that for every factor of four fewer terms, never below 2^3.
inline int default_requant_significance(int inter, int top_k) {
    int s = 7;
    for (long terms = (long)inter * top_k; terms < 16384 && s > 3; terms *= 4) --s;
    return s;
}

// smallest scaled magnitude, in e4m3 code units, an element must reach for MARK_NEAR (config with the
// significance bits set)
inline float requant_min_magnitude(int config) {
    const int sig = (config & CONFIG_SIGNIF_MASK) >> CONFIG_SIGNIF_SHIFT;
    return (float)(1 << (sig ? sig : 7));
}

// Error of a gate/up pre-activation as the e4m3 matrix core computes it, as a multiple of the root mean square
// of the pair's 256 pre-activations of the row block. Measured on gfx950: the partial of one 128-block is off by
// 1.4e-6 of the block's sum of |products| on average (13 times that at most), without a preferred sign. For
// operands without a common sign the errors of the K/128 blocks add up like a random walk while the result
// grows with sqrt(K) as well, so one standard deviation of the error is about 1.3e-5 of the root mean square
// of the results whatever K is; the band takes 4.5 of them (times `width`). This is an error model, not a
// bound: operands of one sign throughout, for which the error grows with K, are outside it.
inline float requant_error_coefficient(int config) {
    static const float width[4] = {1.f, 0.5f, 2.f, 4.f};
    return width[(config & CONFIG_BAND_MASK) >> CONFIG_BAND_SHIFT] * 4.5f * 1.3e-5f;
}

#ifdef __HIPCC__
// Marks of one element of h for the exact requantisation, everything in units of the group's scale (code units):
// v = |h| / scale as computed, sg = silu(g) and u as computed, err_s the error bound of g and of u, dh_max_s a bound
// of the error of any element of the group (both divided by the scale), tau_s the relative amount by which the
// exact scale may differ (0 if it cannot), v_min the magnitude below which an element is not repaired.
__device__ __forceinline__ uint32_t requant_marks(float v, float sg, float u, float err_s, float dh_max_s, float tau_s,
                                                  bool scale_uncertain, float v_min) {
    // |d silu / d g| <= 1.1
    const float tau = fmaf(fmaf(1.1f, fabsf(u), fabsf(sg)), err_s, v * tau_s);
    const float lo = fmaxf(v - tau, 0.f);
    const float hi = fminf(v + tau, E4M3_MAX);
    const int codes = __builtin_amdgcn_cvt_pk_fp8_f32(lo, hi, 0, false);
    uint32_t m = ((codes ^ (codes >> 8)) & 0xff) != 0 && hi >= v_min ? MARK_NEAR : 0u;
    // (the group's maximum has v = 448 by construction)
    if (scale_uncertain && v + 2.f * dh_max_s >= E4M3_MAX) m |= MARK_CANDIDATE;
    return m;
}
#endif

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
    float* y;             // [T*k*H] expert outputs, rows in sorted order: fp32 from the streaming down GEMM; from
                          //         the tiled one fp16 of y / y_scale in the first half of the buffer
    float* y_scale;       // [T*k][H/256] power of two above the largest |y| of each run of 256 columns (tiled)
    int* tile_start;      // [2E+1] first 256-pair tile of every slot of the dispatch order, then the slots' experts
                          //        (tiled path)
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
    w.tile_start = reinterpret_cast<int*>(take((2 * (size_t)n_experts + 1) * 4));
    w.xs_t = reinterpret_cast<float*>(take((size_t)(hidden / GROUP) * w.scale_stride * 4));
    w.hs_t = reinterpret_cast<float*>(take((size_t)(inter / GROUP) * w.scale_stride * 4));
    w.y_scale = reinterpret_cast<float*>(take(pairs * ((hidden + 255) / 256) * 4));
    w.bytes = off;
    return w;
}

}  // namespace moe
