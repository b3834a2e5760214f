// Weighted combine of the expert outputs, and the launcher that runs the whole FP8 MoE layer:
//   route -> sort -> quantise x -> gate/up GEMM (+SiLU*mul, requantise) -> down GEMM -> combine.
#include <hip/hip_bf16.h>

#include "launch_status.hpp"
#include "moe_common.hpp"

extern "C" void moe_route_launcher(int* ids, float* weights, const float* logits, int tokens,
                                   int n_experts, int top_k, int config, hipStream_t stream);
extern "C" void moe_sort_launcher(int* sorted_pairs, int* pair_pos, int* expert_offsets,
                                  int* chunk_scratch, const int* ids, int tokens, int n_experts,
                                  int top_k, int config, hipStream_t stream);
extern "C" void moe_route_sort_launcher(int* ids, float* weights, int* sorted_pairs, int* pair_pos,
                                        int* expert_offsets, int* chunk_scratch, const float* logits,
                                        int tokens, int n_experts, int top_k, int config,
                                        hipStream_t stream);
extern "C" void moe_quant_bf16_launcher(void* q, float* scales, const void* x, int rows, int cols,
                                        int config, hipStream_t stream);
extern "C" void moe_gate_up_launcher(void* h_q, float* h_s, const void* x_q, const float* x_s,
                                     const void* w13_q, const float* w13_s, const int* sorted_pairs,
                                     const int* expert_offsets, int tokens, int hidden, int inter,
                                     int n_experts, int top_k, int config, hipStream_t stream);
extern "C" void moe_down_launcher(float* y, const void* h_q, const float* h_s, const void* w2_q,
                                  const float* w2_s, const int* expert_offsets, int tokens, int hidden,
                                  int inter, int n_experts, int top_k, int config, hipStream_t stream);

extern "C" void moe_tiled_prepare_launcher(int* tile_start, float* xs_t, const float* x_s,
                                           const int* sorted_pairs, const int* expert_offsets,
                                           int tokens, int hidden, int n_experts, int top_k,
                                           int scale_stride, hipStream_t stream);
extern "C" void moe_gate_up_tiled_launcher(void* h_q, float* h_s, float* hs_t, const void* x_q,
                                           const float* xs_t, const void* w13_q, const float* w13_s,
                                           const int* sorted_pairs, const int* expert_offsets,
                                           const int* tile_start, int tokens, int hidden, int inter,
                                           int n_experts, int top_k, int scale_stride, int ue8m0,
                                           int requant_config, hipStream_t stream);
extern "C" void moe_down_tiled_launcher(void* y, float* y_scale, const void* h_q, const float* hs_t,
                                        const void* w2_q, const float* w2_s, const int* expert_offsets,
                                        const int* tile_start, int tokens, int hidden, int inter,
                                        int n_experts, int top_k, int scale_stride, int ue8m0,
                                        hipStream_t stream);

namespace {

using namespace moe;

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

// the "sort" of a single expert that takes every token once: identity order, offsets {0, tokens}
__global__ __launch_bounds__(256) void moe_identity_sort_kernel(int* __restrict__ sorted_pairs,
                                                                int* __restrict__ pair_pos,
                                                                int* __restrict__ expert_offsets,
                                                                int tokens) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < tokens) {
        sorted_pairs[i] = i;
        pair_pos[i] = i;
    }
    if (i < 2) expert_offsets[i] = i * tokens;
}

typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));

// Four consecutive values of row `row` of an expert-output buffer at column c: fp32 rows, or (HALF) fp16 rows
// with one power-of-two scale per row and run of 256 columns, as the tiled down GEMM stores them.
template <bool HALF>
__device__ __forceinline__ floatx4 load_y4(const void* y, const float* y_scale, size_t row, int hidden, int c) {
    if constexpr (HALF) {
        const halfx4 v = __builtin_nontemporal_load(
            reinterpret_cast<const halfx4*>(static_cast<const _Float16*>(y) + row * hidden + c));
        const float s = y_scale[row * (size_t)(hidden / 256) + (c >> 8)];
        return floatx4{(float)v.x * s, (float)v.y * s, (float)v.z * s, (float)v.w * s};
    } else {
        return __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(static_cast<const float*>(y) + row * hidden + c));
    }
}

// out[t, :] = sum_k weights[t, k] * y[pair_pos[t*top_k + k], :] (k ascending) + y_shared[t, :], fp32.
// blockIdx.x is the token, blockIdx.y a 1024-column slice; 4 columns per lane.
// YH / SH: the routed / the shared expert outputs are in the fp16 form (see load_y4).
template <typename OUT, bool YH, bool SH>
__global__ __launch_bounds__(256) void moe_combine_kernel(const void* __restrict__ y,
                                                          const float* __restrict__ y_scale,
                                                          const float* __restrict__ weights,
                                                          const int* __restrict__ pair_pos,
                                                          const void* __restrict__ y_shared,
                                                          const float* __restrict__ ys_scale,
                                                          OUT* __restrict__ out, int hidden,
                                                          int top_k) {
    const int t = blockIdx.x;
    for (int c = (blockIdx.y * 256 + threadIdx.x) * 4; c < hidden; c += gridDim.y * 1024) {
        floatx4 acc = {0.f, 0.f, 0.f, 0.f};
        // four rows are fetched at a time (independent loads); the sum still runs in ascending k
        for (int k0 = 0; k0 < top_k; k0 += 4) {
            floatx4 v[4];
            float w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int k = k0 + j < top_k ? k0 + j : k0;
                const int pos = pair_pos[(size_t)t * top_k + k];
                w[j] = weights[(size_t)t * top_k + k];
                v[j] = load_y4<YH>(y, y_scale, (size_t)pos, hidden, c);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (k0 + j < top_k) acc += v[j] * w[j];
            }
        }
        // the shared expert's row, if there is one, is added last
        if (y_shared != nullptr) acc += load_y4<SH>(y_shared, ys_scale, (size_t)t, hidden, c);
        OUT* dst = out + (size_t)t * hidden + c;
        if constexpr (sizeof(OUT) == 4) {
            *reinterpret_cast<floatx4*>(dst) = acc;
        } else {
            bf16x4 r = {(__bf16)acc.x, (__bf16)acc.y, (__bf16)acc.z, (__bf16)acc.w};
            *reinterpret_cast<bf16x4*>(dst) = r;
        }
    }
}

// y_scale / ys_scale null: that buffer holds fp32 rows; else the fp16 form with these scales (hidden % 256 == 0)
void launch_combine(void* out, const void* y, const float* y_scale, const float* weights, const int* pair_pos,
                    const void* y_shared, const float* ys_scale, int tokens, int hidden, int top_k, int out_dtype,
                    hipStream_t stream) {
    const dim3 grid(tokens, (hidden + 1023) / 1024);
#define MOE_COMBINE(OUT_T, YH, SH)                                                                              \
    moe_combine_kernel<OUT_T, YH, SH><<<grid, 256, 0, stream>>>(y, y_scale, weights, pair_pos, y_shared, ys_scale, \
                                                               static_cast<OUT_T*>(out), hidden, top_k)
#define MOE_COMBINE_FORMS(OUT_T)                             \
    if (y_scale && ys_scale) MOE_COMBINE(OUT_T, true, true); \
    else if (y_scale) MOE_COMBINE(OUT_T, true, false);       \
    else if (ys_scale) MOE_COMBINE(OUT_T, false, true);      \
    else MOE_COMBINE(OUT_T, false, false)
    if (out_dtype == 0) {
        MOE_COMBINE_FORMS(__bf16);
    } else {
        MOE_COMBINE_FORMS(float);
    }
#undef MOE_COMBINE_FORMS
#undef MOE_COMBINE
}

}  // namespace

// out [tokens, hidden] (bf16 if out_dtype == 0, fp32 if 1) from y [tokens*top_k, hidden] fp32 in
// sorted order, weights [tokens, top_k], pair_pos [tokens*top_k]; y_shared [tokens, hidden] fp32
// (or null) is added to every token's sum last.
extern "C" void moe_combine_shared_launcher(void* out, const float* y, const float* weights,
                                            const int* pair_pos, const float* y_shared, int tokens,
                                            int hidden, int top_k, int out_dtype, int config,
                                            hipStream_t stream) {
    (void)config;
    if (tokens <= 0) return;
    if (hidden <= 0 || hidden % 4 != 0 || top_k <= 0 || (out_dtype != 0 && out_dtype != 1)) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!out || !y || !weights || !pair_pos || (reinterpret_cast<uintptr_t>(y) & 15u) ||
        (reinterpret_cast<uintptr_t>(out) & 15u) || (reinterpret_cast<uintptr_t>(y_shared) & 15u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    launch_combine(out, y, nullptr, weights, pair_pos, y_shared, nullptr, tokens, hidden, top_k, out_dtype, stream);
}

extern "C" void moe_combine_launcher(void* out, const float* y, const float* weights,
                                     const int* pair_pos, int tokens, int hidden, int top_k,
                                     int out_dtype, int config, hipStream_t stream) {
    moe_combine_shared_launcher(out, y, weights, pair_pos, nullptr, tokens, hidden, top_k, out_dtype,
                                config, stream);
}

extern "C" size_t moe_fp8_workspace_bytes(int tokens, int hidden, int inter, int n_experts,
                                          int top_k) {
    if (tokens <= 0 || hidden <= 0 || inter <= 0 || n_experts <= 0 || top_k <= 0) return 0;
    return moe::carve_workspace(nullptr, tokens, hidden, inter, n_experts, top_k).bytes;
}

// Byte offsets of the intermediate buffers inside the workspace, in the order
// ids, weights, expert_offsets, sorted_pairs, pair_pos, x_q, x_s, h_q, h_s, y, y_scale
// (for checkers that compare the stages against a reference). Writes min(n_offsets, 11) entries and returns
// the number of entries the layout has, so that a caller built against another version of this list notices.
extern "C" int moe_fp8_workspace_layout(size_t* offsets, int n_offsets, int tokens, int hidden, int inter,
                                        int n_experts, int top_k) {
    char* base = reinterpret_cast<char*>(uintptr_t{4096});
    const moe::Workspace w = moe::carve_workspace(base, tokens, hidden, inter, n_experts, top_k);
    const void* ptrs[11] = {w.ids, w.weights, w.expert_offsets, w.sorted_pairs, w.pair_pos, w.x_q,
                            w.x_s, w.h_q,     w.h_s,            w.y,            w.y_scale};
    for (int i = 0; i < 11 && i < n_offsets; ++i) offsets[i] = static_cast<const char*>(ptrs[i]) - base;
    return 11;
}

namespace {

// How the expert GEMMs of one group of experts run: LDS-tiled or weight-streaming form. Resolved, and checked
// against what the chosen kernels support, before the first launch of a layer, so that a shape one stage rejects
// launches nothing at all.
struct GemmPlan {
    bool ok;
    bool tiled;
};

GemmPlan plan_expert_gemms(int tokens, int hidden, int inter, int n_experts, int top_k, int config) {
    const int form = config & ~(CONFIG_UE8M0 | CONFIG_LAST_EXPERT_FIRST | CONFIG_REQUANT_BITS);
    // (the tiled kernels address activations with 32-bit byte offsets and scan the tiles of at most 1024 experts)
    const bool tiled_ok = hidden % 256 == 0 && n_experts <= 1024 &&
                          (unsigned long long)tokens * hidden < (1ull << 32) &&
                          (unsigned long long)tokens * top_k * inter < (1ull << 32);
    GemmPlan plan{};
    plan.tiled = form == 16 || (form == 0 && (long)tokens * top_k > 32L * n_experts && tiled_ok);
    plan.ok = !plan.tiled || tiled_ok;
    return plan;
}

// gate/up and down GEMMs of the experts over the quantised activations and the sort in `w`; result
// in w.y. Many pairs per expert: LDS-tiled GEMMs (256 x 256 tiles). Few: the weight-streaming form.
void run_expert_gemms(const moe::Workspace& w, const GemmPlan& plan, const void* w13_q, const float* w13_s,
                      const void* w2_q, const float* w2_s, int tokens, int hidden, int inter,
                      int n_experts, int top_k, int config, hipStream_t stream) {
    const int ue8m0 = config & CONFIG_UE8M0;  // power-of-two block scales, see moe_fp8_launcher
    const int order = config & CONFIG_LAST_EXPERT_FIRST;
    int requant = config & CONFIG_REQUANT_BITS;
    if (!(requant & CONFIG_SIGNIF_MASK)) requant |= default_requant_significance(inter, top_k) << CONFIG_SIGNIF_SHIFT;
    const int approx = config & CONFIG_APPROX_REQUANT;
    config &= ~(CONFIG_UE8M0 | CONFIG_LAST_EXPERT_FIRST | CONFIG_REQUANT_BITS);
    if (plan.tiled) {
        moe_tiled_prepare_launcher(w.tile_start, w.xs_t, w.x_s, w.sorted_pairs, w.expert_offsets, tokens,
                                   hidden, n_experts, top_k, w.scale_stride, stream);
        moe_gate_up_tiled_launcher(w.h_q, w.h_s, w.hs_t, w.x_q, w.xs_t, w13_q, w13_s, w.sorted_pairs,
                                   w.expert_offsets, w.tile_start, tokens, hidden, inter, n_experts, top_k,
                                   w.scale_stride, ue8m0, requant, stream);
        moe_down_tiled_launcher(w.y, w.y_scale, w.h_q, w.hs_t, w2_q, w2_s, w.expert_offsets, w.tile_start, tokens,
                                hidden, inter, n_experts, top_k, w.scale_stride, ue8m0, stream);
    } else {
        moe_gate_up_launcher(w.h_q, w.h_s, w.x_q, w.x_s, w13_q, w13_s, w.sorted_pairs, w.expert_offsets,
                             tokens, hidden, inter, n_experts, top_k, config | ue8m0 | order | approx, stream);
        moe_down_launcher(w.y, w.h_q, w.h_s, w2_q, w2_s, w.expert_offsets, tokens, hidden, inter,
                          n_experts, top_k, config | order, stream);
    }
}

bool layer_shape_ok(int hidden, int inter, int n_experts, int top_k, int tokens, int out_dtype) {
    return hidden > 0 && inter > 0 && hidden % GROUP == 0 && inter % GROUP == 0 && n_experts > 0 &&
           n_experts <= 512 && top_k > 0 && top_k <= 64 && top_k <= n_experts &&
           (long)tokens * top_k <= 0x7fffffffL / 4 && (out_dtype == 0 || out_dtype == 1);
}

}  // namespace

// 1 if moe_fp8_launcher runs these sizes and this config on the LDS-tiled GEMMs, 0 if on the weight-streaming
// ones (for checkers: the form decides how the workspace's y buffer is laid out), -1 for an unsupported shape.
extern "C" int moe_fp8_uses_tiled_gemms(int tokens, int hidden, int inter, int n_experts, int top_k, int config) {
    if (tokens <= 0 || !layer_shape_ok(hidden, inter, n_experts, top_k, tokens, 0)) return -1;
    const GemmPlan plan = plan_expert_gemms(tokens, hidden, inter, n_experts, top_k, config);
    return plan.ok ? (plan.tiled ? 1 : 0) : -1;
}

// The whole layer. out [tokens, hidden] bf16 (out_dtype 0) or fp32 (out_dtype 1).
// config: 0 = choose by the average number of pairs per expert (above 32: LDS-tiled GEMMs, else
// weight streaming); 16 forces the tiled GEMMs; 1, 2, 4 (+8) force streaming, see moe_gate_up_launcher.
// +256: with the tiled GEMMs, the exact requantisation pass (CONFIG_EXACT_REQUANT in moe_common.hpp; the
// streaming gate/up GEMM is exact by itself); +512: the streaming gate/up GEMM on the e4m3 matrix core.
// +32: all block scales are powers of two (UE8M0). The caller's weight scales must be; x and h are
// then quantised with the smallest power-of-two scale >= amax/448, and the tiled GEMMs let the MFMA
// apply the scales (no per-block multiply-add on the VALU).
extern "C" void moe_fp8_launcher(void* out, const void* x, const float* logits, const void* w13_q,
                                 const float* w13_s, const void* w2_q, const float* w2_s,
                                 void* workspace, size_t workspace_bytes, int tokens, int hidden,
                                 int inter, int n_experts, int top_k, int out_dtype, int config,
                                 hipStream_t stream) {
    if (tokens <= 0) return;
    const GemmPlan plan = plan_expert_gemms(tokens, hidden, inter, n_experts, top_k, config);
    if (!layer_shape_ok(hidden, inter, n_experts, top_k, tokens, out_dtype) || !plan.ok) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!out || !x || !logits || !w13_q || !w13_s || !w2_q || !w2_s || !workspace ||
        (reinterpret_cast<uintptr_t>(workspace) & 255u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const moe::Workspace w = moe::carve_workspace(workspace, tokens, hidden, inter, n_experts, top_k);
    if (workspace_bytes < w.bytes) {
        caa::set_status(CAA_WORKSPACE_TOO_SMALL);
        return;
    }
    moe_route_sort_launcher(w.ids, w.weights, w.sorted_pairs, w.pair_pos, w.expert_offsets, w.chunk_hist,
                            logits, tokens, n_experts, top_k, 0, stream);
    moe_quant_bf16_launcher(w.x_q, w.x_s, x, tokens, hidden, config & CONFIG_UE8M0, stream);
    run_expert_gemms(w, plan, w13_q, w13_s, w2_q, w2_s, tokens, hidden, inter, n_experts, top_k, config, stream);
    launch_combine(out, w.y, plan.tiled ? w.y_scale : nullptr, w.weights, w.pair_pos, nullptr, nullptr, tokens, hidden,
                   top_k, out_dtype, stream);
}

// Workspace of moe_fp8_shared_launcher: the routed experts' workspace followed by the same
// structure for one expert that takes every token once.
extern "C" size_t moe_fp8_shared_workspace_bytes(int tokens, int hidden, int inter, int shared_inter,
                                                 int n_experts, int top_k) {
    if (tokens <= 0 || hidden <= 0 || inter <= 0 || shared_inter <= 0 || n_experts <= 0 || top_k <= 0)
        return 0;
    return moe::carve_workspace(nullptr, tokens, hidden, inter, n_experts, top_k).bytes +
           moe::carve_workspace(nullptr, tokens, hidden, shared_inter, 1, 1).bytes;
}

// The layer with a shared expert: out = sum_k w[t,k] * expert_k(x[t]) + shared(x[t]), where the
// shared expert is one more block-scaled MLP (sw13_q [2*shared_inter, hidden], sw13_s
// [2*shared_inter/128, hidden/128], sw2_q [hidden, shared_inter], sw2_s [hidden/128,
// shared_inter/128]) applied to every token with weight 1. It runs through the same kernels as
// the routed experts (as a group of one expert holding all tokens, on the activations quantised
// once for both) and its fp32 row is added last in the combine.
extern "C" void moe_fp8_shared_launcher(void* out, const void* x, const float* logits,
                                        const void* w13_q, const float* w13_s, const void* w2_q,
                                        const float* w2_s, const void* sw13_q, const float* sw13_s,
                                        const void* sw2_q, const float* sw2_s, void* workspace,
                                        size_t workspace_bytes, int tokens, int hidden, int inter,
                                        int shared_inter, int n_experts, int top_k, int out_dtype,
                                        int config, hipStream_t stream) {
    if (tokens <= 0) return;
    const GemmPlan plan = plan_expert_gemms(tokens, hidden, inter, n_experts, top_k, config);
    const GemmPlan shared_plan = plan_expert_gemms(tokens, hidden, shared_inter > 0 ? shared_inter : 1, 1, 1, config);
    if (!layer_shape_ok(hidden, inter, n_experts, top_k, tokens, out_dtype) || shared_inter <= 0 ||
        shared_inter % GROUP != 0 || !plan.ok || !shared_plan.ok) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!out || !x || !logits || !w13_q || !w13_s || !w2_q || !w2_s || !sw13_q || !sw13_s || !sw2_q ||
        !sw2_s || !workspace || (reinterpret_cast<uintptr_t>(workspace) & 255u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const moe::Workspace w = moe::carve_workspace(workspace, tokens, hidden, inter, n_experts, top_k);
    moe::Workspace sh = moe::carve_workspace(static_cast<char*>(workspace) + w.bytes, tokens, hidden,
                                             shared_inter, 1, 1);
    if (workspace_bytes < w.bytes + sh.bytes) {
        caa::set_status(CAA_WORKSPACE_TOO_SMALL);
        return;
    }
    moe_route_sort_launcher(w.ids, w.weights, w.sorted_pairs, w.pair_pos, w.expert_offsets, w.chunk_hist,
                            logits, tokens, n_experts, top_k, 0, stream);
    moe_quant_bf16_launcher(w.x_q, w.x_s, x, tokens, hidden, config & CONFIG_UE8M0, stream);
    run_expert_gemms(w, plan, w13_q, w13_s, w2_q, w2_s, tokens, hidden, inter, n_experts, top_k, config, stream);
    sh.x_q = w.x_q;
    sh.x_s = w.x_s;
    moe_identity_sort_kernel<<<(tokens + 255) / 256, 256, 0, stream>>>(sh.sorted_pairs, sh.pair_pos,
                                                                      sh.expert_offsets, tokens);
    run_expert_gemms(sh, shared_plan, sw13_q, sw13_s, sw2_q, sw2_s, tokens, hidden, shared_inter, 1, 1, config,
                     stream);
    launch_combine(out, w.y, plan.tiled ? w.y_scale : nullptr, w.weights, w.pair_pos, sh.y,
                   shared_plan.tiled ? sh.y_scale : nullptr, tokens, hidden, top_k, out_dtype, stream);
}

// The layer with a shared expert stored as expert number n_experts behind the routed ones
// (w13_q [n_experts + 1, 2*inter, hidden] and so on; same inter): every token takes it as one more
// slot with weight 1 after its top_k, so it runs inside the routed experts' launches instead of as
// under-filled launches of its own. out = sum_k w[t,k] * expert_k(x[t]) + expert_{n_experts}(x[t]),
// the same sum as moe_fp8_shared_launcher. workspace: moe_fp8_workspace_bytes(tokens, hidden,
// inter, n_experts + 1, top_k + 1) bytes with the layout of that shape. logits [tokens, n_experts].
extern "C" void moe_fp8_fused_shared_launcher(void* out, const void* x, const float* logits,
                                              const void* w13_q, const float* w13_s,
                                              const void* w2_q, const float* w2_s, void* workspace,
                                              size_t workspace_bytes, int tokens, int hidden,
                                              int inter, int n_experts, int top_k, int out_dtype,
                                              int config, hipStream_t stream) {
    if (tokens <= 0) return;
    const GemmPlan plan = plan_expert_gemms(tokens, hidden, inter, n_experts + 1, top_k + 1, config);
    if (!layer_shape_ok(hidden, inter, n_experts, top_k, tokens, out_dtype) || n_experts >= 512 ||
        top_k >= 64 || (long)tokens * (top_k + 1) > 0x7fffffffL / 4 || !plan.ok) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!out || !x || !logits || !w13_q || !w13_s || !w2_q || !w2_s || !workspace ||
        (reinterpret_cast<uintptr_t>(workspace) & 255u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const moe::Workspace w =
        moe::carve_workspace(workspace, tokens, hidden, inter, n_experts + 1, top_k + 1);
    if (workspace_bytes < w.bytes) {
        caa::set_status(CAA_WORKSPACE_TOO_SMALL);
        return;
    }
    moe_route_sort_launcher(w.ids, w.weights, w.sorted_pairs, w.pair_pos, w.expert_offsets, w.chunk_hist,
                            logits, tokens, n_experts, top_k, CONFIG_SHARED_SLOT, stream);
    moe_quant_bf16_launcher(w.x_q, w.x_s, x, tokens, hidden, config & CONFIG_UE8M0, stream);
    run_expert_gemms(w, plan, w13_q, w13_s, w2_q, w2_s, tokens, hidden, inter, n_experts + 1, top_k + 1,
                     (config & ~CONFIG_LAST_EXPERT_FIRST) | CONFIG_LAST_EXPERT_FIRST, stream);
    launch_combine(out, w.y, plan.tiled ? w.y_scale : nullptr, w.weights, w.pair_pos, nullptr, nullptr, tokens, hidden,
                   top_k + 1, out_dtype, stream);
}

