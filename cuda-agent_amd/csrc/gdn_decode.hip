// Gated DeltaNet single-token decode: one recurrent step per (request, value head).
//
//   S <- g*S;  u = S^T k;  delta = beta*(v - u);  S <- S + k delta^T;  o = S^T q * dk^-1/2
//
// with S the fp32 [dk, dv] state of the head (row-major, dv contiguous), q/k shared by
// `n_v_heads / n_qk_heads` consecutive value heads, g the decay itself (not its log).
//
// The step is a pure HBM stream: 2*dk*dv*4 bytes of state traffic per head against
// O(dk*dv) flops. The kernel reads every state element exactly once and writes it exactly
// once. Both reductions over dk are taken on the *old* state while it sits in registers:
//
//   a = S0^T k,  c = S0^T q,  kq = k.q
//   delta = beta*(v - g*a)
//   o     = dk^-1/2 * (g*c + kq*delta)
//   S1    = g*S0 + k delta^T
//
// which is the same update with the read-out folded in, so no second pass over S is needed.
//
// Work decomposition: a workgroup of 256 lanes (4 wavefronts) owns COLS consecutive value
// columns of one head, all DK rows. Lane t holds the float4 column group (t % (COLS/4)) of
// rows (t / (COLS/4)) + m*ROWS_PER_PASS. A wavefront load instruction therefore covers
// 64/(COLS/4) full row segments of COLS*4 contiguous bytes: with COLS = 128 that is two
// complete 512-byte state rows per instruction, 16 bytes per lane. Column sums are reduced
// across the lanes of a wavefront with lane permutes and across the 4 wavefronts through
// 4 KB of LDS. q, k are staged in LDS as fp32.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "launch_status.hpp"

namespace {

constexpr int DK = 128;
constexpr int DV = 128;

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(__hip_bfloat16 x) { return __bfloat162float(x); }
__device__ __forceinline__ void from_f32(float& d, float x) { d = x; }
__device__ __forceinline__ void from_f32(__hip_bfloat16& d, float x) { d = __float2bfloat16(x); }

typedef float floatx4 __attribute__((ext_vector_type(4)));

// NT marks the access as streaming (no reuse expected), one 16-byte instruction either way.
__device__ __forceinline__ float4 load_state(const float* p, bool nt) {
    if (nt) {
        const floatx4 r = __builtin_nontemporal_load(reinterpret_cast<const floatx4*>(p));
        return make_float4(r.x, r.y, r.z, r.w);
    }
    return *reinterpret_cast<const float4*>(p);
}

__device__ __forceinline__ void store_state(float* p, float4 x, bool nt) {
    if (nt) {
        floatx4 r = {x.x, x.y, x.z, x.w};
        __builtin_nontemporal_store(r, reinterpret_cast<floatx4*>(p));
    } else {
        *reinterpret_cast<float4*>(p) = x;
    }
}

// FUSED: q and k arrive unnormalised and are scaled by rsqrt(sum x^2 + 1e-6) here (the factors are
// applied to the reductions, not to the 128 values); `g` and `beta` are then the per-request
// gate inputs a and b, and g = exp(-exp(a_log[h]) * softplus(a + dt_bias[h])), beta = sigmoid(b).
//
// NORM (needs COLS == DV, one workgroup per head): the layer's gated RMS normalisation of the read-out
// is applied before it is stored: out = norm_w * o * rsqrt(mean(o^2) + eps) * silu(z), written in
// the storage type of q/k/v to o_norm; the fp32 o is not written.
template <typename T, int COLS, int THREADS, int NT, bool FUSED = false, bool NORM = false>
__global__ __launch_bounds__(THREADS) void gdn_decode_kernel(
    float* __restrict__ o, float* __restrict__ state, const T* __restrict__ q,
    const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ g,
    const float* __restrict__ beta, int n_v_heads, int n_qk_heads, float scale,
    const float* __restrict__ a_log = nullptr, const float* __restrict__ dt_bias = nullptr,
    const T* __restrict__ z = nullptr, const T* __restrict__ norm_w = nullptr, float norm_eps = 0.f,
    T* __restrict__ o_norm = nullptr) {
    static_assert(!NORM || COLS == DV, "the normalisation needs a head's whole read-out in one workgroup");
    constexpr int WAVES = THREADS / 64;
    constexpr int CG = COLS / 4;            // float4 column groups per row segment
    constexpr int RPP = THREADS / CG;       // rows covered by one pass of the workgroup
    constexpr int NP = DK / RPP;            // passes; float4 values held per lane
    constexpr int ROWS_PER_WAVE = 64 / CG;  // rows of one pass that fall into one wavefront
    constexpr int TILES = DV / COLS;        // workgroups per head

    __shared__ float s_q[DK];
    __shared__ float s_k[DK];
    __shared__ float s_kq[WAVES];
    __shared__ float s_qq[WAVES];  // FUSED: sums of squares
    __shared__ float s_kk[WAVES];
    __shared__ float s_gate[2];    // FUSED: g and beta of the unit, computed by one lane
    __shared__ float4 s_red[2][WAVES][CG];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int cg = tid % CG;
    const int r0 = tid / CG;

    const int unit = blockIdx.x / TILES;  // b * n_v_heads + hv
    const int tile = blockIdx.x % TILES;
    const int b = unit / n_v_heads;
    const int hv = unit % n_v_heads;
    const int hq = hv / (n_v_heads / n_qk_heads);

    float* S = state + (size_t)unit * (DK * DV) + tile * COLS + cg * 4;

    // The small vectors are requested first and the state tile right behind them: loads return in
    // order, so q, k and the gates can be reduced while the 64 KB of state are still on their way
    // (the other way round, the two wavefronts that hold q and k would wait for their state rows
    // before they could start the k.q reduction everybody else then waits for).
    const T* qh = q + ((size_t)b * n_qk_heads + hq) * DK;
    const T* kh = k + ((size_t)b * n_qk_heads + hq) * DK;
    // FUSED with at least 6 wavefronts: lanes DK..2DK-1 read q and lanes 2DK..3DK-1 read k a second
    // time and reduce the sums of squares, in parallel with the k.q reduction of lanes 0..DK-1
    constexpr bool SPLIT_NORMS = FUSED && THREADS >= 3 * DK;
    float qv = 0.f, kv = 0.f;
    if (tid < DK) {
        qv = to_f32(qh[tid]);
        kv = to_f32(kh[tid]);
    } else if (SPLIT_NORMS && tid < 2 * DK) {
        qv = to_f32(qh[tid - DK]);
    } else if (SPLIT_NORMS && tid < 3 * DK) {
        kv = to_f32(kh[tid - 2 * DK]);
    }
    float gate_a = 0.f, gate_b = 0.f, gate_alog = 0.f, gate_dt = 0.f;
    if (!FUSED || tid == THREADS - 1) {
        gate_a = g[unit];
        gate_b = beta[unit];
        if (FUSED) {
            gate_alog = a_log[hv];
            gate_dt = dt_bias[hv];
        }
    }

    float4 s[NP];
#pragma unroll
    for (int m = 0; m < NP; ++m) {
        s[m] = load_state(S + (size_t)(r0 + m * RPP) * DV, NT == 1 || NT == 2);
    }
    // NORM: the lanes that will hold the read-out (r0 == 0) fetch their gate and weight values now
    float4 zj = make_float4(0.f, 0.f, 0.f, 0.f), wj = zj;
    if (NORM && r0 == 0) {
        const T* zh = z + (size_t)unit * DV + cg * 4;
        const T* wh = norm_w + cg * 4;
        zj = make_float4(to_f32(zh[0]), to_f32(zh[1]), to_f32(zh[2]), to_f32(zh[3]));
        wj = make_float4(to_f32(wh[0]), to_f32(wh[1]), to_f32(wh[2]), to_f32(wh[3]));
    }

    float kq_part = 0.f;
    if (tid < DK) {
        s_q[tid] = qv;
        s_k[tid] = kv;
        kq_part = qv * kv;
    }
    if (tid < DK) {  // waves 0 and 1 (DK == 128): wavefront sum of k_i*q_i
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) kq_part += __shfl_xor(kq_part, off);
        if (lane == 0) s_kq[wave] = kq_part;
    }
    if (FUSED && (SPLIT_NORMS ? (tid >= DK && tid < 3 * DK) : tid < DK)) {
        float qq_part = qv * qv, kk_part = kv * kv;  // (one of them is 0 when the work is split)
        if (SPLIT_NORMS) {
            float part = qq_part + kk_part;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) part += __shfl_xor(part, off);
            if (lane == 0) (tid < 2 * DK ? s_qq : s_kk)[wave & 1] = part;
        } else {
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                qq_part += __shfl_xor(qq_part, off);
                kk_part += __shfl_xor(kk_part, off);
            }
            if (lane == 0) {
                s_qq[wave] = qq_part;
                s_kk[wave] = kk_part;
            }
        }
    }
    const float4 vj = [&] {
        const T* vh = v + (size_t)unit * DV + tile * COLS + cg * 4;
        return make_float4(to_f32(vh[0]), to_f32(vh[1]), to_f32(vh[2]), to_f32(vh[3]));
    }();
    float gh = gate_a, bh = gate_b;
    if (FUSED && tid == THREADS - 1) {  // one lane of a wavefront that has no q/k work
        // hardware exp/log (about 1 ulp of fp32 on the ranges met here); log(1 + e^x) instead of
        // log1p loses at most 1e-7 absolute, far below the fp32 noise of the 128-term sums
        const float x = gate_a + gate_dt;
        const float softplus = x > 20.f ? x : __logf(1.f + __expf(x));
        s_gate[0] = __expf(-__expf(gate_alog) * softplus);
        s_gate[1] = 1.f / (1.f + __expf(-gate_b));
    }
    __syncthreads();
    float inv_q = 1.f, inv_k = 1.f;
    if (FUSED) {
        gh = s_gate[0];
        bh = s_gate[1];
        inv_q = rsqrtf(s_qq[0] + s_qq[1] + 1e-6f);
        inv_k = rsqrtf(s_kk[0] + s_kk[1] + 1e-6f);
    }

    // a = S0^T k and c = S0^T q over this lane's rows
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 c = make_float4(0.f, 0.f, 0.f, 0.f);
    float kr[NP];
#pragma unroll
    for (int m = 0; m < NP; ++m) {
        const int r = r0 + m * RPP;
        kr[m] = s_k[r] * inv_k;
        const float qr = s_q[r] * inv_q;
        a.x += s[m].x * kr[m]; a.y += s[m].y * kr[m]; a.z += s[m].z * kr[m]; a.w += s[m].w * kr[m];
        c.x += s[m].x * qr;    c.y += s[m].y * qr;    c.z += s[m].z * qr;    c.w += s[m].w * qr;
    }
    // across the rows that share a wavefront (lane bits >= log2(CG))
#pragma unroll
    for (int off = 32; off >= CG; off >>= 1) {
        a.x += __shfl_xor(a.x, off); a.y += __shfl_xor(a.y, off);
        a.z += __shfl_xor(a.z, off); a.w += __shfl_xor(a.w, off);
        c.x += __shfl_xor(c.x, off); c.y += __shfl_xor(c.y, off);
        c.z += __shfl_xor(c.z, off); c.w += __shfl_xor(c.w, off);
    }
    if (lane < CG) {
        s_red[0][wave][lane] = a;
        s_red[1][wave][lane] = c;
    }
    __syncthreads();
    a = s_red[0][0][cg];
    c = s_red[1][0][cg];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
        const float4 aw = s_red[0][w][cg];
        const float4 cw = s_red[1][w][cg];
        a.x += aw.x; a.y += aw.y; a.z += aw.z; a.w += aw.w;
        c.x += cw.x; c.y += cw.y; c.z += cw.z; c.w += cw.w;
    }
    const float kq = (s_kq[0] + s_kq[1]) * (inv_q * inv_k);

    float4 d;
    d.x = bh * (vj.x - gh * a.x);
    d.y = bh * (vj.y - gh * a.y);
    d.z = bh * (vj.z - gh * a.z);
    d.w = bh * (vj.w - gh * a.w);

    float4 ov;
    ov.x = scale * (gh * c.x + kq * d.x);
    ov.y = scale * (gh * c.y + kq * d.y);
    ov.z = scale * (gh * c.z + kq * d.z);
    ov.w = scale * (gh * c.w + kq * d.w);
    if (!NORM && r0 == 0) {
        *reinterpret_cast<float4*>(o + (size_t)unit * DV + tile * COLS + cg * 4) = ov;
    }

#pragma unroll
    for (int m = 0; m < NP; ++m) {
        float4 n;
        n.x = gh * s[m].x + kr[m] * d.x;
        n.y = gh * s[m].y + kr[m] * d.y;
        n.z = gh * s[m].z + kr[m] * d.z;
        n.w = gh * s[m].w + kr[m] * d.w;
        store_state(S + (size_t)(r0 + m * RPP) * DV, n, NT == 1 || NT == 3);
    }

    if (NORM && r0 == 0) {
        // lanes 0..CG-1 (CG == 32: the lower half of wavefront 0) hold the head's 128 values
        float ss = ov.x * ov.x + ov.y * ov.y + ov.z * ov.z + ov.w * ov.w;
#pragma unroll
        for (int off = CG / 2; off >= 1; off >>= 1) ss += __shfl_xor(ss, off);
        const float rinv = rsqrtf(ss * (1.f / DV) + norm_eps);
        auto gated = [&](float x, float w, float zz) { return w * (x * rinv) * (zz / (1.f + __expf(-zz))); };
        T* dst = o_norm + (size_t)unit * DV + cg * 4;
        const float r[4] = {gated(ov.x, wj.x, zj.x), gated(ov.y, wj.y, zj.y), gated(ov.z, wj.z, zj.z),
                            gated(ov.w, wj.w, zj.w)};
#pragma unroll
        for (int i = 0; i < 4; ++i) from_f32(dst[i], r[i]);
    }
}

template <typename T, int COLS, int THREADS, int NT>
void launch_variant(float* o, float* state, const T* q, const T* k, const T* v, const float* g,
                    const float* beta, const float* a_log, const float* dt_bias, int units,
                    int n_v_heads, int n_qk_heads, hipStream_t stream) {
    const float scale = 0.08838834764831845f;  // 128^-1/2
    const dim3 grid(units * (DV / COLS));
    if (a_log) {
        gdn_decode_kernel<T, COLS, THREADS, NT, true><<<grid, THREADS, 0, stream>>>(
            o, state, q, k, v, g, beta, n_v_heads, n_qk_heads, scale, a_log, dt_bias);
    } else {
        gdn_decode_kernel<T, COLS, THREADS, NT, false><<<grid, THREADS, 0, stream>>>(
            o, state, q, k, v, g, beta, n_v_heads, n_qk_heads, scale);
    }
}

// a_log != nullptr selects the fused form (g and beta are then the gate inputs a and b)
template <typename T>
void launch(float* o, float* state, const void* q, const void* k, const void* v, const float* g,
            const float* beta, const float* a_log, const float* dt_bias, int batch, int n_v_heads,
            int n_qk_heads, int config, hipStream_t stream) {
    const int units = batch * n_v_heads;
    const T* qt = static_cast<const T*>(q);
    const T* kt = static_cast<const T*>(k);
    const T* vt = static_cast<const T*>(v);
    if (config <= 0 || config > 12) config = units >= 2048 ? 9 : 12;  // few heads: smaller tiles
#define GDN_VARIANT(id, cols, threads, nt)                                                         \
    case id:                                                                                       \
        launch_variant<T, cols, threads, nt>(o, state, qt, kt, vt, g, beta, a_log, dt_bias, units, \
                                             n_v_heads, n_qk_heads, stream);                       \
        break;
    switch (config) {
        GDN_VARIANT(1, 128, 256, 0)
        GDN_VARIANT(2, 64, 256, 0)
        GDN_VARIANT(3, 32, 256, 0)
        GDN_VARIANT(4, 128, 512, 0)
        GDN_VARIANT(5, 128, 256, 1)
        GDN_VARIANT(6, 128, 512, 1)
        GDN_VARIANT(7, 64, 512, 0)
        GDN_VARIANT(8, 128, 1024, 0)
        GDN_VARIANT(9, 128, 1024, 1)
        GDN_VARIANT(10, 128, 1024, 2)
        GDN_VARIANT(11, 128, 1024, 3)
        GDN_VARIANT(12, 32, 256, 1)
    }
#undef GDN_VARIANT
}

bool gdn_shape_ok(int batch, int n_v_heads, int n_qk_heads, int dk, int dv, int qkv_dtype) {
    return dk == DK && dv == DV && n_qk_heads > 0 && n_v_heads % n_qk_heads == 0 &&
           (qkv_dtype == 0 || qkv_dtype == 1) && (long)batch * n_v_heads * 4 <= 0x7fffffffL;
}

}  // namespace

// o      [batch, n_v_heads, 128] fp32, written
// state  [batch, n_v_heads, 128, 128] fp32, updated in place
// q, k   [batch, n_qk_heads, 128]; v [batch, n_v_heads, 128]; all three fp32 (qkv_dtype 0)
//        or bf16 (qkv_dtype 1)
// g, beta [batch, n_v_heads] fp32
// config: 0 picks the column tiling from the number of heads; 1, 2, 3 force workgroups of
//         128, 64, 32 value columns.
extern "C" void gdn_decode_launcher(float* o, float* state, const void* q, const void* k,
                                    const void* v, const float* g, const float* beta, int batch,
                                    int n_v_heads, int n_qk_heads, int dk, int dv, int qkv_dtype,
                                    int config, hipStream_t stream) {
    if (batch <= 0 || n_v_heads <= 0) return;
    if (!gdn_shape_ok(batch, n_v_heads, n_qk_heads, dk, dv, qkv_dtype)) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(o) | reinterpret_cast<uintptr_t>(state);
    if (!o || !state || !q || !k || !v || !g || !beta || (bits & 15u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    if (qkv_dtype == 0) {
        launch<float>(o, state, q, k, v, g, beta, nullptr, nullptr, batch, n_v_heads, n_qk_heads, config,
                      stream);
    } else {
        launch<__hip_bfloat16>(o, state, q, k, v, g, beta, nullptr, nullptr, batch, n_v_heads, n_qk_heads,
                               config, stream);
    }
}

// The same step with the caller's pre-step fused in: q and k [batch, n_qk_heads, 128] arrive
// unnormalised and are scaled by rsqrt(sum x^2 + 1e-6); a, b [batch, n_v_heads] fp32 are the gate
// inputs, a_log, dt_bias [n_v_heads] fp32 the per-head parameters:
//   g = exp(-exp(a_log[h]) * softplus(a + dt_bias[h])),  beta = sigmoid(b).
// Everything else as gdn_decode_launcher.
extern "C" void gdn_decode_fused_launcher(float* o, float* state, const void* q, const void* k,
                                          const void* v, const float* a, const float* b,
                                          const float* a_log, const float* dt_bias, int batch,
                                          int n_v_heads, int n_qk_heads, int dk, int dv,
                                          int qkv_dtype, int config, hipStream_t stream) {
    if (batch <= 0 || n_v_heads <= 0) return;
    if (!gdn_shape_ok(batch, n_v_heads, n_qk_heads, dk, dv, qkv_dtype)) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(o) | reinterpret_cast<uintptr_t>(state);
    if (!o || !state || !q || !k || !v || !a || !b || !a_log || !dt_bias || (bits & 15u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    if (qkv_dtype == 0) {
        launch<float>(o, state, q, k, v, a, b, a_log, dt_bias, batch, n_v_heads, n_qk_heads, config, stream);
    } else {
        launch<__hip_bfloat16>(o, state, q, k, v, a, b, a_log, dt_bias, batch, n_v_heads, n_qk_heads, config,
                               stream);
    }
}


// gdn_decode_fused_launcher followed by the layer's gated RMS normalisation of the read-out, in the
// same kernel: out [batch, n_v_heads, 128] in the storage type of q/k/v (qkv_dtype) =
//   norm_w * o * rsqrt(mean_j(o_j^2) + eps) * silu(z),   o the step's fp32 read-out (not stored),
// z [batch, n_v_heads, 128] the output gate and norm_w [128] the norm's weight, both of that type.
// config is accepted for the launcher pattern and has one value (one workgroup of 1024 lanes per head).
extern "C" void gdn_decode_fused_norm_launcher(void* out, float* state, const void* q, const void* k,
                                               const void* v, const float* a, const float* b,
                                               const float* a_log, const float* dt_bias,
                                               const void* z, const void* norm_w, float eps, int batch,
                                               int n_v_heads, int n_qk_heads, int dk, int dv,
                                               int qkv_dtype, int config, hipStream_t stream) {
    (void)config;
    if (batch <= 0 || n_v_heads <= 0) return;
    if (!gdn_shape_ok(batch, n_v_heads, n_qk_heads, dk, dv, qkv_dtype)) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(state);
    if (!out || !state || !q || !k || !v || !a || !b || !a_log || !dt_bias || !z || !norm_w ||
        (bits & 15u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const int units = batch * n_v_heads;
    const float scale = 0.08838834764831845f;  // 128^-1/2
    if (qkv_dtype == 0) {
        typedef float T;
        gdn_decode_kernel<T, 128, 1024, 1, true, true><<<units, 1024, 0, stream>>>(
            nullptr, state, static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v), a,
            b, n_v_heads, n_qk_heads, scale, a_log, dt_bias, static_cast<const T*>(z),
            static_cast<const T*>(norm_w), eps, static_cast<T*>(out));
    } else {
        typedef __hip_bfloat16 T;
        gdn_decode_kernel<T, 128, 1024, 1, true, true><<<units, 1024, 0, stream>>>(
            nullptr, state, static_cast<const T*>(q), static_cast<const T*>(k), static_cast<const T*>(v), a,
            b, n_v_heads, n_qk_heads, scale, a_log, dt_bias, static_cast<const T*>(z),
            static_cast<const T*>(norm_w), eps, static_cast<T*>(out));
    }
}
