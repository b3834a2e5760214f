// Short causal depthwise convolution, single-token update: the step that produces q, k, v of a
// Gated DeltaNet layer from the layer's input projection while decoding.
//
// Per request b and channel c, with the channel's last L inputs kept in conv_state[b, c, 0..L-1]
// (oldest first) and the new input x[b, c]:
//
//   seq  = [conv_state[b, c, 0..L-1], x[b, c]]                    L + 1 values
//   conv_state[b, c, :] <- seq[1..L]                              (shift by one, in place)
//   y    = bias[c] + sum_{j<K} weight[c, j] * seq[L + 1 - K + j]  (the K newest values)
//   out[b, c] = y * sigmoid(y)  (activation 1)  or  y  (activation 0)
//
// L >= K - 1; a cache may keep L = K values (one more than the convolution needs), as the eager
// layer does. Channels [0, key_dim) of the result are q, [key_dim, 2*key_dim) k, the rest v; they
// are written to three separate dense arrays so that the decode step that follows reads them
// without a slicing copy.
//
// The update is a pure HBM stream (2*L + 2 values moved per channel for K multiply-adds). A lane
// owns the fewest consecutive channels of one request whose state fills whole 16-byte vectors (2
// channels for bf16 and L = 4, 8 for L = 3), so a load instruction of a wavefront covers consecutive
// bytes. Arithmetic is fp32 whatever the storage type; the state is moved, never recomputed, so it
// stays bit-exact.
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "launch_status.hpp"

namespace {

constexpr int CH_GRAIN = 8;  // key_dim and value_dim are multiples of this

// storage types: float, or the 16 bits of a bf16 value (plain integers, so that packs of them are
// moved with whole vector instructions)
typedef uint16_t bf16_bits;

__device__ __forceinline__ float conv_to_f32(float x) { return x; }
__device__ __forceinline__ float conv_to_f32(bf16_bits x) { return __uint_as_float((uint32_t)x << 16); }
__device__ __forceinline__ void conv_from_f32(float& d, float x) { d = x; }
__device__ __forceinline__ void conv_from_f32(bf16_bits& d, float x) {
    const __hip_bfloat16 r = __float2bfloat16(x);  // round to nearest even
    d = *reinterpret_cast<const bf16_bits*>(&r);
}

template <int BYTES>
struct VecOf {
    typedef uint32_t type __attribute__((ext_vector_type(BYTES / 4)));
};
template <>
struct VecOf<4> {
    typedef uint32_t type;
};

// N values of T moved as whole vectors of 16, 8 or 4 bytes (the widest that divides the pack)
template <typename T, int N>
union Pack {
    static constexpr int BYTES = sizeof(T) * N;
    static constexpr int VEC = BYTES % 16 == 0 ? 16 : BYTES % 8 == 0 ? 8 : 4;
    static_assert(BYTES % 4 == 0, "packs are whole dwords");
    typedef typename VecOf<VEC>::type vec_t;
    T v[N];
    vec_t raw[BYTES / VEC];

    __device__ __forceinline__ void load(const T* p) {  // streaming
#pragma unroll
        for (int i = 0; i < BYTES / VEC; ++i)
            raw[i] = __builtin_nontemporal_load(reinterpret_cast<const vec_t*>(p) + i);
    }
    __device__ __forceinline__ void load_cached(const T* p) {
#pragma unroll
        for (int i = 0; i < BYTES / VEC; ++i) raw[i] = reinterpret_cast<const vec_t*>(p)[i];
    }
    __device__ __forceinline__ void store(T* p) const {
#pragma unroll
        for (int i = 0; i < BYTES / VEC; ++i)
            __builtin_nontemporal_store(raw[i], reinterpret_cast<vec_t*>(p) + i);
    }
};

// channels per lane: the fewest whose L state values fill whole 16-byte vectors, so that one load
// instruction of a wavefront covers 1 KB of consecutive state
template <typename T, int L>
constexpr int channels_per_lane() {
    for (int c = 1; c < CH_GRAIN; c *= 2)
        if ((c * L * (int)sizeof(T)) % 16 == 0) return c;
    return CH_GRAIN;
}

constexpr int REQS = 4;  // requests per lane: their loads are issued together, weights read once

// grid: x = blocks of 256 lanes over channels / CH, y = groups of REQS requests
template <typename T, int L, int K>
__global__ __launch_bounds__(256) void causal_conv1d_update_kernel(
    T* __restrict__ q_out, T* __restrict__ k_out, T* __restrict__ v_out, T* __restrict__ conv_state,
    const T* __restrict__ x, const T* __restrict__ weight, const T* __restrict__ bias, int batch,
    int channels, int key_dim, int activation) {
    static_assert(L >= K - 1, "the state must hold the K-1 previous inputs");
    constexpr int CH = channels_per_lane<T, L>();
    const int c0 = (blockIdx.x * 256 + threadIdx.x) * CH;
    if (c0 >= channels) return;
    const int b0 = blockIdx.y * REQS;

    // the big stream first, the small vectors behind it
    Pack<T, CH * L> st[REQS];
    Pack<T, CH> xin[REQS];
    Pack<T, CH * K> w;
    Pack<T, CH> bs;
#pragma unroll
    for (int r = 0; r < REQS; ++r)
        if (b0 + r < batch) st[r].load(conv_state + ((size_t)(b0 + r) * channels + c0) * L);
#pragma unroll
    for (int r = 0; r < REQS; ++r)
        if (b0 + r < batch) xin[r].load(x + (size_t)(b0 + r) * channels + c0);
    w.load_cached(weight + (size_t)c0 * K);
    if (bias != nullptr) bs.load_cached(bias + c0);

    // channels [0, key_dim) are q, [key_dim, 2*key_dim) k, the rest v (a lane's channels fall into one)
    T* dst;
    size_t dst_row, dst_off;
    if (c0 < key_dim) {
        dst = q_out, dst_row = key_dim, dst_off = c0;
    } else if (c0 < 2 * key_dim) {
        dst = k_out, dst_row = key_dim, dst_off = c0 - key_dim;
    } else {
        dst = v_out, dst_row = channels - 2 * key_dim, dst_off = c0 - 2 * key_dim;
    }

#pragma unroll
    for (int r = 0; r < REQS; ++r) {
        if (b0 + r >= batch) break;
        Pack<T, CH * L> st_new;
        Pack<T, CH> res;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            float y = bias != nullptr ? conv_to_f32(bs.v[c]) : 0.f;
#pragma unroll
            for (int j = 0; j < K; ++j) {
                const int pos = L + 1 - K + j;  // position in seq
                const float s = pos < L ? conv_to_f32(st[r].v[c * L + pos]) : conv_to_f32(xin[r].v[c]);
                y = fmaf(conv_to_f32(w.v[c * K + j]), s, y);
            }
            if (activation == 1) y = y / (1.f + __expf(-y));
            conv_from_f32(res.v[c], y);
#pragma unroll
            for (int i = 0; i + 1 < L; ++i) st_new.v[c * L + i] = st[r].v[c * L + i + 1];
            st_new.v[c * L + L - 1] = xin[r].v[c];
        }
        st_new.store(conv_state + ((size_t)(b0 + r) * channels + c0) * L);
        res.store(dst + (size_t)(b0 + r) * dst_row + dst_off);
    }
}

template <typename T, int L, int K>
void launch_lk(void* q_out, void* k_out, void* v_out, void* conv_state, const void* x,
               const void* weight, const void* bias, int batch, int channels, int key_dim,
               int activation, hipStream_t stream) {
    constexpr int CH = channels_per_lane<T, L>();
    const dim3 grid((channels / CH + 255) / 256, (batch + REQS - 1) / REQS);
    causal_conv1d_update_kernel<T, L, K><<<grid, 256, 0, stream>>>(
        static_cast<T*>(q_out), static_cast<T*>(k_out), static_cast<T*>(v_out),
        static_cast<T*>(conv_state), static_cast<const T*>(x), static_cast<const T*>(weight),
        static_cast<const T*>(bias), batch, channels, key_dim, activation);
}

template <typename T>
bool launch_t(void* q_out, void* k_out, void* v_out, void* conv_state, const void* x,
              const void* weight, const void* bias, int batch, int channels, int key_dim,
              int state_len, int kernel_size, int activation, hipStream_t stream) {
#define CONV_CASE(LL, KK)                                                                       \
    if (state_len == LL && kernel_size == KK) {                                                 \
        launch_lk<T, LL, KK>(q_out, k_out, v_out, conv_state, x, weight, bias, batch, channels, \
                             key_dim, activation, stream);                                      \
        return true;                                                                            \
    }
    CONV_CASE(1, 2)
    CONV_CASE(2, 2)
    CONV_CASE(2, 3)
    CONV_CASE(3, 3)
    CONV_CASE(3, 4)
    CONV_CASE(4, 4)
#undef CONV_CASE
    return false;
}

}  // namespace

// q_out [batch, key_dim], k_out [batch, key_dim], v_out [batch, value_dim], written
// conv_state [batch, 2*key_dim + value_dim, state_len], updated in place
// x      [batch, 2*key_dim + value_dim] the new input of every channel
// weight [2*key_dim + value_dim, kernel_size], bias [2*key_dim + value_dim] or null
// All arrays of one storage type: dtype 0 = fp32, 1 = bf16. activation 0 = none, 1 = SiLU.
// key_dim and value_dim multiples of 8 (key_dim may be 0: then everything goes to v_out and
// q_out, k_out may be null). kernel_size 2..4, state_len = kernel_size - 1 or kernel_size.
// All pointers 16-byte aligned. config is accepted for the launcher pattern and has one value.
extern "C" void causal_conv1d_update_launcher(void* q_out, void* k_out, void* v_out,
                                              void* conv_state, const void* x, const void* weight,
                                              const void* bias, int batch, int key_dim,
                                              int value_dim, int state_len, int kernel_size,
                                              int activation, int dtype, int config,
                                              hipStream_t stream) {
    (void)config;
    if (batch <= 0 || (key_dim <= 0 && value_dim <= 0)) return;
    const long long channels = 2ll * key_dim + value_dim;
    if (key_dim < 0 || value_dim < 0 || key_dim % CH_GRAIN != 0 || value_dim % CH_GRAIN != 0 ||
        channels > 0x7fffffffll / 8 || batch > 65535 || (dtype != 0 && dtype != 1) ||
        (activation != 0 && activation != 1)) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    uintptr_t bits = reinterpret_cast<uintptr_t>(conv_state) | reinterpret_cast<uintptr_t>(x) |
                     reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(bias) |
                     reinterpret_cast<uintptr_t>(q_out) | reinterpret_cast<uintptr_t>(k_out) |
                     reinterpret_cast<uintptr_t>(v_out);
    if (!conv_state || !x || !weight || (key_dim > 0 && (!q_out || !k_out)) ||
        (value_dim > 0 && !v_out) || (bits & 15u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const bool ok =
        dtype == 0
            ? launch_t<float>(q_out, k_out, v_out, conv_state, x, weight, bias, batch, (int)channels,
                              key_dim, state_len, kernel_size, activation, stream)
            : launch_t<bf16_bits>(q_out, k_out, v_out, conv_state, x, weight, bias, batch,
                                       (int)channels, key_dim, state_len, kernel_size, activation,
                                       stream);
    if (!ok) caa::set_status(CAA_UNSUPPORTED_SHAPE);
}
