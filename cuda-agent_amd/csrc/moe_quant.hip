// Activation quantisation: bf16 rows -> e4m3 codes with one fp32 scale per 128-wide group.
//   scale = max(amax, 1e-12) * fp32(1/448);  code = e4m3_rne(clamp(v / scale, -448, 448))
//   (or, on request, scale = the smallest power of two >= max(amax, 1e-12) / 448)
// One wavefront per (row, group), two elements per lane. The division is IEEE fp32 so that the
// codes are bit-identical to a CPU evaluation of the same formula; v_cvt_pk_fp8_f32 rounds to
// nearest even but does not saturate (465 -> NaN), hence the clamp.
#include <hip/hip_bf16.h>

#include "launch_status.hpp"
#include "moe_common.hpp"

namespace {

using namespace moe;

__global__ __launch_bounds__(256) void moe_quant_bf16_kernel(const __hip_bfloat16* __restrict__ x,
                                                             uint8_t* __restrict__ q,
                                                             float* __restrict__ scales,
                                                             long n_groups, bool pow2) {
    const int lane = threadIdx.x & 63;
    const long g = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (g >= n_groups) return;
    const unsigned raw = *reinterpret_cast<const unsigned*>(x + g * GROUP + 2 * lane);
    const float v0 = __uint_as_float(raw << 16);
    const float v1 = __uint_as_float(raw & 0xffff0000u);
    float amax = fmaxf(fabsf(v0), fabsf(v1));
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const float scale = group_scale(amax, pow2);
    const float a = fminf(fmaxf(v0 / scale, -E4M3_MAX), E4M3_MAX);
    const float b = fminf(fmaxf(v1 / scale, -E4M3_MAX), E4M3_MAX);
    const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    *reinterpret_cast<uint16_t*>(q + g * GROUP + 2 * lane) = (uint16_t)(packed & 0xffff);
    if (lane == 0) scales[g] = scale;
}

// Same result with 16 lanes per group: a lane loads 8 values (16 bytes) and stores 8 codes.
__global__ __launch_bounds__(256) void moe_quant_bf16_vec_kernel(const __hip_bfloat16* __restrict__ x,
                                                                 uint8_t* __restrict__ q,
                                                                 float* __restrict__ scales,
                                                                 long n_groups, bool pow2) {
    typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
    typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
    const int sub = threadIdx.x & 15;
    const long g = (long)blockIdx.x * 16 + (threadIdx.x >> 4);
    if (g >= n_groups) return;
    const uintx4 raw = *reinterpret_cast<const uintx4*>(x + g * GROUP + 8 * sub);
    float v[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float(raw[j] << 16);
        v[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
    }
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const float scale = group_scale(amax, pow2);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = fminf(fmaxf(v[j] / scale, -E4M3_MAX), E4M3_MAX);
    uintx2 packed;
    int lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], lo, true);
    int hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], 0, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], hi, true);
    packed[0] = (unsigned)lo;
    packed[1] = (unsigned)hi;
    *reinterpret_cast<uintx2*>(q + g * GROUP + 8 * sub) = packed;
    if (sub == 0) scales[g] = scale;
}

}  // namespace

// q [rows, cols] e4m3 codes and scales [rows, cols/128] fp32 from x [rows, cols] bf16.
// config bit 32: power-of-two scales (the smallest power of two >= amax / 448).
extern "C" void moe_quant_bf16_launcher(void* q, float* scales, const void* x, int rows, int cols,
                                        int config, hipStream_t stream) {
    const bool pow2 = (config & CONFIG_UE8M0) != 0;
    if (rows <= 0 || cols <= 0) return;
    if (cols % GROUP != 0) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!q || !scales || !x || (reinterpret_cast<uintptr_t>(x) & 3u) ||
        (reinterpret_cast<uintptr_t>(q) & 1u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const long n_groups = (long)rows * (cols / GROUP);
    if (!(reinterpret_cast<uintptr_t>(x) & 15u) && !(reinterpret_cast<uintptr_t>(q) & 7u)) {
        moe_quant_bf16_vec_kernel<<<dim3((unsigned)((n_groups + 15) / 16)), 256, 0, stream>>>(
            static_cast<const __hip_bfloat16*>(x), static_cast<uint8_t*>(q), scales, n_groups, pow2);
        return;
    }
    const long blocks = (n_groups + 3) / 4;
    moe_quant_bf16_kernel<<<dim3((unsigned)blocks), 256, 0, stream>>>(
        static_cast<const __hip_bfloat16*>(x), static_cast<uint8_t*>(q), scales, n_groups, pow2);
}

namespace {

// RMS normalisation of a row followed by the activation quantisation of the result, one workgroup of 1024
// lanes per row (cols <= 8192): y = w * bf16(x * rsqrt(mean(x^2) + eps)) rounded to bf16 (the two roundings
// of a bf16 norm layer), then per 128-wide group of y the scale and the e4m3 codes of moe_quant_bf16. A lane
// owns 8 consecutive values (16 lanes per group); the row is read once and y, the codes and the scales are
// written once.
__global__ __launch_bounds__(1024) void moe_rmsnorm_quant_kernel(const __hip_bfloat16* __restrict__ x,
                                                                 const __hip_bfloat16* __restrict__ weight,
                                                                 __hip_bfloat16* __restrict__ y,
                                                                 uint8_t* __restrict__ q,
                                                                 float* __restrict__ scales, int cols,
                                                                 float eps, bool pow2) {
    typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
    typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
    __shared__ float s_part[16];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const size_t row = blockIdx.x;
    const int c0 = tid * 8;
    const bool live = c0 < cols;
    float v[8], w[8];
    float ss = 0.f;
    if (live) {
        const uintx4 raw = *reinterpret_cast<const uintx4*>(x + row * cols + c0);
        const uintx4 wraw = *reinterpret_cast<const uintx4*>(weight + c0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = __uint_as_float(raw[j] << 16);
            v[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
            w[2 * j] = __uint_as_float(wraw[j] << 16);
            w[2 * j + 1] = __uint_as_float(wraw[j] & 0xffff0000u);
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) ss = fmaf(v[j], v[j], ss);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off);
    if (lane == 0) s_part[wave] = ss;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) total += s_part[i];
    const float rinv = 1.f / sqrtf(total / (float)cols + eps);  // correctly rounded, as a CPU evaluation
    if (!live) return;
    float amax = 0.f;
    unsigned packed_y[4];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float n = __bfloat162float(__float2bfloat16(v[j] * rinv));  // the norm's result in bf16
        const __hip_bfloat16 yb = __float2bfloat16(w[j] * n);            // times the weight, in bf16
        v[j] = __bfloat162float(yb);
        amax = fmaxf(amax, fabsf(v[j]));
        const unsigned bits = (unsigned)(__float_as_uint(v[j]) >> 16);
        if (j & 1) packed_y[j >> 1] |= bits << 16; else packed_y[j >> 1] = bits;
    }
    if (y != nullptr) {
        *reinterpret_cast<uintx4*>(y + row * cols + c0) = uintx4{packed_y[0], packed_y[1], packed_y[2], packed_y[3]};
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    const float scale = group_scale(amax, pow2);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = fminf(fmaxf(v[j] / scale, -E4M3_MAX), E4M3_MAX);
    uintx2 packed;
    int lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[0], v[1], 0, false);
    lo = __builtin_amdgcn_cvt_pk_fp8_f32(v[2], v[3], lo, true);
    int hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[4], v[5], 0, false);
    hi = __builtin_amdgcn_cvt_pk_fp8_f32(v[6], v[7], hi, true);
    packed[0] = (unsigned)lo;
    packed[1] = (unsigned)hi;
    *reinterpret_cast<uintx2*>(q + row * cols + c0) = packed;
    if ((tid & 15) == 0) scales[row * (cols / GROUP) + (c0 / GROUP)] = scale;
}

}  // namespace

// The norm in front of the layer fused with the layer's activation quantiser:
//   y [rows, cols] bf16 (or null) = weight * bf16(x * rsqrt(mean(x^2) + eps)), rounded to bf16
//   q [rows, cols] e4m3 codes and scales [rows, cols/128] fp32: moe_quant_bf16_launcher applied to y
// x [rows, cols] bf16, weight [cols] bf16; cols a multiple of 128, at most 8192; x, weight, y 16-byte and
// q 8-byte aligned. config bit 32: power-of-two scales.
extern "C" void moe_rmsnorm_quant_launcher(void* q, float* scales, void* y, const void* x,
                                           const void* weight, float eps, int rows, int cols,
                                           int config, hipStream_t stream) {
    const bool pow2 = (config & CONFIG_UE8M0) != 0;
    if (rows <= 0 || cols <= 0) return;
    if (cols % GROUP != 0 || cols > 8192) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(weight) |
                           reinterpret_cast<uintptr_t>(y);
    if (!q || !scales || !x || !weight || (bits & 15u) || (reinterpret_cast<uintptr_t>(q) & 7u)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    moe_rmsnorm_quant_kernel<<<rows, 1024, 0, stream>>>(
        static_cast<const __hip_bfloat16*>(x), static_cast<const __hip_bfloat16*>(weight),
        static_cast<__hip_bfloat16*>(y), static_cast<uint8_t*>(q), scales, cols, eps, pow2);
}
