// Measured ceilings for the roofline figures: a stream of e4m3 (or bf16) MFMAs on random operands, alone or
// beside wavefronts that stream a buffer from HBM for as long as the MFMAs run. What the matrix cores sustain
// depends on the clock the chip holds under the load, so this is measured, not taken from the data sheet.
#include "launch_status.hpp"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ unsigned long long wall_ticks() { return wall_clock64(); }  // 100 MHz

// One workgroup of 512 lanes per CU. Wavefronts 0-3 (one per SIMD) issue `iters` rounds of four independent
// MFMAs on operands read once from `operands` (random bytes); wavefronts 4-7 stream `stream_src` in 16-byte
// loads, eight in flight per lane, until wavefront 0 says the MFMAs are done (they leave at once when
// stream_bytes == 0). Per workgroup: result[0] = ticks of the MFMA loop, result[1] = bytes streamed meanwhile.
template <bool BF16>
__global__ __launch_bounds__(512) void calibrate_mfma_kernel(const intx8* __restrict__ operands,
                                                             const intx4* __restrict__ stream_src,
                                                             size_t stream_chunks,
                                                             unsigned long long* __restrict__ result,
                                                             float* __restrict__ sink, int iters) {
    __shared__ volatile int s_done;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) s_done = 0;
    __syncthreads();
    if (wave < 4) {
        const intx8 a = operands[(blockIdx.x * 4 + wave) * 128 + lane];
        const intx8 b = operands[(blockIdx.x * 4 + wave) * 128 + 64 + lane];
        floatx16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
        const unsigned long long t0 = wall_ticks();
        for (int i = 0; i < iters; ++i) {
            if constexpr (BF16) {
                const bf16x8 ab = __builtin_bit_cast(bf16x8, intx4{a[0], a[1], a[2], a[3]});
                const bf16x8 bb = __builtin_bit_cast(bf16x8, intx4{b[0], b[1], b[2], b[3]});
                const bf16x8 ab2 = __builtin_bit_cast(bf16x8, intx4{a[4], a[5], a[6], a[7]});
                const bf16x8 bb2 = __builtin_bit_cast(bf16x8, intx4{b[4], b[5], b[6], b[7]});
                c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab, bb, c0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab2, bb, c1, 0, 0, 0);
                c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab, bb2, c2, 0, 0, 0);
                c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab2, bb2, c3, 0, 0, 0);
            } else {
                c0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c0, 0, 0, 0, 0, 0, 0);
                c1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, a, c1, 0, 0, 0, 0, 0, 0);
                c2 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, a, c2, 0, 0, 0, 0, 0, 0);
                c3 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b, b, c3, 0, 0, 0, 0, 0, 0);
            }
        }
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
        const unsigned long long t1 = wall_ticks();
        if (s == 1.2345f) sink[0] = s;  // (keeps the MFMAs alive)
        if (wave == 0 && lane == 0) {
            result[2 * blockIdx.x] = t1 - t0;
            s_done = 1;
        }
    } else {
        unsigned long long bytes = 0;
        intx4 acc = {0, 0, 0, 0};
        if (stream_chunks != 0) {
            // every streaming wavefront of the grid walks the buffer from its own starting point
            const size_t waves = (size_t)gridDim.x * 4;
            size_t pos = ((size_t)blockIdx.x * 4 + (wave - 4)) * (stream_chunks / waves);
            while (!s_done) {
                intx4 v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    size_t c = pos + (size_t)j * 64 + lane;
                    c = c < stream_chunks ? c : c - stream_chunks;
                    v[j] = __builtin_nontemporal_load(stream_src + c);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) acc ^= v[j];
                pos += 512;
                if (pos >= stream_chunks) pos -= stream_chunks;
                bytes += 8192;
            }
        }
        if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345) sink[1] = 1.f;
        if (lane == 0) atomicAdd(&result[2 * blockIdx.x + 1], bytes);
    }
}

}  // namespace

// Runs the calibration kernel once on `n_cus` workgroups of 512 lanes.
//   operands     n_cus * 4 * 128 * 32 bytes of random e4m3 codes (no NaN codes) or bf16 values
//   stream_src   buffer to stream beside the MFMAs, stream_bytes of it (a multiple of 16; 0: no streaming)
//   result       [n_cus][2] 64-bit words, cleared by the caller: ticks (100 MHz) of each workgroup's MFMA loop,
//                bytes its streaming wavefronts read meanwhile
//   iters        rounds of four MFMAs per wavefront; each round is 4 * 2 * 32 * 32 * 64 flop (e4m3,
//                v_mfma_f32_32x32x64_f8f6f4) or 4 * 2 * 32 * 32 * 16 (bf16, config 1)
// No counterpart in the reference workspace: a measuring aid of bench.py.
extern "C" void calibrate_mfma_launcher(const void* operands, const void* stream_src, size_t stream_bytes,
                                        void* result, float* sink, int n_cus, int iters, int config,
                                        hipStream_t stream) {
    if (n_cus <= 0 || iters <= 0) return;
    if (!operands || !result || !sink || (stream_bytes != 0 && !stream_src) || (stream_bytes & 15u) ||
        (stream_bytes != 0 && stream_bytes / 16 < (size_t)n_cus * 4 * 1024)) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const auto kernel = config == 1 ? calibrate_mfma_kernel<true> : calibrate_mfma_kernel<false>;
    kernel<<<n_cus, 512, 0, stream>>>(static_cast<const intx8*>(operands), static_cast<const intx4*>(stream_src),
                                      stream_bytes / 16, static_cast<unsigned long long*>(result), sink, iters);
}
