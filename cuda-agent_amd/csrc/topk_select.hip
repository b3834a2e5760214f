// Top-k selection of index scores: the step that produces the row indices sparse-MLA decode
// gathers. Per request, the k largest of n fp32 scores, ties going to the lower index, listed in
// ascending index order; everything is integer work on the scores' bit patterns, so the result
// is exact.
//
//   key(x)  = the 32-bit pattern of x mapped monotonically to an unsigned integer (-0 = +0;
//             NaN maps to 0, below every number, so a NaN is chosen only when nothing else is left)
//   T       = the k-th largest key, found by a radix select: four passes over the row, most
//             significant byte first, each a 256-bin histogram of the keys that share the prefix
//             found so far, and a scan from the top bin for the bin that holds the k-th key
//   chosen  = keys > T, plus the first (k - #greater) keys == T in index order
//
// One workgroup of 1024 lanes per request. Rows of up to 32768 scores are held in registers: lane
// t owns the consecutive entries [t*P, (t+1)*P) (P = 4, 8, 16 or 32), read once with all loads in
// flight; the histograms are LDS atomics into 8 interleaved copies of the 256 bins (scores share
// few exponents, so a single copy would serialise on two or three bins); the output needs one
// workgroup-wide exclusive scan of the lanes' counts, after which every lane writes its chosen
// entries in order. Longer rows are read five times from memory (four histograms, one output
// pass walking the row 1024 entries per round with a prefix count per round). Either way the
// output order does not depend on timing.
// Entries beyond a request's valid length (lengths[b], optional) are not candidates; if fewer
// than k candidates exist the remaining outputs are -1, which the attention treats as padding.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch_status.hpp"

namespace {

constexpr int SELECT_THREADS = 1024;
constexpr int SELECT_WAVES = SELECT_THREADS / 64;

__device__ __forceinline__ uint32_t score_key(float x) {
    if (x != x) return 0u;
    x += 0.f;  // -0 -> +0
    const uint32_t u = __float_as_uint(x);
    // monotone in the float order; the smallest number (-inf) maps to 0x007fffff, above NaN's 0
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// Inclusive prefix sum over the lanes of a wavefront: running sums inside each row of 16 lanes on DPP row
// shifts (vector ALU; the __shfl_up form is six dependent trips through the LDS crossbar), then the totals of
// the rows before a lane's own, read as scalars.
__device__ __forceinline__ int wave_inclusive_sum(int v, int lane) {
#define ROW_SHR_ADD(n) v += __builtin_amdgcn_update_dpp(0, v, 0x110 + (n), 0xf, 0xf, false);
    ROW_SHR_ADD(1)
    ROW_SHR_ADD(2)
    ROW_SHR_ADD(4)
    ROW_SHR_ADD(8)
#undef ROW_SHR_ADD
    const int r0 = __builtin_amdgcn_readlane(v, 15);
    const int r1 = __builtin_amdgcn_readlane(v, 31);
    const int r2 = __builtin_amdgcn_readlane(v, 47);
    const int row = lane >> 4;
    return v + (row >= 1 ? r0 : 0) + (row >= 2 ? r1 : 0) + (row >= 3 ? r2 : 0);
}

__global__ __launch_bounds__(SELECT_THREADS) void topk_select_kernel(
    const float* __restrict__ scores, const int* __restrict__ lengths, int* __restrict__ idx_out,
    int n, int k) {
    __shared__ int s_hist[256];
    __shared__ uint32_t s_prefix;   // key bits fixed so far
    __shared__ int s_remaining;     // how many more keys are wanted from the bins below the prefix
    __shared__ int s_wave_gt[2][SELECT_WAVES];
    __shared__ int s_wave_eq[2][SELECT_WAVES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int b = blockIdx.x;
    const float* row = scores + (size_t)b * n;
    int valid = lengths != nullptr ? lengths[b] : n;
    valid = valid < 0 ? 0 : (valid > n ? n : valid);
    const int want = k < valid ? k : valid;  // entries that will be chosen

    if (tid == 0) {
        s_prefix = 0u;
        s_remaining = want;
    }
    // radix select of the want-th largest key, most significant byte first
    for (int pass = 0; pass < 4 && want > 0; ++pass) {
        const int shift = 24 - 8 * pass;
        if (tid < 256) s_hist[tid] = 0;
        __syncthreads();
        const uint32_t prefix = s_prefix;
        const uint32_t prefix_mask = pass == 0 ? 0u : 0xffffffffu << (shift + 8);
        for (int base = 0; base < valid; base += SELECT_THREADS) {
            const int i = base + tid;
            uint32_t bin = 0u;
            bool active = false;
            if (i < valid) {
                const uint32_t key = score_key(row[i]);
                active = (key & prefix_mask) == prefix;
                bin = (key >> shift) & 255u;
            }
            if (active) atomicAdd(&s_hist[bin], 1);
        }
        __syncthreads();
        if (wave == 0) {
            // lane l owns bins 255-4l .. 252-4l (descending); suffix counts from the top bin
            int c[4];
            int mine = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                c[j] = s_hist[255 - 4 * lane - j];
                mine += c[j];
            }
            int above = mine;  // inclusive scan over lanes (lane 0 = top bins)
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int v = __shfl_up(above, d);
                if (lane >= d) above += v;
            }
            above -= mine;  // keys in bins above this lane's four
            const int remaining = s_remaining;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                // the bin where the running count reaches `remaining` holds the wanted key
                if (above < remaining && above + c[j] >= remaining) {
                    s_prefix = prefix | ((uint32_t)(255 - 4 * lane - j) << shift);
                    s_remaining = remaining - above;
                }
                above += c[j];
            }
        }
        __syncthreads();
    }
    const uint32_t threshold = s_prefix;  // the want-th largest key
    const int need_eq = s_remaining;      // how many keys equal to it are chosen (>= 1 if want > 0)

    // output pass in index order
    int run_gt = 0, run_eq = 0;
    const unsigned long long below = (1ull << lane) - 1ull;
    int round = 0;
    for (int base = 0; base < valid && want > 0; base += SELECT_THREADS, ++round) {
        const int i = base + tid;
        bool gt = false, eq = false;
        if (i < valid) {
            const uint32_t key = score_key(row[i]);
            gt = key > threshold;
            eq = key == threshold;
        }
        const unsigned long long m_gt = __ballot(gt);
        const unsigned long long m_eq = __ballot(eq);
        const int buf = round & 1;
        if (lane == 0) {
            s_wave_gt[buf][wave] = __popcll(m_gt);
            s_wave_eq[buf][wave] = __popcll(m_eq);
        }
        __syncthreads();  // (one barrier per round: the two buffers alternate)
        int gt_before = run_gt + __popcll(m_gt & below);
        int eq_before = run_eq + __popcll(m_eq & below);
        int tot_gt = 0, tot_eq = 0;
#pragma unroll
        for (int w = 0; w < SELECT_WAVES; ++w) {
            const int g = s_wave_gt[buf][w];
            const int e = s_wave_eq[buf][w];
            if (w < wave) {
                gt_before += g;
                eq_before += e;
            }
            tot_gt += g;
            tot_eq += e;
        }
        if (gt || (eq && eq_before < need_eq)) {
            const int pos = gt_before + (eq_before < need_eq ? eq_before : need_eq);
            idx_out[(size_t)b * k + pos] = i;
        }
        run_gt += tot_gt;
        run_eq += tot_eq;
    }
    for (int j = want + tid; j < k; j += SELECT_THREADS) idx_out[(size_t)b * k + j] = -1;
}

constexpr int HIST_COPIES = 8;

// P entries per lane, row in registers (n <= 1024 * P)
template <int P>
__global__ __launch_bounds__(SELECT_THREADS) void topk_select_regs_kernel(
    const float* __restrict__ scores, const int* __restrict__ lengths, int* __restrict__ idx_out,
    int n, int k) {
    __shared__ int s_hist[256 * HIST_COPIES];  // [bin][copy]: the copies of a bin sit in different banks
    __shared__ uint32_t s_prefix;
    __shared__ int s_remaining;
    __shared__ int s_wave_gt[SELECT_WAVES];
    __shared__ int s_wave_eq[SELECT_WAVES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int b = blockIdx.x;
    const float* row = scores + (size_t)b * n;
    int valid = lengths != nullptr ? lengths[b] : n;
    valid = valid < 0 ? 0 : (valid > n ? n : valid);
    const int want = k < valid ? k : valid;
    const int first = tid * P;

    // Keys of this lane's entries; entries that are no candidates are marked in `live`.
    uint32_t key[P];
    uint32_t live = 0u;
    if (first + P <= n && (reinterpret_cast<uintptr_t>(row + first) & 15u) == 0) {
        typedef float floatx4 __attribute__((ext_vector_type(4)));
        floatx4 v[P / 4];
#pragma unroll
        for (int j = 0; j < P / 4; ++j) v[j] = reinterpret_cast<const floatx4*>(row + first)[j];
#pragma unroll
        for (int j = 0; j < P; ++j) key[j] = score_key(v[j / 4][j % 4]);
    } else {
#pragma unroll
        for (int j = 0; j < P; ++j) key[j] = first + j < n ? score_key(row[first + j]) : 0u;
    }
#pragma unroll
    for (int j = 0; j < P; ++j) live |= (first + j < valid ? 1u : 0u) << j;
    // Entries that are no candidates get the smallest key: the passes below then need no test of `live`
    // (such an entry lands in the lowest bin of every digit, below the `want` largest live keys, or among
    // the ties of key 0, of which the emission takes live ones only).
#pragma unroll
    for (int j = 0; j < P; ++j) key[j] = ((live >> j) & 1u) ? key[j] : 0u;

    if (tid == 0) {
        s_prefix = 0u;
        s_remaining = want;
    }
    const int copy = lane & (HIST_COPIES - 1);
    for (int pass = 0; pass < 4 && want > 0; ++pass) {
        const int shift = 24 - 8 * pass;
        for (int i = tid; i < 256 * HIST_COPIES; i += SELECT_THREADS) s_hist[i] = 0;
        __syncthreads();
        const uint32_t prefix = s_prefix;
        const uint32_t prefix_mask = pass == 0 ? 0u : 0xffffffffu << (shift + 8);
        if (pass == 0) {
#pragma unroll
            for (int j = 0; j < P; ++j) atomicAdd(&s_hist[(key[j] >> 24) * HIST_COPIES + copy], 1);
        } else {
#pragma unroll
            for (int j = 0; j < P; ++j) {
                if ((key[j] & prefix_mask) == prefix)
                    atomicAdd(&s_hist[((key[j] >> shift) & 255u) * HIST_COPIES + copy], 1);
            }
        }
        __syncthreads();
        if (wave == 0) {
            int c[4];
            int mine = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int bin = 255 - 4 * lane - j;
                c[j] = 0;
#pragma unroll
                for (int h = 0; h < HIST_COPIES; ++h) c[j] += s_hist[bin * HIST_COPIES + h];
                mine += c[j];
            }
            int above = wave_inclusive_sum(mine, lane) - mine;
            const int remaining = s_remaining;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (above < remaining && above + c[j] >= remaining) {
                    s_prefix = prefix | ((uint32_t)(255 - 4 * lane - j) << shift);
                    s_remaining = remaining - above;
                }
                above += c[j];
            }
        }
        __syncthreads();
    }
    const uint32_t threshold = s_prefix;
    const int need_eq = s_remaining;

    if (want > 0) {
        int n_gt = 0, n_eq = 0;
#pragma unroll
        for (int j = 0; j < P; ++j) {
            const bool on = (live >> j) & 1u;
            n_gt += (on && key[j] > threshold) ? 1 : 0;
            n_eq += (on && key[j] == threshold) ? 1 : 0;
        }
        // exclusive scan of (n_gt, n_eq) over the 1024 lanes, in lane order = index order
        // (both counts fit 16 bits: one scan of the packed pair)
        const int packed_before = wave_inclusive_sum(n_gt | (n_eq << 16), lane);
        int gt_before = packed_before & 0xffff, eq_before = packed_before >> 16;
        if (lane == 63) {
            s_wave_gt[wave] = gt_before;
            s_wave_eq[wave] = eq_before;
        }
        gt_before -= n_gt;
        eq_before -= n_eq;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < SELECT_WAVES; ++w) {
            if (w < wave) {
                gt_before += s_wave_gt[w];
                eq_before += s_wave_eq[w];
            }
        }
        int* dst = idx_out + (size_t)b * k;
#pragma unroll
        for (int j = 0; j < P; ++j) {
            const bool on = (live >> j) & 1u;
            const bool gt = on && key[j] > threshold;
            const bool eq = on && key[j] == threshold;
            if (gt || (eq && eq_before < need_eq))
                dst[gt_before + (eq_before < need_eq ? eq_before : need_eq)] = first + j;
            gt_before += gt ? 1 : 0;
            eq_before += eq ? 1 : 0;
        }
    }
    for (int j = want + tid; j < k; j += SELECT_THREADS) idx_out[(size_t)b * k + j] = -1;
}

}  // namespace

// idx_out [batch, k] int32: per request the indices of the k largest scores among the first
// lengths[b] (or n, if lengths is null) entries of scores [batch, n] fp32; ties go to the lower
// index; listed in ascending index order; -1 where fewer than k candidates exist.
// config is accepted for the launcher pattern and has one value.
extern "C" void topk_select_launcher(int* idx_out, const float* scores, const int* lengths,
                                     int batch, int n, int k, int config, hipStream_t stream) {
    (void)config;
    if (batch <= 0 || k <= 0) return;
    if (n <= 0) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!idx_out || !scores) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    if (n <= 4 * SELECT_THREADS) {
        topk_select_regs_kernel<4><<<batch, SELECT_THREADS, 0, stream>>>(scores, lengths, idx_out, n, k);
    } else if (n <= 8 * SELECT_THREADS) {
        topk_select_regs_kernel<8><<<batch, SELECT_THREADS, 0, stream>>>(scores, lengths, idx_out, n, k);
    } else if (n <= 16 * SELECT_THREADS) {
        topk_select_regs_kernel<16><<<batch, SELECT_THREADS, 0, stream>>>(scores, lengths, idx_out, n, k);
    } else if (n <= 32 * SELECT_THREADS) {
        topk_select_regs_kernel<32><<<batch, SELECT_THREADS, 0, stream>>>(scores, lengths, idx_out, n, k);
    } else {
        topk_select_kernel<<<batch, SELECT_THREADS, 0, stream>>>(scores, lengths, idx_out, n, k);
    }
}
