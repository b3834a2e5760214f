// Grouped FP8 GEMMs of the MoE layer, LDS-tiled form (many pairs per expert: prefill).
//
// A workgroup of 8 wavefronts computes a 256 (weight rows) x 256 (pairs) tile of one expert:
// per 128-block of K it brings 32 KB of weights, 32 KB of activations and the 256 activation
// scales of the block into LDS with global->LDS loads in which 8 lanes fetch one full 128-byte
// line of a row (two stages; weights are requested two blocks ahead and activations one, see
// the comment at `block` in the kernel), and each wavefront multiplies a 64-row x 128-pair slice on v_mfma_f32_32x32x64_f8f6f4:
//
//   weights are the A operand (rows -> M), activations the B operand (pairs -> N), so that in the
//   result layout a lane holds 16 weight rows of ONE pair and the block's scale product
//   x_s[pair, kb] * w_s[row block, kb] is a per-lane scalar;
//   the unscaled partial of one 128-block (two MFMAs of K = 64) is folded into the fp32
//   accumulator with one multiply-add per value (the block scales are arbitrary fp32 and vary
//   along K, so they can be applied neither once at the end nor by the hardware's
//   power-of-two block scaling; when the caller declares them powers of two, the UE8M0 form
//   of the kernel hands them to the MFMA instead);
//   the two A tiles of a wavefront stay in registers for the whole block while the four B
//   tiles stream through: 24 KB of LDS reads per wavefront and block, 16 MFMAs.
//
// LDS slot of 16-byte chunk c of row r: r*8 + (c ^ ((r >> 1) & 7)) (a ds_read_b128 serves 16
// consecutive lanes per cycle from 64 banks, i.e. two 128-byte rows per bank row, so the 8 rows of
// equal parity among 16 consecutive rows must use 8 different chunks), conflict-free for the fill and
// for both operand reads. For gate/up the 256 rows are 128 gate rows and the matching 128 up
// rows, each wavefront holding 32 of either, so SiLU(gate)*up and the e4m3 requantisation of
// the 128-column group happen in the epilogue without leaving the workgroup.
#include "launch_status.hpp"
#include "moe_common.hpp"

namespace {

using namespace moe;

typedef int intx8 __attribute__((ext_vector_type(8)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;
typedef const __attribute__((address_space(3))) uint8_t* lds_bytes;
typedef const __attribute__((address_space(3))) intx4* lds_x4;

constexpr int TILE_PAIRS = 256;
constexpr int TILE_ROWS = 256;
constexpr int STAGE_A = TILE_ROWS * GROUP;    // 32 KB
constexpr int STAGE_B = TILE_PAIRS * GROUP;   // 32 KB
constexpr int STAGE_S = TILE_PAIRS * 4;       // 1 KB of scales
constexpr int STAGE_BYTES = STAGE_A + STAGE_B + STAGE_S;
constexpr int SUPER_ROWS = 4;   // row tiles and pair tiles of the block of workgroups that
constexpr int SUPER_PAIRS = 8;  // share one XCD's L2

inline int tiled_grid(int row_tiles, int max_pair_tiles) {
    const int supers = ((row_tiles + SUPER_ROWS - 1) / SUPER_ROWS) * ((max_pair_tiles + SUPER_PAIRS - 1) / SUPER_PAIRS);
    return ((supers + 7) / 8) * 8 * SUPER_ROWS * SUPER_PAIRS;
}

template <int N>
struct IntConstant {
    static constexpr int value = N;
};

__device__ __forceinline__ intx8 join(intx4 lo, intx4 hi) {
    return intx8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// x / (1 + exp(-x)) on the hardware's exp2 and reciprocal (a few units in the last place of the exact value:
// far inside what the e4m3 matrix core leaves of the pre-activation; the library routines for exp and the IEEE
// division were a tenth of a full tile's time in the gate/up epilogue)
__device__ __forceinline__ float silu(float x) {
    return x * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}

// 8 e4m3 codes (two dwords) -> 8 bf16, exactly (every e4m3 value is a bf16 value)
__device__ __forceinline__ bf16x8 e4m3x8_to_bf16(int lo, int hi) {
    const bf16x2 a = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false);
    const bf16x2 b = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true);
    const bf16x2 c = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false);
    const bf16x2 d = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true);
    return bf16x8{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

// sum over 16 e4m3 pairs of a * b, in fp32 (the products are exact, the sum is rounded 15 times)
__device__ __forceinline__ float dot16(intx4 a, intx4 b) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const floatx2 a0 = __builtin_amdgcn_cvt_pk_f32_fp8(a[j], false);
        const floatx2 a1 = __builtin_amdgcn_cvt_pk_f32_fp8(a[j], true);
        const floatx2 b0 = __builtin_amdgcn_cvt_pk_f32_fp8(b[j], false);
        const floatx2 b1 = __builtin_amdgcn_cvt_pk_f32_fp8(b[j], true);
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

__device__ __forceinline__ void wait_all_loads() {
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));  // vmcnt(0)
    asm volatile("" ::: "memory");
}

// 64 lanes x 16 bytes, global -> LDS (lds_base + lane*16); asm so that the compiler does not
// make every later LDS read wait for it: completion is awaited once per block, before the barrier.
__device__ __forceinline__ void dma16(const void* base, uint32_t lane_byte_offset, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(lane_byte_offset), "s"(base), "s"(lds_base)
                 : "memory", "m0");
}
__device__ __forceinline__ void dma16_ptr(const void* lane_ptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(lane_ptr), "s"(lds_base)
                 : "memory", "m0");
}

// The order in which the experts' pair tiles are numbered, and with it dispatched. Experts with two or more
// 256-pair tiles (the heavily loaded ones, whose tiles are bound by the matrix cores) are spread evenly among the
// others (one tile each, bound by the stream of their weights) instead of standing wherever their numbers put them:
// slot s of the order holds expert slot_expert[s], and tile_start[s] = number of tiles of the slots before s
// (tile_start[E] = total). Measured on the prefill workload: 2.4 % of the layer's time between the heavily loaded
// experts evenly spread and all in a row.
// tile_table: tile_start [n_experts + 1], then slot_expert [n_experts].
__global__ __launch_bounds__(1024) void moe_tile_start_kernel(const int* __restrict__ expert_offsets,
                                                              int* __restrict__ tile_table, int n_experts) {
    __shared__ int s_scan[1024];
    __shared__ int s_list[2][1024];  // experts with several tiles, and the others, each in ascending order
    __shared__ int s_slot_expert[1024];
    const int t = threadIdx.x;
    // inclusive prefix sum of v over the first n_experts lanes
    auto scan = [&](int v) {
        if (t < n_experts) s_scan[t] = v;
        __syncthreads();
        for (int d = 1; d < n_experts; d <<= 1) {
            const int add = (t >= d && t < n_experts) ? s_scan[t - d] : 0;
            __syncthreads();
            v += add;
            if (t < n_experts) s_scan[t] = v;
            __syncthreads();
        }
        return v;
    };
    const int mine = t < n_experts ? (expert_offsets[t + 1] - expert_offsets[t] + TILE_PAIRS - 1) / TILE_PAIRS : 0;
    const bool loaded = mine >= 2;
    const int loaded_upto = scan(loaded ? 1 : 0);  // experts with several tiles among 0..t
    const int n_loaded = s_scan[n_experts - 1];
    if (t < n_experts) s_list[loaded ? 0 : 1][loaded ? loaded_upto - 1 : t - loaded_upto] = t;
    __syncthreads();
    // slot s is taken by loaded expert j if s == j * n_experts / n_loaded
    int j = -1;
    if (t < n_experts && n_loaded > 0) {
        const int cand = (int)(((long)t * n_loaded + n_experts - 1) / n_experts);  // smallest j with j*E/n >= t
        if (cand < n_loaded && (int)((long)cand * n_experts / n_loaded) == t) j = cand;
    }
    const int free_upto = scan(j < 0 ? 1 : 0);  // slots not taken among 0..t
    if (t < n_experts) s_slot_expert[t] = j >= 0 ? s_list[0][j] : s_list[1][free_upto - 1];
    __syncthreads();
    const int tiles_here = t < n_experts ? (expert_offsets[s_slot_expert[t] + 1] - expert_offsets[s_slot_expert[t]] +
                                            TILE_PAIRS - 1) / TILE_PAIRS
                                         : 0;
    const int upto = scan(tiles_here);
    if (t < n_experts) {
        tile_table[t] = upto - tiles_here;
        tile_table[n_experts + 1 + t] = s_slot_expert[t];
    }
    if (t == n_experts - 1) tile_table[n_experts] = upto;
}

// xs_t[kb][pos] = x_s[token of sorted position pos][kb]
__global__ __launch_bounds__(256) void moe_gather_scales_kernel(const float* __restrict__ x_s,
                                                                const int* __restrict__ sorted_pairs,
                                                                float* __restrict__ xs_t, int pairs,
                                                                int stride, int kb_count, int top_k) {
    const int pos = blockIdx.x * 256 + threadIdx.x;
    if (pos >= pairs) return;
    const int token = sorted_pairs[pos] / top_k;
    for (int kb = 0; kb < kb_count; ++kb) {
        xs_t[(size_t)kb * stride + pos] = x_s[(size_t)token * kb_count + kb];
    }
}

// Phase timing build (-DMOE_PHASE_TIMING): every wavefront of workgroup 0 adds up the core clock
// cycles it spends in each phase of the K loop and leaves them in g_phase_cycles.
#ifdef MOE_PHASE_TIMING
__device__ unsigned long long g_phase_cycles[8][8];
// and every workgroup leaves its start and end on the 100 MHz wall clock, its pair count and its hardware id
__device__ unsigned long long g_wg_trace[16384][3];
#define PHASE_TIMING_BEGIN()                                                              \
    unsigned long long phase_t0 = __builtin_readcyclecounter(), phase_acc[8] = {};        \
    const unsigned long long phase_wall0 = wall_clock64(), phase_core0 = phase_t0
#define PHASE_MARK(n)                                                      \
    {                                                                      \
        const unsigned long long phase_now = __builtin_readcyclecounter(); \
        phase_acc[n] += phase_now - phase_t0;                              \
        phase_t0 = phase_now;                                              \
    }
#define PHASE_TIMING_END(wave, lane)                                        \
    if (blockIdx.x == 0 && (lane) == 0) {                                   \
        for (int i = 0; i < 7; ++i) g_phase_cycles[wave][i] = phase_acc[i]; \
        /* core clock in kHz over the workgroup's life: the wall clock counts at 100 MHz */ \
        g_phase_cycles[wave][7] = (__builtin_readcyclecounter() - phase_core0) * 100000ull / (wall_clock64() - phase_wall0); \
    }                                                                       \
    if ((wave) == 0 && (lane) == 0 && blockIdx.x < 16384) {                 \
        g_wg_trace[blockIdx.x][0] = phase_wall0;                            \
        g_wg_trace[blockIdx.x][1] = wall_clock64();                         \
        g_wg_trace[blockIdx.x][2] = ((unsigned long long)cnt << 32) | __builtin_amdgcn_s_getreg((31 << 11) | 4); \
    }
#else
#define PHASE_TIMING_BEGIN()
#define PHASE_MARK(n)
#define PHASE_TIMING_END(wave, lane)
#endif

// grid: 1-D, see the mapping at the top of the kernel
// UE8M0: all block scales are powers of two. They then go into the MFMA as its per-operand block scale
// (v_mfma_scale_f32_32x32x64_f8f6f4: each lane's 32 values of A and of B are multiplied by
// 2^(byte - 127)), the products of all K blocks add up in the accumulator itself, and the per-block
// multiply-add on the VALU (128 per wavefront and K block) disappears.
// FIX (gate/up only): the epilogue also writes the marks of the exact requantisation (moe_common.hpp).
template <bool GATE_UP, bool UE8M0, bool FIX = false, bool BF16 = false>
__global__ __launch_bounds__(512) void moe_tiled_gemm_kernel(
    const uint8_t* __restrict__ w_q, const float* __restrict__ w_s, const uint8_t* __restrict__ a_q,
    const float* __restrict__ as_t, const int* __restrict__ sorted_pairs,
    const int* __restrict__ expert_offsets, const int* __restrict__ tile_start,
    uint8_t* __restrict__ h_q, float* __restrict__ h_s, float* __restrict__ hs_t, float* __restrict__ y,
    float* __restrict__ y_scale, int K, int n_rows, int inter, int top_k, int n_experts, int scale_stride,
    float err_coef, float v_min) {
    __shared__ __attribute__((aligned(16))) uint8_t s_stage[2 * STAGE_BYTES];

    // Workgroup -> (row tile, pair tile). Consecutive workgroup ids go round-robin to the 8 XCDs,
    // each with its own L2, so the 32 workgroups that run together on one XCD are given a
    // 4 x 8 block of (row tile, pair tile): they share 4 weight tiles and 8 activation tiles
    // through that L2 instead of pulling 18 different ones.
    const int total_tiles = tile_start[n_experts];
    const int row_tiles = GATE_UP ? inter / GROUP : n_rows / TILE_ROWS;
    const int row_blocks4 = (row_tiles + SUPER_ROWS - 1) / SUPER_ROWS;
    const int linear = blockIdx.x;
    const int super = ((linear >> 3) / (SUPER_ROWS * SUPER_PAIRS)) * 8 + (linear & 7);
    const int within = (linear >> 3) % (SUPER_ROWS * SUPER_PAIRS);
    const int rb = (super % row_blocks4) * SUPER_ROWS + within % SUPER_ROWS;
    const int pt = (super / row_blocks4) * SUPER_PAIRS + within / SUPER_ROWS;
    if (rb >= row_tiles || pt >= total_tiles) return;
    int lo = 0, hi = n_experts;  // largest slot with tile_start[slot] <= pt
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tile_start[mid] <= pt) lo = mid; else hi = mid;
    }
    const int e = tile_start[n_experts + 1 + lo];  // the expert in that slot of the dispatch order
    const int begin = expert_offsets[e] + (pt - tile_start[lo]) * TILE_PAIRS;
    int cnt = expert_offsets[e + 1] - begin;
    cnt = cnt > TILE_PAIRS ? TILE_PAIRS : cnt;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int rg = wave & 3;   // 64-row group (gate/up: 32 gate + 32 up rows)
    const int th = wave >> 2;  // 128-pair half
    const int KB = K / GROUP;
    const int row_blocks = n_rows / GROUP;
    const int r32 = lane & 31;
    const int half = lane >> 5;

    // ---- fill side -------------------------------------------------------------------------
    // instruction j of a region covers its rows 8j..8j+7; lane -> row 8j + lane/8, chunk
    // (lane%8) ^ ((row >> 1) & 7). This wavefront issues instructions 4*wave .. 4*wave+3 of A and of B.
    const uint32_t ld_row = lane >> 3;
    // the row's swizzle term ((row >> 1) & 7) is (ld_row >> 1) for even and 4 ^ (ld_row >> 1) for
    // odd instructions of a wavefront (its first instruction index is a multiple of 4)
    const uint32_t ld_chunk_even = (lane & 7) ^ (ld_row >> 1);
    const uint32_t ld_off_even = ld_row * (uint32_t)K + 16 * ld_chunk_even;
    const uint32_t ld_off_odd = ld_row * (uint32_t)K + 16 * (ld_chunk_even ^ 4);
    const uint8_t* a_src[4];
    uint32_t b_off[4];  // byte offset of this lane's activation row and chunk (the buffers are < 4 GB)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ar = (4 * wave + i) * 8;  // first of the 8 tile rows of this instruction
        int row;
        if (GATE_UP) row = (ar < 128 ? 0 : inter - 128) + rb * GROUP + ar;
        else row = rb * TILE_ROWS + ar;
        a_src[i] = w_q + ((size_t)e * n_rows + row) * K;
        int p = (4 * wave + i) * 8 + (int)ld_row;
        p = begin + (p < cnt ? p : cnt - 1);  // rows past the tile's end repeat the last one
        const int arow = GATE_UP ? sorted_pairs[p] / top_k : p;
        b_off[i] = (uint32_t)arow * (uint32_t)K + 16 * (ld_chunk_even ^ (4 * (i & 1)));
    }
    const float* s_src = as_t + begin;  // + kb*scale_stride; 256 floats, the tail is padding
    const float* ws0;
    const float* ws1;
    if (GATE_UP) {
        ws0 = w_s + ((size_t)e * row_blocks + rb) * KB;
        ws1 = w_s + ((size_t)e * row_blocks + inter / GROUP + rb) * KB;
    } else {
        ws0 = w_s + ((size_t)e * row_blocks + rb * 2 + (rg >> 1)) * KB;
        ws1 = ws0;
    }

    const uint32_t stage_base = (uint32_t)(size_t)((lds_void_ptr)s_stage);
    // load i (0..7) of this wavefront's share of stage kb: 0..3 weights, 4..7 activations
    // Tiles of at most 128 pairs (the last tile of most experts holds a few dozen) use only the first half of a
    // stage's activation rows and pair scales. Their K loop is bound by load latency, not by the matrix pipe, so
    // they request activations and scales two blocks ahead like the weights: block kb's go to stage kb % 2, half
    // (kb / 2) % 2 (`sub`), and the wavefronts of the first pair half read them there.
    const bool half_tile = cnt <= TILE_PAIRS / 2;
    auto issue_load = [&](int kb, int i, int slot_parity, int sub = 0) {
        const uint32_t st = stage_base + (slot_parity & 1) * STAGE_BYTES;
        if (i < 4) {
            dma16(a_src[i] + (size_t)kb * GROUP, (i & 1) ? ld_off_odd : ld_off_even, st + (4 * wave + i) * 1024);
        } else if ((4 * wave + i - 4) * 8 < cnt) {
            // (8-row groups past the tile's last pair are not fetched: their LDS rows feed output
            // columns that are never stored. A third of the prefill workload's tile rows is such
            // padding; leaving it out lowers the L2 traffic, the kernel time did not change.)
            dma16(a_q + (size_t)kb * GROUP, b_off[i - 4], st + STAGE_A + sub * (STAGE_B / 2) + (4 * wave + i - 4) * 1024);
        }
    };
    auto issue_scales = [&](int kb, int slot_parity, bool half = false, int sub = 0) {
        const uint32_t st = stage_base + (slot_parity & 1) * STAGE_BYTES;
        if (wave == 0) {
            if (!half) dma16(s_src + (size_t)kb * scale_stride, lane * 16, st + STAGE_A + STAGE_B);
            else if (lane < 32) dma16(s_src + (size_t)kb * scale_stride, lane * 16, st + STAGE_A + STAGE_B + sub * (STAGE_S / 2));
        }
    };
    // loads of one block that a half tile's wavefront may leave in flight at the top of the block before:
    // its weights (4), its activation row groups and, in wavefront 0, its pair scales
    int half_tile_in_flight = 4 + (wave == 0 ? 1 : 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) half_tile_in_flight += (4 * wave + i) * 8 < cnt ? 1 : 0;

    // ---- read side -------------------------------------------------------------------------
    // operand of k-step s, 16-byte piece j: chunk 4s + 2*half + j of row r32 (+32*tile)
    const uint32_t rd = (r32 * 8 + ((2 * half) ^ ((r32 >> 1) & 7))) * 16;
    const uint32_t a_row0 = GATE_UP ? rg * 32 : rg * 64;        // A tile 0 of this wavefront
    const uint32_t a_row1 = GATE_UP ? 128 + rg * 32 : rg * 64 + 32;
    const lds_bytes stage_ptr = (lds_bytes)s_stage;

    int active_b = (cnt - th * 128 + 31) / 32;  // B tiles of this wavefront that hold pairs
    active_b = active_b < 0 ? 0 : active_b > 4 ? 4 : active_b;

    floatx16 acc[2][4];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 4; ++b) acc[a][b] = floatx16{0};

    // One K block for a wavefront with NB (compile time) active B tiles.
    //  * Weights are in flight for two blocks, activations for one. A wavefront copies its A
    //    operands of the block into registers at the top, so after a second barrier the weight
    //    half of the stage is free again and the weights of block kb+2 are loaded into it, while
    //    the activations and pair scales of block kb+1 go to the other stage. One stage in
    //    flight (65 KB per CU) at 1.5-2 us of loaded HBM latency was 35 GB/s per CU and bound the
    //    kernel; weights are the part that comes from HBM.
    //  * The activation loads are issued before the weight loads, so "at most 4 loads
    //    outstanding" at the top of a block means everything but the weights of block kb+1.
    //  * The loads go out between MFMA pairs (a load holds the wavefront for 60-130 cycles until
    //    the memory pipeline has taken it).
    //  * The next B tile is read from LDS as soon as the last MFMA of the current one has been
    //    issued; the partial of A tile 0 is promoted (acc += partial * scale) while the MFMAs of
    //    A tile 1 run, and the partial of A tile 1 while the next step's first MFMAs run, so the
    //    VALU work hides behind the matrix pipeline with two partial accumulators only.
    // kb1, kb2: kb+1 and kb+2, or 0 past the end (harmless loads that keep the body branch-free;
    // the epilogue waits for them before it reuses the stages).
    PHASE_TIMING_BEGIN();
    auto block = [&](auto nb_tag, auto half_tag, int kb, int kb1, int kb2) {
        constexpr int NB = decltype(nb_tag)::value;
        constexpr bool HALF = decltype(half_tag)::value != 0;  // a half tile (compile time: full tiles keep their code)
        const lds_bytes st = stage_ptr + (kb & 1) * STAGE_BYTES;
        intx8 A[2][2];  // [tile][k-step]
        intx8 B[2];     // [k-step]
        float bs = 0.f;
        const int rh = HALF ? (kb >> 1) & 1 : th;  // half of the stage's pair rows this wavefront reads
        auto read_b = [&](int b) {
            const lds_bytes bt = st + STAGE_A + (rh * 128 + b * 32) * GROUP;
            B[0] = join(*(lds_x4)(bt + rd), *(lds_x4)(bt + (rd ^ 16)));
            B[1] = join(*(lds_x4)(bt + (rd ^ 64)), *(lds_x4)(bt + (rd ^ 64 ^ 16)));
        };
        auto read_bs = [&](int b) {
            return *(const __attribute__((address_space(3))) float*)(st + STAGE_A + STAGE_B +
                                                                     (rh * 128 + b * 32 + r32) * 4);
        };
        if (NB > 0) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                A[0][s] = join(*(lds_x4)(st + a_row0 * GROUP + (rd ^ (64 * s))),
                               *(lds_x4)(st + a_row0 * GROUP + (rd ^ (64 * s) ^ 16)));
                A[1][s] = join(*(lds_x4)(st + a_row1 * GROUP + (rd ^ (64 * s))),
                               *(lds_x4)(st + a_row1 * GROUP + (rd ^ (64 * s) ^ 16)));
            }
            if constexpr (!BF16) read_b(0);
            bs = read_bs(0);
        }
        // every wavefront holds its A operands: the weight half of this stage may be refilled
        __builtin_amdgcn_s_waitcnt((63 & 15) | ((63 >> 4) << 14) | (7 << 4) | (0 << 8));  // lgkmcnt(0)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // load sequence of the block: pair scales and activations of block kb+1 (load numbers
        // 0..3), then the weights of block kb+2 (4..7), spread over the MFMA pairs
        auto load_number = [&](int n) {
            if constexpr (HALF) {
                if (n == 0) issue_scales(kb2, kb, true, ((kb + 2) >> 1) & 1);
                if (n < 4) issue_load(kb2, 4 + n, kb, ((kb + 2) >> 1) & 1);
                else issue_load(kb2, n - 4, kb);
            } else {
                if (n == 0) issue_scales(kb1, kb + 1);
                if (n < 4) issue_load(kb1, 4 + n, kb + 1);
                else issue_load(kb2, n - 4, kb);
            }
        };
        constexpr int PER_SLOT = NB >= 3 ? 2 : NB == 2 ? 2 : NB == 1 ? 4 : 8;
        auto loads = [&](int slot) {
#pragma unroll
            for (int j = 0; j < PER_SLOT; ++j) {
                // NB >= 3: activations two per slot (slots 0, 1), weights one per slot (slots 2..5)
                const int n = NB >= 3 ? (slot < 2 ? 2 * slot + j : (j == 0 ? slot + 2 : 8)) : slot * PER_SLOT + j;
                if (n < 8) load_number(n);
            }
        };
        if (NB == 0) {
            loads(0);
            return;
        }
        const float w0 = ws0[kb];
        const float w1 = ws1[kb];
        if constexpr (BF16) {
            // Gate/up on the bf16 matrix core: every e4m3 code is a bf16 value, and v_mfma_f32_32x32x16_bf16 adds
            // the products of a 128-block to fp32 accuracy (the e4m3 instruction keeps about 16 bits), so that the
            // requantised h agrees with an fp32 evaluation. A lane's 32 operand bytes of a k-step, eight at a time,
            // are the operands of four such MFMAs (A and B take the same bytes of their lanes, so the products
            // pair up the same k whichever order the matrix core walks them in).
            // Schedule: the A operands are converted once per block (64 registers); per B tile the 8 MFMAs of A
            // tile 0 run as one chain into p0, then the 8 of A tile 1 into p1. B arrives 16 bytes (two MFMAs) at
            // a time, just in time, and is read and converted once per chain, so that only 8 + 8 registers hold B.
            // The partial of one chain is promoted under the MFMAs of the next: per MFMA (32 cycles) the wavefront
            // issues 4 conversions and 2 multiply-adds, which is what fits beside it.
            bf16x8 Ab[2][8];
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int j = 0; j < 4; ++j) Ab[a][4 * s + j] = e4m3x8_to_bf16(A[a][s][2 * j], A[a][s][2 * j + 1]);
            // piece u (0..3) of B tile b: the 16 bytes that feed MFMAs 2u and 2u+1 of a chain
            auto b_piece = [&](int b, int u) {
                const lds_bytes bt = st + STAGE_A + (rh * 128 + b * 32) * GROUP;
                return *(lds_x4)(bt + (rd ^ (64 * (u >> 1)) ^ (16 * (u & 1))));
            };
            floatx16 p0, p1;
            float s0 = 0.f, s1_prev = 0.f;
            intx4 q = b_piece(0, 0);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
#pragma unroll
                for (int u = 0; u < 4; ++u) {  // chain of A tile 0; p1 of the tile before is promoted meanwhile
                    const bf16x8 f0 = e4m3x8_to_bf16(q[0], q[1]);
                    const bf16x8 f1 = e4m3x8_to_bf16(q[2], q[3]);
                    q = b_piece(b, (u + 1) & 3);
                    p0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ab[0][2 * u], f0, u == 0 ? floatx16{0} : p0, 0, 0, 0);
                    if (b > 0) {
#pragma unroll
                        for (int i = 4 * u; i < 4 * u + 2; ++i) acc[1][b - 1][i] += p1[i] * s1_prev;
                    }
                    p0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ab[0][2 * u + 1], f1, p0, 0, 0, 0);
                    if (b > 0) {
#pragma unroll
                        for (int i = 4 * u + 2; i < 4 * u + 4; ++i) acc[1][b - 1][i] += p1[i] * s1_prev;
                    }
                    if (u == 1) loads(2 * b);
                    __builtin_amdgcn_sched_barrier(0);
                }
                s0 = bs * w0;
                s1_prev = bs * w1;
                if (b + 1 < NB) bs = read_bs(b + 1);
#pragma unroll
                for (int u = 0; u < 4; ++u) {  // chain of A tile 1; p0 is promoted meanwhile
                    const bf16x8 f0 = e4m3x8_to_bf16(q[0], q[1]);
                    const bf16x8 f1 = e4m3x8_to_bf16(q[2], q[3]);
                    if (u < 3) q = b_piece(b, u + 1);
                    else if (b + 1 < NB) q = b_piece(b + 1, 0);
                    p1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ab[1][2 * u], f0, u == 0 ? floatx16{0} : p1, 0, 0, 0);
#pragma unroll
                    for (int i = 4 * u; i < 4 * u + 2; ++i) acc[0][b][i] += p0[i] * s0;
                    p1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(Ab[1][2 * u + 1], f1, p1, 0, 0, 0);
#pragma unroll
                    for (int i = 4 * u + 2; i < 4 * u + 4; ++i) acc[0][b][i] += p0[i] * s0;
                    if (u == 1) loads(2 * b + 1);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            acc[1][NB - 1] += p1 * s1_prev;
            return;
        }
        if constexpr (UE8M0) {
            // exponent bytes of the three scales; opsel 0 = byte 0 of the scale register
            const int e0 = (int)((__float_as_uint(w0) >> 23) & 255u);
            const int e1 = (int)((__float_as_uint(w1) >> 23) & 255u);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int eb = (int)((__float_as_uint(bs) >> 23) & 255u);
                acc[0][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[0][0], B[0], acc[0][b], 0, 0, 0, e0, 0, eb);
                acc[1][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[1][0], B[0], acc[1][b], 0, 0, 0, e1, 0, eb);
                loads(2 * b);
                __builtin_amdgcn_sched_barrier(0);
                acc[0][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[0][1], B[1], acc[0][b], 0, 0, 0, e0, 0, eb);
                acc[1][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[1][1], B[1], acc[1][b], 0, 0, 0, e1, 0, eb);
                if (b + 1 < NB) {
                    read_b(b + 1);
                    bs = read_bs(b + 1);
                }
                loads(2 * b + 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            return;
        }
        floatx16 p0, p1;
        float s1_prev = 0.f;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            p0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[0][0], B[0], floatx16{0}, 0, 0, 0, 0, 0, 0);
            p0 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[0][1], B[1], p0, 0, 0, 0, 0, 0, 0);
            if (b > 0) {
                acc[1][b - 1] += p1 * s1_prev;  // runs under the two MFMAs above
                asm volatile("" : "+v"(acc[1][b - 1]));
            }
            loads(2 * b);
            __builtin_amdgcn_sched_barrier(0);
            p1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[1][0], B[0], floatx16{0}, 0, 0, 0, 0, 0, 0);
            p1 = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A[1][1], B[1], p1, 0, 0, 0, 0, 0, 0);
            const float s0 = bs * w0;
            s1_prev = bs * w1;
            if (b + 1 < NB) {
                read_b(b + 1);
                bs = read_bs(b + 1);
            }
            acc[0][b] += p0 * s0;  // p0 is complete by the time the MFMAs above are in
            asm volatile("" : "+v"(acc[0][b]));
            loads(2 * b + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        acc[1][NB > 0 ? NB - 1 : 0] += p1 * s1_prev;
    };

    issue_scales(0, 0, half_tile, 0);
#pragma unroll
    for (int i = 4; i < 8; ++i) issue_load(0, i, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) issue_load(0, i, 0);
    if (KB > 1) {
        if (half_tile) {
            issue_scales(1, 1, true, 0);
#pragma unroll
            for (int i = 4; i < 8; ++i) issue_load(1, i, 1);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) issue_load(1, i, 1);
    }
    PHASE_MARK(0);  // prologue
    // the K loop exists once per value of NB, so that the accumulators live in one place per copy
    auto k_loop = [&](auto nb_tag, auto half_tag) {
        constexpr bool HALF = decltype(half_tag)::value != 0;
        for (int kb = 0; kb < KB; ++kb) {
            if (KB > 1) {
                // everything but the 4 weight loads of block kb+1 (past the end: harmless ones); in a half tile
                // everything but the loads of block kb+1
                if constexpr (!HALF) {
                    __builtin_amdgcn_s_waitcnt((4 & 15) | ((4 >> 4) << 14) | (7 << 4) | (15 << 8));
                } else {
                    switch (half_tile_in_flight) {
                        case 4: __builtin_amdgcn_s_waitcnt(4 | (7 << 4) | (15 << 8)); break;
                        case 5: __builtin_amdgcn_s_waitcnt(5 | (7 << 4) | (15 << 8)); break;
                        case 6: __builtin_amdgcn_s_waitcnt(6 | (7 << 4) | (15 << 8)); break;
                        case 7: __builtin_amdgcn_s_waitcnt(7 | (7 << 4) | (15 << 8)); break;
                        case 8: __builtin_amdgcn_s_waitcnt(8 | (7 << 4) | (15 << 8)); break;
                        default: __builtin_amdgcn_s_waitcnt(9 | (7 << 4) | (15 << 8)); break;
                    }
                }
                asm volatile("" ::: "memory");
            } else {
                wait_all_loads();
            }
            PHASE_MARK(1);  // wait for this wavefront's own loads
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            PHASE_MARK(2);  // wait for the other wavefronts
            block(nb_tag, half_tag, kb, kb + 1 < KB ? kb + 1 : 0, kb + 2 < KB ? kb + 2 : 0);
            asm volatile("" ::: "memory");
            PHASE_MARK(4);  // operand reads, MFMAs, promotion, loads of later blocks
        }
    };
    if (!half_tile) {
        switch (active_b) {
            case 4: k_loop(IntConstant<4>{}, IntConstant<0>{}); break;
            case 3: k_loop(IntConstant<3>{}, IntConstant<0>{}); break;
            case 2: k_loop(IntConstant<2>{}, IntConstant<0>{}); break;
            case 1: k_loop(IntConstant<1>{}, IntConstant<0>{}); break;
            default: k_loop(IntConstant<0>{}, IntConstant<0>{}); break;
        }
    } else {
        switch (active_b) {
            case 4: k_loop(IntConstant<4>{}, IntConstant<1>{}); break;
            case 3: k_loop(IntConstant<3>{}, IntConstant<1>{}); break;
            case 2: k_loop(IntConstant<2>{}, IntConstant<1>{}); break;
            case 1: k_loop(IntConstant<1>{}, IntConstant<1>{}); break;
            default: k_loop(IntConstant<0>{}, IntConstant<1>{}); break;
        }
    }
    wait_all_loads();
    __syncthreads();  // the stages are free: reuse them for the epilogue exchange
    PHASE_MARK(5);

    // result layout: register i of acc[a][b] is row 8*(i/4) + 4*half + i%4 of A tile a, pair
    // th*128 + b*32 + r32 of the tile. In that layout a store instruction would touch 32 or 64
    // different output rows with 4 to 32 bytes each, so both epilogues transpose through LDS and
    // write every output row as one contiguous run.
    if (GATE_UP) {
        float* s_amax = reinterpret_cast<float*>(s_stage);                      // [4 row groups][256 pairs]
        constexpr int CODE_ROW = GROUP + 16;                                    // bytes per pair row of codes
        uint8_t* s_codes = s_stage + 4 * TILE_PAIRS * sizeof(float);            // [256 pairs][CODE_ROW]
        // FIX: three more per-pair statistics, the marks of every lane's 16 elements as bit masks, the pairs'
        // scales and the list of pairs that hold a marked element
        float* s_sumsq = reinterpret_cast<float*>(s_codes + TILE_PAIRS * CODE_ROW);
        float* s_umax = s_sumsq + 4 * TILE_PAIRS;
        float* s_sgmax = s_umax + 4 * TILE_PAIRS;
        uint16_t* s_near = reinterpret_cast<uint16_t*>(s_sgmax + 4 * TILE_PAIRS);  // [256 pairs][4 row groups][2 halves]
        uint16_t* s_cand = s_near + 8 * TILE_PAIRS;
        float* s_scale = reinterpret_cast<float*>(s_cand + 8 * TILE_PAIRS);      // [256 pairs]
        int* s_token = reinterpret_cast<int*>(s_scale + TILE_PAIRS);             // [256] token of a listed pair
        float* s_tau = reinterpret_cast<float*>(s_token + TILE_PAIRS);           // [256] relative uncertainty of the scale
        int* s_count = reinterpret_cast<int*>(s_tau + TILE_PAIRS);               // items listed
        constexpr int MAX_ITEMS = 8192;  // items beyond it (a tile with that many marks) stay unrepaired
        uint16_t* s_items = reinterpret_cast<uint16_t*>(s_count + 4);            // [MAX_ITEMS] pair << 7 | column
        static_assert(19 * TILE_PAIRS * sizeof(float) + 16 * TILE_PAIRS * sizeof(uint16_t) + TILE_PAIRS * CODE_ROW + 16 +
                              MAX_ITEMS * sizeof(uint16_t) <= 2 * STAGE_BYTES, "epilogue LDS");
        // column, within the group of 128, of bit `bit` of a lane's mark mask number `part` (= 2 * row group + half)
        auto mark_column = [](int part, int bit) { return (part >> 1) * 32 + 8 * (bit >> 2) + 4 * (part & 1) + (bit & 3); };
        if constexpr (FIX) {
            if (threadIdx.x == 0) *s_count = 0;
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            float m = 0.f, sumsq = 0.f, umax = 0.f, sgmax = 0.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float sg = silu(acc[0][b][i]);
                const float v = sg * acc[1][b][i];
                if constexpr (FIX) {
                    // (the gate value stays in its register: the second pass needs silu(g) and u again)
                    sumsq += acc[0][b][i] * acc[0][b][i] + acc[1][b][i] * acc[1][b][i];
                    umax = fmaxf(umax, fabsf(acc[1][b][i]));
                    sgmax = fmaxf(sgmax, fabsf(sg));
                } else {
                    acc[0][b][i] = v;
                }
                m = fmaxf(m, fabsf(v));
            }
            m = fmaxf(m, __shfl_xor(m, 32));
            const int at = rg * TILE_PAIRS + th * 128 + b * 32 + r32;
            if (half == 0) s_amax[at] = m;
            if constexpr (FIX) {
                sumsq += __shfl_xor(sumsq, 32);
                umax = fmaxf(umax, __shfl_xor(umax, 32));
                sgmax = fmaxf(sgmax, __shfl_xor(sgmax, 32));
                if (half == 0) s_sumsq[at] = sumsq, s_umax[at] = umax, s_sgmax[at] = sgmax;
            }
        }
        __syncthreads();
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const int pl = th * 128 + b * 32 + r32;
            const float m = fmaxf(fmaxf(s_amax[pl], s_amax[TILE_PAIRS + pl]),
                                  fmaxf(s_amax[2 * TILE_PAIRS + pl], s_amax[3 * TILE_PAIRS + pl]));
            const float scale = group_scale(m, UE8M0);
            // (v * (1 / scale) is within an ulp of v / scale, which the exact forms use: they can differ only
            // where fp32 itself does not decide the code)
            const float inv_scale = 1.f / scale;
            float err = 0.f, dh_max = 0.f;
            bool uncertain = false;
            if constexpr (FIX) {
                const float sumsq = s_sumsq[pl] + s_sumsq[TILE_PAIRS + pl] + s_sumsq[2 * TILE_PAIRS + pl] +
                                    s_sumsq[3 * TILE_PAIRS + pl];
                const float umax = fmaxf(fmaxf(s_umax[pl], s_umax[TILE_PAIRS + pl]),
                                         fmaxf(s_umax[2 * TILE_PAIRS + pl], s_umax[3 * TILE_PAIRS + pl]));
                const float sgmax = fmaxf(fmaxf(s_sgmax[pl], s_sgmax[TILE_PAIRS + pl]),
                                          fmaxf(s_sgmax[2 * TILE_PAIRS + pl], s_sgmax[3 * TILE_PAIRS + pl]));
                err = err_coef * sqrtf(sumsq * (1.f / 256.f));
                dh_max = (1.1f * umax + sgmax) * err;
                uncertain = !UE8M0 || group_scale(m + dh_max, true) != group_scale(m - dh_max, true);
            }
            uint32_t near_bits = 0, cand_bits = 0;
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                float q[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    float v = acc[0][b][4 * qd + r];
                    if constexpr (FIX) {
                        const float sg = silu(v);
                        v = sg * acc[1][b][4 * qd + r];
                        const uint32_t marks = requant_marks(fminf(fabsf(v) * inv_scale, E4M3_MAX), sg, acc[1][b][4 * qd + r],
                                                             err * inv_scale, dh_max * inv_scale,
                                                             uncertain ? dh_max / fmaxf(m, AMAX_FLOOR) : 0.f, uncertain, v_min);
                        near_bits |= (marks & MARK_NEAR ? 1u : 0u) << (4 * qd + r);
                        cand_bits |= (marks & MARK_CANDIDATE ? 1u : 0u) << (4 * qd + r);
                    }
                    q[r] = fminf(fmaxf(v * inv_scale, -E4M3_MAX), E4M3_MAX);
                }
                int packed = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
                packed = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], packed, true);
                *reinterpret_cast<int*>(s_codes + pl * CODE_ROW + rg * 32 + 8 * qd + 4 * half) = packed;
            }
            if constexpr (FIX) {
                s_near[pl * 8 + rg * 2 + half] = (uint16_t)near_bits;
                s_cand[pl * 8 + rg * 2 + half] = (uint16_t)cand_bits;
                if (rg == 0 && half == 0) s_scale[pl] = scale, s_tau[pl] = dh_max / fmaxf(m, AMAX_FLOOR);
            }
            if (rg == 0 && half == 0 && pl < cnt) {
                const size_t pos = (size_t)begin + pl;
                h_s[pos * (inter / GROUP) + rb] = scale;
                hs_t[(size_t)rb * scale_stride + pos] = scale;
            }
        }
        __syncthreads();
        if constexpr (FIX) {
            // Exact requantisation of the marked elements: a list of (pair, column) items that the wavefronts take
            // in turn. An item is recomputed by one wavefront as fp32 products of the codes summed in fp64 (the dot
            // product itself to fp32 accuracy), all of its loads in flight at once: the activation row and the two
            // weight rows (3 K bytes) and the block scales. The pair keeps the scale the matrix core's maximum gave
            // it (off by about 1e-5 of itself, which moves no dequantised value by more than that); the code is the
            // rounding of exact value / that scale unless the exact scale, which may differ by the relative amount
            // s_tau, could give another code: only then the elements that may be the pair's maximum are recomputed as
            // well and the code is taken with the exact scale (a power-of-two scale does not move with the maximum's
            // 5th digit, so that form never does this).
            if (threadIdx.x < TILE_PAIRS) {
                const int pl = threadIdx.x;
                const uint16_t* masks = s_near + pl * 8;
                const intx4 nm = *reinterpret_cast<const intx4*>(masks);
                if (pl < cnt && (nm[0] | nm[1] | nm[2] | nm[3]) != 0) {
                    s_token[pl] = sorted_pairs[(size_t)begin + pl] / top_k;
                    int n = 0;
                    for (int part = 0; part < 8; ++part) n += __builtin_popcount(masks[part]);
                    int slot = atomicAdd(s_count, n);
                    for (int part = 0; part < 8; ++part) {
                        for (uint32_t m = masks[part]; m != 0; m &= m - 1) {
                            if (slot < MAX_ITEMS) s_items[slot] = (uint16_t)((pl << 7) | mark_column(part, __builtin_ctz(m)));
                            ++slot;
                        }
                    }
                }
            }
            __syncthreads();
            const int n_chunks = K / 16;
            const uint8_t* gate_rows = w_q + ((size_t)e * n_rows + rb * GROUP) * K;
            auto exact_h = [&](int pl, int col) {  // every lane returns the same value
                const uint8_t* x_row = a_q + (size_t)s_token[pl] * K;
                const float* xs = as_t + begin + pl;  // [kb * scale_stride]
                const uint8_t* gate_row = gate_rows + (size_t)col * K;
                const uint8_t* up_row = gate_row + (size_t)inter * K;
                double g = 0.0, u = 0.0;
                for (int c0 = 0; c0 < n_chunks; c0 += 512) {
                    // (a load instruction costs a wavefront 150-300 cycles to issue whatever it fetches: the scale
                    // products of the 64 K blocks of this stretch are fetched by one lane each, three loads, and
                    // handed to the lanes that need them by shuffles, instead of three loads per 1 KB of a row)
                    const int kb = (c0 >> 3) + lane;
                    float sg_kb = 0.f, su_kb = 0.f;
                    if (kb < KB) {
                        const float x_scale = xs[(size_t)kb * scale_stride];
                        sg_kb = x_scale * ws0[kb];
                        su_kb = x_scale * ws1[kb];
                    }
                    intx4 xq[8], wg[8], wu[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const int c = c0 + 64 * j + lane;
                        xq[j] = wg[j] = wu[j] = intx4{0, 0, 0, 0};
                        if (c < n_chunks) {
                            xq[j] = *reinterpret_cast<const intx4*>(x_row + 16 * c);
                            wg[j] = *reinterpret_cast<const intx4*>(gate_row + 16 * c);
                            wu[j] = *reinterpret_cast<const intx4*>(up_row + 16 * c);
                        }
                    }
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        g += (double)(dot16(xq[j], wg[j]) * __shfl(sg_kb, 8 * j + (lane >> 3)));
                        u += (double)(dot16(xq[j], wu[j]) * __shfl(su_kb, 8 * j + (lane >> 3)));
                    }
                }
                const float gf = (float)wave_sum(g);
                const float uf = (float)wave_sum(u);
                return gf / (1.f + expf(-gf)) * uf;
            };
            const int n_items = min(*s_count, MAX_ITEMS);
            for (int it = wave; it < n_items; it += 8) {
                const int item = __builtin_amdgcn_readfirstlane((int)s_items[it]);
                const int pl = item >> 7, col = item & 127;
                const float h = exact_h(pl, col);
                float scale = s_scale[pl];
                if constexpr (!UE8M0) {
                    const float v = fminf(fabsf(h) / scale, E4M3_MAX), tau = v * s_tau[pl];
                    const int codes = __builtin_amdgcn_cvt_pk_fp8_f32(fmaxf(v - tau, 0.f), fminf(v + tau, E4M3_MAX), 0, false);
                    if (((codes ^ (codes >> 8)) & 0xff) != 0) {  // (uniform over the wavefront: h is)
                        float amax = 0.f;
                        for (int part = 0; part < 8; ++part) {
                            for (uint32_t cm = __builtin_amdgcn_readfirstlane((uint32_t)s_cand[pl * 8 + part]); cm != 0;
                                 cm &= cm - 1) {
                                amax = fmaxf(amax, fabsf(exact_h(pl, mark_column(part, __builtin_ctz(cm)))));
                            }
                        }
                        if (amax > 0.f) scale = group_scale(amax, false);
                    }
                }
                const float v = fminf(fmaxf(h / scale, -E4M3_MAX), E4M3_MAX);
                const int code = __builtin_amdgcn_cvt_pk_fp8_f32(v, v, 0, false);
                if (lane == 0) s_codes[pl * CODE_ROW + col] = (uint8_t)(code & 0xff);
            }
            __syncthreads();
        }
        // 8 lanes write the 128 codes of one pair: 8 pairs per instruction, 4 instructions per wavefront
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int pl = (wave * 4 + it) * 8 + (lane >> 3);
            if (pl < cnt) {
                const size_t at = ((size_t)begin + pl) * inter + rb * GROUP + (lane & 7) * 16;
                *reinterpret_cast<intx4*>(h_q + at) =
                    *reinterpret_cast<const intx4*>(s_codes + pl * CODE_ROW + (lane & 7) * 16);
            }
        }
    } else {
        // The tile leaves as fp16 of y / 2^e, 2^e the power of two above the largest magnitude of the pair's 256
        // values of this tile (kept per pair and column tile for the combine): half the bytes of fp32 to write
        // here and to read there, 11 significant bits relative to that maximum. The maximum of a pair: over a
        // lane's 32 values, the lane holding the pair's other rows of this wavefront, and through LDS the four
        // wavefronts that hold its other row groups. Then two passes of 128 pairs: the wavefronts of one pair
        // half put their 64 x 128 results into LDS as [pair][256 rows], and all 8 wavefronts write whole
        // 512-byte rows.
        typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
        constexpr int Y_ROW = TILE_ROWS + 8;  // halfs per staged pair row (16 bytes of padding)
        _Float16* s_y = reinterpret_cast<_Float16*>(s_stage);
        float* s_max = reinterpret_cast<float*>(s_stage + 128 * Y_ROW * sizeof(_Float16));  // [4 row groups][256 pairs]
        static_assert(128 * Y_ROW * sizeof(_Float16) + 4 * TILE_PAIRS * sizeof(float) <= 2 * STAGE_BYTES, "epilogue LDS");
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            float m = 0.f;
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int i = 0; i < 16; ++i) m = fmaxf(m, fabsf(acc[a][b][i]));
            m = fmaxf(m, __shfl_xor(m, 32));
            if (half == 0) s_max[rg * TILE_PAIRS + th * 128 + b * 32 + r32] = m;
        }
        __syncthreads();
        auto pair_exponent = [&](int pl) {  // biased exponent of 2^e for pair pl of the tile
            const float m = fmaxf(fmaxf(s_max[pl], s_max[TILE_PAIRS + pl]),
                                  fmaxf(s_max[2 * TILE_PAIRS + pl], s_max[3 * TILE_PAIRS + pl]));
            const uint32_t e_bits = ((__float_as_uint(m) >> 23) & 255u) + 1u;
            return m > 0.f ? (e_bits > 253u ? 253u : e_bits) : 127u;
        };
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            if (pass == 1) __syncthreads();
            if (th == pass) {
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const float inv = __uint_as_float((254u - pair_exponent(th * 128 + b * 32 + r32)) << 23);
                    _Float16* dst = s_y + (b * 32 + r32) * Y_ROW + rg * 64 + 4 * half;
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
#pragma unroll
                        for (int qd = 0; qd < 4; ++qd) {
                            *reinterpret_cast<halfx4*>(dst + a * 32 + 8 * qd) =
                                halfx4{(_Float16)(acc[a][b][4 * qd] * inv), (_Float16)(acc[a][b][4 * qd + 1] * inv),
                                       (_Float16)(acc[a][b][4 * qd + 2] * inv), (_Float16)(acc[a][b][4 * qd + 3] * inv)};
                        }
                    }
                }
            }
            __syncthreads();
            // 32 lanes write the 512 bytes of one pair: two pairs per instruction, 8 instructions per wavefront
#pragma unroll
            for (int it = 0; it < 8; ++it) {
                const int pr = wave * 16 + 2 * it + half;  // pair within this half
                const int pl = pass * 128 + pr;
                if (pl < cnt) {
                    const size_t row = (size_t)begin + pl;
                    *reinterpret_cast<intx4*>(reinterpret_cast<_Float16*>(y) + row * n_rows + rb * TILE_ROWS + r32 * 8) =
                        *reinterpret_cast<const intx4*>(s_y + pr * Y_ROW + r32 * 8);
                    if (r32 == 0) y_scale[row * (n_rows / TILE_ROWS) + rb] = __uint_as_float(pair_exponent(pl) << 23);
                }
            }
        }
    }
    PHASE_MARK(6);  // epilogue
    PHASE_TIMING_END(wave, lane);
}

}  // namespace

// Scratch the tiled path needs beyond the layer's common workspace:
//   tile_start [2*n_experts+1] ints (moe_tile_start_kernel); xs_t [hidden/128][stride] and hs_t [inter/128][stride] floats
//   with stride = pairs rounded up to 256, plus 256.
extern "C" void moe_tiled_prepare_launcher(int* tile_start, float* xs_t, const float* x_s,
                                           const int* sorted_pairs, const int* expert_offsets,
                                           int tokens, int hidden, int n_experts, int top_k,
                                           int scale_stride, hipStream_t stream) {
    if (tokens <= 0) return;
    if (n_experts <= 0 || n_experts > 1024 || hidden <= 0 || hidden % GROUP != 0 || top_k <= 0) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);  // (the tile scan is one workgroup of 1024 lanes)
        return;
    }
    const int pairs = tokens * top_k;
    moe_tile_start_kernel<<<1, 1024, 0, stream>>>(expert_offsets, tile_start, n_experts);
    moe_gather_scales_kernel<<<(pairs + 255) / 256, 256, 0, stream>>>(x_s, sorted_pairs, xs_t, pairs,
                                                                    scale_stride, hidden / GROUP, top_k);
}

// requant_config: the CONFIG_*_REQUANT, band and significance bits of the layer's config (moe_common.hpp):
// neither requant bit: e4m3 matrix core, the marked elements repaired in the epilogue; CONFIG_EXACT_REQUANT: bf16
// matrix core; CONFIG_APPROX_REQUANT: e4m3 matrix core, codes as they come.
extern "C" void moe_gate_up_tiled_launcher(void* h_q, float* h_s, float* hs_t, const void* x_q,
                                           const float* xs_t, const void* w13_q, const float* w13_s,
                                           const int* sorted_pairs, const int* expert_offsets,
                                           const int* tile_start, int tokens, int hidden, int inter,
                                           int n_experts, int top_k, int scale_stride, int ue8m0,
                                           int requant_config, hipStream_t stream) {
    if (tokens <= 0) return;
    if (hidden % GROUP != 0 || inter % GROUP != 0 || hidden <= 0 || inter <= 0 ||
        (unsigned long long)tokens * hidden >= (1ull << 32)) {  // 32-bit activation offsets
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const int max_tiles = (tokens * top_k) / TILE_PAIRS + n_experts;
    const dim3 grid(tiled_grid(inter / GROUP, max_tiles));
    const bool bf16_core = (requant_config & CONFIG_EXACT_REQUANT) != 0 && !(requant_config & CONFIG_APPROX_REQUANT);
    const bool repair = !bf16_core && !(requant_config & CONFIG_APPROX_REQUANT);
    const auto kernel = bf16_core ? (ue8m0 ? moe_tiled_gemm_kernel<true, true, false, true> : moe_tiled_gemm_kernel<true, false, false, true>)
                        : repair  ? (ue8m0 ? moe_tiled_gemm_kernel<true, true, true> : moe_tiled_gemm_kernel<true, false, true>)
                                  : (ue8m0 ? moe_tiled_gemm_kernel<true, true, false> : moe_tiled_gemm_kernel<true, false, false>);
    kernel<<<grid, 512, 0, stream>>>(
        static_cast<const uint8_t*>(w13_q), w13_s, static_cast<const uint8_t*>(x_q), xs_t, sorted_pairs,
        expert_offsets, tile_start, static_cast<uint8_t*>(h_q), h_s, hs_t, nullptr, nullptr, hidden, 2 * inter,
        inter, top_k, n_experts, scale_stride, requant_error_coefficient(requant_config),
        requant_min_magnitude(requant_config));
}

// y [pairs, hidden] as fp16 of y / y_scale (the buffer's first pairs * hidden * 2 bytes), y_scale
// [pairs, hidden/256] fp32 powers of two: value = fp16 * y_scale[row][column / 256].
extern "C" void moe_down_tiled_launcher(void* y, float* y_scale, const void* h_q, const float* hs_t,
                                        const void* w2_q, const float* w2_s, const int* expert_offsets,
                                        const int* tile_start, int tokens, int hidden, int inter,
                                        int n_experts, int top_k, int scale_stride, int ue8m0,
                                        hipStream_t stream) {
    if (tokens <= 0) return;
    if (hidden % TILE_ROWS != 0 || inter % GROUP != 0 || hidden <= 0 || inter <= 0 ||
        (unsigned long long)tokens * top_k * inter >= (1ull << 32)) {  // 32-bit activation offsets
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const int max_tiles = (tokens * top_k) / TILE_PAIRS + n_experts;
    const dim3 grid(tiled_grid(hidden / TILE_ROWS, max_tiles));
    const auto kernel = ue8m0 ? moe_tiled_gemm_kernel<false, true> : moe_tiled_gemm_kernel<false, false>;
    kernel<<<grid, 512, 0, stream>>>(
        static_cast<const uint8_t*>(w2_q), w2_s, static_cast<const uint8_t*>(h_q), hs_t, nullptr,
        expert_offsets, tile_start, nullptr, nullptr, nullptr, static_cast<float*>(y), y_scale, inter, hidden,
        inter, top_k, n_experts, scale_stride, 0.f, 0.f);
}
