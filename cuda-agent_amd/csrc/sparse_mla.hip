// Sparse-MLA decode attention: per request, every head attends to the same top-k rows of the
// request's latent KV cache.
//
//   K_g = kv[b, idx[b, :]]            [topk, 576]  (gathered rows, bf16)
//   s   = q[b] K_g^T * sm_scale       [heads, topk]
//   p   = softmax(s)                  over the selected rows
//   out = p K_g[:, :512]              [heads, 512] -> bf16
//
// The gathered rows are the only large stream (topk*1152 bytes per request) and are read from
// HBM once per (request, split): a workgroup owns ALL heads of one head group (32 heads per
// wavefront, up to 4 wavefronts = 128 heads) for a contiguous slice of the selected rows.
//
// Data path of one 32-row tile:
//   * rows go straight from global memory to LDS (16 bytes per lane, no VGPR staging), three
//     tiles in flight, 16-byte chunks XOR-swizzled by row so that both access patterns below
//     are bank-conflict free;
//   * QK^T on v_mfma_f32_32x32x16_bf16 as S^T[row, head] = K[row, :] Q^T: K is the A operand,
//     read from LDS 16 bytes per lane, Q^T is the B operand and stays in registers for the
//     whole kernel (144 VGPRs). In the result layout every lane holds 16 scores of ONE head,
//     so the online-softmax state (running max, running sum, rescale factor) is per-lane
//     scalar work with a single cross-lane exchange per tile;
//   * PV as O^T[dv, head] = V^T[dv, row] P^T[row, head]: the probabilities never leave the
//     registers they were computed in (converted to bf16 in place they are already the B
//     operand), V^T is the A operand and comes from the same LDS tile through the transposing
//     LDS read (ds_read_b64_tr_b16). The 32x512 fp32 accumulator of a wavefront is 256
//     registers.
// Each split writes a normalised partial output and its log2-sum-exp; a merge kernel combines
// the splits and converts to bf16.
//
// Two split kernels share this data path. sparse_mla_split_kernel<NW> is the form described
// above (one wavefront per 32 heads; used for 32 and 64 heads and for caches of 4 GB and more
// per request). sparse_mla_split8_kernel, further down, is the default for multiples of 128
// heads: two wavefronts per 32 heads that split Q by d and the accumulator by dv.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "launch_status.hpp"
#include "mla_addressing.hpp"

namespace {

using mla::KvAddressing;
using mla::resolve_key;

constexpr int D_QK = 576;
constexpr int D_V = 512;
constexpr int ROW_BYTES = D_QK * 2;        // 1152
constexpr int ROW_CHUNKS = ROW_BYTES / 16;  // 72 chunks of 16 bytes
constexpr int TILE_ROWS = 32;
constexpr int TILE_CHUNKS = TILE_ROWS * ROW_CHUNKS;  // 2304
constexpr int K_STEPS = D_QK / 16;                   // 36 MFMA k-steps for QK^T
constexpr int DV_TILES = D_V / 32;                   // 16 accumulator tiles per wavefront
constexpr int MAX_SPLIT_ROWS = 2048;                 // indices of one split staged in LDS

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_void_ptr;

// position of 16-byte chunk `chunk` of row `row` inside a tile (in 16-byte units). A row is 1152
// bytes = 4.5 x 256, so two consecutive rows share a row of the 64 LDS banks like rows of 128
// bytes would; a ds_read_b128 serves 16 consecutive lanes per cycle, so among 16 consecutive
// tile rows the 8 of equal parity must use 8 different chunk positions: the swizzle term is a
// permutation of (row >> 1) & 7 (with row & 7 the K operand reads ran at 2/3 of the conflict-free rate).
// The permutation is a rotation right by one bit, so that rows 2 apart differ in bit 2 of the term: a
// transposing 8-byte read of the V^T operand takes 64 bytes from each of 4 consecutive rows per 32 lanes,
// and rows of equal parity must take them from different halves of a 128-byte stretch (with the plain
// (row >> 1) & 7 every such read cost two more LDS cycles, a fifth of the kernel's LDS time).
__device__ __forceinline__ int row_swizzle(int row) { return ((row & 2) << 1) | ((row >> 2) & 3); }
__device__ __forceinline__ int swizzled_slot(int row, int chunk) {
    return row * ROW_CHUNKS + ((chunk & ~7) | ((chunk ^ row_swizzle(row)) & 7));
}

// One wavefront's share of a tile: with NW wavefronts each owns 32/NW consecutive rows, fetched by
// PER_WAVE global->LDS instructions of 64 lanes x 16 bytes.
template <int NW>
struct TileLoader {
    static constexpr int PER_WAVE = TILE_CHUNKS / 64 / NW;  // 36 / NW
    const char* kv_b;
    int wave;
    int lane;

    // Instruction i of this wavefront's share of `tile`.
    __device__ __forceinline__ void issue(uint4* tile, const int* s_idx_tile, bool has_padding,
                                          int i) const {
        // Hiding the lane number from the optimiser keeps the slot -> (row, chunk) arithmetic
        // (a handful of integer operations) from being precomputed for all loads before the
        // tile loop, which would hold two registers per load for the whole kernel.
        int l = lane;
        asm volatile("" : "+v"(l));
        const int inst = wave * PER_WAVE + i;
        const int slot = inst * 64 + l;
        const int row = slot / ROW_CHUNKS;
        const int pos = slot - row * ROW_CHUNKS;
        const int chunk = (pos & ~7) | ((pos ^ row_swizzle(row)) & 7);
        const int key = s_idx_tile[row];
        const char* src = kv_b + (size_t)(key < 0 ? 0 : key) * ROW_BYTES + chunk * 16;
        // Each lane's 16 bytes land at lds_base + lane*16 (M0 carries the wavefront's base).
        // Written as an asm statement so that the loads stay outside the compiler's own
        // bookkeeping of outstanding memory operations: completion is awaited explicitly, per
        // tile, by wait_vmcnt<>() in the main loop, and LDS reads of one tile do not wait
        // for the loads of the tiles behind it.
        const uint32_t lds_base = (uint32_t)(size_t)((lds_void_ptr)(tile + inst * 64));
        if (!has_padding || key >= 0) {
            asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off"
                         :
                         : "v"(src), "s"(lds_base)
                         : "memory", "m0");
        } else {
            // Padding rows are zero-filled rather than fetched: their probabilities are 0, and
            // 0 times whatever a cache row happens to hold (NaN, Inf) would not be.
            tile[slot] = make_uint4(0u, 0u, 0u, 0u);
        }
    }

    __device__ __forceinline__ void issue_all(uint4* tile, const int* s_idx_tile,
                                              bool has_padding) const {
#pragma unroll
        for (int i = 0; i < PER_WAVE; ++i) issue(tile, s_idx_tile, has_padding, i);
    }
};

struct SoftmaxState {
    float m;  // reference exponent of the accumulator (log2 domain); same in lanes l and l^32
    float l;  // running sum of exp2(s - m) over the rows this lane has seen
};

// The accumulator is kept relative to a per-head reference exponent m, which moves whenever a
// score exceeds it by more than FRAME_SLACK powers of two. With slack 0 this is the usual strict
// running maximum: the largest probability of a head is exactly 1, which is what keeps the
// bf16 rounding of the probabilities below the 2e-2*rms bound on heads that one row dominates
// (a slack of 8 measured 2.0e-2 on the full workload against 0.9e-2 for slack 0). The price is
// the 256-register rescale of the accumulator on almost every tile, since some head out of a
// wavefront's 32 nearly always sees a new maximum.
constexpr float FRAME_SLACK = 0.f;

// Per-lane byte offsets into a tile, computed once. With the XOR swizzle every LDS address of
// the inner loops is one of these six values plus a compile-time constant, so the reads use
// the instruction's immediate offset field and no address arithmetic.
struct LaneOffsets {
    uint32_t qk[4];  // K operand of k-step ks: qk[ks & 3] + (ks >> 2) * 128
    uint32_t pv[2];  // V^T operand of dv tile t, k-step ks, half-read rr:
                     //   (pv[t & 1] ^ 32*rr) + (16*ks + 8*rr) * ROW_BYTES + (t >> 1) * 128
                     // (8 rows further down the swizzle term has bit 1 flipped)
};

__device__ __forceinline__ LaneOffsets make_lane_offsets(int lane) {
    LaneOffsets o;
    const int r32 = lane & 31;
    const int half = lane >> 5;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        o.qk[c] = r32 * ROW_BYTES + (((2 * c + half) ^ row_swizzle(r32)) & 7) * 16;
    }
    const int g2 = (lane >> 4) & 1;
    const int s16 = lane & 15;
    const int row = 4 * half + (s16 >> 2);  // tile row of this lane's address, modulo 8
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int chunk = 4 * u + 2 * g2 + ((s16 & 3) >> 1);
        o.pv[u] = row * ROW_BYTES + ((chunk ^ row_swizzle(row)) & 7) * 16 + 8 * (s16 & 1);
    }
    return o;
}

typedef const __attribute__((address_space(3))) char* lds_bytes;

// Everything a wavefront does with one resident tile. `prefetch(i)` issues instruction i of the
// wavefront's share of a later tile; the calls are spread over the QK^T loop so that the
// address arithmetic overlaps the matrix pipeline and the memory system sees a steady stream.
// LDS reads run two groups ahead of the MFMAs that consume them; the scheduling fences keep the
// compiler from hoisting all 36 + 64 reads to the top (which would need more registers than
// the ~110 left beside Q and the accumulator).
template <int PREFETCH_COUNT, typename Prefetch>
__device__ __forceinline__ void process_tile(const uint4* tile, const int* s_idx_tile, bool masked,
                                             const bf16x8 (&qreg)[K_STEPS], floatx16 (&acc)[DV_TILES],
                                             SoftmaxState& st, const LaneOffsets& off,
                                             float scale_log2, int lane, Prefetch prefetch) {
    typedef const __attribute__((address_space(3))) uintx4* lds_x4;
    typedef shortx4 __attribute__((address_space(3)))* lds_s4;
    const int half = lane >> 5;
    const lds_bytes base = (lds_bytes)tile;

#pragma unroll
    for (int t = 0; t < DV_TILES; ++t) asm volatile("" : "+a"(acc[t]));

    // S^T[row, head] = sum_d K[row, d] Q[head, d]
    floatx16 s = {0};
    asm volatile("" : "+v"(s));  // keep S out of the accumulation registers
    {
        constexpr int G = 2;                 // MFMAs per group
        constexpr int GROUPS = K_STEPS / G;  // 18
        constexpr int DEPTH = 2;             // groups of LDS reads in flight
        uintx4 kbuf[DEPTH][G];
        auto k_read = [&](int g) {
#pragma unroll
            for (int j = 0; j < G; ++j) {
                const int ks = G * g + j;
                kbuf[g % DEPTH][j] = *(lds_x4)(base + off.qk[ks & 3] + (ks >> 2) * 128);
            }
        };
#pragma unroll
        for (int g = 0; g < DEPTH - 1; ++g) k_read(g);
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            if (g + DEPTH - 1 < GROUPS) k_read(g + DEPTH - 1);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kbuf[g % DEPTH][0]),
                                                        qreg[G * g], s, 0, 0, 0);
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kbuf[g % DEPTH][1]),
                                                        qreg[G * g + 1], s, 0, 0, 0);
#pragma unroll
            for (int i = g * PREFETCH_COUNT / GROUPS; i < (g + 1) * PREFETCH_COUNT / GROUPS; ++i) {
                prefetch(i);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    asm volatile("" : "+v"(s));  // the softmax arithmetic below wants S in ordinary VGPRs

    // register i of `s` is row 8*(i/4) + 4*half + i%4 of the tile, head = lane % 32
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] *= scale_log2;
    if (masked) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int row = 8 * (i / 4) + 4 * half + (i % 4);
            if (s_idx_tile[row] < 0) s[i] = -INFINITY;
        }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, s[i]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));

    // Move the reference exponent only when this tile exceeds it by more than FRAME_SLACK (or
    // when it is still unset). alpha rescales what has been accumulated so far.
    const bool move = tmax > st.m + FRAME_SLACK || st.m == -INFINITY;
    const float m_new = move ? tmax : st.m;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // every row so far was padding
    const float alpha = move ? __builtin_amdgcn_exp2f(st.m - m_use) : 1.f;
    const bool rescale = move && st.l != 0.f;  // nothing accumulated yet: nothing to rescale
    st.m = m_new;

    float psum = 0.f;
    bf16x8 p[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const __bf16 e = (__bf16)__builtin_amdgcn_exp2f(s[i] - m_use);
        p[i / 8][i % 8] = e;
        // The normaliser sums the probabilities as rounded, i.e. exactly the weights the PV
        // product uses: the output is then a true convex combination of rows, and where one row
        // dominates a head the rounding error of its weight cancels between numerator and
        // denominator.
        psum += (float)e;
    }
    st.l = st.l * alpha + psum;

    if (__builtin_amdgcn_ballot_w64(rescale) != 0) {
#pragma unroll
        for (int t = 0; t < DV_TILES; ++t) {
            // The empty asm statements pin the tile to accumulation registers on both sides
            // of the multiply, so only 16 values at a time pass through ordinary VGPRs.
            asm volatile("" : "+a"(acc[t]));
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[t][i] *= alpha;
            asm volatile("" : "+a"(acc[t]));
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // O^T[dv, head] += V^T[dv, row] P^T[row, head]; k index 8*half + 4*rr + e of k-step ks is
    // tile row 16*ks + 8*rr + 4*half + e for both operands.
    constexpr int PV_STEPS = 2 * DV_TILES;  // (k-step, dv tile) pairs, 32 MFMAs
    constexpr int PV_GROUP = 4;
    shortx4 vbuf[2][PV_GROUP][2];
    auto pv_read = [&](int step, shortx4 (&dst)[2]) {
        const int ks = step / DV_TILES;
        const int t = step % DV_TILES;
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
            dst[rr] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (lds_s4)(base + (off.pv[t & 1] ^ (32 * rr)) + (16 * ks + 8 * rr) * ROW_BYTES + (t >> 1) * 128));
        }
    };
#pragma unroll
    for (int j = 0; j < PV_GROUP; ++j) pv_read(j, vbuf[0][j]);
#pragma unroll
    for (int g = 0; g < PV_STEPS / PV_GROUP; ++g) {
        if (g + 1 < PV_STEPS / PV_GROUP) {
#pragma unroll
            for (int j = 0; j < PV_GROUP; ++j) pv_read((g + 1) * PV_GROUP + j, vbuf[(g + 1) & 1][j]);
        }
#pragma unroll
        for (int j = 0; j < PV_GROUP; ++j) {
            const int step = g * PV_GROUP + j;
            const int ks = step / DV_TILES;
            const int t = step % DV_TILES;
            const bf16x4 lo = __builtin_bit_cast(bf16x4, vbuf[g & 1][j][0]);
            const bf16x4 hi = __builtin_bit_cast(bf16x4, vbuf[g & 1][j][1]);
            const bf16x8 a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, p[ks], acc[t], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// wait until at most `n` of this wavefront's vector-memory operations are outstanding
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// all of this wavefront's vector-memory AND LDS operations have completed (tiles with padding
// rows are completed by ordinary LDS stores of zeros, which the other wavefronts read)
__device__ __forceinline__ void wait_all_memory() {
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8));
}

// grid: x = split, y = request, z = head group of 32*NW heads
template <int NW>
__global__ __launch_bounds__(64 * NW) void sparse_mla_split_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ idx,
    float* __restrict__ o_part, float* __restrict__ lse_part, int n_heads, int n_kv_rows, int topk,
    int rows_per_split, float scale_log2, KvAddressing kva) {
    constexpr int PER_WAVE = TileLoader<NW>::PER_WAVE;
    // Three separately named tile buffers: the compiler then knows which in-flight
    // global->LDS loads an LDS read can depend on and does not drain all of them.
    __shared__ uint4 tile0[TILE_CHUNKS];
    __shared__ uint4 tile1[TILE_CHUNKS];
    __shared__ uint4 tile2[TILE_CHUNKS];
    __shared__ int s_idx[MAX_SPLIT_ROWS];
    __shared__ int s_first_masked_tile;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int split = blockIdx.x;
    const int n_splits = gridDim.x;
    const int b = blockIdx.y;
    const int head0 = blockIdx.z * (32 * NW) + wave * 32;

    const int row_begin = split * rows_per_split;
    int row_end = row_begin + rows_per_split;
    if (row_end > topk) row_end = topk;
    const int n_rows = row_end > row_begin ? row_end - row_begin : 0;
    const int n_tiles = (n_rows + TILE_ROWS - 1) / TILE_ROWS;

    if (tid == 0) s_first_masked_tile = n_tiles;
    __syncthreads();
    for (int i = tid; i < n_tiles * TILE_ROWS; i += 64 * NW) {
        int key = -1;  // out-of-range selections are treated as padding
        if (i < n_rows) key = resolve_key(idx[(size_t)b * topk + row_begin + i], b, kva, n_kv_rows);
        if (key < 0) atomicMin(&s_first_masked_tile, i / TILE_ROWS);
        s_idx[i] = key;
    }
    __syncthreads();
    const int first_masked_tile = s_first_masked_tile;

    const TileLoader<NW> loader{
        reinterpret_cast<const char*>(kv) + (size_t)b * kva.batch_rows * ROW_BYTES, wave, lane};

    // prologue: tiles 0 and 1 in flight
    if (n_tiles > 0) loader.issue_all(tile0, s_idx, 0 >= first_masked_tile);
    if (n_tiles > 1) loader.issue_all(tile1, s_idx + TILE_ROWS, 1 >= first_masked_tile);

    // Q^T operand: lane holds Q[head0 + lane%32][16*ks + 8*(lane/32) .. +7]
    bf16x8 qreg[K_STEPS];
    {
        const __bf16* qrow = q + ((size_t)b * n_heads + head0 + (lane & 31)) * D_QK + 8 * (lane >> 5);
#pragma unroll
        for (int ks = 0; ks < K_STEPS; ++ks) {
            qreg[ks] = *reinterpret_cast<const bf16x8*>(qrow + 16 * ks);
        }
    }
    // Make the Q loads complete here, once (the empty asm statements are uses of the loaded
    // registers): a wait for them inside the tile loop would also wait, on every pass, for
    // the tile loads issued behind them.
#pragma unroll
    for (int ks = 0; ks < K_STEPS; ++ks) asm volatile("" : "+v"(qreg[ks]));

    floatx16 acc[DV_TILES];
#pragma unroll
    for (int t = 0; t < DV_TILES; ++t) acc[t] = floatx16{0};
    SoftmaxState st{-INFINITY, 0.f};
    const LaneOffsets off = make_lane_offsets(lane);

    // Three-stage ring. At the top of step t the loads of tiles t and t+1 are outstanding;
    // waiting until at most one tile's worth of loads is in flight therefore completes tile t.
    // (A tile with padding rows issues an unknown number of loads, so next to such a tile the
    // wait is for everything.) Tile t+2 is issued during step t, after the barrier, into the
    // buffer every wavefront finished reading in step t-1.
#define MLA_STEP(CUR, NXT2, T)                                                                  \
    {                                                                                           \
        if ((T) + 1 < n_tiles && (T) + 1 < first_masked_tile)                                   \
            wait_vmcnt<PER_WAVE>();                                                             \
        else                                                                                    \
            wait_all_memory();                                                                  \
        __builtin_amdgcn_s_barrier();                                                           \
        asm volatile("" ::: "memory");                                                          \
        const bool more = (T) + 2 < n_tiles;                                                    \
        const bool pad2 = (T) + 2 >= first_masked_tile;                                         \
        const int* idx2 = s_idx + ((T) + 2) * TILE_ROWS;                                        \
        process_tile<PER_WAVE>(CUR, s_idx + (T) * TILE_ROWS, (T) >= first_masked_tile, qreg, acc, \
                               st, off, scale_log2, lane, [&](int i) {                          \
                                   if (more) loader.issue(NXT2, idx2, pad2, i);                 \
                               });                                                              \
    }
    for (int t = 0; t < n_tiles; t += 3) {
        MLA_STEP(tile0, tile2, t)
        if (t + 1 < n_tiles) MLA_STEP(tile1, tile0, t + 1)
        if (t + 2 < n_tiles) MLA_STEP(tile2, tile1, t + 2)
    }
#undef MLA_STEP

    // Epilogue: normalise and write the partial output [b, split, head, dv] and the
    // log2-sum-exp. The accumulator is O^T (a lane holds 4 consecutive dv of one head, lanes
    // run over heads), so it goes through LDS, 128 dv at a time in a region private to the
    // wavefront, to leave as 512-byte row segments.
    const float l_total = st.l + __shfl_xor(st.l, 32);
    const float inv_l = l_total > 0.f ? 1.f / l_total : 0.f;
    const int half = lane >> 5;
    const size_t part0 = ((size_t)b * n_splits + split) * n_heads + head0;
    if (half == 0) {
        // v_log_f32 is a base-2 logarithm
        lse_part[part0 + lane] = l_total > 0.f ? st.m + __builtin_amdgcn_logf(l_total) : -INFINITY;
    }
    __syncthreads();  // every wavefront is done with the tile buffers
    constexpr int STAGE_STRIDE = 128 + 4;  // floats per staged head row (padded against conflicts)
    float* stage = reinterpret_cast<float*>(wave < 2 ? tile0 : tile1) + (wave & 1) * (32 * STAGE_STRIDE);
    float* o_rows = o_part + part0 * D_V;
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) {
            const floatx16 a = acc[4 * ps + tt];
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                floatx4 v = {a[4 * qd] * inv_l, a[4 * qd + 1] * inv_l, a[4 * qd + 2] * inv_l,
                             a[4 * qd + 3] * inv_l};
                *reinterpret_cast<floatx4*>(stage + (lane & 31) * STAGE_STRIDE + 32 * tt + 8 * qd +
                                            4 * half) = v;
            }
        }
#pragma unroll
        for (int it = 0; it < 16; ++it) {
            const int r = 2 * it + half;
            const floatx4 v = *reinterpret_cast<const floatx4*>(stage + r * STAGE_STRIDE + 4 * (lane & 31));
            *reinterpret_cast<floatx4*>(o_rows + (size_t)r * D_V + 128 * ps + 4 * (lane & 31)) = v;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// 128 heads per workgroup, 8 wavefronts (two per SIMD).
//
// The per-head-group state of the kernel above (Q: 144 registers, O^T: 256) fills a SIMD's
// whole register file with one wavefront, so nothing can overlap: MFMA, softmax arithmetic, LDS
// reads and the issue of the gather loads simply add up. Here each head group is a PAIR of
// wavefronts (w, w^1, on different SIMDs) that splits that state: each keeps alternating
// 32-element slices of d of Q (72 registers) and one half of dv of O^T (128 registers, ordinary
// VGPRs, so the running-max rescale is one multiply per register). Per 32-row tile a wavefront
// computes the partial scores of its d slices (18 MFMAs) into an exchange buffer in LDS; after a
// workgroup barrier both partners add the two partials in the same order, do the softmax on the
// full scores (bit-identical in both) and multiply P with their half of V^T (16 MFMAs). No MFMA
// is duplicated.
// Wavefronts 0-3 (lead) and 4-7 (lag; w and w+4 share a SIMD) run half a tile apart, so that on
// every SIMD one wavefront is in its QK^T half-step while the other is in its softmax/PV
// half-step. The lag group also gathers: each of its wavefronts loads 8 whole rows of a tile.
// Measured per wavefront and tile (core clock cycles, 16-tile splits): gather issue 2 000 (the
// memory pipeline accepts one 1 KB load of a wavefront per 150-300 cycles, whatever the
// addresses), QK^T 950-1 200, softmax + rescale 1 750-1 950, PV 650-900, barriers 500-2 800;
// the prologue (indices, Q, first tiles) is 10 us and the epilogue (131 KB of fp16 partials) 3 us.
// ---------------------------------------------------------------------------------------------
// Phase timing build (-DMLA_PHASE_TIMING): every wavefront of workgroup (0,0,0) adds up the core
// clock cycles it spends in each phase of the loop and leaves them in g_phase_cycles.
#ifdef MLA_PHASE_TIMING
__device__ unsigned long long g_phase_cycles[8][12];
#define PHASE_TIMING_BEGIN() unsigned long long phase_t0 = __builtin_readcyclecounter(), phase_acc[12] = {}
#define PHASE_MARK(n)                                                    \
    {                                                                    \
        const unsigned long long phase_now = __builtin_readcyclecounter(); \
        phase_acc[n] += phase_now - phase_t0;                            \
        phase_t0 = phase_now;                                            \
    }
#define PHASE_TIMING_END(wave, lane)                                                     \
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && (lane) == 0) {          \
        for (int i = 0; i < 11; ++i) g_phase_cycles[wave][i] = phase_acc[i];             \
        g_phase_cycles[wave][11] = __builtin_amdgcn_s_getreg((31 << 11) | 4); /* HW_ID */ \
    }
#else
#define PHASE_TIMING_BEGIN()
#define PHASE_MARK(n)
#define PHASE_TIMING_END(wave, lane)
#endif

constexpr int HALF_K_STEPS = K_STEPS / 2;   // 18
constexpr int HALF_DV_TILES = DV_TILES / 2;  // 8

// Gather of one tile by the four wavefronts of the lag group: wavefront `quarter` loads rows
// 8*quarter .. 8*quarter+7, which are 576 16-byte chunks = exactly 9 load instructions. `tab`
// holds, for chunk c = 64*i + lane of that span, (4 * (c / 72)) << 16 | byte offset of the
// swizzled source chunk within the row; it is the same for every tile and every wavefront.
// The loads address the request's cache block as 64-bit scalar base + 32-bit lane offset, so a
// prepared tile costs 9 registers; gather_prepare() reads table and indices for all nine loads
// at once, so that the nine address chains overlap.
constexpr int GATHER_INSTR = 9;
constexpr int GATHER_TAB = GATHER_INSTR * 64;
constexpr uint32_t GATHER_MASKED = 0xffffffffu;  // offset sentinel of a padding row

__device__ __forceinline__ void gather_prepare(uint32_t (&off)[GATHER_INSTR], const int* s_idx_tile,
                                               const uint32_t* tab, bool has_padding, int quarter, int lane) {
    const char* keys = reinterpret_cast<const char*>(s_idx_tile + 8 * quarter);
    uint32_t e[GATHER_INSTR];
#pragma unroll
    for (int i = 0; i < GATHER_INSTR; ++i) e[i] = tab[64 * i + lane];
#pragma unroll
    for (int i = 0; i < GATHER_INSTR; ++i) {
        const int key = *reinterpret_cast<const int*>(keys + (e[i] >> 16));
        off[i] = (uint32_t)key * (uint32_t)ROW_BYTES + ((e[i] & 0xffffu) ^ ((quarter & 1) << 5));
        if (has_padding && key < 0) off[i] = GATHER_MASKED;
    }
}

__device__ __forceinline__ void gather_issue(uint4* tile, const char* kv_b, uint32_t off, int i,
                                             bool has_padding, int quarter, int lane) {
    uint4* dst = tile + quarter * GATHER_TAB + i * 64;
    if (!has_padding || off != GATHER_MASKED) {
        const uint32_t lds_base = (uint32_t)(size_t)((lds_void_ptr)dst);
        // (non-temporal: a selected row is read once per launch; 66.6 -> 65.1 us per step)
        asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     :
                     : "v"(off), "s"(kv_b), "s"(lds_base)
                     : "memory", "m0");
    } else {
        dst[lane] = make_uint4(0u, 0u, 0u, 0u);
    }
}

// ---- e4m3 storage form of the cache (rows of 656 bytes: 512 codes, 4 fp32 scales, 64 bf16 rope values) ----
// A wavefront gathers the 8 rows of its quarter of a tile as 328 consecutive 16-byte chunks (row r at chunks
// 41*r .. 41*r + 40) at the start of the quarter's own region of the tile, with 6 load instructions of 64 lanes
// (the last one of 8): a load instruction costs the same to issue whether 41 or 64 of its lanes fetch. The same
// wavefront then reads all of it into registers (4 code chunks, their scales and one rope chunk per lane) and
// writes the 8 rows in the tile's bf16 layout over the region (a wavefront's LDS operations execute in order, and
// every read is issued before the first write). No LDS beyond the tile ring is needed.
constexpr int FP8_ROW_BYTES = 656;
constexpr int FP8_ROW_CHUNKS = FP8_ROW_BYTES / 16;  // 41
constexpr int FP8_STAGE_CHUNKS = 8 * FP8_ROW_CHUNKS;  // 328 chunks of a quarter
constexpr int FP8_GATHER_INSTR = (FP8_STAGE_CHUNKS + 63) / 64;  // 6

// quarter `quarter` of a tile. pad: the tile has padding entries (key < 0): their lanes fetch row 0, and the
// dequantisation writes zeros for them.
__device__ __forceinline__ void gather_quarter_fp8(uint4* tile, const char* kv_b, const int* s_idx_tile, bool pad,
                                                   int quarter, int lane) {
    // (the lane number is hidden from the optimiser: per-lane row and chunk numbers would otherwise be kept
    // across the tile loop, spilled, and a scratch reload in front of a load waits for all loads in flight)
    asm volatile("" : "+v"(lane));
    uint32_t off[FP8_GATHER_INSTR];
#pragma unroll
    for (int k = 0; k < FP8_GATHER_INSTR; ++k) {
        const int g = 64 * k + lane;       // chunk of the quarter
        int r = (g * 25) >> 10;            // g / 41 for g < 328
        r = r > 7 ? 7 : r;                 // (idle lanes of the last instruction)
        int key = s_idx_tile[8 * quarter + r];
        if (pad) key = key < 0 ? 0 : key;
        off[k] = (uint32_t)key * (uint32_t)FP8_ROW_BYTES + 16u * (uint32_t)(g - FP8_ROW_CHUNKS * r);
    }
    const uint32_t lds_base = (uint32_t)(size_t)((lds_void_ptr)(tile + 8 * quarter * ROW_CHUNKS));
#pragma unroll
    for (int k = 0; k < FP8_GATHER_INSTR; ++k) {
        if (64 * k + 64 <= FP8_STAGE_CHUNKS || lane < FP8_STAGE_CHUNKS - 64 * k) {
            asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                         :
                         : "v"(off[k]), "s"(kv_b), "s"(lds_base + 1024u * k)
                         : "memory", "m0");
        }
    }
}

// two e4m3 codes (one half of a dword) times a scale -> two bf16 (round to nearest even) in one dword
__device__ __forceinline__ uint32_t dequant_pair(uint32_t codes, bool upper, float scale) {
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const floatx2 f = upper ? __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, true)
                            : __builtin_amdgcn_cvt_pk_f32_fp8((int)codes, false);
    const bf16x2 r = {(__bf16)(f[0] * scale), (__bf16)(f[1] * scale)};
    return __builtin_bit_cast(uint32_t, r);
}

// the 8 rows of quarter `quarter` from the gathered form (see above) to the tile's bf16 layout, rows 4..7 first and
// then rows 0..3: the bf16 form of rows 4..7 (chunks 288..575 of the region) does not reach the gathered form of
// rows 0..3 (chunks 0..163), and within a step every read is issued before the first write. Codes: lanes 0-31
// take one row and lanes 32-63 the next; a lane converts 16 codes with the scale of their block of 128, read
// straight from the row's scale chunk. Rope values: 8 bytes per lane, row lane / 16 of the step.
__device__ __forceinline__ void dequant_quarter(uint4* tile, const int* s_idx_tile, bool pad, int quarter, int lane) {
    asm volatile("" : "+v"(lane));  // (as in gather_quarter_fp8)
    const int sub = lane & 31;
    const int x = 2 * sub;  // bf16 chunks 2*sub and 2*sub + 1 of the row
    const int hi = lane >> 5;
    const int piece = lane & 15;
    uint4* region = tile + 8 * quarter * ROW_CHUNKS;
#pragma unroll
    for (int step = 1; step >= 0; --step) {
        const int rope_row = 4 * step + (lane >> 4);
        uint4 c[2];
        float sc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint4* src = region + (4 * step + 2 * j + hi) * FP8_ROW_CHUNKS;
            c[j] = src[sub];
            sc[j] = reinterpret_cast<const float*>(src + 32)[sub >> 3];
        }
        uint2 rope = reinterpret_cast<const uint2*>(region + rope_row * FP8_ROW_CHUNKS + 33)[piece];
        if (pad) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t keep = s_idx_tile[8 * quarter + 4 * step + 2 * j + hi] < 0 ? 0u : ~0u;
                c[j].x &= keep, c[j].y &= keep, c[j].z &= keep, c[j].w &= keep;
            }
            const uint32_t keep = s_idx_tile[8 * quarter + rope_row] < 0 ? 0u : ~0u;
            rope.x &= keep, rope.y &= keep;
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = 4 * step + 2 * j + hi;
            uint4* slots = region + row * ROW_CHUNKS;
            const int swz = row_swizzle(8 * quarter + row);
            slots[(x & ~7) | ((x ^ swz) & 7)] =
                make_uint4(dequant_pair(c[j].x, false, sc[j]), dequant_pair(c[j].x, true, sc[j]),
                           dequant_pair(c[j].y, false, sc[j]), dequant_pair(c[j].y, true, sc[j]));
            slots[(x & ~7) | (((x + 1) ^ swz) & 7)] =
                make_uint4(dequant_pair(c[j].z, false, sc[j]), dequant_pair(c[j].z, true, sc[j]),
                           dequant_pair(c[j].w, false, sc[j]), dequant_pair(c[j].w, true, sc[j]));
        }
        reinterpret_cast<uint2*>(region + rope_row * ROW_CHUNKS + 64 +
                                 ((piece >> 1) ^ row_swizzle(8 * quarter + rope_row)))[piece & 1] = rope;
        __builtin_amdgcn_sched_barrier(0);
    }
}

// grid: x = split, y = request, z = group of 128 heads; 512 lanes. FP8: kv is a cache in the 656-byte e4m3 form.
template <bool FP8>
__global__ __launch_bounds__(512) void sparse_mla_split8_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ idx,
    _Float16* __restrict__ o_part, float* __restrict__ lse_part, float* __restrict__ scale_part,
    int n_heads, int n_kv_rows, int topk, int rows_per_split, float scale_log2, KvAddressing kva) {
    typedef const __attribute__((address_space(3))) uintx4* lds_x4;
    typedef shortx4 __attribute__((address_space(3)))* lds_s4;
    __shared__ uint4 tiles[3 * TILE_CHUNKS];  // ring of three resident tiles
    __shared__ floatx4 s_xchg[8][4 * 64];     // partial scores of every wavefront, 4 KB each
    __shared__ int s_idx[MAX_SPLIT_ROWS];
    __shared__ uint32_t s_gather_tab[GATHER_TAB];
    __shared__ float s_head_max[8][32];  // epilogue: largest |O^T| of every head in a wavefront's half
    __shared__ int s_first_masked_tile;

    PHASE_TIMING_BEGIN();
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // wavefronts w and w^1 are a pair (they sit on different SIMDs); wavefronts w and w+4 share
    // a SIMD and belong to the lead (0-3) and the lag (4-7) group
    const int dh = wave & 1;   // which slices of d (QK^T) and which half of dv (PV) this wavefront owns
    const int hg = wave >> 1;  // 32-head group
    const int group = wave >> 2;
    const int n_splits = gridDim.x;
    int split = blockIdx.x;
    int b = blockIdx.y;
    // Consecutive workgroup ids go round-robin to the 8 XCDs, each with its own L2. With the plain mapping the
    // splits of a request land on four XCDs and each of them fetches the request's 147 KB of Q; with a batch
    // that is a multiple of 8 the splits of request b all run on XCD b % 8 (one fetch of Q per XCD, and the
    // request's partials are written through one L2, where the merge kernel looks for them).
    if ((gridDim.y & 7) == 0) {
        const int linear = blockIdx.x + gridDim.x * blockIdx.y;
        const int j = linear >> 3;
        split = j % n_splits;
        b = (linear & 7) + 8 * (j / n_splits);
    }
    const int head0 = blockIdx.z * 128 + hg * 32;
    const int half = lane >> 5;

    const int row_begin = split * rows_per_split;
    int row_end = row_begin + rows_per_split;
    if (row_end > topk) row_end = topk;
    const int n_rows = row_end > row_begin ? row_end - row_begin : 0;
    const int n_tiles = (n_rows + TILE_ROWS - 1) / TILE_ROWS;

    // indices of the split first: everything else in the prologue queues up behind them
    int raw_key[MAX_SPLIT_ROWS / 512];
#pragma unroll
    for (int j = 0; j < MAX_SPLIT_ROWS / 512; ++j) {
        const int i = tid + 512 * j;
        raw_key[j] = i < n_rows ? idx[(size_t)b * topk + row_begin + i] : -1;
    }
    // Q^T operand of this wavefront's share of d: local step l is k-step 4*(l/2) + 2*dh + l%2,
    // i.e. the two wavefronts of a pair alternate 32-element slices of d. The wait for Q also
    // waits for the two tiles issued above (loads return in order), which the loop needs anyway.
    // (requested here, behind the indices: Q does not depend on them, so its latency overlaps theirs)
    // The loads take the wavefront's 64 bytes of every 128-byte line of Q from 16 rows per instruction
    // (lane -> row 16*(l&1) + lane/4, 16-byte piece lane%4 of line l/2: 16 line requests instead of the 32 that
    // loading the operand layout directly needs); the operand layout is made below through LDS.
    uintx4 qraw[HALF_K_STEPS];
    {
        const char* qsrc = reinterpret_cast<const char*>(q + ((size_t)b * n_heads + head0) * D_QK) +
                           (size_t)(lane >> 2) * ROW_BYTES + 64 * dh + 16 * (lane & 3);
#pragma unroll
        for (int l = 0; l < HALF_K_STEPS; ++l) {
            qraw[l] = *reinterpret_cast<const uintx4*>(qsrc + (size_t)(16 * (l & 1)) * ROW_BYTES + 128 * (l >> 1));
        }
    }
    if (kva.block_table != nullptr) {
#pragma unroll
        for (int j = 0; j < MAX_SPLIT_ROWS / 512; ++j)
            raw_key[j] = resolve_key(raw_key[j], b, kva, n_kv_rows);
    }
    if (tid == 0) s_first_masked_tile = n_tiles;
    for (int c = tid; c < (FP8 ? 0 : GATHER_TAB); c += 512) {  // (the e4m3 gather computes its offsets itself)
        const int row = c / ROW_CHUNKS;  // 0..7; the tile row is 8*quarter + row: for odd quarters the
        const int pos = c - row * ROW_CHUNKS;  // swizzle term has bit 1 flipped (gather_prepare)
        const int chunk = (pos & ~7) | ((pos ^ row_swizzle(row)) & 7);
        s_gather_tab[c] = ((uint32_t)(4 * row) << 16) | (uint32_t)(chunk * 16);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < MAX_SPLIT_ROWS / 512; ++j) {
        const int i = tid + 512 * j;
        if (i < n_tiles * TILE_ROWS) {
            int key = raw_key[j];
            if (key < 0 || key >= n_kv_rows) {
                key = -1;
                atomicMin(&s_first_masked_tile, i / TILE_ROWS);
            }
            s_idx[i] = key;
        }
    }
    __syncthreads();
    const int first_masked_tile = s_first_masked_tile;
    const char* kv_b = reinterpret_cast<const char*>(kv) + (size_t)b * kva.batch_rows * (FP8 ? FP8_ROW_BYTES : ROW_BYTES);
    PHASE_MARK(7);  // index staging

    // The first two tiles are on their way before Q is fetched: tile 0 by the lead group, tile 1
    // by the lag group (a cold load instruction takes several hundred cycles to issue, so the
    // two groups share the work; from tile 2 on the lag group gathers alone).
    if (group < n_tiles) {
        if constexpr (FP8) {
            gather_quarter_fp8(tiles + group * TILE_CHUNKS, kv_b, s_idx + group * TILE_ROWS, group >= first_masked_tile,
                               wave & 3, lane);
        } else {
            uint32_t off[GATHER_INSTR];
            const bool pad = group >= first_masked_tile;
            gather_prepare(off, s_idx + group * TILE_ROWS, s_gather_tab, pad, wave & 3, lane);
#pragma unroll
            for (int i = 0; i < GATHER_INSTR; ++i) {
                gather_issue(tiles + group * TILE_CHUNKS, kv_b, off[i], i, pad, wave & 3, lane);
            }
        }
    }
    PHASE_MARK(9);  // first gather issue

    // Q into operand layout (lane = head lane%32, 16-byte piece 2*(l&1) + half of line l/2), one line of the
    // 32 heads at a time through this wavefront's exchange buffer, which the loop does not use yet: rows of
    // 64 bytes, piece p of row r at slot p ^ ((r >> 2) & 3) so that the 16 rows a read serves per cycle hit
    // 16 different bank groups. No barrier: the LDS operations of a wavefront execute in order.
    bf16x8 qreg[HALF_K_STEPS];
    {
        uintx4* stage = reinterpret_cast<uintx4*>(&s_xchg[wave][0]);
        const int r = lane & 31;
#pragma unroll
        for (int j = 0; j < HALF_K_STEPS / 2; ++j) {
#pragma unroll
            for (int sl = 0; sl < 2; ++sl) {
                const int wr = 16 * sl + (lane >> 2);
                stage[wr * 4 + ((lane & 3) ^ ((wr >> 2) & 3))] = qraw[2 * j + sl];
            }
#pragma unroll
            for (int sl = 0; sl < 2; ++sl) {
                qreg[2 * j + sl] = __builtin_bit_cast(bf16x8, stage[r * 4 + ((2 * sl + half) ^ ((r >> 2) & 3))]);
            }
        }
    }
#pragma unroll
    for (int ks = 0; ks < HALF_K_STEPS; ++ks) asm volatile("" : "+v"(qreg[ks]));
    PHASE_MARK(8);  // wait for Q

    floatx16 acc[HALF_DV_TILES];
#pragma unroll
    for (int t = 0; t < HALF_DV_TILES; ++t) acc[t] = floatx16{0};
    SoftmaxState st{-INFINITY, 0.f};
    const LaneOffsets off = make_lane_offsets(lane);
    // K operand of local step l: qk_l[l & 1] + (l >> 1) * 128
    // V^T operand of local dv tile tl: (pv_l[tl & 1] ^ 32*rr) + (16*ks + 8*rr) * ROW_BYTES + (tl >> 1) * 128
    const uint32_t qk_l[2] = {dh ? off.qk[2] : off.qk[0], dh ? off.qk[3] : off.qk[1]};
    const uint32_t pv_l[2] = {off.pv[0] + 512u * dh, off.pv[1] + 512u * dh};
    floatx4* my_xchg = &s_xchg[wave][0];
    const floatx4* pair_xchg = &s_xchg[wave & ~1][0];  // d-slices 0 partial, then d-slices 1 partial

    // The loop runs in half-steps with one workgroup barrier each. A wavefront alternates between
    // a QK^T half-step (partial scores of one tile into its exchange buffer) and a softmax + PV
    // half-step (which starts by reading both partners' partials, so the exchange crosses exactly
    // one barrier). The lag group runs one half-step behind the lead group: on every SIMD one
    // wavefront is in its MFMA-bound phase while the other is in its VALU-bound phase.
    //   half-step h, lead: h even -> QK^T(h/2), h odd -> softmax/PV((h-1)/2)
    //                lag:  h odd  -> QK^T((h-1)/2), h even -> softmax/PV(h/2 - 1)
    // Tile t is last read in half-step 2t+2, so its ring slot is refilled (tile t+3) after the
    // barrier of half-step 2t+3.
    for (int h = 0; h <= 2 * n_tiles; ++h) {
        PHASE_MARK(6);
        if ((h & 1) == 0 && h < 2 * n_tiles) {
            // tile h/2 must be resident: everything but this wavefront's share of the next tile
            const int t = h >> 1;
            if constexpr (FP8) {
                // tile 0 was gathered by the lead group: it turns its rows into bf16 here, before the barrier
                // below hands the tile to everyone; every later tile is converted by the lag group inside the
                // half-step before (see there)
                if (h == 0 && group == 0) {
                    wait_all_memory();
                    asm volatile("" ::: "memory");  // the reads below stay behind the wait above
                    dequant_quarter(tiles, s_idx, 0 >= first_masked_tile, wave & 3, lane);
                }
            } else {
                const bool plain_wait = t + 1 < n_tiles && t + 1 < first_masked_tile;
                if (plain_wait) {
                    wait_vmcnt<GATHER_INSTR>();  // (the lead group has no loads in flight)
                } else {
                    wait_all_memory();
                }
            }
        }
        __builtin_amdgcn_s_waitcnt((63 & 15) | ((63 >> 4) << 14) | (7 << 4) | (0 << 8));  // lgkmcnt(0)
        PHASE_MARK(0);  // wait for this wavefront's own gather loads and LDS stores
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        PHASE_MARK(1);  // wait for the other wavefronts
        // the lag group's QK^T half-steps (odd h) also gather tile (h-1)/2 + 2 into the slot
        // that tile (h-1)/2 - 1 has left after the barrier above
        const int t2 = (h >> 1) + 2;
        const bool gather = (h & 1) && group == 1 && t2 < n_tiles;
        const bool gather_pad = t2 >= first_masked_tile;
        uint4* gather_tile = tiles + ((gather ? t2 : 0) % 3) * TILE_CHUNKS;
        const int mine = h - group;  // this wavefront's own half-step counter
        const int t = mine >> 1;
        const bool active = mine >= 0 && t < n_tiles;
        const lds_bytes base = (lds_bytes)(tiles + ((active ? t : 0) % 3) * TILE_CHUNKS);

        if (active && (mine & 1) == 0) {
            // partial S^T over this wavefront's slices of d
            floatx16 s = {0};
            // Gather of tile t2 first: the memory pipeline takes the nine loads of a wavefront
            // at one per ~150 cycles whether or not MFMAs are issued in between (measured), so
            // they go out back to back and the QK^T loop stays free of them.
            if (gather) {
                if constexpr (FP8) {
                    gather_quarter_fp8(gather_tile, kv_b, s_idx + t2 * TILE_ROWS, gather_pad, wave & 3, lane);
                } else {
                    uint32_t goff[GATHER_INSTR];
                    gather_prepare(goff, s_idx + t2 * TILE_ROWS, s_gather_tab, gather_pad, wave & 3, lane);
#pragma unroll
                    for (int i = 0; i < GATHER_INSTR; ++i) {
                        gather_issue(gather_tile, kv_b, goff[i], i, gather_pad, wave & 3, lane);
                    }
                }
            }
            PHASE_MARK(2);  // gather issue
            uintx4 kbuf[3];  // K operands are read two MFMAs ahead
            auto k_read = [&](int l) { kbuf[l % 3] = *(lds_x4)(base + qk_l[l & 1] + (l >> 1) * 128); };
            k_read(0);
            k_read(1);
#pragma unroll
            for (int l = 0; l < HALF_K_STEPS; ++l) {
                if (l + 2 < HALF_K_STEPS) k_read(l + 2);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kbuf[l % 3]), qreg[l], s,
                                                            0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                my_xchg[qd * 64 + lane] = floatx4{s[4 * qd], s[4 * qd + 1], s[4 * qd + 2], s[4 * qd + 3]};
            }
            __builtin_amdgcn_sched_barrier(0);  // (the scores leave their registers before the conversion needs them)
            if constexpr (FP8) {
                // the lag group gathered tile t + 1 two half-steps ago: its rows become bf16 here, next to the lead
                // group's softmax and P V of tile t, and the next barrier hands the tile to everyone
                if (group == 1 && t + 1 < n_tiles) {
                    if (gather) {
                        wait_vmcnt<FP8_GATHER_INSTR>();  // all but the loads of tile t + 2 issued above
                    } else {
                        wait_all_memory();
                    }
                    asm volatile("" ::: "memory");  // the reads below stay behind the wait above
                    dequant_quarter(tiles + ((t + 1) % 3) * TILE_CHUNKS, s_idx + (t + 1) * TILE_ROWS,
                                    t + 1 >= first_masked_tile, wave & 3, lane);
                }
            }
            PHASE_MARK(3);  // QK^T
        }
        if (!(active && (mine & 1) == 1)) continue;

        // full scores = partial of d-slices 0 + partial of d-slices 1, in that order in both
        // partners, so that they compute bit-identical probabilities
        const int* s_idx_tile = s_idx + t * TILE_ROWS;
        floatx16 s;
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            const floatx4 lo = pair_xchg[qd * 64 + lane];
            const floatx4 hi = pair_xchg[4 * 64 + qd * 64 + lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) s[4 * qd + r] = (lo[r] + hi[r]) * scale_log2;
        }

        // softmax on the tile's scores; register i of `s` is row 8*(i/4) + 4*half + i%4
        float tmax = -INFINITY;
        if (t >= first_masked_tile) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int row = 8 * (i / 4) + 4 * half + (i % 4);
                if (s_idx_tile[row] < 0) s[i] = -INFINITY;
            }
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) tmax = fmaxf(tmax, s[i]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const bool move = tmax > st.m + FRAME_SLACK || st.m == -INFINITY;
        const float m_new = move ? tmax : st.m;
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = move ? __builtin_amdgcn_exp2f(st.m - m_use) : 1.f;
        const bool rescale = move && st.l != 0.f;
        st.m = m_new;
        float psum = 0.f;
        bf16x8 p[2];
#pragma unroll
        for (int i = 0; i < 16; ++i) p[i / 8][i % 8] = (__bf16)__builtin_amdgcn_exp2f(s[i] - m_use);
        // the normaliser sums the probabilities as rounded (see process_tile); v_dot2c_f32_bf16 adds two of
        // them per instruction
        {
            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
            const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                const bf16x2 pair = {p[i / 8][i % 8], p[i / 8][i % 8 + 1]};
                psum = __builtin_amdgcn_fdot2_f32_bf16(pair, ones, psum, false);
            }
        }
        st.l = st.l * alpha + psum;
        if (__builtin_amdgcn_ballot_w64(rescale) != 0) {
#pragma unroll
            for (int tt = 0; tt < HALF_DV_TILES; ++tt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) acc[tt][i] *= alpha;
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        PHASE_MARK(4);  // exchange read, softmax, rescale

        // O^T[dv half] += V^T P^T
        shortx4 vbuf[2][2][2];
        auto pv_read = [&](int stepi, shortx4 (&dst)[2][2]) {
            // two MFMAs per group: (ks, dv tile) = stepi*2, stepi*2+1 in (ks major) order
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int idx2 = stepi * 2 + j;
                const int ks = idx2 / HALF_DV_TILES;
                const int tl = idx2 % HALF_DV_TILES;
#pragma unroll
                for (int rr = 0; rr < 2; ++rr) {
                    dst[j][rr] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (lds_s4)(base + (pv_l[tl & 1] ^ (32 * rr)) + (16 * ks + 8 * rr) * ROW_BYTES + (tl >> 1) * 128));
                }
            }
        };
        pv_read(0, vbuf[0]);
#pragma unroll
        for (int g = 0; g < HALF_DV_TILES; ++g) {  // 8 groups of 2 MFMAs
            if (g + 1 < HALF_DV_TILES) pv_read(g + 1, vbuf[(g + 1) & 1]);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int idx2 = g * 2 + j;
                const int ks = idx2 / HALF_DV_TILES;
                const int tl = idx2 % HALF_DV_TILES;
                const bf16x4 lo = __builtin_bit_cast(bf16x4, vbuf[g & 1][j][0]);
                const bf16x4 hi = __builtin_bit_cast(bf16x4, vbuf[g & 1][j][1]);
                const bf16x8 a = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                acc[tl] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, p[ks], acc[tl], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        PHASE_MARK(5);  // PV
    }

    // epilogue: normalise; O^T half -> LDS (64 dv at a time, region private to the wavefront)
    // -> 128-byte row segments of the partial output. The partial is stored as fp16 of
    // O / 2^e with 2^e the power of two above the head's largest magnitude (kept next to the
    // log-sum-exp): half the bytes of fp32 for the split kernel to write and the merge to read, and
    // an error of at most 2^-12 of that magnitude.
    const float l_total = st.l + __shfl_xor(st.l, 32);
    const float inv_l = l_total > 0.f ? 1.f / l_total : 0.f;
    const size_t part0 = ((size_t)b * n_splits + split) * n_heads + head0;
    float amax = 0.f;
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(acc[t][i]));
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    if (half == 0) s_head_max[wave][lane] = amax;
    if (dh == 0 && half == 0) {
        lse_part[part0 + lane] = l_total > 0.f ? st.m + __builtin_amdgcn_logf(l_total) : -INFINITY;
    }
    __syncthreads();
    // exponent field of the bound + 1: 2^e > |O| for every element of the head (1 if the head is 0)
    const float bound = fmaxf(s_head_max[wave][lane & 31], s_head_max[wave ^ 1][lane & 31]) * inv_l;
    uint32_t e_bits = ((__float_as_uint(bound) >> 23) & 255u) + 1u;
    e_bits = bound > 0.f ? (e_bits > 253u ? 253u : e_bits) : 127u;
    const float inv_scale = __uint_as_float((254u - e_bits) << 23) * inv_l;
    if (dh == 0 && half == 0) scale_part[part0 + lane] = __uint_as_float(e_bits << 23);
    constexpr int STAGE_STRIDE = 64 + 4;
    float* stage = reinterpret_cast<float*>(tiles + (wave >> 2) * TILE_CHUNKS) + (wave & 3) * (32 * STAGE_STRIDE);
    _Float16* o_rows = o_part + part0 * D_V + 256 * dh;
    typedef _Float16 halfx4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            const floatx16 a = acc[2 * ps + tt];
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                floatx4 v = {a[4 * qd] * inv_scale, a[4 * qd + 1] * inv_scale, a[4 * qd + 2] * inv_scale,
                             a[4 * qd + 3] * inv_scale};
                *reinterpret_cast<floatx4*>(stage + (lane & 31) * STAGE_STRIDE + 32 * tt + 8 * qd +
                                            4 * half) = v;
            }
        }
#pragma unroll
        for (int it = 0; it < 8; ++it) {
            const int r = 4 * it + (lane >> 4);
            const floatx4 v = *reinterpret_cast<const floatx4*>(stage + r * STAGE_STRIDE + 4 * (lane & 15));
            const halfx4 h = {(_Float16)v.x, (_Float16)v.y, (_Float16)v.z, (_Float16)v.w};
            *reinterpret_cast<halfx4*>(o_rows + (size_t)r * D_V + 64 * ps + 4 * (lane & 15)) = h;
        }
    }
    PHASE_MARK(10);  // epilogue
    PHASE_TIMING_END(wave, lane);
}

// out[b, h, :] = sum_s w_s o_part[b, s, h, :],  w_s = exp2(lse_s - max) / sum. One wavefront per
// (b, h), 8 output columns per lane, 4 heads per workgroup (grid x = n_heads / 4, y = request): the
// rows of all splits are requested before the first is used. PART is the type the split kernel
// stored: float, or fp16 of O / scale with the per-head scale in scale_part.
// BATCH = splits whose rows a lane requests at once.
template <typename OUT, typename PART, int BATCH>
__global__ __launch_bounds__(256) void sparse_mla_merge_kernel(const PART* __restrict__ o_part,
                                                               const float* __restrict__ lse_part,
                                                               const float* __restrict__ scale_part,
                                                               OUT* __restrict__ out, int n_heads,
                                                               int n_splits) {
    typedef PART partx8 __attribute__((ext_vector_type(8)));
    typedef float floatx8 __attribute__((ext_vector_type(8)));
    const int lane = threadIdx.x & 63;
    int hg = blockIdx.x;
    int b = blockIdx.y;
    // request b on XCD b % 8, where the split kernel wrote its partials (see there)
    if ((gridDim.y & 7) == 0) {
        const int linear = blockIdx.x + gridDim.x * blockIdx.y;
        const int j = linear >> 3;
        hg = j % (int)gridDim.x;
        b = (linear & 7) + 8 * (j / (int)gridDim.x);
    }
    const int h = hg * 4 + (threadIdx.x >> 6);
    const size_t base = (size_t)b * n_splits * n_heads + h;
    floatx8 o = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float wsum = 0.f;
    partx8 rows[BATCH];
    auto load_rows = [&](int s0) {
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
            // (splits past the end repeat the last one; their weight is 0)
            const int s = s0 + j < n_splits ? s0 + j : n_splits - 1;
            rows[j] = __builtin_nontemporal_load(
                reinterpret_cast<const partx8*>(o_part + (base + (size_t)s * n_heads) * D_V) + lane);
        }
    };
    // the first rows are requested before anything depends on the log-sum-exps
    load_rows(0);
    float mx = -INFINITY;
    for (int s = 0; s < n_splits; ++s) mx = fmaxf(mx, lse_part[base + (size_t)s * n_heads]);
    for (int s0 = 0; s0 < n_splits; s0 += BATCH) {
        if (s0 > 0) load_rows(s0);
        float w[BATCH], sc[BATCH];
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
            const int s = s0 + j < n_splits ? s0 + j : n_splits - 1;
            const size_t row = base + (size_t)s * n_heads;
            // (mx = -inf: every split is empty, all weights 0)
            w[j] = s0 + j < n_splits && mx > -INFINITY ? __builtin_amdgcn_exp2f(lse_part[row] - mx) : 0.f;
            sc[j] = 1.f;
            if constexpr (sizeof(PART) == 2) sc[j] = scale_part[row];
        }
#pragma unroll
        for (int j = 0; j < BATCH; ++j) {
            if (w[j] > 0.f) {  // (a split without rows has weight 0 and is not looked at)
                const float ws = w[j] * sc[j];  // sc is a power of two
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] += (float)rows[j][i] * ws;
                wsum += w[j];
            }
        }
    }
    if (wsum > 0.f) o *= 1.f / wsum;
    OUT* dst = out + ((size_t)b * n_heads + h) * D_V + lane * 8;
    if constexpr (sizeof(OUT) == 4) {
        reinterpret_cast<floatx4*>(dst)[0] = floatx4{o[0], o[1], o[2], o[3]};
        reinterpret_cast<floatx4*>(dst)[1] = floatx4{o[4], o[5], o[6], o[7]};
    } else {
        const bf16x8 r = {(__bf16)o[0], (__bf16)o[1], (__bf16)o[2], (__bf16)o[3],
                          (__bf16)o[4], (__bf16)o[5], (__bf16)o[6], (__bf16)o[7]};
        *reinterpret_cast<bf16x8*>(dst) = r;
    }
}

int pick_splits(int batch, int head_groups, int topk, int config) {
    const int tiles = (topk + TILE_ROWS - 1) / TILE_ROWS;
    int splits = config > 0 ? config : 0;
    if (splits == 0) {
        // fill the 256 CUs once (one resident workgroup per CU)
        const int wgs = batch * head_groups;
        splits = (256 + wgs - 1) / wgs;
    }
    const int min_splits = (topk + MAX_SPLIT_ROWS - 1) / MAX_SPLIT_ROWS;
    if (splits < min_splits) splits = min_splits;
    if (splits > tiles) splits = tiles;
    if (splits < 1) splits = 1;
    return splits;
}

}  // namespace

extern "C" int sparse_mla_decode_num_splits(int batch, int n_heads, int topk, int config) {
    if (batch <= 0 || n_heads <= 0 || topk <= 0) return 0;
    if (config >= 1000) config -= 1000;  // 1000 + n: n splits on the one-wavefront-per-head-group kernel
    const int head_groups = n_heads <= 128 ? 1 : n_heads / 128;
    return pick_splits(batch, head_groups, topk, config);
}

// bytes of scratch sparse_mla_decode_launcher needs for these sizes
extern "C" size_t sparse_mla_decode_workspace_bytes(int batch, int n_heads, int topk, int config) {
    const int splits = sparse_mla_decode_num_splits(batch, n_heads, topk, config);
    // partial outputs (sized for fp32), log-sum-exp and scale of every (request, split, head)
    return (size_t)batch * splits * n_heads * (D_V + 2) * sizeof(float);
}

namespace {

// shared by the two launchers: n_kv_rows is the number of rows of the block a request's keys
// resolve into (the request's own cache, or the whole pool)
// fp8_cache: kv is in the 656-byte e4m3 form, which only the 128-head kernel reads (the caller has checked
// the shape with fp8_cache_fused_ok)
void launch_sparse_mla(void* out, const void* q, const void* kv, const int* idx, void* workspace,
                       size_t workspace_bytes, int batch, int n_heads, int n_kv_rows, int topk,
                       int d_qk, int d_v, float sm_scale, int out_dtype, int config,
                       const KvAddressing& kva, hipStream_t stream, bool fp8_cache = false) {
    if (batch <= 0 || n_heads <= 0 || topk <= 0) return;
    const bool heads_ok = n_heads == 32 || n_heads == 64 || (n_heads % 128 == 0);
    if (d_qk != D_QK || d_v != D_V || !heads_ok || n_kv_rows <= 0 || batch > 65535 ||
        (out_dtype != 0 && out_dtype != 1) ||
        n_heads / 128 > 65535) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    const uintptr_t bits = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(q) |
                           reinterpret_cast<uintptr_t>(kv) | reinterpret_cast<uintptr_t>(workspace);
    if (!out || !q || !kv || !idx || !workspace || (bits & 15u) != 0) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    if (workspace_bytes < sparse_mla_decode_workspace_bytes(batch, n_heads, topk, config)) {
        caa::set_status(CAA_WORKSPACE_TOO_SMALL);
        return;
    }
    // config >= 1000: the one-wavefront-per-SIMD kernel for 128 heads (config - 1000 is then the
    // split count)
    // The 8-wavefront kernel addresses a request's cache block with 32-bit byte offsets.
    const bool four_wave_kernel =
        config >= 1000 ||
        (unsigned long long)n_kv_rows * (fp8_cache ? FP8_ROW_BYTES : ROW_BYTES) >= 0xffffffffull;
    if (config >= 1000) config -= 1000;
    const int head_groups = n_heads <= 128 ? 1 : n_heads / 128;
    const int splits = pick_splits(batch, head_groups, topk, config);
    const int tiles = (topk + TILE_ROWS - 1) / TILE_ROWS;
    const int rows_per_split = ((tiles + splits - 1) / splits) * TILE_ROWS;
    float* o_part = static_cast<float*>(workspace);
    float* lse_part = o_part + (size_t)batch * splits * n_heads * D_V;
    float* scale_part = lse_part + (size_t)batch * splits * n_heads;
    const float scale_log2 = sm_scale * 1.4426950408889634f;
    const __bf16* qb = static_cast<const __bf16*>(q);
    const __bf16* kvb = static_cast<const __bf16*>(kv);
    const dim3 grid(splits, batch, head_groups);
    const dim3 merge_grid(n_heads / 4, batch);
    bool half_parts = false;
    if (n_heads == 32) {
        sparse_mla_split_kernel<1><<<grid, 64, 0, stream>>>(qb, kvb, idx, o_part, lse_part, n_heads,
                                                            n_kv_rows, topk, rows_per_split,
                                                            scale_log2, kva);
    } else if (n_heads == 64) {
        sparse_mla_split_kernel<2><<<grid, 128, 0, stream>>>(qb, kvb, idx, o_part, lse_part, n_heads,
                                                             n_kv_rows, topk, rows_per_split,
                                                             scale_log2, kva);
    } else if (four_wave_kernel) {
        sparse_mla_split_kernel<4><<<grid, 256, 0, stream>>>(qb, kvb, idx, o_part, lse_part, n_heads,
                                                             n_kv_rows, topk, rows_per_split,
                                                             scale_log2, kva);
    } else {
        half_parts = true;  // this kernel stores its partials as scaled fp16
        if (fp8_cache) {
            sparse_mla_split8_kernel<true><<<grid, 512, 0, stream>>>(
                qb, kvb, idx, reinterpret_cast<_Float16*>(o_part), lse_part, scale_part, n_heads, n_kv_rows,
                topk, rows_per_split, scale_log2, kva);
        } else {
            sparse_mla_split8_kernel<false><<<grid, 512, 0, stream>>>(
                qb, kvb, idx, reinterpret_cast<_Float16*>(o_part), lse_part, scale_part, n_heads, n_kv_rows,
                topk, rows_per_split, scale_log2, kva);
        }
    }
    // rows requested at once per lane: as many as there are splits, up to 8
#define MLA_MERGE(OUT_T, PART_T, PARTS, SCALES)                                                   \
    if (splits <= 2)                                                                              \
        sparse_mla_merge_kernel<OUT_T, PART_T, 2><<<merge_grid, 256, 0, stream>>>(                \
            PARTS, lse_part, SCALES, static_cast<OUT_T*>(out), n_heads, splits);                  \
    else if (splits <= 4)                                                                         \
        sparse_mla_merge_kernel<OUT_T, PART_T, 4><<<merge_grid, 256, 0, stream>>>(                \
            PARTS, lse_part, SCALES, static_cast<OUT_T*>(out), n_heads, splits);                  \
    else                                                                                          \
        sparse_mla_merge_kernel<OUT_T, PART_T, 8><<<merge_grid, 256, 0, stream>>>(                \
            PARTS, lse_part, SCALES, static_cast<OUT_T*>(out), n_heads, splits);
    if (half_parts) {
        const _Float16* parts = reinterpret_cast<const _Float16*>(o_part);
        if (out_dtype == 0) {
            MLA_MERGE(__bf16, _Float16, parts, scale_part)
        } else {
            MLA_MERGE(float, _Float16, parts, scale_part)
        }
    } else if (out_dtype == 0) {
        MLA_MERGE(__bf16, float, o_part, nullptr)
    } else {
        MLA_MERGE(float, float, o_part, nullptr)
    }
#undef MLA_MERGE
}

}  // namespace

// out  [batch, n_heads, 512], written; bf16 if out_dtype == 0 (the operator's output type),
//      fp32 if out_dtype == 1 (the same values before the final rounding, for measuring
//      arithmetic error apart from output rounding)
// q    [batch, n_heads, 576] bf16
// kv   [batch, n_kv_rows, 576] bf16 (latent cache: 512 latent + 64 rope dims per row)
// idx  [batch, topk] int32 row numbers into the request's cache; values < 0 or >= n_kv_rows
//      are padding and take no part in the softmax
// workspace: sparse_mla_decode_workspace_bytes(...) bytes of device scratch, 16-byte aligned
// config: 0 picks the number of key splits so that one workgroup per CU is resident;
//         n > 0 forces n splits.
extern "C" void sparse_mla_decode_launcher(void* out, const void* q, const void* kv, const int* idx,
                                           void* workspace, size_t workspace_bytes, int batch,
                                           int n_heads, int n_kv_rows, int topk, int d_qk, int d_v,
                                           float sm_scale, int out_dtype, int config,
                                           hipStream_t stream) {
    const KvAddressing kva{nullptr, 0, 0, n_kv_rows};
    launch_sparse_mla(out, q, kv, idx, workspace, workspace_bytes, batch, n_heads, n_kv_rows, topk,
                      d_qk, d_v, sm_scale, out_dtype, config, kva, stream);
}

// The same attention over a paged latent cache: one pool of pages shared by all requests.
// kv_pool     [n_pages, page_size, 576] bf16, page_size a power of two
// block_table [batch, max_pages_per_request] int32: physical page of each logical page of a
//             request, negative where no page is mapped; or null
// idx         [batch, topk] int32. With a block table: logical positions of the request
//             (position p is row p % page_size of page block_table[b][p / page_size]). Without:
//             rows of the pool, page * page_size + row, as an indexer that already works on
//             physical rows hands them over. Negative entries, positions beyond the block
//             table, unmapped pages and rows beyond the pool are padding.
// Everything else as sparse_mla_decode_launcher; the workspace size is the same function of
// (batch, n_heads, topk, config).
extern "C" void sparse_mla_decode_paged_launcher(void* out, const void* q, const void* kv_pool,
                                                 const int* block_table, const int* idx,
                                                 void* workspace, size_t workspace_bytes, int batch,
                                                 int n_heads, int n_pages, int page_size,
                                                 int max_pages_per_request, int topk, int d_qk,
                                                 int d_v, float sm_scale, int out_dtype, int config,
                                                 hipStream_t stream) {
    if (batch <= 0 || n_heads <= 0 || topk <= 0) return;
    if (n_pages <= 0 || page_size <= 0 || (page_size & (page_size - 1)) != 0 ||
        (long long)n_pages * page_size > 0x7fffffffll ||
        (block_table != nullptr && max_pages_per_request <= 0)) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    const KvAddressing kva{block_table, max_pages_per_request, page_shift, 0};
    launch_sparse_mla(out, q, kv_pool, idx, workspace, workspace_bytes, batch, n_heads,
                      n_pages * page_size, topk, d_qk, d_v, sm_scale, out_dtype, config, kva, stream);
}

// ---- the entry point that allocates nothing ------------------------------------------------------------------
// Scratch of sparse_mla_decode_static_launcher: the partial outputs of the key splits live in this array of the
// library's own instead of in a caller-provided workspace. Every GPU the library runs on holds one copy from
// module load to process end. 72 MiB covers 64 requests x 128 heads x 2048 selected rows in 4 splits
// (67 371 008 bytes) with some room.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)72 << 20;
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

namespace {

constexpr int MAX_SCRATCH_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[MAX_SCRATCH_DEVICES];  // device address of `scratch` on every device, once known

// Device address of this device's copy of `scratch` (the array's name is a host-side stand-in, not an address a
// kernel could use). Looked up once per device, with that device current; null on failure.
void* static_scratch() {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= MAX_SCRATCH_DEVICES) return nullptr;
    void* ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return nullptr;
        g_scratch_ptr[device].store(ptr, std::memory_order_release);  // (a concurrent first call stores the same value)
    }
    return ptr;
}

}  // namespace

// sparse_mla_decode_launcher for callers that cannot allocate device memory (code under HIP graph capture,
// serving loops with a fixed memory plan, harnesses that forbid it): same arguments without the workspace, same
// kernels, same result bit for bit. The split partials go to a static device array of STATIC_SCRATCH_BYTES.
// Limits and rules that follow from that:
//   * sparse_mla_decode_workspace_bytes(batch, n_heads, topk, config) must not exceed
//     sparse_mla_decode_static_scratch_bytes(); a larger problem is rejected (status CAA_SCRATCH_LIMIT) and
//     nothing is launched;
//   * all calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two
//     threads) race; calls on one stream are ordered and safe. Nothing in the array has to start at zero (every
//     partial the merge reads was written by the split kernel of the same call), so it is never cleared;
//   * the first call on a device looks up the array's device address (hipGetSymbolAddress): make that call
//     outside a graph capture. No call allocates or frees memory.
extern "C" size_t sparse_mla_decode_static_scratch_bytes(void) { return STATIC_SCRATCH_BYTES; }

extern "C" void sparse_mla_decode_static_launcher(void* out, const void* q, const void* kv, const int* idx,
                                                  int batch, int n_heads, int n_kv_rows, int topk, int d_qk,
                                                  int d_v, float sm_scale, int out_dtype, int config,
                                                  hipStream_t stream) {
    if (batch <= 0 || n_heads <= 0 || topk <= 0) return;
    if (sparse_mla_decode_workspace_bytes(batch, n_heads, topk, config) > STATIC_SCRATCH_BYTES) {
        caa::set_status(CAA_SCRATCH_LIMIT);
        return;
    }
    void* ptr = static_scratch();
    if (ptr == nullptr) {
        caa::set_status(CAA_RUNTIME_ERROR);
        return;
    }
    const KvAddressing kva{nullptr, 0, 0, n_kv_rows};
    launch_sparse_mla(out, q, kv, idx, ptr, STATIC_SCRATCH_BYTES, batch, n_heads, n_kv_rows, topk, d_qk, d_v,
                      sm_scale, out_dtype, config, kva, stream);
}

// Decode over a cache in the 656-byte e4m3 form with the dequantisation inside the 128-head kernel (see
// gather_quarter_fp8 / dequant_quarter). Internal to the library: mla_fp8_cache.hip calls it from
// sparse_mla_decode_fp8_launcher and its paged form; it is not part of the public header. Returns 1 if the launch was made (or rejected with a status), 0 if
// this shape has to take the two-step form of sparse_mla_decode_fp8_launcher: head counts other than
// multiples of 128, config >= 1000, caches of 4 GB and more per addressed block.
// block_table / table_stride / page_shift / batch_rows: the addressing of the cache, as in KvAddressing.
extern "C" int sparse_mla_decode_fp8_fused(void* out, const void* q, const void* kv_fp8, const int* idx,
                                           void* workspace, size_t workspace_bytes, int batch, int n_heads,
                                           int n_kv_rows, int topk, int d_qk, int d_v, float sm_scale,
                                           int out_dtype, int config, const int* block_table,
                                           int table_stride, int page_shift, int batch_rows,
                                           hipStream_t stream) {
    if (n_heads <= 0 || n_heads % 128 != 0 || config >= 1000 || n_kv_rows <= 0 ||
        (unsigned long long)n_kv_rows * FP8_ROW_BYTES >= 0xffffffffull)
        return 0;
    const KvAddressing kva{block_table, table_stride, page_shift, batch_rows};
    launch_sparse_mla(out, q, kv_fp8, idx, workspace, workspace_bytes, batch, n_heads, n_kv_rows, topk, d_qk,
                      d_v, sm_scale, out_dtype, config, kva, stream, true);
    return 1;
}
