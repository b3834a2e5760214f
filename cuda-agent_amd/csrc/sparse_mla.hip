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
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "launch_status.hpp"

namespace {

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

// position of 16-byte chunk `chunk` of row `row` inside a tile (in 16-byte units)
__device__ __forceinline__ int swizzled_slot(int row, int chunk) {
    return row * ROW_CHUNKS + ((chunk & ~7) | ((chunk ^ row) & 7));
}

// One wavefront's share of a tile load: LDS slots [first_slot, first_slot + 64*N) in lane order.
template <int NW>
__device__ __forceinline__ void issue_tile_load(uint4* tile, const char* kv_b, const int* s_idx_tile,
                                                bool has_padding, int wave, int lane) {
    constexpr int PER_WAVE = TILE_CHUNKS / 64 / NW;  // 36 wave-instructions per tile
    // The slot -> (row, chunk) arithmetic is a handful of integer operations per load. Hiding the
    // lane number from the optimiser here keeps it from precomputing all of them before the
    // tile loop and holding (or spilling) two registers per load for the whole kernel.
    asm volatile("" : "+v"(lane));
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i) {
        const int inst = wave * PER_WAVE + i;
        const int slot = inst * 64 + lane;
        const int row = slot / ROW_CHUNKS;
        const int pos = slot - row * ROW_CHUNKS;
        const int chunk = (pos & ~7) | ((pos ^ row) & 7);
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
}

struct SoftmaxState {
    float m;  // running max of the scaled scores (log2 domain); same in lanes l and l^32
    float l;  // running sum of exp2(s - m) over the rows this lane has seen
};

// Per-lane byte offsets into a tile, computed once. With the XOR swizzle every LDS address of
// the inner loops is one of these six values plus a compile-time constant, so the reads use
// the instruction's immediate offset field and no address arithmetic.
struct LaneOffsets {
    uint32_t qk[4];  // K operand of k-step ks: qk[ks & 3] + (ks >> 2) * 128
    uint32_t pv[2];  // V^T operand of dv tile t, k-step ks, half-read rr:
                     //   pv[t & 1] + (16*ks + 8*rr) * ROW_BYTES + (t >> 1) * 128
};

__device__ __forceinline__ LaneOffsets make_lane_offsets(int lane) {
    LaneOffsets o;
    const int r32 = lane & 31;
    const int half = lane >> 5;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        o.qk[c] = r32 * ROW_BYTES + (((2 * c + half) ^ r32) & 7) * 16;
    }
    const int g2 = (lane >> 4) & 1;
    const int s16 = lane & 15;
    const int row = 4 * half + (s16 >> 2);  // tile row of this lane's address, modulo 8
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int chunk = 4 * u + 2 * g2 + ((s16 & 3) >> 1);
        o.pv[u] = row * ROW_BYTES + ((chunk ^ row) & 7) * 16 + 8 * (s16 & 1);
    }
    return o;
}

typedef const __attribute__((address_space(3))) char* lds_bytes;

// Everything a wavefront does with one resident tile. LDS reads run one group of four MFMAs
// ahead of their use; the scheduling fences keep the compiler from hoisting all 36 + 64 reads
// to the top (which would need more registers than the 112 left beside Q and the accumulator).
__device__ __forceinline__ void process_tile(const uint4* tile, const int* s_idx_tile, bool masked,
                                             const bf16x8 (&qreg)[K_STEPS], floatx16 (&acc)[DV_TILES],
                                             SoftmaxState& st, const LaneOffsets& off,
                                             float scale_log2, int lane) {
    typedef const __attribute__((address_space(3))) uintx4* lds_x4;
    typedef shortx4 __attribute__((address_space(3)))* lds_s4;
    const int half = lane >> 5;
    const lds_bytes base = (lds_bytes)tile;

#pragma unroll
    for (int t = 0; t < DV_TILES; ++t) asm volatile("" : "+a"(acc[t]));

    // S^T[row, head] = sum_d K[row, d] Q[head, d]
    floatx16 s = {0};
    asm volatile("" : "+v"(s));  // keep S out of the accumulation registers, which O^T fills
    {
        constexpr int G = 2;
        constexpr int GROUPS = K_STEPS / G;  // 18
        uintx4 kbuf[2][G];
#pragma unroll
        for (int j = 0; j < G; ++j) kbuf[0][j] = *(lds_x4)(base + off.qk[j & 3] + (j >> 2) * 128);
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            if (g + 1 < GROUPS) {
#pragma unroll
                for (int j = 0; j < G; ++j) {
                    const int ks = G * (g + 1) + j;
                    kbuf[(g + 1) & 1][j] = *(lds_x4)(base + off.qk[ks & 3] + (ks >> 2) * 128);
                }
            }
#pragma unroll
            for (int j = 0; j < G; ++j) {
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kbuf[g & 1][j]),
                                                            qreg[G * g + j], s, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    constexpr int PV_STEPS = 2 * DV_TILES;  // (k-step, dv tile) pairs, 32 MFMAs
    constexpr int PV_GROUP = 4;
    shortx4 vbuf[2][PV_GROUP][2];
    auto pv_read = [&](int step, shortx4 (&dst)[2]) {
        const int ks = step / DV_TILES;
        const int t = step % DV_TILES;
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
            dst[rr] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (lds_s4)(base + off.pv[t & 1] + (16 * ks + 8 * rr) * ROW_BYTES + (t >> 1) * 128));
        }
    };

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
    const float m_new = fmaxf(st.m, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // all rows masked so far
    const float alpha = __builtin_amdgcn_exp2f(st.m - m_use);
    st.m = m_new;

    float psum = 0.f;
    bf16x8 p[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float e = __builtin_amdgcn_exp2f(s[i] - m_use);
        psum += e;
        p[i / 8][i % 8] = (__bf16)e;
    }
    st.l = st.l * alpha + psum;

    // rescale the accumulator only when some head's maximum moved
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
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

// grid: x = split, y = request, z = head group of 32*NW heads
template <int NW>
__global__ __launch_bounds__(64 * NW) void sparse_mla_split_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ idx,
    float* __restrict__ o_part, float* __restrict__ lse_part, int n_heads, int n_kv_rows, int topk,
    int rows_per_split, float scale_log2) {
    constexpr int PER_WAVE = TILE_CHUNKS / 64 / NW;
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
        int key = -1;
        if (i < n_rows) {
            key = idx[(size_t)b * topk + row_begin + i];
            if (key >= n_kv_rows) key = -1;  // out-of-range selections are treated as padding
        }
        if (key < 0) {
            key = -1;
            atomicMin(&s_first_masked_tile, i / TILE_ROWS);
        }
        s_idx[i] = key;
    }
    __syncthreads();
    const int first_masked_tile = s_first_masked_tile;

    const char* kv_b = reinterpret_cast<const char*>(kv) + (size_t)b * n_kv_rows * ROW_BYTES;

    // prologue: tiles 0 and 1 in flight
    if (n_tiles > 0) issue_tile_load<NW>(tile0, kv_b, s_idx, 0 >= first_masked_tile, wave, lane);
    if (n_tiles > 1)
        issue_tile_load<NW>(tile1, kv_b, s_idx + TILE_ROWS, 1 >= first_masked_tile, wave, lane);

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
    // wait is for everything.) Tile t+2 is issued after the barrier, into the buffer every
    // wavefront finished reading in step t-1.
#define MLA_STEP(CUR, NXT2, T)                                                                  \
    {                                                                                           \
        if ((T) + 1 < n_tiles && (T) + 1 < first_masked_tile)                                   \
            wait_vmcnt<PER_WAVE>();                                                             \
        else                                                                                    \
            wait_vmcnt<0>();                                                                    \
        __builtin_amdgcn_s_barrier();                                                           \
        asm volatile("" ::: "memory");                                                          \
        if ((T) + 2 < n_tiles)                                                                  \
            issue_tile_load<NW>(NXT2, kv_b, s_idx + ((T) + 2) * TILE_ROWS,                      \
                                (T) + 2 >= first_masked_tile, wave, lane);                      \
        process_tile(CUR, s_idx + (T) * TILE_ROWS, (T) >= first_masked_tile, qreg, acc, st, off,  \
                     scale_log2, lane);                                                         \
    }
    for (int t = 0; t < n_tiles; t += 3) {
        MLA_STEP(tile0, tile2, t)
        if (t + 1 < n_tiles) MLA_STEP(tile1, tile0, t + 1)
        if (t + 2 < n_tiles) MLA_STEP(tile2, tile1, t + 2)
    }
#undef MLA_STEP

    // epilogue: normalise, write partial output [b, split, head, dv] and log2-sum-exp
    const float l_total = st.l + __shfl_xor(st.l, 32);
    const float inv_l = l_total > 0.f ? 1.f / l_total : 0.f;
    const int head = head0 + (lane & 31);
    const int half = lane >> 5;
    const size_t part = ((size_t)b * n_splits + split) * n_heads + head;
    float* o_row = o_part + part * D_V;
#pragma unroll
    for (int t = 0; t < DV_TILES; ++t) {
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            floatx4 v = {acc[t][4 * qd] * inv_l, acc[t][4 * qd + 1] * inv_l,
                         acc[t][4 * qd + 2] * inv_l, acc[t][4 * qd + 3] * inv_l};
            *reinterpret_cast<floatx4*>(o_row + 32 * t + 8 * qd + 4 * half) = v;
        }
    }
    if (half == 0) {
        lse_part[part] = l_total > 0.f ? st.m + __builtin_amdgcn_logf(l_total) : -INFINITY;
    }
}

// out[b, h, :] = sum_s w_s o_part[b, s, h, :],  w_s = exp2(lse_s - max) / sum; one workgroup of
// 128 lanes per (b, h), 4 output columns per lane.
template <typename OUT>
__global__ __launch_bounds__(128) void sparse_mla_merge_kernel(const float* __restrict__ o_part,
                                                               const float* __restrict__ lse_part,
                                                               OUT* __restrict__ out, int n_heads,
                                                               int n_splits) {
    const int h = blockIdx.x;
    const int b = blockIdx.y;
    const size_t base = (size_t)b * n_splits * n_heads + h;
    float mx = -INFINITY;
    for (int s = 0; s < n_splits; ++s) mx = fmaxf(mx, lse_part[base + (size_t)s * n_heads]);
    float wsum = 0.f;
    floatx4 o = {0.f, 0.f, 0.f, 0.f};
    if (mx > -INFINITY) {
        for (int s = 0; s < n_splits; ++s) {
            const float w = __builtin_amdgcn_exp2f(lse_part[base + (size_t)s * n_heads] - mx);
            if (w > 0.f) {
                const floatx4 v = *reinterpret_cast<const floatx4*>(
                    o_part + (base + (size_t)s * n_heads) * D_V + threadIdx.x * 4);
                o += v * w;
                wsum += w;
            }
        }
        o *= 1.f / wsum;
    }
    OUT* dst = out + ((size_t)b * n_heads + h) * D_V + threadIdx.x * 4;
    if constexpr (sizeof(OUT) == 4) {
        *reinterpret_cast<floatx4*>(dst) = o;
    } else {
        bf16x4 r = {(__bf16)o.x, (__bf16)o.y, (__bf16)o.z, (__bf16)o.w};
        *reinterpret_cast<bf16x4*>(dst) = r;
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
    const int head_groups = n_heads <= 128 ? 1 : n_heads / 128;
    return pick_splits(batch, head_groups, topk, config);
}

// bytes of scratch sparse_mla_decode_launcher needs for these sizes
extern "C" size_t sparse_mla_decode_workspace_bytes(int batch, int n_heads, int topk, int config) {
    const int splits = sparse_mla_decode_num_splits(batch, n_heads, topk, config);
    return (size_t)batch * splits * n_heads * (D_V + 1) * sizeof(float);
}

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
    const int head_groups = n_heads <= 128 ? 1 : n_heads / 128;
    const int splits = pick_splits(batch, head_groups, topk, config);
    const int tiles = (topk + TILE_ROWS - 1) / TILE_ROWS;
    const int rows_per_split = ((tiles + splits - 1) / splits) * TILE_ROWS;
    float* o_part = static_cast<float*>(workspace);
    float* lse_part = o_part + (size_t)batch * splits * n_heads * D_V;
    const float scale_log2 = sm_scale * 1.4426950408889634f;
    const __bf16* qb = static_cast<const __bf16*>(q);
    const __bf16* kvb = static_cast<const __bf16*>(kv);
    const dim3 grid(splits, batch, head_groups);
    if (n_heads == 32) {
        sparse_mla_split_kernel<1><<<grid, 64, 0, stream>>>(qb, kvb, idx, o_part, lse_part, n_heads,
                                                            n_kv_rows, topk, rows_per_split,
                                                            scale_log2);
    } else if (n_heads == 64) {
        sparse_mla_split_kernel<2><<<grid, 128, 0, stream>>>(qb, kvb, idx, o_part, lse_part, n_heads,
                                                             n_kv_rows, topk, rows_per_split,
                                                             scale_log2);
    } else {
        sparse_mla_split_kernel<4><<<grid, 256, 0, stream>>>(qb, kvb, idx, o_part, lse_part, n_heads,
                                                             n_kv_rows, topk, rows_per_split,
                                                             scale_log2);
    }
    if (out_dtype == 0) {
        sparse_mla_merge_kernel<__bf16><<<dim3(n_heads, batch), 128, 0, stream>>>(
            o_part, lse_part, static_cast<__bf16*>(out), n_heads, splits);
    } else {
        sparse_mla_merge_kernel<float><<<dim3(n_heads, batch), 128, 0, stream>>>(
            o_part, lse_part, static_cast<float*>(out), n_heads, splits);
    }
}
