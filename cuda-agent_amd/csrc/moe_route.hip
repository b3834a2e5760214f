// MoE routing and the deterministic sort of (token, slot) pairs by expert.
//
// route:  one wavefront per token. The token's 8 experts are its 8 largest logits, ties going
//         to the lower expert id, listed in that order; weight = sigmoid(logit) normalised over
//         the 8. Ranking uses the logits themselves, which orders exactly as an exact sigmoid
//         would and does not depend on how a sigmoid implementation rounds.
// sort:   stable counting sort in three small kernels, all integer and order-independent:
//         per-chunk histograms (256 tokens per chunk), an exclusive scan over chunks and
//         experts, and a scatter in which lane e of a workgroup walks its chunk's pairs in
//         flat order and hands out expert e's positions one by one.
#include "launch_status.hpp"
#include "moe_common.hpp"

namespace {

using namespace moe;

__device__ __forceinline__ unsigned long long rank_key(float logit, int id) {
    logit += 0.f;  // -0 -> +0, so that the two zeros tie
    unsigned u = __float_as_uint(logit);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // monotone in the float order
    return ((unsigned long long)u << 32) | (unsigned)(0x7fffffff - id);  // lower id wins a tie
}

// the logit a key was made from (-0 comes back as +0, which has the same sigmoid)
__device__ __forceinline__ float key_logit(unsigned long long key) {
    const unsigned u = (unsigned)(key >> 32);
    return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

// Maximum of a 32-bit unsigned value over the wavefront, returned as the same value in every lane. The
// running maximum inside each row of 16 lanes goes through the DPP row shifts of the vector ALU, and the
// last lanes of the four rows are read as scalars: no LDS crossbar, which the __shfl exchanges use and
// which made a dependent chain of them cost about 100 cycles per step.
__device__ __forceinline__ unsigned wave_max_u32(unsigned v) {
    // dpp control 0x110 + n = row_shr:n; lanes without a source lane take `old` = 0, the identity
#define ROW_SHR_MAX(n)                                                                              \
    {                                                                                               \
        const unsigned o = (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, 0x110 + (n), 0xf, 0xf, false); \
        v = o > v ? o : v;                                                                          \
    }
    ROW_SHR_MAX(1)
    ROW_SHR_MAX(2)
    ROW_SHR_MAX(4)
    ROW_SHR_MAX(8)
#undef ROW_SHR_MAX
    const unsigned r0 = (unsigned)__builtin_amdgcn_readlane((int)v, 15);
    const unsigned r1 = (unsigned)__builtin_amdgcn_readlane((int)v, 31);
    const unsigned r2 = (unsigned)__builtin_amdgcn_readlane((int)v, 47);
    const unsigned r3 = (unsigned)__builtin_amdgcn_readlane((int)v, 63);
    const unsigned a = r0 > r1 ? r0 : r1;
    const unsigned b = r2 > r3 ? r2 : r3;
    return a > b ? a : b;
}

// maximum of the 64-bit rank keys of a wavefront: the largest upper half, then the largest lower half
// among the lanes that hold it
__device__ __forceinline__ unsigned long long wave_max_key(unsigned long long key) {
    const unsigned hi = (unsigned)(key >> 32);
    const unsigned hi_max = wave_max_u32(hi);
    const unsigned lo_max = wave_max_u32(hi == hi_max ? (unsigned)key : 0u);
    return ((unsigned long long)hi_max << 32) | lo_max;
}

template <int PER_LANE>
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits,
                                                        int* __restrict__ ids,
                                                        float* __restrict__ weights, int tokens,
                                                        int n_experts, int top_k, int shared) {
    // shared == 1: every token gets one more slot, expert number n_experts with weight 1 (a shared
    // expert stored behind the routed ones); rows of ids/weights then have top_k + 1 entries
    const int slots = top_k + shared;
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= tokens) return;
    unsigned long long key[PER_LANE];
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int e = j * 64 + lane;
        key[j] = e < n_experts ? rank_key(logits[(size_t)t * n_experts + e], e) : 0ull;
    }
    float my_score = 0.f;  // lane k keeps the k-th choice
    int my_id = 0;
    float total = 0.f;
    for (int k = 0; k < top_k; ++k) {
        unsigned long long best = 0ull;
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) best = key[j] > best ? key[j] : best;
        best = wave_max_key(best);
        const int id = 0x7fffffff - (int)(unsigned)(best & 0xffffffffull);
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            if (j * 64 + lane == id) key[j] = 0ull;  // taken
        }
        const float logit = key_logit(best);
        const float score = 1.f / (1.f + expf(-logit));
        total += score;
        if (lane == k) {
            my_score = score;
            my_id = id;
        }
    }
    if (lane < top_k) {
        ids[(size_t)t * slots + lane] = my_id;
        weights[(size_t)t * slots + lane] = my_score / total;
    } else if (lane == top_k && shared) {
        ids[(size_t)t * slots + lane] = n_experts;
        weights[(size_t)t * slots + lane] = 1.f;
    }
}

// Group-limited routing with a selection bias (the DeepSeek-V3 router): one wavefront per token.
//   score = sigmoid(logit);  choice = score + bias
//   group value = sum of the 2 largest choice values of the group (groups are runs of
//                 n_experts / n_group consecutive experts)
//   the topk_group groups with the largest value stay (ties to the lower group), the others are out
//   ids = the top_k largest choice values among the experts that stay, descending, ties to the
//         lower expert id
//   weights = score[ids] (the unbiased score), divided by their sum + 1e-20 if normalise, times scale
// LDS per wavefront: the token's choice values and scores, n_experts floats each.
template <int PER_LANE>
__global__ __launch_bounds__(256) void moe_route_grouped_kernel(
    const float* __restrict__ logits, const float* __restrict__ bias, int* __restrict__ ids,
    float* __restrict__ weights, int tokens, int n_experts, int top_k, int n_group, int topk_group,
    int normalise, float scale) {
    extern __shared__ float s_route[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= tokens) return;  // (no workgroup barrier below: a wavefront only reads what it wrote)
    float* s_choice = s_route + (size_t)wave * 2 * n_experts;
    float* s_score = s_choice + n_experts;
    const int group_size = n_experts / n_group;

    float choice[PER_LANE];
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int e = j * 64 + lane;
        choice[j] = -INFINITY;
        if (e < n_experts) {
            const float score = 1.f / (1.f + expf(-logits[(size_t)t * n_experts + e]));
            choice[j] = score + (bias != nullptr ? bias[e] : 0.f);
            s_choice[e] = choice[j];
            s_score[e] = score;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // lane g: value of group g
    float value = -INFINITY;
    if (lane < n_group) {
        float first = -INFINITY, second = -INFINITY;
        for (int i = 0; i < group_size; ++i) {
            const float c = s_choice[lane * group_size + i];
            if (c > first) {
                second = first;
                first = c;
            } else if (c > second) {
                second = c;
            }
        }
        value = group_size > 1 ? first + second : first;
    }
    // rank of group `lane` among the groups; the topk_group best stay
    int better = 0;
    for (int g = 0; g < n_group; ++g) {
        const float other = __shfl(value, g);
        better += (other > value || (other == value && g < lane)) ? 1 : 0;
    }
    const unsigned long long stay_mask = __ballot(lane < n_group && better < topk_group);

    unsigned long long key[PER_LANE];
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
        const int e = j * 64 + lane;
        const bool stays = e < n_experts && ((stay_mask >> (e / group_size)) & 1ull);
        key[j] = stays ? rank_key(choice[j], e) : 0ull;
    }
    float my_score = 0.f;  // lane k keeps the k-th choice
    int my_id = 0;
    float total = 0.f;
    for (int k = 0; k < top_k; ++k) {
        unsigned long long best = 0ull;
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) best = key[j] > best ? key[j] : best;
        best = wave_max_key(best);
        const int id = 0x7fffffff - (int)(unsigned)(best & 0xffffffffull);
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            if (j * 64 + lane == id) key[j] = 0ull;  // taken
        }
        const float score = s_score[id];
        total += score;
        if (lane == k) {
            my_score = score;
            my_id = id;
        }
    }
    if (lane < top_k) {
        ids[(size_t)t * top_k + lane] = my_id;
        const float w = normalise ? my_score / (total + 1e-20f) : my_score;
        weights[(size_t)t * top_k + lane] = w * scale;
    }
}

// chunk_hist[chunk][e] = number of pairs of chunk `chunk` routed to expert e
__global__ __launch_bounds__(256) void moe_hist_kernel(const int* __restrict__ ids,
                                                       int* __restrict__ chunk_hist, int pairs,
                                                       int pairs_per_chunk, int n_experts) {
    extern __shared__ int s_hist[];
    for (int e = threadIdx.x; e < n_experts; e += 256) s_hist[e] = 0;
    __syncthreads();
    const int begin = blockIdx.x * pairs_per_chunk;
    int end = begin + pairs_per_chunk;
    if (end > pairs) end = pairs;
    for (int p = begin + threadIdx.x; p < end; p += 256) atomicAdd(&s_hist[ids[p]], 1);
    __syncthreads();
    for (int e = threadIdx.x; e < n_experts; e += 256) {
        chunk_hist[(size_t)blockIdx.x * n_experts + e] = s_hist[e];
    }
}

// Exclusive prefix sum of s[0..n) in place (n <= 1024, blockDim.x == 1024); s[n] = total.
__device__ __forceinline__ void block_exclusive_scan(int* s, int n) {
    const int t = threadIdx.x;
    const int mine = t < n ? s[t] : 0;
    int v = mine;
    __syncthreads();
    for (int d = 1; d < n; d <<= 1) {
        const int add = (t >= d && t < n) ? s[t - d] : 0;
        __syncthreads();
        v += add;
        if (t < n) s[t] = v;
        __syncthreads();
    }
    if (t < n) s[t] = v - mine;
    if (t == n - 1) s[n] = v;
    __syncthreads();
}

// In place: chunk_hist[chunk][e] becomes the first sorted position of expert e's pairs from
// that chunk; expert_offsets[e] the first position of the expert. One workgroup; the loads of a
// column are issued in independent batches (a read-modify-write loop over the chunks is one
// memory latency per chunk).
__global__ __launch_bounds__(1024) void moe_scan_kernel(int* __restrict__ chunk_hist,
                                                        int* __restrict__ expert_offsets,
                                                        int chunks, int n_experts) {
    __shared__ int s_count[1024 + 1];
    constexpr int BATCH = 8;
    const int e = threadIdx.x;
    int total = 0;
    if (e < n_experts) {
        for (int c0 = 0; c0 < chunks; c0 += BATCH) {
            int v[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                v[j] = c0 + j < chunks ? chunk_hist[(size_t)(c0 + j) * n_experts + e] : 0;
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) total += v[j];
        }
        s_count[e] = total;
    }
    __syncthreads();
    block_exclusive_scan(s_count, n_experts);
    if (e < n_experts) {
        int running = s_count[e];
        expert_offsets[e] = running;
        for (int c0 = 0; c0 < chunks; c0 += BATCH) {
            int v[BATCH];
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                v[j] = c0 + j < chunks ? chunk_hist[(size_t)(c0 + j) * n_experts + e] : 0;
            }
#pragma unroll
            for (int j = 0; j < BATCH; ++j) {
                if (c0 + j < chunks) chunk_hist[(size_t)(c0 + j) * n_experts + e] = running;
                running += v[j];
            }
        }
    }
    if (e == 0) expert_offsets[n_experts] = s_count[n_experts];
}

// rank of this lane's pair among the pairs of the same 64-pair group with the same expert
// (`earlier`), and whether a later lane of the group has the same expert
__device__ __forceinline__ void group_rank(int e, int lane, int& earlier, bool& later) {
    earlier = 0;
    later = false;
#pragma unroll 8
    for (int k = 0; k < 64; ++k) {
        const int ek = __builtin_amdgcn_readlane(e, k);
        earlier += (ek == e && k < lane) ? 1 : 0;
        later = later || (ek == e && k > lane);
    }
}

// Stable scatter of one chunk in three parallel phases. The chunk's pairs are taken in groups of
// 64 in flat order: (1) one wavefront per group ranks its pairs among equal experts of the group
// and leaves the group's count per expert in LDS; (2) one lane per expert turns the counts into
// first positions, group after group, starting from the chunk's first position for that expert;
// (3) every pair is written to (first position of its expert in its group) + (its rank).
// LDS: [groups][n_experts] counts + [groups*64] ranks.
__global__ __launch_bounds__(1024) void moe_scatter_kernel(const int* __restrict__ ids,
                                                           const int* __restrict__ chunk_base,
                                                           int* __restrict__ sorted_pairs,
                                                           int* __restrict__ pair_pos, int pairs,
                                                           int pairs_per_chunk, int n_experts) {
    extern __shared__ int s_mem[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int begin = blockIdx.x * pairs_per_chunk;
    int count = pairs - begin;
    if (count > pairs_per_chunk) count = pairs_per_chunk;
    const int groups = (count + 63) / 64;
    int* s_first = s_mem;                       // [groups][n_experts]
    int* s_rank = s_mem + groups * n_experts;   // [groups * 64]
    for (int i = threadIdx.x; i < groups * n_experts; i += 1024) s_first[i] = 0;
    __syncthreads();
    for (int g = wave; g < groups; g += 16) {
        const int i = g * 64 + lane;
        const int e = i < count ? ids[begin + i] : -1 - lane;  // lanes past the end match nobody
        int earlier;
        bool later;
        group_rank(e, lane, earlier, later);
        s_rank[i] = earlier;
        if (i < count && !later) s_first[g * n_experts + e] = earlier + 1;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < n_experts; e += 1024) {
        int running = chunk_base[(size_t)blockIdx.x * n_experts + e];
        for (int g = 0; g < groups; ++g) {
            const int v = s_first[g * n_experts + e];
            s_first[g * n_experts + e] = running;
            running += v;
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < count; i += 1024) {
        const int pos = s_first[(i >> 6) * n_experts + ids[begin + i]] + s_rank[i];
        sorted_pairs[pos] = begin + i;
        pair_pos[begin + i] = pos;
    }
}

// The same order with one wavefront per chunk and n_experts ints of LDS, for chunks whose group
// table would not fit: a pair's position is (next free position of its expert) + (its rank in the
// group); the last lane of every expert present then advances that expert's position.
__global__ __launch_bounds__(64) void moe_scatter_serial_kernel(const int* __restrict__ ids,
                                                                const int* __restrict__ chunk_base,
                                                                int* __restrict__ sorted_pairs,
                                                                int* __restrict__ pair_pos, int pairs,
                                                                int pairs_per_chunk, int n_experts) {
    extern __shared__ int s_next[];  // [n_experts]
    const int lane = threadIdx.x;
    const int begin = blockIdx.x * pairs_per_chunk;
    int count = pairs - begin;
    if (count > pairs_per_chunk) count = pairs_per_chunk;
    for (int e = lane; e < n_experts; e += 64) s_next[e] = chunk_base[(size_t)blockIdx.x * n_experts + e];
    __syncthreads();
    for (int g = 0; g < count; g += 64) {
        const int i = g + lane;
        const int e = i < count ? ids[begin + i] : -1 - lane;
        int earlier;
        bool later;
        group_rank(e, lane, earlier, later);
        if (i < count) {
            const int pos = s_next[e] + earlier;
            sorted_pairs[pos] = begin + i;
            pair_pos[begin + i] = pos;
            if (!later) s_next[e] = pos + 1;
        }
        __syncthreads();
    }
}

// Routing and sort of a small batch in one workgroup (tokens*top_k <= 1024 pairs): wavefronts
// route tokens round-robin, keeping the expert ids in LDS; each pair then finds its position as
// (first position of its expert) + (number of earlier pairs with the same expert), which is
// the same stable order the chunked path produces.
template <int PER_LANE>
__global__ __launch_bounds__(1024) void moe_route_sort_small_kernel(
    const float* __restrict__ logits, int* __restrict__ ids, float* __restrict__ weights,
    int* __restrict__ sorted_pairs, int* __restrict__ pair_pos, int* __restrict__ expert_offsets,
    int tokens, int n_experts, int top_k, int shared) {
    __shared__ int s_ids[1024];
    __shared__ int s_count[512 + 2];
    __shared__ int s_wave_count[16][512 + 1];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int slots = top_k + shared;        // see moe_route_kernel
    const int sorted_experts = n_experts + shared;
    const int pairs = tokens * slots;
    for (int e = threadIdx.x; e <= sorted_experts; e += 1024) s_count[e] = 0;
    for (int i = threadIdx.x; i < 16 * (512 + 1); i += 1024) (&s_wave_count[0][0])[i] = 0;
    for (int t = wave; t < tokens; t += 16) {
        unsigned long long key[PER_LANE];
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            const int e = j * 64 + lane;
            key[j] = e < n_experts ? rank_key(logits[(size_t)t * n_experts + e], e) : 0ull;
        }
        float my_score = 0.f, total = 0.f;
        int my_id = 0;
        for (int k = 0; k < top_k; ++k) {
            unsigned long long best = 0ull;
#pragma unroll
            for (int j = 0; j < PER_LANE; ++j) best = key[j] > best ? key[j] : best;
            best = wave_max_key(best);
            const int id = 0x7fffffff - (int)(unsigned)(best & 0xffffffffull);
#pragma unroll
            for (int j = 0; j < PER_LANE; ++j) {
                if (j * 64 + lane == id) key[j] = 0ull;
            }
            const float score = 1.f / (1.f + expf(-key_logit(best)));
            total += score;
            if (lane == k) {
                my_score = score;
                my_id = id;
            }
        }
        if (lane < top_k) {
            ids[(size_t)t * slots + lane] = my_id;
            weights[(size_t)t * slots + lane] = my_score / total;
            s_ids[t * slots + lane] = my_id;
        } else if (lane == top_k && shared) {
            ids[(size_t)t * slots + lane] = n_experts;
            weights[(size_t)t * slots + lane] = 1.f;
            s_ids[t * slots + lane] = n_experts;
        }
    }
    __syncthreads();
    // Stable rank of every pair inside its expert without walking the earlier pairs: the rank among
    // the 64 pairs of the wavefront (lane compares), plus the expert's pairs in earlier wavefronts
    // (a 16 x experts table, prefix-summed per expert).
    const int p = threadIdx.x;
    const int mine = p < pairs ? s_ids[p] : -1;
    int rank;
    bool later;
    group_rank(mine, lane, rank, later);
    if (mine >= 0 && !later) s_wave_count[wave][mine] = rank + 1;  // this wavefront's pairs of the expert
    __syncthreads();
    for (int e = threadIdx.x; e < sorted_experts; e += 1024) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) {
            const int c = s_wave_count[w][e];
            s_wave_count[w][e] = run;
            run += c;
        }
        s_count[e] = run;
    }
    __syncthreads();
    if (mine >= 0) rank += s_wave_count[wave][mine];
    block_exclusive_scan(s_count, sorted_experts);  // in place; s_count[sorted_experts] = number of pairs
    for (int e = threadIdx.x; e <= sorted_experts; e += 1024) expert_offsets[e] = s_count[e];
    if (p < pairs) {
        const int pos = s_count[mine] + rank;
        sorted_pairs[pos] = p;
        pair_pos[p] = pos;
    }
}

// The sort of a small batch alone (tokens*slots <= 1024 pairs, one workgroup): ids come from the routing
// kernel, which spreads the tokens over many CUs (on one CU the 8 arg-max rounds of 64 tokens are bound by
// that CU's instruction issue rate: 24 of the 31 us the fused kernel above takes).
__global__ __launch_bounds__(1024) void moe_sort_small_kernel(const int* __restrict__ ids,
                                                              int* __restrict__ sorted_pairs,
                                                              int* __restrict__ pair_pos,
                                                              int* __restrict__ expert_offsets, int pairs,
                                                              int sorted_experts) {
    __shared__ int s_count[512 + 2];
    __shared__ int s_wave_count[16][512 + 1];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int p = threadIdx.x;
    const int mine = p < pairs ? ids[p] : -1;  // (requested before the tables are cleared)
    for (int e = threadIdx.x; e <= sorted_experts; e += 1024) s_count[e] = 0;
    for (int i = threadIdx.x; i < 16 * (512 + 1); i += 1024) (&s_wave_count[0][0])[i] = 0;
    __syncthreads();
    int rank;
    bool later;
    group_rank(mine, lane, rank, later);
    if (mine >= 0 && !later) s_wave_count[wave][mine] = rank + 1;  // this wavefront's pairs of the expert
    __syncthreads();
    for (int e = threadIdx.x; e < sorted_experts; e += 1024) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) {
            const int c = s_wave_count[w][e];
            s_wave_count[w][e] = run;
            run += c;
        }
        s_count[e] = run;
    }
    __syncthreads();
    if (mine >= 0) rank += s_wave_count[wave][mine];
    block_exclusive_scan(s_count, sorted_experts);  // in place; s_count[sorted_experts] = number of pairs
    for (int e = threadIdx.x; e <= sorted_experts; e += 1024) expert_offsets[e] = s_count[e];
    if (p < pairs) {
        const int pos = s_count[mine] + rank;
        sorted_pairs[pos] = p;
        pair_pos[p] = pos;
    }
}

}  // namespace

// Routing followed by the sort. Small batches (tokens*top_k <= 1024): the routing kernel, then the
// single-workgroup sort (config 2: one kernel that does both in one workgroup); otherwise
// moe_route_launcher + moe_sort_launcher. Same outputs in every form.
extern "C" void moe_route_sort_launcher(int* ids, float* weights, int* sorted_pairs, int* pair_pos,
                                        int* expert_offsets, int* chunk_scratch, const float* logits,
                                        int tokens, int n_experts, int top_k, int config,
                                        hipStream_t stream);

// ids [tokens, top_k] int32 and weights [tokens, top_k] fp32 from logits [tokens, n_experts] fp32.
extern "C" void moe_route_launcher(int* ids, float* weights, const float* logits, int tokens,
                                   int n_experts, int top_k, int config, hipStream_t stream) {
    const int shared = (config & CONFIG_SHARED_SLOT) ? 1 : 0;
    if (tokens <= 0) return;
    if (n_experts <= 0 || n_experts > 512 - shared || top_k <= 0 || top_k > 64 - shared ||
        top_k > n_experts) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!ids || !weights || !logits) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const int blocks = (tokens + 3) / 4;
    if (n_experts <= 256) {
        moe_route_kernel<4><<<blocks, 256, 0, stream>>>(logits, ids, weights, tokens, n_experts, top_k,
                                                        shared);
    } else {
        moe_route_kernel<8><<<blocks, 256, 0, stream>>>(logits, ids, weights, tokens, n_experts, top_k,
                                                        shared);
    }
}

// Group-limited routing with a selection bias (see moe_route_grouped_kernel).
// bias [n_experts] fp32 or null. n_experts a multiple of n_group, n_group <= 64,
// topk_group <= n_group, top_k <= topk_group * (n_experts / n_group).
extern "C" void moe_route_grouped_launcher(int* ids, float* weights, const float* logits,
                                           const float* bias, int tokens, int n_experts, int top_k,
                                           int n_group, int topk_group, int normalise,
                                           float routed_scaling_factor, int config,
                                           hipStream_t stream) {
    (void)config;
    if (tokens <= 0) return;
    if (n_experts <= 0 || n_experts > 512 || top_k <= 0 || top_k > 64 || n_group <= 0 ||
        n_group > 64 || n_experts % n_group != 0 || topk_group <= 0 || topk_group > n_group ||
        (long long)topk_group * (n_experts / n_group) < top_k) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!ids || !weights || !logits) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const int blocks = (tokens + 3) / 4;
    const size_t lds = (size_t)4 * 2 * n_experts * sizeof(float);
    if (n_experts <= 256) {
        moe_route_grouped_kernel<4><<<blocks, 256, lds, stream>>>(
            logits, bias, ids, weights, tokens, n_experts, top_k, n_group, topk_group, normalise,
            routed_scaling_factor);
    } else {
        moe_route_grouped_kernel<8><<<blocks, 256, lds, stream>>>(
            logits, bias, ids, weights, tokens, n_experts, top_k, n_group, topk_group, normalise,
            routed_scaling_factor);
    }
}

// Stable counting sort of the tokens*top_k pairs by expert id.
//   sorted_pairs[pos] = flat pair index (token*top_k + slot); pair_pos is its inverse;
//   expert_offsets[e] .. expert_offsets[e+1] are expert e's positions.
//   chunk_scratch: ceil(tokens/256) * n_experts ints.
extern "C" void moe_sort_launcher(int* sorted_pairs, int* pair_pos, int* expert_offsets,
                                  int* chunk_scratch, const int* ids, int tokens, int n_experts,
                                  int top_k, int config, hipStream_t stream) {
    (void)config;
    if (tokens <= 0) return;
    if (n_experts <= 0 || n_experts > 1024 || top_k <= 0 || top_k > 64) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!sorted_pairs || !pair_pos || !expert_offsets || !chunk_scratch || !ids) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    const int pairs = tokens * top_k;
    const int pairs_per_chunk = moe::SORT_CHUNK_TOKENS * top_k;
    const int chunks = (tokens + moe::SORT_CHUNK_TOKENS - 1) / moe::SORT_CHUNK_TOKENS;
    moe_hist_kernel<<<chunks, 256, n_experts * sizeof(int), stream>>>(ids, chunk_scratch, pairs,
                                                                     pairs_per_chunk, n_experts);
    moe_scan_kernel<<<1, 1024, 0, stream>>>(chunk_scratch, expert_offsets, chunks, n_experts);
    const size_t group_table = ((size_t)(pairs_per_chunk / 64) * n_experts + pairs_per_chunk) * sizeof(int);
    if (group_table <= 64 * 1024) {
        moe_scatter_kernel<<<chunks, 1024, group_table, stream>>>(ids, chunk_scratch, sorted_pairs, pair_pos,
                                                                  pairs, pairs_per_chunk, n_experts);
    } else {
        moe_scatter_serial_kernel<<<chunks, 64, n_experts * sizeof(int), stream>>>(
            ids, chunk_scratch, sorted_pairs, pair_pos, pairs, pairs_per_chunk, n_experts);
    }
}

extern "C" void moe_route_sort_launcher(int* ids, float* weights, int* sorted_pairs, int* pair_pos,
                                        int* expert_offsets, int* chunk_scratch, const float* logits,
                                        int tokens, int n_experts, int top_k, int config,
                                        hipStream_t stream) {
    const int shared = (config & CONFIG_SHARED_SLOT) ? 1 : 0;
    config &= ~CONFIG_SHARED_SLOT;
    if (tokens <= 0) return;
    if (n_experts <= 0 || n_experts > 512 - shared || top_k <= 0 || top_k > 64 - shared ||
        top_k > n_experts) {
        caa::set_status(CAA_UNSUPPORTED_SHAPE);
        return;
    }
    if (!ids || !weights || !sorted_pairs || !pair_pos || !expert_offsets || !chunk_scratch || !logits) {
        caa::set_status(CAA_BAD_ARGUMENT);
        return;
    }
    if ((long)tokens * (top_k + shared) <= 1024 && config != 1 && config != 2) {
        // two launches: routing over many CUs, then the single-workgroup sort (config 2: the fused kernel)
        moe_route_launcher(ids, weights, logits, tokens, n_experts, top_k, shared ? CONFIG_SHARED_SLOT : 0, stream);
        moe_sort_small_kernel<<<1, 1024, 0, stream>>>(ids, sorted_pairs, pair_pos, expert_offsets,
                                                      tokens * (top_k + shared), n_experts + shared);
        return;
    }
    if ((long)tokens * (top_k + shared) <= 1024 && config == 2) {
        if (n_experts <= 256) {
            moe_route_sort_small_kernel<4><<<1, 1024, 0, stream>>>(
                logits, ids, weights, sorted_pairs, pair_pos, expert_offsets, tokens, n_experts, top_k,
                shared);
        } else {
            moe_route_sort_small_kernel<8><<<1, 1024, 0, stream>>>(
                logits, ids, weights, sorted_pairs, pair_pos, expert_offsets, tokens, n_experts, top_k,
                shared);
        }
        return;
    }
    moe_route_launcher(ids, weights, logits, tokens, n_experts, top_k, shared ? CONFIG_SHARED_SLOT : 0, stream);
    moe_sort_launcher(sorted_pairs, pair_pos, expert_offsets, chunk_scratch, ids, tokens,
                      n_experts + shared, top_k + shared, 0, stream);
}
