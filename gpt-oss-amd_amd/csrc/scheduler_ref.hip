// The reference's bucketing steps under their own argument lists (src/hip/scheduler.hip:11-61,
// 112-184; launched inline at src/forward.cpp:333-376), for a host loop that keeps those call sites:
// flatten + histogram, exclusive scan, compaction, heavy/light work queues.  Same inputs, same
// outputs; the one difference is that the compaction here lists every bucket in ascending
// assignment index instead of in the order atomic slot claims happen to finish, so the whole
// sequence is a pure function of its inputs.  moe_bucket_by_expert (bucket.hip) does the first three
// steps in one launch and is what the fused block uses.
#include "common.h"
#include "kernels.h"

namespace moe {

namespace {

// out_expert/out_token/out_w[idx] = (topk_i, idx / K, topk_v)[idx]; counts[e] += assignments to e.
// A block counts in LDS and adds each non-zero total once (integer adds: the sums do not depend on
// their order).  grid = ceil(BK / 4096) blocks of 1024 threads, dynamic LDS = E ints.
__global__ __launch_bounds__(1024) void flatten_count_kernel(const int* __restrict__ topk_i,
                                                             const float* __restrict__ topk_v, int BK, int K,
                                                             int* __restrict__ out_expert,
                                                             int* __restrict__ out_token,
                                                             float* __restrict__ out_w, int* __restrict__ counts,
                                                             int E) {
    extern __shared__ int hist[];
    for (int e = threadIdx.x; e < E; e += blockDim.x) hist[e] = 0;
    __syncthreads();
    const int base = blockIdx.x * 4096;
    int ids[4];
    float wv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {  // all loads first
        const int idx = base + u * 1024 + threadIdx.x;
        ids[u] = idx < BK ? topk_i[idx] : -1;
        wv[u] = idx < BK ? topk_v[idx] : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int idx = base + u * 1024 + threadIdx.x;
        if (idx < BK) {
            out_expert[idx] = ids[u];
            out_token[idx] = idx / K;
            out_w[idx] = wv[u];
            if ((unsigned)ids[u] < (unsigned)E) atomicAdd(&hist[ids[u]], 1);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x)
        if (hist[e]) atomicAdd(&counts[e], hist[e]);
}

// offsets[0] = 0, offsets[i + 1] = counts[0] + .. + counts[i]; counts[i] = 0.  One wave, 64 experts per
// step: inclusive scan on the data-parallel-primitive path, running total in a scalar.
__global__ __launch_bounds__(64) void scan_offsets_kernel(int* __restrict__ counts, int* __restrict__ offsets, int E) {
    const int lane = threadIdx.x;
    int total = 0;
    if (lane == 0) offsets[0] = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        const int e = e0 + lane;
        const int c = e < E ? counts[e] : 0;
        int incl = c;
        // shifts by 1, 2, 4, 8 inside rows of 16 lanes, then the sums of the rows before
        incl += (int)dpp_move<0x111, 0xf>(0u, (uint32_t)incl);
        incl += (int)dpp_move<0x112, 0xf>(0u, (uint32_t)incl);
        incl += (int)dpp_move<0x114, 0xf>(0u, (uint32_t)incl);
        incl += (int)dpp_move<0x118, 0xf>(0u, (uint32_t)incl);
        const int r0 = __builtin_amdgcn_readlane(incl, 15), r1 = __builtin_amdgcn_readlane(incl, 31),
                  r2 = __builtin_amdgcn_readlane(incl, 47), r3 = __builtin_amdgcn_readlane(incl, 63);
        const int row = lane >> 4;
        incl += (row > 0 ? r0 : 0) + (row > 1 ? r1 : 0) + (row > 2 ? r2 : 0);
        if (e < E) {
            offsets[e + 1] = total + incl;
            counts[e] = 0;
        }
        total += r0 + r1 + r2 + r3;
    }
}

// Bucket e = the assignments i with expert_ids[i] == e, in ascending i, at offsets[e] .. ; block per
// expert, 1024 assignments per step, positions from wave ballots and prefix counts.
// write_counters[e] ends up increased by the bucket's size, as after the reference's slot claims.
__global__ __launch_bounds__(1024) void compact_ordered_kernel(const int* __restrict__ expert_ids,
                                                               const int* __restrict__ tokens,
                                                               const float* __restrict__ weights, int BK,
                                                               const int* __restrict__ offsets,
                                                               int* __restrict__ write_counters,
                                                               int* __restrict__ tokens_flat,
                                                               float* __restrict__ weights_flat) {
    __shared__ int wave_cnt[16];
    const int e = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int first = offsets[e];
    int base = 0;
    for (int i0 = 0; i0 < BK; i0 += 4 * 1024) {
        int ids[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int i = i0 + u * 1024 + tid;
            ids[u] = i < BK ? expert_ids[i] : -1;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (i0 + u * 1024 >= BK) break;  // block-uniform
            const int i = i0 + u * 1024 + tid;
            const bool mine = ids[u] == e;
            const unsigned long long ballot = __ballot(mine);
            if (lane == 0) wave_cnt[wave] = __popcll(ballot);
            __syncthreads();
            int wave_base = 0, total = 0;
#pragma unroll
            for (int w = 0; w < 16; ++w) {
                const int c = wave_cnt[w];
                if (w < wave) wave_base += c;
                total += c;
            }
            if (mine) {
                const int dst = first + base + wave_base + __popcll(ballot & ((1ull << lane) - 1ull));
                tokens_flat[dst] = tokens[i];
                weights_flat[dst] = weights[i];
            }
            base += total;
            __syncthreads();
        }
    }
    if (tid == 0) write_counters[e] += base;
}

// Heavy / light work queues and their statistics (src/hip/scheduler.hip:112-184): an expert with rows
// is heavy if the active experts are at most very_sparse_cutoff, or if it has at least
// ceil(factor * average rows per active expert) rows, the factor being 1 up to very_sparse_cutoff
// active experts, heavy_factor_sparse up to 12, heavy_factor_default beyond.  Entries are (expert,
// row_offset, row_count) in ascending expert id.  One wave; counts by wave sums, positions by ballots.
__global__ __launch_bounds__(64) void classify_queues_kernel(const int* __restrict__ expert_offsets, int E,
                                                             int very_sparse_cutoff, float heavy_factor_sparse,
                                                             float heavy_factor_default, int* __restrict__ wq_heavy,
                                                             int* __restrict__ wq_light,
                                                             moe_queue_stats* __restrict__ stats_out) {
    const int lane = threadIdx.x;
    int active = 0, sum = 0;
    for (int e = lane; e < E; e += 64) {
        const int ne = expert_offsets[e + 1] - expert_offsets[e];
        if (ne > 0) {
            active += 1;
            sum += ne;
        }
    }
    active = wave_sum(active);
    sum = wave_sum(sum);
    if (active == 0) {  // wave-uniform
        if (lane == 0) *stats_out = moe_queue_stats{0, 0, 0, 0, 0};
        return;
    }
    const float avg = (float)(long long)sum / (float)active;
    float factor = heavy_factor_default;
    if (active <= very_sparse_cutoff) factor = 1.0f;
    else if (active <= 12) factor = heavy_factor_sparse;
    const int heavy_thresh = (int)ceilf(factor * avg);
    int n_heavy = 0, n_light = 0, heavy_max = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        const int e = e0 + lane;
        int off = 0, ne = 0;
        if (e < E) {
            off = expert_offsets[e];
            ne = expert_offsets[e + 1] - off;
        }
        const bool heavy = ne > 0 && (active <= very_sparse_cutoff || ne >= heavy_thresh);
        const bool light = ne > 0 && !heavy;
        const unsigned long long bh = __ballot(heavy), bl = __ballot(light);
        const unsigned long long below = (1ull << lane) - 1ull;
        if (heavy || light) {
            int* q = heavy ? wq_heavy : wq_light;
            const int dst = heavy ? n_heavy + __popcll(bh & below) : n_light + __popcll(bl & below);
            q[3 * dst + 0] = e;
            q[3 * dst + 1] = off;
            q[3 * dst + 2] = ne;
        }
        if (heavy) heavy_max = max(heavy_max, ne);
        n_heavy += __popcll(bh);
        n_light += __popcll(bl);
    }
#define MOE_STEP(C, M) heavy_max = max(heavy_max, (int)dpp_move<C, M>(0u, (uint32_t)heavy_max));
    MOE_DPP_STEPS(MOE_STEP)  // maximum of non-negative values: a lane without a source sees 0
#undef MOE_STEP
    heavy_max = __builtin_amdgcn_readlane(heavy_max, 63);
    if (lane == 0) *stats_out = moe_queue_stats{n_heavy, n_light, heavy_max, active, (long long)sum};
}

}  // namespace

int launch_count_tokens_per_expert(const int* topk_i, const float* topk_v, int B, int K, int* out_expert,
                                   int* out_token, float* out_w, int* counts, int E, hipStream_t stream) {
    const int BK = B * K;
    hipLaunchKernelGGL(flatten_count_kernel, dim3(ceil_div(BK, 4096)), dim3(1024), (size_t)E * sizeof(int), stream,
                       topk_i, topk_v, BK, K, out_expert, out_token, out_w, counts, E);
    return launch_status();
}

int launch_exclusive_scan_expert_offsets(int* counts, int* offsets, int E, hipStream_t stream) {
    hipLaunchKernelGGL(scan_offsets_kernel, dim3(1), dim3(64), 0, stream, counts, offsets, E);
    return launch_status();
}

int launch_compact_by_expert(const int* expert_ids, const int* tokens, const float* weights, int BK, const int* offsets,
                             int* write_counters, int* tokens_flat, float* weights_flat, int E, hipStream_t stream) {
    hipLaunchKernelGGL(compact_ordered_kernel, dim3(E), dim3(1024), 0, stream, expert_ids, tokens, weights, BK, offsets,
                       write_counters, tokens_flat, weights_flat);
    return launch_status();
}

int launch_classify_and_build_queues(const int* expert_offsets, int E, int very_sparse_cutoff,
                                     float heavy_factor_sparse, float heavy_factor_default, int* wq_heavy,
                                     int* wq_light, moe_queue_stats* stats, hipStream_t stream) {
    hipLaunchKernelGGL(classify_queues_kernel, dim3(1), dim3(64), 0, stream, expert_offsets, E, very_sparse_cutoff,
                       heavy_factor_sparse, heavy_factor_default, wq_heavy, wq_light, stats);
    return launch_status();
}

}  // namespace moe
