// Expert token bucketing: histogram, exclusive scan, ordered compaction and the token-block map
// of the expert kernels in one launch.  Replaces count_tokens_per_expert /
// exclusive_scan_expert_offsets / compact_by_expert_kernel (src/hip/scheduler.hip:11-61), whose
// slot claim by atomicAdd leaves the order inside a bucket to chance; here every bucket lists its
// tokens in ascending token id (wave ballot + lane prefix count), so the output is a pure function
// of topk_i.
#include "common.h"
#include "kernels.h"

namespace moe {

// Copies of the histogram in LDS: a wave's atomic adds go to random experts, and adds of several
// lanes to one counter run one after the other; with one copy per lane (mod kHistCopies, the copy
// index being the bank) two lanes meet only when they are 32 apart.
constexpr int kHistCopies = 32;
static int hist_copies(int E) { return E <= 256 ? kHistCopies : E <= 512 ? 16 : 8; }

// grid = E blocks (one expert each), block = 1024 threads, dynamic LDS = (E * copies + E + 32) ints.
// Tile map order: every full tile first (ascending expert), then the experts' partial last tiles from
// the largest to the smallest (equal sizes: ascending expert).  An expert kernel that takes tiles in
// this order runs its shortest blocks last, next to compute units that have already run out of work.
// With map.second > 0 the same tiles are listed a second time, from index map.second of the three
// arrays, in bucket order (an expert's tiles together, the partial one last).
__global__ __launch_bounds__(1024) void bucket_kernel(const int* __restrict__ topk_i,
                                                      const float* __restrict__ topk_v, int T, int K, int E,
                                                      int copies, int* __restrict__ expert_offsets,
                                                      int* __restrict__ tokens_flat,
                                                      float* __restrict__ weights_flat,
                                                      int* __restrict__ slot_of, TileMap map) {
    extern __shared__ int lds[];
    __shared__ int wave_cnt[4 * 16];  // matches per wave of the four compaction steps in flight
    int* hist = lds;                  // [E]
    int* scal = lds + E + 16;         // [0] rows before this expert, [1] full tiles before it, [2] full tiles in all,
                                      // [3] partial tiles ahead of this expert's (by size), [4] partial tiles in all,
                                      // [5] partial tiles of the experts before this one
    int* hist_c = lds + E + 32;       // [E][copies]
    const int e = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int A = T * K;

    for (int i = tid; i < E * copies; i += blockDim.x) hist_c[i] = 0;
    if (tid < 8) scal[tid] = 0;
    __syncthreads();
    const int my_copy = tid & (copies - 1);
    // eight loads per thread in flight: the pass costs memory round trips, not adds
    for (int a0 = tid; a0 < A; a0 += 8 * 1024) {
        int id[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) id[u] = a0 + u * 1024 < A ? topk_i[a0 + u * 1024] : -1;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if ((unsigned)id[u] < (unsigned)E) atomicAdd(&hist_c[id[u] * copies + my_copy], 1);
    }
    __syncthreads();
    for (int i = tid; i < E; i += blockDim.x) {
        int c = 0;
        for (int j = 0; j < copies; ++j) c += hist_c[i * copies + ((j + i) & (copies - 1))];  // rotated: no common bank
        hist[i] = c;
    }
    __syncthreads();
    const int nb = map.tile_tokens;
    const int my_cnt = hist[e];
    {
        const int my_rem = nb > 0 ? my_cnt % nb : 0;
        int rows_before = 0, full_before = 0, full_all = 0, part_ahead = 0, part_all = 0, part_before = 0;
        for (int i = tid; i < E; i += blockDim.x) {
            const int c = hist[i];
            if (i < e) rows_before += c;
            if (nb > 0) {
                const int full = c / nb, rem = c - full * nb;
                full_all += full;
                if (i < e) full_before += full;
                if (rem > 0) {
                    part_all += 1;
                    if (i < e) part_before += 1;
                    if (rem > my_rem || (rem == my_rem && i < e)) part_ahead += 1;
                }
            }
        }
        // wave sums first, one add per wave and quantity (an atomic add of a different value per lane
        // is carried out lane by lane)
        int sums[6] = {rows_before, full_before, full_all, part_ahead, part_all, part_before};
        if (wave * 64 < E) {  // wave-uniform: later waves hold zeros
#pragma unroll
            for (int i = 0; i < 6; ++i) {
                const int total = wave_sum(sums[i]);
                if (lane == 0 && total) atomicAdd(&scal[i], total);
            }
        }
    }
    __syncthreads();
    const int my_off = scal[0];
    if (tid == 0) {
        expert_offsets[e] = my_off;
        if (e == E - 1) expert_offsets[E] = my_off + my_cnt;
    }
    if (nb > 0) {
        const int my_full = my_cnt / nb;
        const int my_rem = my_cnt - my_full * nb;
        for (int j = tid; j < my_full; j += blockDim.x) {
            map.tile_expert[scal[1] + j] = e;
            map.tile_row0[scal[1] + j] = my_off + j * nb;
            map.tile_rows[scal[1] + j] = nb;
        }
        if (my_rem > 0 && tid == 0) {
            const int at = scal[2] + scal[3];
            map.tile_expert[at] = e;
            map.tile_row0[at] = my_off + my_full * nb;
            map.tile_rows[at] = my_rem;
        }
        if (map.second > 0) {  // the same tiles in bucket order: an expert's tiles together, its partial one last
            const int first = map.second + scal[1] + scal[5];
            for (int j = tid; j < my_full + (my_rem > 0); j += blockDim.x) {
                map.tile_expert[first + j] = e;
                map.tile_row0[first + j] = my_off + j * nb;
                map.tile_rows[first + j] = min(nb, my_cnt - j * nb);
            }
        }
        if (e == E - 1 && tid == 0) *map.n_tiles = scal[2] + scal[4];
    }

    // ordered compaction: tokens visited in ascending id, 1024 tokens per step; the ids of four steps
    // are fetched together (K <= 8 per token)
    int base = my_off;
    for (int t00 = 0; t00 < T; t00 += 4 * 1024) {
        int mk4[4];
        float wv4[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = t00 + u * 1024 + tid;
            int ids[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) ids[k] = (t < T && k < K) ? topk_i[(size_t)t * K + k] : -1;
            int mk = -1;
#pragma unroll
            for (int k = 7; k >= 0; --k) mk = ids[k] == e ? k : mk;  // the first k that names this expert
            mk4[u] = mk;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {  // the matching routing weights, again before anything waits
            const int t = t00 + u * 1024 + tid;
            wv4[u] = mk4[u] >= 0 ? topk_v[(size_t)t * K + mk4[u]] : 0.f;
        }
        // the four steps' wave counts go through LDS together: one exchange (two barriers) per 4096 tokens
        int prefix4[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const unsigned long long ballot = __ballot(mk4[u] >= 0);
            prefix4[u] = __popcll(ballot & ((1ull << lane) - 1ull));
            if (lane == 0) wave_cnt[u * 16 + wave] = __popcll(ballot);
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int t = t00 + u * 1024 + tid;
            int wave_base = 0, total = 0;
#pragma unroll
            for (int w = 0; w < 16; ++w) {
                const int c = wave_cnt[u * 16 + w];
                if (w < wave) wave_base += c;
                total += c;
            }
            if (mk4[u] >= 0) {
                const int dst = base + wave_base + prefix4[u];
                tokens_flat[dst] = t;
                weights_flat[dst] = wv4[u];
                if (slot_of) slot_of[(size_t)t * K + mk4[u]] = dst;
            }
            base += total;
        }
        __syncthreads();
    }
}

int launch_bucket(const int* topk_i, const float* topk_v, int T, int K, int E, int* expert_offsets,
                  int* tokens_flat, float* weights_flat, int* slot_of, TileMap map, hipStream_t stream) {
    const int copies = hist_copies(E);
    hipLaunchKernelGGL(bucket_kernel, dim3(E), dim3(1024), (size_t)(E * copies + E + 32) * sizeof(int), stream, topk_i,
                       topk_v, T, K, E, copies, expert_offsets, tokens_flat, weights_flat, slot_of, map);
    return launch_status();
}

// Y[row,:] = X[idx[row],:], fp32 rows of H (H % 4 == 0).  src/hip/scheduler.hip:63-85.
__global__ void gather_rows_kernel(const float4* __restrict__ X, const int* __restrict__ idx,
                                   float4* __restrict__ Y, int rows, int H4) {
    const int row = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows || c >= H4) return;
    Y[(size_t)row * H4 + c] = X[(size_t)idx[row] * H4 + c];
}

// One grid row per table row: launched in slabs of kMaxGridRows rows (the grid's y limit).
constexpr int kMaxGridRows = 65535;

int launch_gather_rows(const float* X, const int* idx, float* Y, int rows, int H, hipStream_t stream) {
    const int H4 = H / 4;
    for (int r0 = 0; r0 < rows; r0 += kMaxGridRows) {
        const int n = rows - r0 < kMaxGridRows ? rows - r0 : kMaxGridRows;
        hipLaunchKernelGGL(gather_rows_kernel, dim3(ceil_div(H4, 256), n), dim3(256), 0, stream,
                           reinterpret_cast<const float4*>(X), idx + r0, reinterpret_cast<float4*>(Y) + (size_t)r0 * H4, n,
                           H4);
    }
    return launch_status();
}

// X[idx[row],:] = Y[row,:]: the inverse of gather_rows (rows of a compact batch back to the table
// rows they were gathered from; idx must not repeat).
__global__ void scatter_rows_kernel(const float4* __restrict__ Y, const int* __restrict__ idx,
                                    float4* __restrict__ X, int rows, int H4) {
    const int row = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows || c >= H4) return;
    X[(size_t)idx[row] * H4 + c] = Y[(size_t)row * H4 + c];
}

int launch_scatter_rows(const float* Y, const int* idx, float* X, int rows, int H, hipStream_t stream) {
    const int H4 = H / 4;
    for (int r0 = 0; r0 < rows; r0 += kMaxGridRows) {
        const int n = rows - r0 < kMaxGridRows ? rows - r0 : kMaxGridRows;
        hipLaunchKernelGGL(scatter_rows_kernel, dim3(ceil_div(H4, 256), n), dim3(256), 0, stream,
                           reinterpret_cast<const float4*>(Y) + (size_t)r0 * H4, idx + r0, reinterpret_cast<float4*>(X), n,
                           H4);
    }
    return launch_status();
}

// (expert, row_offset, row_count) triples of the non-empty experts, ascending expert id
// (entry format of src/hip/scheduler.hip:163-166).  One wave; ballot + prefix count per 64 experts.
__global__ __launch_bounds__(64) void work_queue_kernel(const int* __restrict__ expert_offsets, int E,
                                                        int* __restrict__ work_queue,
                                                        int* __restrict__ work_count) {
    const int lane = threadIdx.x;
    int base = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
        const int e = e0 + lane;
        int off = 0, ne = 0;
        if (e < E) {
            off = expert_offsets[e];
            ne = expert_offsets[e + 1] - off;
        }
        const unsigned long long ballot = __ballot(ne > 0);
        if (ne > 0) {
            const int dst = base + __popcll(ballot & ((1ull << lane) - 1ull));
            work_queue[3 * dst + 0] = e;
            work_queue[3 * dst + 1] = off;
            work_queue[3 * dst + 2] = ne;
        }
        base += __popcll(ballot);
    }
    if (lane == 0) *work_count = base;
}

int launch_build_work_queue(const int* expert_offsets, int E, int* work_queue, int* work_count,
                            hipStream_t stream) {
    hipLaunchKernelGGL(work_queue_kernel, dim3(1), dim3(64), 0, stream, expert_offsets, E, work_queue, work_count);
    return launch_status();
}

}  // namespace moe
