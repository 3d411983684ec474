// Expert token bucketing: histogram, exclusive scan, ordered compaction and the token-block map
// of the expert kernels in one launch.  Replaces count_tokens_per_expert /
// exclusive_scan_expert_offsets / compact_by_expert_kernel (src/hip/scheduler.hip:11-61), whose
// slot claim by atomicAdd leaves the order inside a bucket to chance; here every bucket lists its
// tokens in ascending token id (wave ballot + lane prefix count), so the output is a pure function
// of topk_i.
#include "common.h"
#include "kernels.h"

namespace moe {

// grid = E blocks (one expert each), block = 1024 threads, dynamic LDS = (E + 32) ints.
__global__ __launch_bounds__(1024) void bucket_kernel(const int* __restrict__ topk_i,
                                                      const float* __restrict__ topk_v, int T, int K, int E,
                                                      int* __restrict__ expert_offsets,
                                                      int* __restrict__ tokens_flat,
                                                      float* __restrict__ weights_flat,
                                                      int* __restrict__ slot_of, TileMap map) {
    extern __shared__ int lds[];
    int* hist = lds;           // [E]
    int* wave_cnt = lds + E;   // [16]
    int* scal = lds + E + 16;  // [0] rows before this expert, [1] tiles before this expert
    const int e = blockIdx.x;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int A = T * K;

    for (int i = tid; i < E; i += blockDim.x) hist[i] = 0;
    if (tid < 2) scal[tid] = 0;
    __syncthreads();
    for (int a = tid; a < A; a += blockDim.x) {
        const int id = topk_i[a];
        if ((unsigned)id < (unsigned)E) atomicAdd(&hist[id], 1);
    }
    __syncthreads();
    const int nb = map.tile_tokens;
    {
        int rows_before = 0, tiles_before = 0;
        for (int i = tid; i < e; i += blockDim.x) {
            const int c = hist[i];
            rows_before += c;
            if (nb > 0) tiles_before += (c + nb - 1) / nb;
        }
        if (rows_before) atomicAdd(&scal[0], rows_before);
        if (tiles_before) atomicAdd(&scal[1], tiles_before);
    }
    __syncthreads();
    const int my_off = scal[0];
    const int my_cnt = hist[e];
    const int my_tile0 = scal[1];
    if (tid == 0) {
        expert_offsets[e] = my_off;
        if (e == E - 1) expert_offsets[E] = my_off + my_cnt;
    }
    if (nb > 0) {
        const int my_tiles = (my_cnt + nb - 1) / nb;
        for (int j = tid; j < my_tiles; j += blockDim.x) {
            map.tile_expert[my_tile0 + j] = e;
            map.tile_row0[my_tile0 + j] = my_off + j * nb;
            map.tile_rows[my_tile0 + j] = min(nb, my_cnt - j * nb);
        }
        if (e == E - 1 && tid == 0) *map.n_tiles = my_tile0 + my_tiles;
    }

    // ordered compaction: tokens visited in ascending id, blockDim tokens per step
    int base = my_off;
    for (int t0 = 0; t0 < T; t0 += blockDim.x) {
        const int t = t0 + tid;
        int mk = -1;
        if (t < T) {
            for (int k = 0; k < K; ++k)
                if (topk_i[(size_t)t * K + k] == e) {
                    mk = k;
                    break;
                }
        }
        const unsigned long long ballot = __ballot(mk >= 0);
        const int prefix = __popcll(ballot & ((1ull << lane) - 1ull));
        if (lane == 0) wave_cnt[wave] = __popcll(ballot);
        __syncthreads();
        int wave_base = 0, total = 0;
        const int n_waves = blockDim.x >> 6;
        for (int w = 0; w < n_waves; ++w) {
            const int c = wave_cnt[w];
            if (w < wave) wave_base += c;
            total += c;
        }
        if (mk >= 0) {
            const int dst = base + wave_base + prefix;
            tokens_flat[dst] = t;
            weights_flat[dst] = topk_v[(size_t)t * K + mk];
            if (slot_of) slot_of[(size_t)t * K + mk] = dst;
        }
        base += total;
        __syncthreads();
    }
}

int launch_bucket(const int* topk_i, const float* topk_v, int T, int K, int E, int* expert_offsets,
                  int* tokens_flat, float* weights_flat, int* slot_of, TileMap map, hipStream_t stream) {
    hipLaunchKernelGGL(bucket_kernel, dim3(E), dim3(1024), (size_t)(E + 32) * sizeof(int), stream, topk_i, topk_v,
                       T, K, E, expert_offsets, tokens_flat, weights_flat, slot_of, map);
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

int launch_gather_rows(const float* X, const int* idx, float* Y, int rows, int H, hipStream_t stream) {
    const int H4 = H / 4;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(ceil_div(H4, 256), rows), dim3(256), 0, stream,
                       reinterpret_cast<const float4*>(X), idx, reinterpret_cast<float4*>(Y), rows, H4);
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
    hipLaunchKernelGGL(scatter_rows_kernel, dim3(ceil_div(H4, 256), rows), dim3(256), 0, stream,
                       reinterpret_cast<const float4*>(Y), idx, reinterpret_cast<float4*>(X), rows, H4);
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
