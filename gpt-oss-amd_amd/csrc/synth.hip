// Device side of the counter-based synthetic tensor generator (include/moe_synth.h): identical
// integer mixing and table lookup as the host loops, so device-filled buffers match host-filled
// ones bit for bit.
#include "common.h"
#include "kernels.h"
#include "../../include/moe_synth.h"

namespace moe {

enum { SYNTH_NORMAL_F32 = 0, SYNTH_NORMAL_BF16 = 1, SYNTH_BYTES = 2, SYNTH_RANGE_BYTES = 3 };

template <int KIND>
__global__ __launch_bounds__(256) void synth_kernel(void* __restrict__ dst, long long n,
                                                    const float* __restrict__ table, float scale, unsigned seed,
                                                    unsigned tensor_id, unsigned lo, unsigned span) {
    // four consecutive elements per thread keep byte stores dword-sized
    const long long i0 = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i0 >= n) return;
    if constexpr (KIND == SYNTH_NORMAL_F32) {
        float* d = static_cast<float*>(dst);
        for (int j = 0; j < 4 && i0 + j < n; ++j)
            d[i0 + j] = moe_synth_normal_f32(table, scale, seed, tensor_id, (uint64_t)(i0 + j));
    } else if constexpr (KIND == SYNTH_NORMAL_BF16) {
        uint16_t* d = static_cast<uint16_t*>(dst);
        for (int j = 0; j < 4 && i0 + j < n; ++j)
            d[i0 + j] = moe_synth_normal_bf16(table, scale, seed, tensor_id, (uint64_t)(i0 + j));
    } else if constexpr (KIND == SYNTH_BYTES) {
        uint8_t* d = static_cast<uint8_t*>(dst);
        if (i0 + 4 <= n) {
            uint32_t w = 0;
            for (int j = 0; j < 4; ++j) w |= (uint32_t)moe_synth_byte(seed, tensor_id, (uint64_t)(i0 + j)) << (8 * j);
            *reinterpret_cast<uint32_t*>(d + i0) = w;
        } else {
            for (int j = 0; i0 + j < n; ++j) d[i0 + j] = moe_synth_byte(seed, tensor_id, (uint64_t)(i0 + j));
        }
    } else {
        uint8_t* d = static_cast<uint8_t*>(dst);
        if (i0 + 4 <= n) {
            uint32_t w = 0;
            for (int j = 0; j < 4; ++j)
                w |= (uint32_t)moe_synth_range_byte(seed, tensor_id, (uint64_t)(i0 + j), lo, span) << (8 * j);
            *reinterpret_cast<uint32_t*>(d + i0) = w;
        } else {
            for (int j = 0; i0 + j < n; ++j)
                d[i0 + j] = moe_synth_range_byte(seed, tensor_id, (uint64_t)(i0 + j), lo, span);
        }
    }
}

int launch_synth(int kind, void* dst, long long n, const float* table, float scale, unsigned seed,
                 unsigned tensor_id, unsigned lo, unsigned span, hipStream_t stream) {
    const long long threads = (n + 3) / 4;
    const long long blocks = (threads + 255) / 256;
    if (blocks > 0x7FFFFFFFll) return MOE_ERR_LIMIT;
    const dim3 grid((unsigned)blocks), block(256);
    switch (kind) {
        case SYNTH_NORMAL_F32:
            hipLaunchKernelGGL(synth_kernel<SYNTH_NORMAL_F32>, grid, block, 0, stream, dst, n, table, scale, seed, tensor_id, lo, span);
            break;
        case SYNTH_NORMAL_BF16:
            hipLaunchKernelGGL(synth_kernel<SYNTH_NORMAL_BF16>, grid, block, 0, stream, dst, n, table, scale, seed, tensor_id, lo, span);
            break;
        case SYNTH_BYTES:
            hipLaunchKernelGGL(synth_kernel<SYNTH_BYTES>, grid, block, 0, stream, dst, n, table, scale, seed, tensor_id, lo, span);
            break;
        case SYNTH_RANGE_BYTES:
            hipLaunchKernelGGL(synth_kernel<SYNTH_RANGE_BYTES>, grid, block, 0, stream, dst, n, table, scale, seed, tensor_id, lo, span);
            break;
        default:
            return MOE_ERR_FORMAT;
    }
    return launch_status();
}

// Sum of a buffer's 32-bit words modulo 2^64: a plain streaming read (every byte fetched once, 16 bytes per lane and
// load, nothing written but one partial per block), so its duration over a buffer much larger than the caches is the
// read rate the memory system sustains.  A block takes chunks of 256 x 4 sixteen-byte words in grid-stride order.
constexpr int kChecksumUnroll = 4;

__global__ __launch_bounds__(256) void synth_checksum_kernel(const u32x4* __restrict__ src, long long n16,
                                                             unsigned long long* __restrict__ partials) {
    unsigned long long acc = 0;
    const long long stride = (long long)gridDim.x * 256 * kChecksumUnroll;
    long long i = (long long)blockIdx.x * 256 * kChecksumUnroll + threadIdx.x;
    for (; i + 256 * (kChecksumUnroll - 1) < n16; i += stride) {
        u32x4 v[kChecksumUnroll];
#pragma unroll
        for (int j = 0; j < kChecksumUnroll; ++j) v[j] = __builtin_nontemporal_load(src + i + 256 * j);
#pragma unroll
        for (int j = 0; j < kChecksumUnroll; ++j)
            acc += (unsigned long long)v[j].x + v[j].y + (unsigned long long)v[j].z + v[j].w;
    }
    // at most one partly filled chunk is left for this thread (the next one starts a whole stride further on)
    for (int j = 0; j < kChecksumUnroll; ++j) {
        const long long k = i + 256 * j;
        if (k < n16) {
            const u32x4 v = __builtin_nontemporal_load(src + k);
            acc += (unsigned long long)v.x + v.y + (unsigned long long)v.z + v.w;
        }
    }
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    __shared__ unsigned long long wave_sum[4];
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) partials[blockIdx.x] = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
}

__global__ __launch_bounds__(256) void synth_checksum_final_kernel(const unsigned long long* __restrict__ partials,
                                                                   int n, unsigned long long* __restrict__ out) {
    unsigned long long acc = 0;
    for (int i = threadIdx.x; i < n; i += 256) acc += partials[i];
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_down(acc, off, 64);
    __shared__ unsigned long long wave_sum[4];
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) out[0] = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
}

int launch_synth_checksum(const void* src, long long n_bytes, unsigned long long* out, int max_partials,
                          hipStream_t stream) {
    const long long n16 = n_bytes / 16;
    const long long chunks = (n16 + 256 * kChecksumUnroll - 1) / (256 * kChecksumUnroll);
    // eight 4-wave blocks per CU fill every wave slot of a 256-CU part; fewer for a short buffer
    const int blocks = (int)(chunks < (long long)max_partials ? chunks : (long long)max_partials);
    if (blocks < 1) return MOE_ERR_SHAPE;
    hipLaunchKernelGGL(synth_checksum_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       static_cast<const u32x4*>(src), n16, out + 1);
    hipLaunchKernelGGL(synth_checksum_final_kernel, dim3(1), dim3(256), 0, stream, out + 1, blocks, out);
    return launch_status();
}

}  // namespace moe
