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

}  // namespace moe
