// MXFP4 (e2m1 codes + e8m0 block scales) support: reference-exact dequantisation, the load-time
// repack into the tiled layout the fused expert kernels stream, its inverse, and a tiled -> bf16
// expansion through the same conversion the fused kernels use.
// Arithmetic contract: tools/model_export/gpt-oss-20b/export_model_bin.py:75-133.
#include "common.h"
#include "kernels.h"

namespace moe {

// ---- canonical layout -> bf16, every scale byte ------------------------------------------------
// One thread per MX block: 16 bytes in, 32 bf16 (64 bytes) out.
__global__ __launch_bounds__(256) void dequant_mxfp4_kernel(const u32x4* __restrict__ blocks,
                                                            const uint8_t* __restrict__ scales,
                                                            long long n_blocks, u32x4* __restrict__ out) {
    const long long b = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n_blocks) return;
    const u32x4 raw = blocks[b];
    const uint32_t s = scales[b];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t w = raw[d];
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t byte = (w >> (8 * i)) & 0xFFu;
            o[i] = mxfp4_code_to_bf16_bits(byte & 0xFu, s) | (mxfp4_code_to_bf16_bits(byte >> 4, s) << 16);
        }
        out[b * 4 + d] = o;
    }
}

int launch_dequant_mxfp4(const uint8_t* blocks, const uint8_t* scales, long long n_blocks, uint16_t* out,
                         hipStream_t stream) {
    const unsigned grid = (unsigned)ceil_div(n_blocks, (long long)256);
    hipLaunchKernelGGL(dequant_mxfp4_kernel, dim3(grid), dim3(256), 0, stream,
                       reinterpret_cast<const u32x4*>(blocks), scales, n_blocks, reinterpret_cast<u32x4*>(out));
    return launch_status();
}

// ---- tiled layout ------------------------------------------------------------------------------
// Per expert, weight rows are taken in groups of 64; each group is four MFMA row tiles of 16 rows
// (row order inside the group: tile_row_in_group).  A tile stores its K/32 MX blocks chunk by
// chunk, a chunk being four consecutive MX blocks (128 elements) of all 16 rows:
//     blocks : tile t, chunk c, lane l = (blk%4)*16 + q, 16 bytes      -> t*G*256 + c*1024 + l*16
//              (a ragged last chunk holds only its G%4 block columns)
//     scales : tile t, chunk quad c/4, lane l, byte c%4               -> t*SQ*256 + (c/4)*256 + l*4 + c%4
// with G = K/32 and SQ = ceil(ceil(G/4)/4).  One wave-wide 128-bit load fetches one chunk of a tile
// (1 KiB, contiguous); one dword load per lane fetches the scales of four chunks.
void mxfp4_tiled_bytes(int rows, int K, size_t* block_bytes, size_t* scale_bytes) {
    const int G = K / 32;
    const size_t tiles = (size_t)(rows / 64) * 4;
    if (block_bytes) *block_bytes = tiles * (size_t)G * 256;
    if (scale_bytes) *scale_bytes = tiles * (size_t)ceil_div(ceil_div(G, 4), 4) * 256;
}

struct TiledAddr {
    size_t block_off;
    size_t scale_off;
};

MOE_DEVICE TiledAddr tiled_addr(int e, int row, int blk, int G, size_t block_bytes, size_t scale_bytes) {
    const int group = row >> 6;
    const int i = row & 63;
    const int r = (i & 15) >> 2;
    const int q = ((i >> 4) << 2) | (i & 3);
    const size_t tile = (size_t)group * 4 + r;
    const int c = blk >> 2;
    const int lane = ((blk & 3) << 4) | q;
    const int SQ = (((G + 3) >> 2) + 3) >> 2;
    TiledAddr a;
    a.block_off = (size_t)e * block_bytes + tile * (size_t)G * 256 + (size_t)c * 1024 + (size_t)lane * 16;
    a.scale_off = (size_t)e * scale_bytes + tile * (size_t)SQ * 256 + (size_t)(c >> 2) * 256 + (size_t)lane * 4 + (c & 3);
    return a;
}

template <bool INVERSE>
__global__ __launch_bounds__(256) void mxfp4_repack_kernel(const uint8_t* __restrict__ src_blocks,
                                                           const uint8_t* __restrict__ src_scales,
                                                           uint8_t* __restrict__ dst_blocks,
                                                           uint8_t* __restrict__ dst_scales, int E, int rows, int G,
                                                           size_t block_bytes, size_t scale_bytes) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long total = (long long)E * rows * G;
    if (idx >= total) return;
    const int blk = (int)(idx % G);
    const long long er = idx / G;
    const int row = (int)(er % rows);
    const int e = (int)(er / rows);
    const TiledAddr t = tiled_addr(e, row, blk, G, block_bytes, scale_bytes);
    if (!INVERSE) {
        *reinterpret_cast<u32x4*>(dst_blocks + t.block_off) = *reinterpret_cast<const u32x4*>(src_blocks + idx * 16);
        dst_scales[t.scale_off] = src_scales[idx];
    } else {
        *reinterpret_cast<u32x4*>(dst_blocks + idx * 16) = *reinterpret_cast<const u32x4*>(src_blocks + t.block_off);
        dst_scales[idx] = src_scales[t.scale_off];
    }
}

__global__ void fill_zero_kernel(uint32_t* __restrict__ p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

int launch_fill_zero(uint32_t* words, size_t n, hipStream_t stream) {
    if (n == 0) return MOE_OK;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)ceil_div(n, (size_t)256)), dim3(256), 0, stream, words, n);
    return launch_status();
}

int launch_mxfp4_repack(const uint8_t* blocks, const uint8_t* scales, int E, int rows, int K,
                        uint8_t* tiled_blocks, uint8_t* tiled_scales, bool inverse, hipStream_t stream) {
    const int G = K / 32;
    size_t bb, sb;
    mxfp4_tiled_bytes(rows, K, &bb, &sb);
    const long long total = (long long)E * rows * G;
    const unsigned grid = (unsigned)ceil_div(total, (long long)256);
    if (!inverse) {
        // scale slots of a ragged last chunk quad are never written by the scatter below
        const size_t nwords = (size_t)E * sb / 4;
        hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)ceil_div(nwords, (size_t)256)), dim3(256), 0, stream,
                           reinterpret_cast<uint32_t*>(tiled_scales), nwords);
        hipLaunchKernelGGL(mxfp4_repack_kernel<false>, dim3(grid), dim3(256), 0, stream, blocks, scales,
                           tiled_blocks, tiled_scales, E, rows, G, bb, sb);
    } else {
        // here `blocks`/`scales` are the canonical destination, tiled_* the source
        hipLaunchKernelGGL(mxfp4_repack_kernel<true>, dim3(grid), dim3(256), 0, stream, tiled_blocks, tiled_scales,
                           const_cast<uint8_t*>(blocks), const_cast<uint8_t*>(scales), E, rows, G, bb, sb);
    }
    return launch_status();
}

// Tiled -> row-major bf16 [E, rows, K] through mxfp4_dword_to_bf16x8, the conversion of the fused
// expert kernels.
__global__ __launch_bounds__(256) void mxfp4_tiled_to_bf16_kernel(const uint8_t* __restrict__ tiled_blocks,
                                                                  const uint8_t* __restrict__ tiled_scales,
                                                                  u32x4* __restrict__ out, int E, int rows, int G,
                                                                  size_t block_bytes, size_t scale_bytes) {
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long total = (long long)E * rows * G;
    if (idx >= total) return;
    const int blk = (int)(idx % G);
    const long long er = idx / G;
    const int row = (int)(er % rows);
    const int e = (int)(er / rows);
    const TiledAddr t = tiled_addr(e, row, blk, G, block_bytes, scale_bytes);
    const u32x4 raw = *reinterpret_cast<const u32x4*>(tiled_blocks + t.block_off);
    const float sc = mxfp4_scale_to_f32(tiled_scales[t.scale_off]);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        uint32_t o[4];
        mxfp4_dword_to_bf16x8(raw[d], sc, o);
        out[idx * 4 + d] = u32x4{o[0], o[1], o[2], o[3]};
    }
}

int launch_mxfp4_tiled_to_bf16(const uint8_t* tiled_blocks, const uint8_t* tiled_scales, int E, int rows, int K,
                               uint16_t* out, hipStream_t stream) {
    const int G = K / 32;
    size_t bb, sb;
    mxfp4_tiled_bytes(rows, K, &bb, &sb);
    const long long total = (long long)E * rows * G;
    hipLaunchKernelGGL(mxfp4_tiled_to_bf16_kernel, dim3((unsigned)ceil_div(total, (long long)256)), dim3(256), 0,
                       stream, tiled_blocks, tiled_scales, reinterpret_cast<u32x4*>(out), E, rows, G, bb, sb);
    return launch_status();
}

}  // namespace moe
