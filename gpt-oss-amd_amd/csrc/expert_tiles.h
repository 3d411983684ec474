// Pieces shared by the expert GEMM kernels (experts_stream.hip, experts_fused.hip): weight formats and
// epilogue kinds, the LDS image of an activation stage, the direct-to-LDS load, and the epilogue that
// turns a wave's accumulators into SwiGLU outputs or per-slot rows.
#pragma once
#include "common.h"
#include "kernels.h"

namespace moe {
namespace {

constexpr int FMT_BF16 = MOE_WEIGHTS_BF16;
constexpr int FMT_MXFP4 = MOE_WEIGHTS_MXFP4_TILED;

// Epilogues: the fused block keeps bf16 SwiGLU outputs and fp32 per-slot rows; the entries that
// keep the reference's data flow write fp32 SwiGLU outputs and scatter with atomics.
enum { EPI_SWIGLU_BF16 = 0, EPI_ROWS_F32 = 1, EPI_SWIGLU_F32 = 2, EPI_SCATTER = 3 };

constexpr int kStageSteps = 4;                                  // MFMA k-steps per LDS stage
constexpr int kStageElems = 32 * kStageSteps;                   // 128 contraction elements
constexpr int kNTMax = 4;                                       // token tiles (of 16) per block
constexpr int kLdsStageBytes = kStageSteps * kNTMax * 1024;     // 16 KiB, two of them per block

// Epilogue shared by the expert kernels: lane (q,g) of the 16x16 accumulator layout holds token
// t*16+q and weight rows group*64 + g*16 + (r0+r)*4 + j (j = 0..3) for its R row tiles.
// The four bias values per row tile of a lane; loaded before the main loop by the kernels that
// want the load latency off the block's tail.
template <int R>
MOE_DEVICE void load_bias(const ExpertGemmArgs& a, int e, int group, int r0, uint2 (&raw)[R]) {
    const int g = (threadIdx.x & 63) >> 4;
    const uint16_t* bias = a.bias + (size_t)e * a.bias_expert_stride + group * 64 + g * 16 + r0 * 4;
#pragma unroll
    for (int r = 0; r < R; ++r) raw[r] = *reinterpret_cast<const uint2*>(bias + 4 * r);
}

// slot_of_row(i): output row (slot) of bucket row i of the token block.
template <int R, int NT, int EPI, class SlotFn>
MOE_DEVICE void stream_epilogue(const ExpertGemmArgs& a, const f32x4 (&acc)[R][NT], int e, SlotFn slot_of_row, int nrows,
                                int group, int r0, const uint2 (&bias_raw)[R]) {
    const int lane = threadIdx.x & 63;
    const int q = lane & 15;
    const int g = lane >> 4;
    const int row_base = group * 64 + g * 16 + r0 * 4;
    float bv[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint2 raw = bias_raw[r];
        bv[r][0] = bf16_bits_to_f32(raw.x & 0xFFFFu);
        bv[r][1] = bf16_bits_to_f32(raw.x >> 16);
        bv[r][2] = bf16_bits_to_f32(raw.y & 0xFFFFu);
        bv[r][3] = bf16_bits_to_f32(raw.y >> 16);
    }
    if constexpr (EPI == EPI_ROWS_F32 && R == 4) {
        // Four row tiles per lane: lane (q, g) holds, for its token, the four 16-byte pieces g*64 + r*16 of a
        // 256-byte stretch of the output row, so one store instruction would touch 64 pieces that are 64 bytes
        // apart.  A 4x4 transpose between the four lane rows (g) and the four row tiles (r), two lane-row
        // swaps per value, leaves lane (q, g) with the pieces r*64 + g*16: a store instruction then writes
        // 64 contiguous bytes per token (four lanes), a quarter of the write requests.
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            uint32_t v[4][4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j) v[r][j] = __float_as_uint(acc[r][t][j] + bv[r][j]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int r = 0; r < 2; ++r) {  // lanes 32..63 of tile r <-> lanes 0..31 of tile r + 2
                    const auto sw = __builtin_amdgcn_permlane32_swap(v[r][j], v[r + 2][j], false, false);
                    v[r][j] = sw[0];
                    v[r + 2][j] = sw[1];
                }
#pragma unroll
                for (int r = 0; r < 4; r += 2) {  // odd lane rows of tile r <-> even lane rows of tile r + 1
                    const auto sw = __builtin_amdgcn_permlane16_swap(v[r][j], v[r + 1][j], false, false);
                    v[r][j] = sw[0];
                    v[r + 1][j] = sw[1];
                }
            }
            const int idx = t * 16 + q;
            if (idx < nrows) {
                float* dst = reinterpret_cast<float*>(a.out) + (size_t)slot_of_row(idx) * a.rows + group * 64 + g * 4;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    *reinterpret_cast<u32x4*>(dst + 16 * r) = u32x4{v[r][0], v[r][1], v[r][2], v[r][3]};
            }
        }
        return;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int idx = t * 16 + q;
        if (idx >= nrows) continue;
        const size_t slot = (size_t)slot_of_row(idx);
        if constexpr (EPI == EPI_SWIGLU_BF16 || EPI == EPI_SWIGLU_F32) {
            const int I = a.rows / 2;
            float h[R][2];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                h[r][0] = swiglu(acc[r][t][0] + bv[r][0], acc[r][t][1] + bv[r][1], a.alpha, a.limit);
                h[r][1] = swiglu(acc[r][t][2] + bv[r][2], acc[r][t][3] + bv[r][3], a.alpha, a.limit);
            }
            if constexpr (EPI == EPI_SWIGLU_BF16) {
                uint32_t* dst =
                    reinterpret_cast<uint32_t*>(reinterpret_cast<uint16_t*>(a.out) + slot * I + row_base / 2);
                if constexpr (R == 4) {
                    *reinterpret_cast<u32x4*>(dst) = u32x4{pack_bf16x2(h[0][0], h[0][1]), pack_bf16x2(h[1][0], h[1][1]),
                                                           pack_bf16x2(h[2][0], h[2][1]), pack_bf16x2(h[3][0], h[3][1])};
                } else if constexpr (R == 2) {
                    *reinterpret_cast<u32x2*>(dst) = u32x2{pack_bf16x2(h[0][0], h[0][1]), pack_bf16x2(h[1][0], h[1][1])};
                } else {
                    dst[0] = pack_bf16x2(h[0][0], h[0][1]);
                }
            } else {
                float* dst = reinterpret_cast<float*>(a.out) + slot * I + row_base / 2;
#pragma unroll
                for (int r = 0; r < R; ++r) *reinterpret_cast<f32x2*>(dst + 2 * r) = f32x2{h[r][0], h[r][1]};
            }
        } else if constexpr (EPI == EPI_ROWS_F32) {
            float* dst = reinterpret_cast<float*>(a.out) + slot * a.rows + row_base;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                f32x4 v = acc[r][t];
                v[0] += bv[r][0];
                v[1] += bv[r][1];
                v[2] += bv[r][2];
                v[3] += bv[r][3];
                *reinterpret_cast<f32x4*>(dst + 4 * r) = v;
            }
        } else {
            const int tok = a.tokens_flat[slot];
            const float wgt = a.weights_flat[slot];
            float* dst = reinterpret_cast<float*>(a.out) + (size_t)tok * a.rows + row_base;
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int j = 0; j < 4; ++j) atomicAdd(dst + 4 * r + j, (acc[r][t][j] + bv[r][j]) * wgt);
        }
    }
}

constexpr int kWsRing = 4;

template <int N>
MOE_DEVICE void wait_vmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// AUX: cache policy of the load (0 = default; 16 = device scope: never served from this compute unit's L1).
template <int AUX = 0>
MOE_DEVICE void dma16(const void* gsrc, uint8_t* lds_dst_wave_uniform) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc,
                                     (__attribute__((address_space(3))) void*)lds_dst_wave_uniform, 16, 0, AUX);
}

// LDS image of one stage of activations: token tile t at t*4096, row q (0..15) of the tile at
// q*256, and inside the row the sixteen 16-byte chunks of the stage's 128 contraction elements,
// chunk c stored at position c ^ q.  A producer instruction moves four rows of 256 contiguous
// bytes (whole cache lines, each fetched once); the XOR spreads the sixteen rows that one
// fragment read touches over all LDS banks.
template <int FMT>
MOE_DEVICE int ws_chunk(int j, int g) {  // chunk holding the operand of MFMA step j for lane group g
    return (FMT == FMT_BF16) ? 8 * (j >> 1) + 2 * g + (j & 1) : 4 * g + j;
}
// MXFP4: the image is built over a permutation of the chunks.  The LDS serves a fragment read with the
// four lane groups of a token row side by side, and the chunks 4g + j that they read in one MFMA step
// are 64 bytes apart: two of the four would share banks (measured: every fragment read took twice its
// cycles).  ws_pos(c) takes the place of c above: chunk 4g + j sits where the bf16 operand order has
// its step-j chunk of group g (32 bytes apart: no conflicts).  ws_chunk_at is the inverse.
template <int FMT>
MOE_DEVICE int ws_pos(int c) {
    return (FMT == FMT_BF16) ? c : 8 * ((c & 3) >> 1) + 2 * (c >> 2) + (c & 1);
}
template <int FMT>
MOE_DEVICE int ws_chunk_at(int p) {
    return (FMT == FMT_BF16) ? p : 4 * ((p >> 1) & 3) + (((p >> 3) << 1) | (p & 1));
}

}  // namespace
}  // namespace moe
