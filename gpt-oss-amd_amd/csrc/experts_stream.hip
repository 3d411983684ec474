// Weight-streaming expert GEMM for decode-sized buckets (tens of rows per expert).
//
// Every weight byte is loaded from HBM exactly once per token block, straight into the MFMA
// A-operand registers with 128-bit loads (no LDS: a weight element is used by one wave only);
// the few activation rows of the bucket are the B operand, read from the L2-resident bf16 copy.
// fp32 accumulation in v_mfma_f32_16x16x32_bf16.  Replaces moe_mlp1_swiglu_mfma_kernel
// (src/hip/moe.hip:9-235) and moe_mlp2_scatter_mfma_kernel (src/hip/moe.hip:261-512) for small
// buckets; the arithmetic contract is the CPU path's (src/run.cpp:657-705): y = W x + b, SwiGLU on
// interleaved gate/up rows, down projection.
//
// Work split: block (x = row unit, y = token block).  A block has 4 waves; each wave owns R MFMA
// row tiles (16R weight rows) over the whole contraction length and up to NT*16 tokens.
// The contraction index is a dummy index, so lanes are free to pick which k each of their eight
// operand elements stands for as long as A and B agree:
//   bf16  : per 64-element chunk, lane group g = lane/16 takes elements [16g, 16g+16): two adjacent
//           128-bit loads per row, a whole 128-byte line per row per chunk;
//   MXFP4 : per 128-element chunk, lane group g takes MX block g of the chunk (32 elements, one
//           128-bit load + one scale byte), dequantised in registers to four A operands.
#include "common.h"
#include "kernels.h"

namespace moe {

namespace {

constexpr int FMT_BF16 = MOE_WEIGHTS_BF16;
constexpr int FMT_MXFP4 = MOE_WEIGHTS_MXFP4_TILED;

template <int FMT>
struct ChunkTraits;
template <>
struct ChunkTraits<FMT_BF16> {
    static constexpr int kElems = 64;   // contraction elements per chunk
    static constexpr int kSteps = 2;    // MFMA k-steps per chunk
    static constexpr int kADwords = 8;  // raw A dwords per lane per row tile per chunk
};
template <>
struct ChunkTraits<FMT_MXFP4> {
    static constexpr int kElems = 128;
    static constexpr int kSteps = 4;
    static constexpr int kADwords = 4;
};

// Epilogues: the fused block keeps bf16 SwiGLU outputs and fp32 per-slot rows; the entries that
// keep the reference's data flow write fp32 SwiGLU outputs and scatter with atomics.
enum { EPI_SWIGLU_BF16 = 0, EPI_ROWS_F32 = 1, EPI_SWIGLU_F32 = 2, EPI_SCATTER = 3 };

template <int FMT, int R, int NT>
struct Frags {
    u32x4 a[R][ChunkTraits<FMT>::kADwords / 4];  // raw weight data
    u32x4 b[NT][ChunkTraits<FMT>::kSteps];       // bf16 activations
};

MOE_DEVICE u32x4 pack_f32x8_to_bf16x8(const float4& lo, const float4& hi) {
    return u32x4{pack_bf16x2(lo.x, lo.y), pack_bf16x2(lo.z, lo.w), pack_bf16x2(hi.x, hi.y), pack_bf16x2(hi.z, hi.w)};
}

// One (row unit, token block) of one expert.  ACT_F32: activations are fp32 rows indexed by slot
// (the reference's x_by_expert / gate_by_expert buffers) and are rounded to bf16 on load.
template <int FMT, int R, int NT, int EPI, bool ACT_F32>
MOE_DEVICE void stream_body(const ExpertGemmArgs& a, int e, int row0, int nrows, int unit) {
    using CT = ChunkTraits<FMT>;
    constexpr int kUnitsPerGroup = 4 / R;
    const int lane = threadIdx.x & 63;
    const int q = lane & 15;
    const int g = lane >> 4;
    const int group = unit / kUnitsPerGroup;
    const int r0 = (unit % kUnitsPerGroup) * R;
    const int K = a.K;

    // ---- operand addressing ----
    const uint8_t* a_ptr[R];
    const uint8_t* s_ptr[R];
    if constexpr (FMT == FMT_BF16) {
        const uint16_t* wbase = reinterpret_cast<const uint16_t*>(a.w) + (size_t)e * a.w_expert_stride;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = group * 64 + tile_row_in_group(r0 + r, q);
            a_ptr[r] = reinterpret_cast<const uint8_t*>(wbase + (size_t)row * K + 16 * g);
            s_ptr[r] = nullptr;
        }
    } else {
        const int G = K / 32;
        const size_t tile_bytes = (size_t)G * 256;
        const size_t stile_bytes = (size_t)ceil_div(ceil_div(G, 4), 4) * 256;
        const uint8_t* wbase = reinterpret_cast<const uint8_t*>(a.w) + (size_t)e * a.w_expert_stride;
        const uint8_t* sbase = a.w_scales + (size_t)e * a.s_expert_stride;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const size_t tile = (size_t)group * 4 + (r0 + r);
            a_ptr[r] = wbase + tile * tile_bytes + (size_t)lane * 16;
            s_ptr[r] = sbase + tile * stile_bytes + (size_t)lane * 4;
        }
    }
    const uint8_t* b_ptr[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int idx = min(t * 16 + q, nrows - 1);
        if constexpr (ACT_F32) {
            b_ptr[t] = reinterpret_cast<const uint8_t*>(a.act_f32 + (size_t)(row0 + idx) * K) +
                       (FMT == FMT_BF16 ? 64 * g : 128 * g);
        } else {
            const int src = a.gather ? a.tokens_flat[row0 + idx] : row0 + idx;
            b_ptr[t] = reinterpret_cast<const uint8_t*>(a.act + (size_t)src * K) +
                       (FMT == FMT_BF16 ? 32 * g : 64 * g);
        }
    }

    f32x4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int n_chunks = ceil_div(K, CT::kElems);
    const int rem_groups = (FMT == FMT_MXFP4) ? ((K / 32) & 3) : 0;  // MX blocks in a ragged last chunk

    uint32_t scale_word[R];  // four scale bytes, one per chunk, reloaded every fourth chunk

    auto load_chunk = [&](Frags<FMT, R, NT>& f, int c) {
        if constexpr (FMT == FMT_BF16) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const u32x4* p = reinterpret_cast<const u32x4*>(a_ptr[r] + (size_t)c * 128);
                f.a[r][0] = p[0];
                f.a[r][1] = p[1];
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if constexpr (ACT_F32) {
                    const float4* p = reinterpret_cast<const float4*>(b_ptr[t] + (size_t)c * 256);
                    f.b[t][0] = pack_f32x8_to_bf16x8(p[0], p[1]);
                    f.b[t][1] = pack_f32x8_to_bf16x8(p[2], p[3]);
                } else {
                    const u32x4* p = reinterpret_cast<const u32x4*>(b_ptr[t] + (size_t)c * 128);
                    f.b[t][0] = p[0];
                    f.b[t][1] = p[1];
                }
            }
        } else {
            const bool live = !(rem_groups != 0 && c == n_chunks - 1 && g >= rem_groups);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                f.a[r][0] = u32x4{0u, 0u, 0u, 0u};
                if (live) f.a[r][0] = *reinterpret_cast<const u32x4*>(a_ptr[r] + (size_t)c * 1024);
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    f.b[t][s] = u32x4{0u, 0u, 0u, 0u};
                    if (live) {
                        if constexpr (ACT_F32) {
                            const float4* p = reinterpret_cast<const float4*>(b_ptr[t] + (size_t)c * 512);
                            f.b[t][s] = pack_f32x8_to_bf16x8(p[2 * s], p[2 * s + 1]);
                        } else {
                            const u32x4* p = reinterpret_cast<const u32x4*>(b_ptr[t] + (size_t)c * 256);
                            f.b[t][s] = p[s];
                        }
                    }
                }
            }
        }
    };

    auto compute_chunk = [&](const Frags<FMT, R, NT>& f, int c) {
        if constexpr (FMT == FMT_BF16) {
#pragma unroll
            for (int s = 0; s < 2; ++s)
#pragma unroll
                for (int r = 0; r < R; ++r)
#pragma unroll
                    for (int t = 0; t < NT; ++t) acc[r][t] = mfma_16x16x32(f.a[r][s], f.b[t][s], acc[r][t]);
        } else {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float sc = mxfp4_scale_to_f32((scale_word[r] >> (8 * (c & 3))) & 0xFFu);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    uint32_t d[4];
                    mxfp4_dword_to_bf16x8(f.a[r][0][s], sc, d);
                    const u32x4 av = {d[0], d[1], d[2], d[3]};
#pragma unroll
                    for (int t = 0; t < NT; ++t) acc[r][t] = mfma_16x16x32(av, f.b[t][s], acc[r][t]);
                }
            }
        }
    };

    auto load_scales = [&](int c) {
        if constexpr (FMT == FMT_MXFP4) {
#pragma unroll
            for (int r = 0; r < R; ++r)
                scale_word[r] = *reinterpret_cast<const uint32_t*>(s_ptr[r] + (size_t)(c >> 2) * 256);
        }
    };

    Frags<FMT, R, NT> f0, f1;
    load_scales(0);
    load_chunk(f0, 0);
    for (int c = 0; c < n_chunks; c += 2) {
        if (c + 1 < n_chunks) load_chunk(f1, c + 1);
        compute_chunk(f0, c);
        if (c + 2 < n_chunks) load_chunk(f0, c + 2);
        if (c + 1 < n_chunks) compute_chunk(f1, c + 1);
        if (((c + 2) & 3) == 0 && c + 2 < n_chunks) load_scales(c + 2);
    }

    // ---- epilogue: lane (q,g) holds token t*16+q, weight rows group*64 + g*16 + (r0+r)*4 + j ----
    const int row_base = group * 64 + g * 16 + r0 * 4;
    const uint16_t* bias = a.bias + (size_t)e * a.bias_expert_stride + row_base;
    float bv[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint2 raw = *reinterpret_cast<const uint2*>(bias + 4 * r);
        bv[r][0] = bf16_bits_to_f32(raw.x & 0xFFFFu);
        bv[r][1] = bf16_bits_to_f32(raw.x >> 16);
        bv[r][2] = bf16_bits_to_f32(raw.y & 0xFFFFu);
        bv[r][3] = bf16_bits_to_f32(raw.y >> 16);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int idx = t * 16 + q;
        if (idx >= nrows) continue;
        const size_t slot = (size_t)row0 + idx;
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

template <int FMT, int R, int EPI, bool ACT_F32>
MOE_DEVICE void stream_dispatch(const ExpertGemmArgs& a, int e, int row0, int nrows, int unit) {
    const int nt = (nrows + 15) >> 4;
    if (nt == 4) {
        stream_body<FMT, R, 4, EPI, ACT_F32>(a, e, row0, nrows, unit);
    } else if (nt == 3) {
        stream_body<FMT, R, 3, EPI, ACT_F32>(a, e, row0, nrows, unit);
    } else if (nt == 2) {
        stream_body<FMT, R, 2, EPI, ACT_F32>(a, e, row0, nrows, unit);
    } else if (nt == 1) {
        stream_body<FMT, R, 1, EPI, ACT_F32>(a, e, row0, nrows, unit);
    }
}

// Token blocks from the bucketing kernel's tile map.  grid = (row units / 4, max_tiles).
template <int FMT, int R, int EPI>
__global__ __launch_bounds__(256) void expert_stream_kernel(ExpertGemmArgs a) {
    const int tile = blockIdx.y;
    if (tile >= *a.n_tiles) return;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = blockIdx.x * 4 + wave;
    if (unit >= (a.rows / 64) * (4 / R)) return;
    stream_dispatch<FMT, R, EPI, false>(a, a.tile_expert[tile], a.tile_row0[tile], a.tile_rows[tile], unit);
}

// Token blocks from a queue of (expert, row_offset, row_count) triples (entry format of
// src/hip/scheduler.hip:163-166).  grid = (row units / 4, token blocks per entry, entries).
template <int FMT, int R, int EPI>
__global__ __launch_bounds__(256) void expert_stream_queue_kernel(ExpertGemmArgs a) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = blockIdx.x * 4 + wave;
    if (unit >= (a.rows / 64) * (4 / R)) return;
    const int* entry = a.work_queue + 3 * (a.work_start + blockIdx.z);
    const int e = entry[0], off = entry[1], n = entry[2];
    for (int tb = blockIdx.y; tb * 64 < n; tb += gridDim.y)
        stream_dispatch<FMT, R, EPI, true>(a, e, off + tb * 64, min(64, n - tb * 64), unit);
}

template <int FMT, int R, int EPI>
int launch_cfg(const ExpertGemmArgs& a, hipStream_t stream) {
    const int units = (a.rows / 64) * (4 / R);
    if (a.work_queue) {
        if (a.work_count <= 0) return MOE_OK;
        dim3 grid(ceil_div(units, 4), max(1, ceil_div(a.max_rows_hint, 64)), a.work_count);
        hipLaunchKernelGGL((expert_stream_queue_kernel<FMT, R, EPI>), grid, dim3(256), 0, stream, a);
    } else {
        dim3 grid(ceil_div(units, 4), a.max_tiles);
        hipLaunchKernelGGL((expert_stream_kernel<FMT, R, EPI>), grid, dim3(256), 0, stream, a);
    }
    return launch_status();
}

template <int FMT>
int launch_fmt(const ExpertGemmArgs& a, int epi, hipStream_t stream) {
    switch (epi) {
        case EPI_SWIGLU_BF16: return launch_cfg<FMT, 2, EPI_SWIGLU_BF16>(a, stream);
        case EPI_ROWS_F32: return launch_cfg<FMT, 2, EPI_ROWS_F32>(a, stream);
        case EPI_SWIGLU_F32: return launch_cfg<FMT, 2, EPI_SWIGLU_F32>(a, stream);
        case EPI_SCATTER: return launch_cfg<FMT, 2, EPI_SCATTER>(a, stream);
    }
    return MOE_ERR_FORMAT;
}

}  // namespace

// epi: 0 fused gate/up (bf16 SwiGLU out), 1 fused down (fp32 rows per slot), 2 gate/up with fp32
// in/out, 3 down with fp32 in and atomic scatter.  Token blocks hold at most 64 rows.
int launch_expert_stream(const ExpertGemmArgs& a, int epi, hipStream_t stream) {
    if (a.rows % 64 != 0) return MOE_ERR_SHAPE;
    const bool queue = a.work_queue != nullptr;
    if (queue != (epi == EPI_SWIGLU_F32 || epi == EPI_SCATTER)) return MOE_ERR_FORMAT;
    if (a.format == FMT_BF16) {
        if (a.K % 64 != 0) return MOE_ERR_SHAPE;
        return launch_fmt<FMT_BF16>(a, epi, stream);
    }
    if (a.format == FMT_MXFP4) {
        if (a.K % 32 != 0) return MOE_ERR_SHAPE;
        return launch_fmt<FMT_MXFP4>(a, epi, stream);
    }
    return MOE_ERR_FORMAT;
}

}  // namespace moe
