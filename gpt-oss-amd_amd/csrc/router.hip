// Router: logits (fp32 products, fp64 accumulation) -> top-k (ties to the lower expert id) ->
// softmax over the k selected logits.  Arithmetic follows the reference CPU path
// (src/run.cpp:321-404, 628-642); the GPU functions replaced are gemm_router
// (src/hip/gemms/gemm_router.hip:184), topk (src/hip/topk.hip:59) and softmax (src/hip/softmax.hip:46).
#include "common.h"
#include "kernels.h"

namespace moe {

// ---------------------------------------------------------------------------------------------
// Partial dot products.  One lane = one token, one wave = EG experts over one k-segment, so every
// accumulator walks its segment in ascending k exactly like the reference loop; with one segment
// the fp64 sum is bit-identical to src/run.cpp:348-351.  The four waves of a block share a
// transposed activation chunk of KC k-values in LDS (row stride 65 floats: conflict-free for the transposing
// store and for the lane-per-token read); weights are wave-uniform 16-byte loads issued one group
// of eight elements ahead (scalar registers: no vector ALU work to unpack them).
// grid = (ceil(T/64), ceil(E/(4*EG)), S), block = 256.
// partial layout: [S][T][E] fp64.
// ---------------------------------------------------------------------------------------------
template <int EG, int KC>
__global__ __launch_bounds__(256) void router_partial_kernel(const float* __restrict__ x,
                                                             const uint16_t* __restrict__ w,
                                                             double* __restrict__ partial,
                                                             uint16_t* __restrict__ x_bf16, int T, int H,
                                                             int E, int seg_len) {
    constexpr int NF = KC / 16;  // float4 loads per thread and chunk
    __shared__ float xs[KC][65];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t0 = blockIdx.x * 64;
    const int e0 = (blockIdx.y * 4 + wave) * EG;  // first expert of the wave
    const int s = blockIdx.z;
    const int kbeg = s * seg_len;
    const int kend = min(H, kbeg + seg_len);

    // the blocks of the first expert group also emit the bf16 copy of the activations that the
    // expert GEMMs consume (every (token tile, segment) pair is visited exactly once by them)
    const bool write_bf16 = x_bf16 != nullptr && blockIdx.y == 0;

    double acc[EG];
#pragma unroll
    for (int j = 0; j < EG; ++j) acc[j] = 0.0;

    // chunk c+1 is fetched into registers while chunk c is consumed from LDS
    float4 xr[NF];
    auto fetch = [&](int k0) {
        const int kc = min(KC, kend - k0);  // multiple of 8
        const int q4 = kc >> 2;
#pragma unroll
        for (int it = 0; it < NF; ++it) {
            const int i = threadIdx.x + 256 * it;
            const int tl = i / q4;
            const int c = i - tl * q4;
            const int tok = t0 + tl;
            xr[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (i < 64 * q4 && tok < T) xr[it] = *reinterpret_cast<const float4*>(x + (size_t)tok * H + k0 + 4 * c);
        }
    };
    auto stash = [&](int k0) {
        const int kc = min(KC, kend - k0);
        const int q4 = kc >> 2;
#pragma unroll
        for (int it = 0; it < NF; ++it) {
            const int i = threadIdx.x + 256 * it;
            if (i < 64 * q4) {
                const int tl = i / q4;
                const int c = i - tl * q4;
                if (write_bf16 && t0 + tl < T) {
                    uint2 o;
                    o.x = pack_bf16x2(xr[it].x, xr[it].y);
                    o.y = pack_bf16x2(xr[it].z, xr[it].w);
                    *reinterpret_cast<uint2*>(x_bf16 + (size_t)(t0 + tl) * H + k0 + 4 * c) = o;
                }
                xs[4 * c + 0][tl] = xr[it].x;
                xs[4 * c + 1][tl] = xr[it].y;
                xs[4 * c + 2][tl] = xr[it].z;
                xs[4 * c + 3][tl] = xr[it].w;
            }
        }
    };
    // weights: wave-uniform addresses (scalar loads), fetched one group of eight ahead
    const uint16_t* wrow[EG];
#pragma unroll
    for (int j = 0; j < EG; ++j) wrow[j] = w + (size_t)min(e0 + j, E - 1) * H;
    uint4 wv[EG], wn[EG];
#pragma unroll
    for (int j = 0; j < EG; ++j) wn[j] = *reinterpret_cast<const uint4*>(wrow[j] + min(kbeg, H - 8));
    if (kbeg < kend) fetch(kbeg);
    for (int k0 = kbeg; k0 < kend; k0 += KC) {
        const int kc = min(KC, kend - k0);
        stash(k0);
        __syncthreads();
        if (k0 + KC < kend) fetch(k0 + KC);
        if (e0 < E) {
            for (int kk = 0; kk < kc; kk += 8) {
#pragma unroll
                for (int j = 0; j < EG; ++j) {
                    wv[j] = wn[j];
                    wn[j] = *reinterpret_cast<const uint4*>(wrow[j] + min(k0 + kk + 8, H - 8));
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const float xv = xs[kk + i][lane];
#pragma unroll
                    for (int j = 0; j < EG; ++j) {
                        const uint32_t word = (i < 2) ? wv[j].x : (i < 4) ? wv[j].y : (i < 6) ? wv[j].z : wv[j].w;
                        const float wf = (i & 1) ? __uint_as_float(word & 0xFFFF0000u)
                                                 : __uint_as_float(word << 16);
                        acc[j] += (double)__fmul_rn(wf, xv);
                    }
                }
            }
        }
        __syncthreads();
    }
    const int tok = t0 + lane;
    if (tok < T) {
#pragma unroll
        for (int j = 0; j < EG; ++j) {
            const int e = e0 + j;
            if (e < E) partial[((size_t)s * T + tok) * E + e] = acc[j];
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Few tokens (a handful of token tiles): every block is latency bound, so it handles one segment
// of at most KS k-values in a single pass: all loads of the activation tile and of the four
// experts' weight segments are issued together, both land in LDS (weights widened to fp32), and
// each wave then walks its expert's segment in ascending k.  Same grid and partial layout as
// router_partial_kernel<1, *>.
// ---------------------------------------------------------------------------------------------
constexpr int kSmallSeg = 192;

__global__ __launch_bounds__(256) void router_partial_small_kernel(const float* __restrict__ x,
                                                                   const uint16_t* __restrict__ w,
                                                                   double* __restrict__ partial,
                                                                   uint16_t* __restrict__ x_bf16, int T, int H,
                                                                   int E, int seg_len) {
    constexpr int KS = kSmallSeg;
    constexpr int NF = KS / 16;
    __shared__ float xs[KS][65];
    __shared__ __align__(16) float wsh[4][KS];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int t0 = blockIdx.x * 64;
    const int e = blockIdx.y * 4 + wave;
    const int s = blockIdx.z;
    const int kbeg = s * seg_len;
    const int kc = min(H, kbeg + seg_len) - kbeg;  // multiple of 8, may be <= 0 for a trailing segment
    const bool write_bf16 = x_bf16 != nullptr && blockIdx.y == 0;
    double acc = 0.0;
    if (kc > 0) {
        const int q4 = kc >> 2;
        const int q8 = kc >> 3;
        float4 xr[NF];
#pragma unroll
        for (int it = 0; it < NF; ++it) {
            const int i = threadIdx.x + 256 * it;
            const int tl = i / q4;
            const int c = i - tl * q4;
            xr[it] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (i < 64 * q4 && t0 + tl < T)
                xr[it] = *reinterpret_cast<const float4*>(x + (size_t)(t0 + tl) * H + kbeg + 4 * c);
        }
        // weights: thread i < 4*q8 loads eight bf16 of expert (blockIdx.y*4 + i/q8)
        uint4 wr = make_uint4(0, 0, 0, 0);
        const int wj = threadIdx.x / q8, wc = threadIdx.x - wj * q8;
        const bool wload = threadIdx.x < 4 * q8;
        if (wload)
            wr = *reinterpret_cast<const uint4*>(w + (size_t)min(blockIdx.y * 4 + wj, E - 1) * H + kbeg + 8 * wc);
#pragma unroll
        for (int it = 0; it < NF; ++it) {
            const int i = threadIdx.x + 256 * it;
            if (i < 64 * q4) {
                const int tl = i / q4;
                const int c = i - tl * q4;
                if (write_bf16 && t0 + tl < T) {
                    uint2 o;
                    o.x = pack_bf16x2(xr[it].x, xr[it].y);
                    o.y = pack_bf16x2(xr[it].z, xr[it].w);
                    *reinterpret_cast<uint2*>(x_bf16 + (size_t)(t0 + tl) * H + kbeg + 4 * c) = o;
                }
                xs[4 * c + 0][tl] = xr[it].x;
                xs[4 * c + 1][tl] = xr[it].y;
                xs[4 * c + 2][tl] = xr[it].z;
                xs[4 * c + 3][tl] = xr[it].w;
            }
        }
        if (wload) {
            float4 lo, hi;
            lo.x = __uint_as_float(wr.x << 16);
            lo.y = __uint_as_float(wr.x & 0xFFFF0000u);
            lo.z = __uint_as_float(wr.y << 16);
            lo.w = __uint_as_float(wr.y & 0xFFFF0000u);
            hi.x = __uint_as_float(wr.z << 16);
            hi.y = __uint_as_float(wr.z & 0xFFFF0000u);
            hi.z = __uint_as_float(wr.w << 16);
            hi.w = __uint_as_float(wr.w & 0xFFFF0000u);
            *reinterpret_cast<float4*>(&wsh[wj][8 * wc]) = lo;
            *reinterpret_cast<float4*>(&wsh[wj][8 * wc + 4]) = hi;
        }
        __syncthreads();
        if (e < E) {
            for (int kk = 0; kk < kc; kk += 8) {
                const float4 wa = *reinterpret_cast<const float4*>(&wsh[wave][kk]);
                const float4 wb = *reinterpret_cast<const float4*>(&wsh[wave][kk + 4]);
                acc += (double)__fmul_rn(wa.x, xs[kk + 0][lane]);
                acc += (double)__fmul_rn(wa.y, xs[kk + 1][lane]);
                acc += (double)__fmul_rn(wa.z, xs[kk + 2][lane]);
                acc += (double)__fmul_rn(wa.w, xs[kk + 3][lane]);
                acc += (double)__fmul_rn(wb.x, xs[kk + 4][lane]);
                acc += (double)__fmul_rn(wb.y, xs[kk + 5][lane]);
                acc += (double)__fmul_rn(wb.z, xs[kk + 6][lane]);
                acc += (double)__fmul_rn(wb.w, xs[kk + 7][lane]);
            }
        }
    }
    const int tok = t0 + lane;
    if (tok < T && e < E) partial[((size_t)s * T + tok) * E + e] = acc;
}

// ---------------------------------------------------------------------------------------------
// Finalise: one wave per token.  score[e] = float(sum_s partial[s][t][e]) + bias[e]
// (src/run.cpp:352, 635-637), then K rounds of wave-wide argmax ordered by (value desc, index
// asc), then the softmax of src/run.cpp:321-339 on the K selected values.
// When `partial` is NULL the scores are read from `scores_in` instead.
// grid = ceil(T/4), block = 256, dynamic LDS = 4*E floats.
// ---------------------------------------------------------------------------------------------
MOE_DEVICE bool better(float va, int ia, float vb, int ib) { return va > vb || (va == vb && ia < ib); }

__global__ __launch_bounds__(256) void router_finalize_kernel(const double* __restrict__ partial, int S,
                                                              const float* __restrict__ scores_in,
                                                              const uint16_t* __restrict__ bias,
                                                              float* __restrict__ scores_out,
                                                              float* __restrict__ topk_v,
                                                              int* __restrict__ topk_i, int T, int E,
                                                              int K, int do_topk, int do_softmax) {
    extern __shared__ float sc[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T) return;  // no block-wide barrier below
    float* my = sc + (size_t)wave * E;

    for (int e = lane; e < E; e += 64) {
        float v;
        if (partial) {
            // all segment partials in flight at once, then summed in segment order
            double part[16];
#pragma unroll
            for (int s = 0; s < 16; ++s) part[s] = s < S ? partial[((size_t)s * T + t) * E + e] : 0.0;
            double sum = 0.0;
#pragma unroll
            for (int s = 0; s < 16; ++s)
                if (s < S) sum += part[s];
            v = (float)sum;
            v += bf16_bits_to_f32(bias[e]);
        } else {
            v = scores_in[(size_t)t * E + e];
        }
        my[e] = v;
        if (scores_out) scores_out[(size_t)t * E + e] = v;
    }
    if (!do_topk) return;
    __builtin_amdgcn_wave_barrier();

    uint32_t taken = 0;  // bit c set: candidate lane + 64*c already selected
    float sel_v[8];
    int sel_i[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        sel_v[r] = 0.f;
        sel_i[r] = 0;
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        if (r < K) {
            float bv = -INFINITY;
            int bi = 0x7FFFFFFF;
            for (int c = 0, e = lane; e < E; ++c, e += 64) {
                if (taken & (1u << c)) continue;
                const float v = my[e];
                if (bi == 0x7FFFFFFF || better(v, e, bv, bi)) {
                    bv = v;
                    bi = e;
                }
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                const float ov = __shfl_xor(bv, off, 64);
                const int oi = __shfl_xor(bi, off, 64);
                if (oi != 0x7FFFFFFF && (bi == 0x7FFFFFFF || better(ov, oi, bv, bi))) {
                    bv = ov;
                    bi = oi;
                }
            }
            sel_v[r] = bv;
            sel_i[r] = bi;
            if ((bi & 63) == lane) taken |= 1u << (bi >> 6);
        }
    }
    float outv[8];
    if (do_softmax) {
        double max_val = sel_v[0];
#pragma unroll
        for (int r = 1; r < 8; ++r)
            if (r < K && sel_v[r] > max_val) max_val = sel_v[r];
        double sum = 0.0;
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if (r < K) {
                outv[r] = expf((float)((double)sel_v[r] - max_val));
                sum += outv[r];
            }
        }
#pragma unroll
        for (int r = 0; r < 8; ++r)
            if (r < K) outv[r] = (float)((double)outv[r] / sum);
    } else {
#pragma unroll
        for (int r = 0; r < 8; ++r) outv[r] = sel_v[r];
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) {
        if (r < K && lane == r) {
            topk_v[(size_t)t * K + r] = outv[r];
            topk_i[(size_t)t * K + r] = sel_i[r];
        }
    }
}

// In-place softmax over the last dimension, one thread per row, the reference's order of
// operations (src/run.cpp:321-339).
__global__ void softmax_rows_kernel(float* __restrict__ x, int B, int size) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= B) return;
    float* r = x + (size_t)b * size;
    double max_val = r[0];
    for (int i = 1; i < size; ++i)
        if (r[i] > max_val) max_val = r[i];
    double sum = 0.0;
    for (int i = 0; i < size; ++i) {
        const float ex = expf((float)((double)r[i] - max_val));
        r[i] = ex;
        sum += ex;
    }
    for (int i = 0; i < size; ++i) r[i] = (float)((double)r[i] / sum);
}

// ---------------------------------------------------------------------------------------------
// Host launchers
// ---------------------------------------------------------------------------------------------
// Experts per wave: the largest group that still leaves about four waves per SIMD once the k range
// is cut into at most 16 segments (a larger group reuses each LDS read of an activation more often).
static int router_expert_group(int T, int E) {
    const long long tiles = ceil_div(T, 64);
    for (int eg = 4; eg > 1; eg >>= 1)
        if (tiles * ceil_div(E, eg) * 16 >= 4096) return eg;
    return 1;
}

int router_segments(int T, int E, int H, bool strict) {
    if (strict) return 1;
    const long long waves_one = (long long)ceil_div(T, 64) * ceil_div(E, router_expert_group(T, E));
    int S = 1;
    while (S < 16 && waves_one * S < 4096 && H / (S * 2) >= 64) S *= 2;
    return S;
}

size_t router_partial_bytes(int T, int E) { return (size_t)16 * T * E * sizeof(double); }

int launch_router_partial(const float* x, const uint16_t* w, double* partial, uint16_t* x_bf16, int T, int H,
                          int E, int S, hipStream_t stream) {
    int seg_len = ceil_div(ceil_div(H, S), 8) * 8;
    const int eg = router_expert_group(T, E);
    dim3 grid(ceil_div(T, 64), ceil_div(E, 4 * eg), S);
    if (eg == 1 && seg_len <= kSmallSeg) {
        hipLaunchKernelGGL(router_partial_small_kernel, grid, dim3(256), 0, stream, x, w, partial, x_bf16, T, H, E,
                           seg_len);
    } else if (eg == 1) {
        hipLaunchKernelGGL((router_partial_kernel<1, 64>), grid, dim3(256), 0, stream, x, w, partial, x_bf16, T, H, E,
                           seg_len);
    } else if (eg == 2) {
        hipLaunchKernelGGL((router_partial_kernel<2, 64>), grid, dim3(256), 0, stream, x, w, partial, x_bf16, T, H, E,
                           seg_len);
    } else {
        hipLaunchKernelGGL((router_partial_kernel<4, 64>), grid, dim3(256), 0, stream, x, w, partial, x_bf16, T, H, E,
                           seg_len);
    }
    return launch_status();
}

int launch_router_finalize(const double* partial, int S, const float* scores_in, const uint16_t* bias,
                           float* scores_out, float* topk_v, int* topk_i, int T, int E, int K, int do_topk,
                           int do_softmax, hipStream_t stream) {
    hipLaunchKernelGGL(router_finalize_kernel, dim3(ceil_div(T, 4)), dim3(256), (size_t)4 * E * sizeof(float),
                       stream, partial, S, scores_in, bias, scores_out, topk_v, topk_i, T, E, K, do_topk,
                       do_softmax);
    return launch_status();
}

int launch_softmax_rows(float* x, int B, int size, hipStream_t stream) {
    hipLaunchKernelGGL(softmax_rows_kernel, dim3(ceil_div(B, 256)), dim3(256), 0, stream, x, B, size);
    return launch_status();
}

}  // namespace moe
