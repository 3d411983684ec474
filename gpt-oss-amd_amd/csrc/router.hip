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

// These kernels run their code once per wave, so their time is instruction fetch as much as
// anything: loops stay rolled (the round and segment counts are wave-uniform anyway).
//
// K rounds of wave-wide argmax over vals[0..E) ordered by (value desc, index asc).  Lane r < K
// ends up holding the winner of round r in (my_v, my_i).
MOE_DEVICE void select_topk(const float* vals, int E, int K, int lane, float& my_v, int& my_i) {
    uint32_t taken = 0;  // bit c set: candidate lane + 64*c already selected
    my_v = -INFINITY;
    my_i = 0;
#pragma nounroll
    for (int r = 0; r < K; ++r) {
        float bv = -INFINITY;
        int bi = 0x7FFFFFFF;
#pragma nounroll
        for (int c = 0, e = lane; e < E; ++c, e += 64) {
            const float v = vals[e];
            if (!(taken & (1u << c)) && (bi == 0x7FFFFFFF || better(v, e, bv, bi))) {
                bv = v;
                bi = e;
            }
        }
        // wave-wide winner on the DPP path; a lane without a source keeps (any, 0x7FFFFFFF)
#define MOE_STEP(C, M)                                                                      \
    {                                                                                       \
        const float ov = __uint_as_float(dpp_move<C, M>(0u, __float_as_uint(bv)));          \
        const int oi = (int)dpp_move<C, M>(0x7FFFFFFFu, (uint32_t)bi);                      \
        const bool take = oi != 0x7FFFFFFF && (bi == 0x7FFFFFFF || better(ov, oi, bv, bi)); \
        bv = take ? ov : bv;                                                                \
        bi = take ? oi : bi;                                                                \
    }
        MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
        bv = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(bv), 63));
        bi = __builtin_amdgcn_readlane(bi, 63);
        if (lane == r) {
            my_v = bv;
            my_i = bi;
        }
        if ((bi & 63) == lane) taken |= 1u << (bi >> 6);
    }
}

MOE_DEVICE float lane_value(float v, int src_lane) {
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), src_lane));
}

// Softmax of src/run.cpp:321-339 over the K selected values in its own order of operations (max,
// then exponentials, then their fp64 sum in index order), or the values themselves; lane r < K
// stores entry r.
MOE_DEVICE void write_topk(float my_v, int my_i, int K, int lane, int do_softmax, float* __restrict__ out_v,
                           int* __restrict__ out_i) {
    float o = my_v;
    if (do_softmax) {
        double max_val = lane_value(my_v, 0);
#pragma nounroll
        for (int r = 1; r < K; ++r) {
            const float v = lane_value(my_v, r);
            if (v > max_val) max_val = v;
        }
        const float ex = expf((float)((double)my_v - max_val));
        double sum = 0.0;
#pragma nounroll
        for (int r = 0; r < K; ++r) sum += (double)lane_value(ex, r);
        o = (float)((double)ex / sum);
    }
    if (lane < K) {
        out_v[lane] = o;
        out_i[lane] = my_i;
    }
}

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
            // summed in segment order; four loads in flight
            double sum = 0.0;
#pragma unroll 4
            for (int s = 0; s < S; ++s) sum += partial[((size_t)s * T + t) * E + e];
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

    float my_v;
    int my_i;
    select_topk(my, E, K, lane, my_v, my_i);
    write_topk(my_v, my_i, K, lane, do_softmax, topk_v + (size_t)t * K, topk_i + (size_t)t * K);
}

// ---------------------------------------------------------------------------------------------
// First pass of the two-pass router: approximate logits of ALL experts on the matrix cores.
// Every activation is split into two bf16 pieces, x = hi + lo + r with |r| <= 2^-16 |x|, and both
// pieces are multiplied with the bf16 router weights (products of two bf16 are exact in fp32) and
// accumulated in fp32 by v_mfma_f32_16x16x32_bf16.  Taking every fp32 addition inside the matrix
// unit and every accumulation to be good to one unit in the last place, a partial over a segment
// of n k-steps is within (33 + 2n) * 2^-23 * sum|w_k x_k| of the products it adds up.
// A wave owns 16 tokens (MFMA rows) and NE tiles of 16 experts (MFMA columns) over one k-segment.
// The same pass writes the bf16 copy of the activations (the hi pieces) for the expert GEMMs, the
// squared norm of every token's segment (xn2 [S][T]) and, in the blocks of the first token tile,
// of every router row's segment (wn2 [S][E]).  partial is [S][T][E] fp32.
// grid = (ceil(T/64), ceil(E/(16*NE)), S), block = 256; seg_len % 32 == 0, H % 32 == 0.
// ---------------------------------------------------------------------------------------------
template <int NE>
__global__ __launch_bounds__(256) void router_screen_kernel(const float* __restrict__ x,
                                                            const uint16_t* __restrict__ w,
                                                            float* __restrict__ partial, float* __restrict__ wn2,
                                                            float* __restrict__ xn2, uint16_t* __restrict__ x_bf16,
                                                            int T, int H, int E, int seg_len) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int t0 = blockIdx.x * 64 + wave * 16;
    const int e_base = blockIdx.y * 16 * NE;
    const int s = blockIdx.z;
    const int kbeg = s * seg_len;
    const int kend = min(H, kbeg + seg_len);
    const bool first_group = blockIdx.y == 0;

    if (blockIdx.x == 0) {  // block-uniform: squared norms of this block's router rows
        for (int i = wave; i < 16 * NE; i += 4) {
            const int e = e_base + i;
            if (e >= E) break;
            float q = 0.f;
            for (int k = kbeg + lane; k < kend; k += 64) {
                const float wf = bf16_bits_to_f32(w[(size_t)e * H + k]);
                q = fmaf(wf, wf, q);
            }
            q = wave_sum(q);
            if (lane == 0) wn2[(size_t)s * E + e] = q;
        }
    }
    if (t0 >= T) return;  // wave-uniform; no block-wide barrier below

    const int tok = min(t0 + r, T - 1);
    const bool tok_ok = t0 + r < T;
    const float* xrow = x + (size_t)tok * H + 8 * g;
    const uint16_t* wrow[NE];
#pragma unroll
    for (int n = 0; n < NE; ++n) wrow[n] = w + (size_t)min(e_base + 16 * n + r, E - 1) * H + 8 * g;

    f32x4 acc[NE];
#pragma unroll
    for (int n = 0; n < NE; ++n) acc[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    float x2 = 0.f;

    // k-steps of 32; the loads of step i+1 are in flight while step i is converted and multiplied
    float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0;
    u32x4 b[NE];
    auto load = [&](int k0) {
        a0 = *reinterpret_cast<const float4*>(xrow + k0);
        a1 = *reinterpret_cast<const float4*>(xrow + k0 + 4);
#pragma unroll
        for (int n = 0; n < NE; ++n) b[n] = *reinterpret_cast<const u32x4*>(wrow[n] + k0);
    };
    if (kbeg < kend) load(kbeg);
    for (int k0 = kbeg; k0 < kend; k0 += 32) {
        const float v[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
        u32x4 bb[NE];
#pragma unroll
        for (int n = 0; n < NE; ++n) bb[n] = b[n];
        if (k0 + 32 < kend) load(k0 + 32);
        u32x4 hi, lo;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t h2 = pack_bf16x2(v[2 * i], v[2 * i + 1]);
            hi[i] = h2;
            lo[i] = pack_bf16x2(v[2 * i] - __uint_as_float(h2 << 16), v[2 * i + 1] - __uint_as_float(h2 & 0xFFFF0000u));
            x2 = fmaf(v[2 * i], v[2 * i], x2);
            x2 = fmaf(v[2 * i + 1], v[2 * i + 1], x2);
        }
        if (first_group && tok_ok && x_bf16) *reinterpret_cast<u32x4*>(x_bf16 + (size_t)tok * H + 8 * g + k0) = hi;
#pragma unroll
        for (int n = 0; n < NE; ++n) {
            acc[n] = mfma_16x16x32(hi, bb[n], acc[n]);
            acc[n] = mfma_16x16x32(lo, bb[n], acc[n]);
        }
    }
    // accumulator layout: lane holds tokens t0 + 4g + i (i = 0..3) for expert e_base + 16n + r
#pragma unroll
    for (int n = 0; n < NE; ++n) {
        const int e = e_base + 16 * n + r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int t = t0 + 4 * g + i;
            if (e < E && t < T) partial[((size_t)s * T + t) * E + e] = acc[n][i];
        }
    }
    if (first_group) {
        x2 += __shfl_xor(x2, 16, 64);
        x2 += __shfl_xor(x2, 32, 64);
        if (g == 0 && tok_ok) xn2[(size_t)s * T + tok] = x2;
    }
}

// ---------------------------------------------------------------------------------------------
// Second pass of the two-pass router: one wave per token.
//   1. approximate scores a[e] = float(sum_s partial[s][t][e]) + bias[e] from the screening pass,
//      each within d of the exact score, d = err_coeff * |x_t|_2 * max_e |w_e|_2 (Cauchy-Schwarz
//      on sum|w_k x_k|; err_coeff from the screening pass's error model) plus the final roundings;
//   2. vK = K-th largest a.  An expert with a[e] < vK - 2d has an exact score below those of the K
//      experts with a >= vK, so the exact top K lies inside C = {e : a[e] >= vK - 2d};
//   3. the exact score (fp32 products, fp64 sum: src/run.cpp:341-354, 635-637) of every member
//      of C, each lane summing its own k in ascending order, lanes combined by a butterfly;
//   4. top-k and softmax over those exact scores, as in router_finalize_kernel.
// The result equals router_partial_kernel + router_finalize_kernel up to the order of
// the fp64 additions; |C| is K except for near-ties at the boundary (every exact tie is in C).
// grid = ceil(T/4), block = 256, dynamic LDS = 4 * 3 * E * 4 bytes.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void router_refine_kernel(const float* __restrict__ partial, int S,
                                                            const float* __restrict__ wn2,
                                                            const float* __restrict__ xn2,
                                                            const float* __restrict__ x,
                                                            const uint16_t* __restrict__ w,
                                                            const uint16_t* __restrict__ bias, float err_coeff,
                                                            float* __restrict__ topk_v, int* __restrict__ topk_i,
                                                            int T, int H, int E, int K, int do_softmax) {
    extern __shared__ float sc[];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int t = blockIdx.x * 4 + wave;
    if (t >= T) return;  // no block-wide barrier below
    float* approx = sc + (size_t)wave * 3 * E;
    float* exact = approx + E;
    int* cand = reinterpret_cast<int*>(exact + E);

    float x2 = 0.f;
#pragma unroll 4
    for (int s = 0; s < S; ++s) x2 += xn2[(size_t)s * T + t];
    float w2max = 0.f, amax = 0.f;
#pragma nounroll
    for (int e = lane; e < E; e += 64) {
        double sum = 0.0;
        float q = 0.f;
#pragma unroll 4
        for (int s = 0; s < S; ++s) {
            sum += (double)partial[((size_t)s * T + t) * E + e];
            q += wn2[(size_t)s * E + e];
        }
        const float v = (float)sum + bf16_bits_to_f32(bias[e]);
        approx[e] = v;
        exact[e] = -INFINITY;
        w2max = fmaxf(w2max, q);
        amax = fmaxf(amax, fabsf(v));
    }
    w2max = wave_max_nonneg(w2max);
    amax = wave_max_nonneg(amax);
    // upper bound of |approx - exact| for every expert of this token; the 1.001 factors cover the
    // rounding of the two norms themselves, the last term the final roundings of both scores
    const float delta = err_coeff * (sqrtf(x2) * 1.001f) * (sqrtf(w2max) * 1.001f) + amax * 0x1p-20f;
    __builtin_amdgcn_wave_barrier();

    float my_v;
    int my_i;
    select_topk(approx, E, K, lane, my_v, my_i);
    const float thr = lane_value(my_v, K - 1) - 2.f * delta;

    int n_cand = 0;
#pragma nounroll
    for (int e0 = 0; e0 < E; e0 += 64) {
        const int e = e0 + lane;
        const bool in = e < E && approx[e] >= thr;
        const unsigned long long ballot = __ballot(in);
        if (in) cand[n_cand + __popcll(ballot & ((1ull << lane) - 1ull))] = e;
        n_cand += __popcll(ballot);
    }
    if (n_cand < K) {  // not-a-number scores: no screening, every expert is scored exactly
        for (int e = lane; e < E; e += 64) cand[e] = e;
        n_cand = E;
    }
    __builtin_amdgcn_wave_barrier();

    // exact scores, four candidates at a time (their loads and reductions overlap); lane l takes
    // float4 number l, l + 64, ... of the token's activations, in ascending order
    const int n4 = H >> 2;
    const float4* xrow = reinterpret_cast<const float4*>(x + (size_t)t * H);
#pragma nounroll
    for (int c0 = 0; c0 < n_cand; c0 += 4) {
        const uint2* wrow[4];
        double acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = __builtin_amdgcn_readfirstlane(cand[min(c0 + i, n_cand - 1)]);
            wrow[i] = reinterpret_cast<const uint2*>(w + (size_t)e * H);
            acc[i] = 0.0;
        }
#pragma unroll 3
        for (int i4 = lane; i4 < n4; i4 += 64) {
            const float4 xv = xrow[i4];
            uint2 wb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) wb[i] = wrow[i][i4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[i] += (double)__fmul_rn(__uint_as_float(wb[i].x << 16), xv.x);
                acc[i] += (double)__fmul_rn(__uint_as_float(wb[i].x & 0xFFFF0000u), xv.y);
                acc[i] += (double)__fmul_rn(__uint_as_float(wb[i].y << 16), xv.z);
                acc[i] += (double)__fmul_rn(__uint_as_float(wb[i].y & 0xFFFF0000u), xv.w);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const double total = wave_sum(acc[i]);
            const int e = __builtin_amdgcn_readfirstlane(cand[min(c0 + i, n_cand - 1)]);
            if (lane == 0) exact[e] = (float)total + bf16_bits_to_f32(bias[e]);
        }
    }
    __builtin_amdgcn_wave_barrier();

    select_topk(exact, E, K, lane, my_v, my_i);
    write_topk(my_v, my_i, K, lane, do_softmax, topk_v + (size_t)t * K, topk_i + (size_t)t * K);
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

// ---- two-pass router -----------------------------------------------------------------------------
// Worth it once the exact pass is throughput bound (three vector instructions per term); small
// batches are latency bound and keep the single exact pass.
bool router_two_pass(int T, int E, int H) { return (long long)T * E >= 65536 && H % 32 == 0; }

static int screen_tiles(int E) { return E <= 16 ? 1 : E <= 32 ? 2 : 4; }  // 16-expert tiles per wave

static int router_screen_segments(int T, int E, int H) {
    const long long waves_one = (long long)ceil_div(T, 16) * ceil_div(E, 16 * screen_tiles(E));
    int S = 1;
    while (S < 16 && waves_one * S < 2048 && H / (S * 2) >= 64) S *= 2;
    return S;
}

size_t router_screen_bytes(int T, int E, int H) {
    const size_t S = router_screen_segments(T, E, H);
    return S * T * E * sizeof(float) + S * E * sizeof(float) + S * T * sizeof(float);
}

int launch_router_two_pass(const float* x, const uint16_t* w, const uint16_t* bias, void* scratch, uint16_t* x_bf16,
                           float* topk_v, int* topk_i, int T, int H, int E, int K, int do_softmax,
                           hipStream_t stream, hipEvent_t between) {
    int S = router_screen_segments(T, E, H);
    const int seg_len = ceil_div(ceil_div(H, S), 32) * 32;
    S = ceil_div(H, seg_len);  // rounding the segment up can empty the last ones
    float* partial = static_cast<float*>(scratch);
    float* wn2 = partial + (size_t)S * T * E;
    float* xn2 = wn2 + (size_t)S * E;
    const int ne = screen_tiles(E);
    dim3 grid(ceil_div(T, 64), ceil_div(E, 16 * ne), S);
    if (ne == 1) {
        hipLaunchKernelGGL((router_screen_kernel<1>), grid, dim3(256), 0, stream, x, w, partial, wn2, xn2, x_bf16, T, H, E,
                           seg_len);
    } else if (ne == 2) {
        hipLaunchKernelGGL((router_screen_kernel<2>), grid, dim3(256), 0, stream, x, w, partial, wn2, xn2, x_bf16, T, H, E,
                           seg_len);
    } else {
        hipLaunchKernelGGL((router_screen_kernel<4>), grid, dim3(256), 0, stream, x, w, partial, wn2, xn2, x_bf16, T, H, E,
                           seg_len);
    }
    int rc = launch_status();
    if (rc) return rc;
    if (between) MOE_RETURN_IF_HIP(hipEventRecord(between, stream));
    // error model of the screening pass per unit of |x| |w|: 33 + 2 * k-steps roundings of 2^-23 inside
    // a segment, the 2^-16 the two bf16 pieces leave out, and 8 * 2^-24 for the product roundings of
    // the exact path; 1 % slack
    const float err_coeff = ((float)(33 + 2 * (seg_len / 32)) * 0x1p-23f + 0x1p-16f + 8 * 0x1p-24f) * 1.01f;
    hipLaunchKernelGGL(router_refine_kernel, dim3(ceil_div(T, 4)), dim3(256),
                       (size_t)4 * 3 * E * sizeof(float), stream, partial, S, wn2, xn2, x, w, bias, err_coeff, topk_v,
                       topk_i, T, H, E, K, do_softmax);
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
