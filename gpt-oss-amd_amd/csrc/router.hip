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

// These kernels run their code once per wave, so their time is instruction fetch as much as
// anything: loops stay rolled (the round and segment counts are wave-uniform anyway).
//
// Sort key of a (score, expert) pair: larger key = better candidate.  High word: the score's bits
// mapped to an unsigned integer in score order (-0 counts as +0, as in the reference's float
// comparison); low word: ~index, so equal scores order by the lower index.  Key 0 is "nothing".
MOE_DEVICE uint64_t rank_key(float v, int e) {
    const uint32_t u = __float_as_uint(v + 0.f);
    const uint32_t m = u ^ ((uint32_t)((int32_t)u >> 31) | 0x80000000u);
    return ((uint64_t)m << 32) | (uint32_t)~e;
}
MOE_DEVICE float rank_key_value(uint64_t key) {
    const uint32_t m = (uint32_t)(key >> 32);
    return __uint_as_float((m & 0x80000000u) ? m ^ 0x80000000u : ~m);
}

// K rounds of wave-wide argmax over vals[0..E) ordered by (value desc, index asc).  Lane r < K
// ends up holding the winner of round r in (my_v, my_i).
MOE_DEVICE void select_topk(const float* vals, int E, int K, int lane, float& my_v, int& my_i) {
    uint32_t taken = 0;  // bit c set: candidate lane + 64*c already selected
    my_v = -INFINITY;
    my_i = 0;
#pragma nounroll
    for (int r = 0; r < K; ++r) {
        uint64_t best = 0;
#pragma nounroll
        for (int c = 0, e = lane; e < E; ++c, e += 64) {
            const uint64_t key = (taken >> c) & 1u ? 0ull : rank_key(vals[e], e);
            best = key > best ? key : best;
        }
        // wave-wide maximum on the DPP path (a lane without a source sees key 0)
#define MOE_STEP(C, M)                                                                          \
    {                                                                                           \
        const uint64_t o = ((uint64_t)dpp_move<C, M>(0u, (uint32_t)(best >> 32)) << 32) |       \
                           dpp_move<C, M>(0u, (uint32_t)best);                                  \
        best = o > best ? o : best;                                                             \
    }
        MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
        const uint32_t hi = __builtin_amdgcn_readlane((uint32_t)(best >> 32), 63);
        const uint32_t lo = __builtin_amdgcn_readlane((uint32_t)best, 63);
        const int bi = (int)~lo;
        if (lane == r) {
            my_v = rank_key_value((uint64_t)hi << 32);
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
// The four waves of a block share the router rows of their segment through LDS.
// grid = (ceil(T/64), ceil(E/(16*NE)), S), block = 256, dynamic LDS = 16*NE*(seg_len+8)*2 bytes;
// seg_len % 32 == 0, H % 32 == 0.
// ---------------------------------------------------------------------------------------------
// D: k-steps whose activation loads are in flight together (the kernel is a chain of memory round
// trips: one for the router rows, then one per D k-steps of its segment).
template <int NE, int D>
__global__ __launch_bounds__(256) void router_screen_kernel(const float* __restrict__ x,
                                                            const uint16_t* __restrict__ w,
                                                            float* __restrict__ partial, float* __restrict__ wn2,
                                                            float* __restrict__ xn2, uint16_t* __restrict__ x_bf16,
                                                            int T, int H, int E, int seg_len) {
    extern __shared__ __attribute__((aligned(16))) uint16_t wl[];  // [16*NE][seg_len + 8]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int t0 = blockIdx.x * 64 + wave * 16;
    const int e_base = blockIdx.y * 16 * NE;
    const int s = blockIdx.z;
    const int kbeg = s * seg_len;
    const int kend = min(H, kbeg + seg_len);  // kend - kbeg is a positive multiple of 32
    const int ldw = seg_len + 8;              // row stride 16 bytes off a multiple of 64: rows r, r+1 land 4 banks apart
    const bool first_group = blockIdx.y == 0;

    // activations first: D k-steps (32 values each) per request group, the next group in flight
    // while the current one is converted and multiplied
    const int tok = min(t0 + r, T - 1);
    const bool tok_ok = t0 + r < T;
    const float* xrow = x + (size_t)tok * H + 8 * g;
    float4 xa[D][2];
    auto load_group = [&](int k0) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int k = min(k0 + 32 * d, kend - 32);
            xa[d][0] = *reinterpret_cast<const float4*>(xrow + k);
            xa[d][1] = *reinterpret_cast<const float4*>(xrow + k + 4);
        }
    };
    load_group(kbeg);

    // this block's router rows over the segment -> LDS, shared by the four waves
    {
        const int cpr = (kend - kbeg) >> 3;  // 16-byte chunks per row
        for (int idx = threadIdx.x; idx < 16 * NE * cpr; idx += 256) {
            const int row = idx / cpr, c = idx - row * cpr;
            const int e = min(e_base + row, E - 1);
            *reinterpret_cast<u32x4*>(wl + row * ldw + 8 * c) =
                *reinterpret_cast<const u32x4*>(w + (size_t)e * H + kbeg + 8 * c);
        }
    }
    __syncthreads();

    if (blockIdx.x == 0) {  // block-uniform: squared norms of this block's router rows
        for (int i = wave; i < 16 * NE; i += 4) {
            const int e = e_base + i;
            if (e >= E) break;
            float q = 0.f;
            for (int k = lane; k < kend - kbeg; k += 64) {
                const float wf = bf16_bits_to_f32(wl[i * ldw + k]);
                q = fmaf(wf, wf, q);
            }
            q = wave_sum(q);
            if (lane == 0) wn2[(size_t)s * E + e] = q;
        }
    }
    if (t0 >= T) return;  // wave-uniform; no block-wide barrier below

    f32x4 acc[NE];
#pragma unroll
    for (int n = 0; n < NE; ++n) acc[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    float x2 = 0.f;
    const int wfrag = r * ldw + 8 * g - kbeg;  // element index of this lane's fragment at k = 0

    for (int k0 = kbeg; k0 < kend; k0 += 32 * D) {
        float4 cur[D][2];
#pragma unroll
        for (int d = 0; d < D; ++d) {
            cur[d][0] = xa[d][0];
            cur[d][1] = xa[d][1];
        }
        if (k0 + 32 * D < kend) load_group(k0 + 32 * D);
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int k = k0 + 32 * d;
            if (k < kend) {  // wave-uniform
                const float v[8] = {cur[d][0].x, cur[d][0].y, cur[d][0].z, cur[d][0].w,
                                    cur[d][1].x, cur[d][1].y, cur[d][1].z, cur[d][1].w};
                u32x4 hi, lo;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t h2 = pack_bf16x2(v[2 * i], v[2 * i + 1]);
                    hi[i] = h2;
                    lo[i] = pack_bf16x2(v[2 * i] - __uint_as_float(h2 << 16),
                                        v[2 * i + 1] - __uint_as_float(h2 & 0xFFFF0000u));
                    x2 = fmaf(v[2 * i], v[2 * i], x2);
                    x2 = fmaf(v[2 * i + 1], v[2 * i + 1], x2);
                }
                if (first_group && tok_ok && x_bf16)
                    *reinterpret_cast<u32x4*>(x_bf16 + (size_t)tok * H + 8 * g + k) = hi;
#pragma unroll
                for (int n = 0; n < NE; ++n) {
                    const u32x4 b = *reinterpret_cast<const u32x4*>(wl + (wfrag + 16 * n * ldw + k));
                    acc[n] = mfma_16x16x32(hi, b, acc[n]);
                    acc[n] = mfma_16x16x32(lo, b, acc[n]);
                }
            }
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

// Exact logits of NE experts for one token, by one wave: fp32 products, fp64 sums
// (src/run.cpp:341-354).  Lane l takes float4 number l, l + 64, ... of the token's activations in
// ascending order; the lanes' sums are combined by wave_sum's fixed tree, so a logit does not depend
// on NE or on which other experts share the call.  The trip count is the same for every lane (a
// lane past the end multiplies zeros), so that the loads of several iterations can be in flight
// together.  Every lane returns all NE totals.
template <int NE>
MOE_DEVICE void exact_dots(const float* __restrict__ x_row, const uint16_t* __restrict__ w, const int (&e)[NE], int H,
                           int lane, double (&total)[NE]) {
    const int n4 = H >> 2;
    const int trips = ceil_div(n4, 64);
    const float4* xrow = reinterpret_cast<const float4*>(x_row);
    const uint2* wrow[NE];
    double acc[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        wrow[i] = reinterpret_cast<const uint2*>(w + (size_t)e[i] * H);
        acc[i] = 0.0;
    }
#pragma unroll 4
    for (int j = 0; j < trips; ++j) {
        const bool live = lane + 64 * j < n4;
        const int i4 = min(lane + 64 * j, n4 - 1);
        const float4 xv = xrow[i4];
        uint2 wb[NE];
#pragma unroll
        for (int i = 0; i < NE; ++i) wb[i] = wrow[i][i4];
#pragma unroll
        for (int i = 0; i < NE; ++i) {
            if (!live) wb[i] = make_uint2(0u, 0u);  // zero products leave the sum unchanged
            acc[i] += (double)__fmul_rn(__uint_as_float(wb[i].x << 16), xv.x);
            acc[i] += (double)__fmul_rn(__uint_as_float(wb[i].x & 0xFFFF0000u), xv.y);
            acc[i] += (double)__fmul_rn(__uint_as_float(wb[i].y << 16), xv.z);
            acc[i] += (double)__fmul_rn(__uint_as_float(wb[i].y & 0xFFFF0000u), xv.w);
        }
    }
#pragma unroll
    for (int i = 0; i < NE; ++i) total[i] = wave_sum(acc[i]);
}

// ---------------------------------------------------------------------------------------------
// Whole router in one launch for batches too small for the two-pass router to pay: one block per
// token.  The block stages the token's activation row in LDS (and writes its row of the bf16 copy
// that the expert GEMMs consume); wave w scores experts NE*w .. NE*w + NE-1 (then NE*(w + waves) ..,
// if there are more) with the arithmetic and the order of additions of exact_dots — the same logits, bit for bit,
// as the exact pass of the two-pass router — and leaves them in LDS; wave 0 then runs top-k and
// softmax and writes the score row if the caller wants it.
// All loads of a wave's first pass (the activation piece it stages, its two router rows) are issued
// before anything waits, so a block costs one memory round trip plus the arithmetic.
// grid = T, block = 64 * waves, dynamic LDS = (H + E) floats; H <= 256 * kFusedTrips.  NE experts per
// wave and pass: two with up to 16 waves (128 registers per lane hold the loads of two rows), four
// with up to 8 waves.
// ---------------------------------------------------------------------------------------------
constexpr int kFusedTrips = 12;  // rows of up to 3072 values

template <int NE>
__global__ __launch_bounds__(NE == 2 ? 1024 : 512) void router_fused_kernel(const float* __restrict__ x, const uint16_t* __restrict__ w,
                                                            const uint16_t* __restrict__ bias,
                                                            uint16_t* __restrict__ x_bf16,
                                                            float* __restrict__ scores_out, float* __restrict__ topk_v,
                                                            int* __restrict__ topk_i, int H, int E, int K,
                                                            int do_softmax) {
    extern __shared__ __attribute__((aligned(16))) float fused_lds[];
    float4* xs = reinterpret_cast<float4*>(fused_lds);  // [H / 4]
    float* sc = fused_lds + H;                           // [E]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int t = blockIdx.x;
    const int n4 = H >> 2;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)t * H);
    const int n_groups = ceil_div(E, NE);

    // activation row: thread i stages float4 number i, i + blockDim, ...
    constexpr int STG = NE == 2 ? 1 : 2;  // enough for a full-size block; smaller blocks take the loops below
    float4 xv_st[STG];
#pragma unroll
    for (int i = 0; i < STG; ++i) {
        const int c = threadIdx.x + i * blockDim.x;
        xv_st[i] = xr[min(c, n4 - 1)];
    }
    // per-lane element index of trip j, clamped into the row; as 32-bit byte offsets next to
    // wave-uniform row bases the loads need no per-lane 64-bit addresses
    uint32_t idx[kFusedTrips];
#pragma unroll
    for (int j = 0; j < kFusedTrips; ++j) idx[j] = (uint32_t)min(lane + 64 * j, n4 - 1);
    uint2 wb[kFusedTrips][NE];
    auto load_rows = [&](int grp) {
#pragma unroll
        for (int i = 0; i < NE; ++i) {
            const char* wrow = reinterpret_cast<const char*>(w + (size_t)min(grp * NE + i, E - 1) * H);
#pragma unroll
            for (int j = 0; j < kFusedTrips; ++j) wb[j][i] = *reinterpret_cast<const uint2*>(wrow + (size_t)(idx[j] * 8u));
        }
    };
    if (wave < n_groups) load_rows(wave);
    for (int c = threadIdx.x + STG * blockDim.x; c < n4; c += blockDim.x) xs[c] = xr[c];  // blocks with few waves
#pragma unroll
    for (int i = 0; i < STG; ++i) {
        const int c = threadIdx.x + i * blockDim.x;
        if (c < n4) {
            xs[c] = xv_st[i];
            if (x_bf16)
                reinterpret_cast<uint2*>(x_bf16 + (size_t)t * H)[c] =
                    make_uint2(pack_bf16x2(xv_st[i].x, xv_st[i].y), pack_bf16x2(xv_st[i].z, xv_st[i].w));
        }
    }
    if (x_bf16)
        for (int c = threadIdx.x + STG * blockDim.x; c < n4; c += blockDim.x) {
            const float4 v = xr[c];
            reinterpret_cast<uint2*>(x_bf16 + (size_t)t * H)[c] = make_uint2(pack_bf16x2(v.x, v.y), pack_bf16x2(v.z, v.w));
        }
    __syncthreads();
    auto score_group = [&](int grp) {
        double acc[NE];
#pragma unroll
        for (int i = 0; i < NE; ++i) acc[i] = 0.0;
#pragma unroll
        for (int j = 0; j < kFusedTrips; ++j) {
            const bool live = lane + 64 * j < n4;
            const float4 xv = xs[idx[j]];
#pragma unroll
            for (int i = 0; i < NE; ++i) {
                const uint2 wv = live ? wb[j][i] : make_uint2(0u, 0u);  // zero products leave the sum unchanged
                acc[i] += (double)__fmul_rn(__uint_as_float(wv.x << 16), xv.x);
                acc[i] += (double)__fmul_rn(__uint_as_float(wv.x & 0xFFFF0000u), xv.y);
                acc[i] += (double)__fmul_rn(__uint_as_float(wv.y << 16), xv.z);
                acc[i] += (double)__fmul_rn(__uint_as_float(wv.y & 0xFFFF0000u), xv.w);
            }
        }
#pragma unroll
        for (int i = 0; i < NE; ++i) {
            const double total = wave_sum(acc[i]);
            const int e = grp * NE + i;
            if (lane == 0 && e < E) sc[e] = (float)total + bf16_bits_to_f32(bias[e]);
        }
    };
    // the usual case, one group per wave, is straight-line code (a loop here makes the compiler hoist
    // every trip's address arithmetic out of it and hold it in registers)
    if (wave < n_groups) score_group(wave);
    if (n_groups > n_waves) {
#pragma nounroll
        for (int grp = wave + n_waves; grp < n_groups; grp += n_waves) {
            load_rows(grp);
            score_group(grp);
        }
    }
    __syncthreads();
    if (wave != 0) return;
    if (scores_out)
        for (int e = lane; e < E; e += 64) scores_out[(size_t)t * E + e] = sc[e];
    float my_v;
    int my_i;
    select_topk(sc, E, K, lane, my_v, my_i);
    write_topk(my_v, my_i, K, lane, do_softmax, topk_v + (size_t)t * K, topk_i + (size_t)t * K);
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
__global__ __launch_bounds__(256, 4) void router_refine_kernel(const float* __restrict__ partial, int S,
                                                            const float* __restrict__ wn2,
                                                            const float* __restrict__ xn2,
                                                            const float* __restrict__ x,
                                                            const uint16_t* __restrict__ w,
                                                            const uint16_t* __restrict__ bias, float err_coeff,
                                                            float* __restrict__ topk_v, int* __restrict__ topk_i,
                                                            int T, int H, int E, int K, int do_softmax,
                                                            float* __restrict__ approx_out,
                                                            float* __restrict__ delta_out,
                                                            int* __restrict__ n_cand_out) {
    extern __shared__ float sc[];
    __shared__ float w2_of_wave[4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int t = min(blockIdx.x * 4 + wave, T - 1);  // a surplus wave repeats the last token
    float* approx = sc + (size_t)wave * 3 * E;
    float* exact = approx + E;
    int* cand = reinterpret_cast<int*>(exact + E);

    // largest squared router-row norm: the same for every token, so the block's threads share it
    float w2max = 0.f;
#pragma nounroll
    for (int e = threadIdx.x; e < E; e += 256) {
        float q = 0.f;
#pragma nounroll
        for (int s0 = 0; s0 < S; s0 += 16) {
            float wq[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) wq[i] = wn2[(size_t)min(s0 + i, S - 1) * E + e];
#pragma unroll
            for (int i = 0; i < 16; ++i) q += s0 + i < S ? wq[i] : 0.f;
        }
        w2max = fmaxf(w2max, q);
    }
    // approximate scores: all loads of up to two experts per lane in flight, summed in segment order
    float amax = 0.f;
#pragma nounroll
    for (int e0 = lane; e0 < E; e0 += 128) {
#pragma nounroll
        for (int s0 = 0; s0 < S; s0 += 16) {
            float part[2][16];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int e = min(e0 + 64 * h, E - 1);
#pragma unroll
                for (int i = 0; i < 16; ++i) part[h][i] = partial[((size_t)min(s0 + i, S - 1) * T + t) * E + e];
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int e = e0 + 64 * h;
                double sum = s0 == 0 ? 0.0 : (double)exact[min(e, E - 1)];  // carries the sum when S > 16
#pragma unroll
                for (int i = 0; i < 16; ++i) sum += s0 + i < S ? (double)part[h][i] : 0.0;
                if (e < E) exact[e] = (float)sum;
            }
        }
    }
    float x2 = 0.f;
#pragma unroll 4
    for (int s = 0; s < S; ++s) x2 += xn2[(size_t)s * T + t];
    w2max = wave_max_nonneg(w2max);
    if (lane == 0) w2_of_wave[wave] = w2max;
    __syncthreads();
    if (blockIdx.x * 4 + wave >= T) return;  // no block-wide barrier below
    w2max = fmaxf(fmaxf(w2_of_wave[0], w2_of_wave[1]), fmaxf(w2_of_wave[2], w2_of_wave[3]));
#pragma nounroll
    for (int e = lane; e < E; e += 64) {
        const float v = exact[e] + bf16_bits_to_f32(bias[e]);
        approx[e] = v;
        exact[e] = -INFINITY;
        amax = fmaxf(amax, fabsf(v));
        if (approx_out) approx_out[(size_t)t * E + e] = v;  // what the screening decides on, for whoever checks the bound
    }
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
    if (lane == 0) {
        if (delta_out) delta_out[t] = delta;
        if (n_cand_out) n_cand_out[t] = n_cand;
    }
    __builtin_amdgcn_wave_barrier();

    // exact scores of the candidates, four at a time
    const float* x_row = x + (size_t)t * H;
#pragma nounroll
    for (int c0 = 0; c0 < n_cand; c0 += 4) {
        int e[4];
        double total[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = __builtin_amdgcn_readfirstlane(cand[min(c0 + i, n_cand - 1)]);
        exact_dots<4>(x_row, w, e, H, lane, total);
        if (lane == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) exact[e[i]] = (float)total[i] + bf16_bits_to_f32(bias[e[i]]);
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

// Segment length (multiple of 32) and count of the screening pass: enough segments for about 2048
// waves, and short enough for the block's router rows to fit 64 KB of LDS.
static void screen_plan(int T, int E, int H, int* seg_len, int* S) {
    const int ne = screen_tiles(E);
    const long long waves_one = (long long)ceil_div(T, 16) * ceil_div(E, 16 * ne);
    int want = 1;
    while (want < 16 && waves_one * want < 2048 && H / (want * 2) >= 64) want *= 2;
    const int seg_max = (65536 / (2 * 16 * ne) - 8) / 32 * 32;
    const int seg = min(seg_max, ceil_div(ceil_div(H, want), 32) * 32);
    *seg_len = seg;
    *S = ceil_div(H, seg);
}

size_t router_screen_bytes(int T, int E, int H) {
    int seg_len, S;
    screen_plan(T, E, H, &seg_len, &S);
    return ((size_t)S * T * E + (size_t)S * E + (size_t)S * T) * sizeof(float);
}

int launch_router_two_pass(const float* x, const uint16_t* w, const uint16_t* bias, void* scratch, uint16_t* x_bf16,
                           float* topk_v, int* topk_i, int T, int H, int E, int K, int do_softmax,
                           hipStream_t stream, hipEvent_t between, float* approx_out, float* delta_out,
                           int* n_cand_out) {
    int seg_len, S;
    screen_plan(T, E, H, &seg_len, &S);
    float* partial = static_cast<float*>(scratch);
    float* wn2 = partial + (size_t)S * T * E;
    float* xn2 = wn2 + (size_t)S * E;
    const int ne = screen_tiles(E);
    dim3 grid(ceil_div(T, 64), ceil_div(E, 16 * ne), S);
    const size_t lds = (size_t)16 * ne * (seg_len + 8) * sizeof(uint16_t);
    // the whole segment in flight where it is short enough for the registers (D * 8 per lane)
    const int steps = seg_len / 32;
    const int depth = steps >= 12 ? 12 : steps >= 6 ? 6 : 4;
#define MOE_SCREEN(NE_, D_)                                                                                          \
    hipLaunchKernelGGL((router_screen_kernel<NE_, D_>), grid, dim3(256), lds, stream, x, w, partial, wn2, xn2, x_bf16, T, H, \
                       E, seg_len)
#define MOE_SCREEN_NE(NE_)          \
    if (depth == 12) {              \
        MOE_SCREEN(NE_, 12);        \
    } else if (depth == 6) {        \
        MOE_SCREEN(NE_, 6);         \
    } else {                        \
        MOE_SCREEN(NE_, 4);         \
    }
    if (ne == 1) {
        MOE_SCREEN_NE(1)
    } else if (ne == 2) {
        MOE_SCREEN_NE(2)
    } else {
        MOE_SCREEN_NE(4)
    }
#undef MOE_SCREEN_NE
#undef MOE_SCREEN
    int rc = launch_status();
    if (rc) return rc;
    if (between) MOE_RETURN_IF_HIP(hipEventRecord(between, stream));
    // error model of the screening pass per unit of |x| |w|: 33 + 2 * k-steps roundings of 2^-23 inside
    // a segment, the 2^-16 the two bf16 pieces leave out, and 8 * 2^-24 for the product roundings of
    // the exact path; 1 % slack
    const float err_coeff = ((float)(33 + 2 * (seg_len / 32)) * 0x1p-23f + 0x1p-16f + 8 * 0x1p-24f) * 1.01f;
    hipLaunchKernelGGL(router_refine_kernel, dim3(ceil_div(T, 4)), dim3(256),
                       (size_t)4 * 3 * E * sizeof(float), stream, partial, S, wn2, xn2, x, w, bias, err_coeff, topk_v,
                       topk_i, T, H, E, K, do_softmax, approx_out, delta_out, n_cand_out);
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

// Rows the fused router can take (all of a wave's loads are held in registers at once).
bool router_fused_fits(int H) { return H % 4 == 0 && H <= 256 * kFusedTrips; }

// Up to 32 experts: two per wave, up to 16 waves (the shortest critical path per token); beyond: four
// per wave, 8 waves, as many passes as that takes.
int launch_router_fused(const float* x, const uint16_t* w, const uint16_t* bias, uint16_t* x_bf16, float* scores_out,
                        float* topk_v, int* topk_i, int T, int H, int E, int K, int do_softmax, hipStream_t stream) {
    if (!router_fused_fits(H)) return MOE_ERR_LIMIT;
    const size_t lds = (size_t)(H + E) * sizeof(float);
    if (E <= 32) {
        hipLaunchKernelGGL(router_fused_kernel<2>, dim3(T), dim3(64 * min(16, ceil_div(E, 2))), lds, stream, x, w, bias,
                           x_bf16, scores_out, topk_v, topk_i, H, E, K, do_softmax);
    } else {
        hipLaunchKernelGGL(router_fused_kernel<4>, dim3(T), dim3(64 * min(8, ceil_div(E, 4))), lds, stream, x, w, bias,
                           x_bf16, scores_out, topk_v, topk_i, H, E, K, do_softmax);
    }
    return launch_status();
}

int launch_softmax_rows(float* x, int B, int size, hipStream_t stream) {
    hipLaunchKernelGGL(softmax_rows_kernel, dim3(ceil_div(B, 256)), dim3(256), 0, stream, x, B, size);
    return launch_status();
}

}  // namespace moe
