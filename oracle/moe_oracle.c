/*
 * moe_oracle.c — CPU restatement of the reference's MoE block arithmetic.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py may load this library, and only as the checker / the timed CPU
 * baseline.  Nothing in the shipped GPU path calls into it.
 *
 * Each function follows one piece of the reference (tuanlda78202/gpt-oss-amd):
 *   oracle_matmul        src/run.cpp:341-354   float product, double accumulation, sequential k
 *   oracle_rmsnorm       src/run.cpp:306-319   double sum of float squares, eps 1e-5f, sqrtf
 *   oracle_softmax       src/run.cpp:321-339   double max / double sum, expf on the float diff
 *   oracle_topk          src/run.cpp:357-404   descending sort of (value,index), first K;
 *                                              equal values keep ascending index (stable order,
 *                                              which is what glibc's merge-sort qsort yields)
 *   oracle_topk_qsort    src/run.cpp:365-399   the same through qsort(3) itself, kept to show
 *                                              that the stable rule is what this libc does
 *   oracle_swiglu        src/run.cpp:666-689   de-interleave (gate = even, up = odd rows), clamp
 *                                              gate from above only, up on both sides,
 *                                              gate*sigmoid(1.702 gate)*(up+1)
 *   oracle_moe_block     src/run.cpp:628-707   router matmul + bias, topk, softmax, experts
 *                                              visited in ascending id, weighted accumulate
 *   oracle_moe_layer     src/run.cpp:626,710-712  rmsnorm in, residual out around the block
 *   oracle_dequant_mxfp4 tools/model_export/gpt-oss-20b/export_model_bin.py:75-133
 *                                              value = LUT[nibble] * 2^(scale-127) as bf16; low
 *                                              nibble is the even element, 16 bytes -> 32
 *                                              consecutive elements sharing one scale byte
 *   oracle_bucket        src/hip/scheduler.hip:11-61 (count, exclusive scan, compaction); the
 *                                              reference claims slots with atomics, so order
 *                                              inside a bucket is unspecified there; here it
 *                                              is ascending token id
 *   oracle_classify_queues src/hip/scheduler.hip:112-184  heavy / light work queues: experts with
 *                                              rows, in ascending id, heavy when at most
 *                                              `very_sparse_cutoff` experts are active or when the
 *                                              expert has at least ceil(factor * mean rows) rows
 *
 * Pinning status (what fixes each function independently of this file):
 *   matmul/moe_block  : fp64 numpy composition, one-hot and zero inputs, brute force (tests)
 *   topk              : numpy stable argsort, crafted ties, glibc qsort agreement
 *   softmax           : scipy.special.softmax in fp64
 *   swiglu            : closed-form special cases (g>7, |u|>7, u=-1, g=0, g<<0)
 *   dequant           : exhaustive 16 codes x 256 scales against exact rational arithmetic and
 *                       against torch.ldexp on bf16 (the library routine the reference calls)
 *   bucket            : integer invariants (bincount, exclusive scan, sortedness, round trip)
 *   classify_queues   : numpy restatement of the rule from its description (partition of the active
 *                       experts, threshold cases at each of the three factor regimes, empty input)
 * The reference holds no golden vectors for this path and its translation unit does not
 * compile as shipped, so nothing here is checked against a reference binary.
 * PARITY UNPINNED (outside every workload's range): the NaN payload that scale byte 255
 * yields for zero codes; tie order of qsort when it falls back to quicksort under memory
 * pressure; last-ulp behaviour of libm expf.
 *
 * Build: see oracle/Makefile (gcc -O3 -fopenmp; the reference's CPU target uses
 * -O3 -fopenmp -march=native, Makefile:22 — here -march is pinned to x86-64-v3 so the same
 * binary runs on the build container and on the GPU host).
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#include "../include/moe_synth.h"

#define ORACLE_API __attribute__((visibility("default")))

ORACLE_API int oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---- src/run.cpp:341-354 ------------------------------------------------------------- */
ORACLE_API void oracle_matmul(float* xout, const float* x, const float* w, int n, int d) {
    int i;
#pragma omp parallel for private(i)
    for (i = 0; i < d; i++) {
        double val = 0.0;
        const float* wr = w + (long long)i * n;
        for (int j = 0; j < n; j++) {
            float prod = wr[j] * x[j]; /* float multiply first, then widened */
            val += prod;
        }
        xout[i] = (float)val;
    }
}

/* ---- src/run.cpp:306-319 ------------------------------------------------------------- */
ORACLE_API void oracle_rmsnorm(float* o, const float* x, const float* weight, int size) {
    double ss = 0.0;
    for (int j = 0; j < size; j++) {
        float sq = x[j] * x[j];
        ss += sq;
    }
    ss /= size;
    ss += 1e-5f;
    ss = 1.0f / sqrtf((float)ss);
    for (int j = 0; j < size; j++) {
        o[j] = (float)(weight[j] * (ss * x[j]));
    }
}

/* ---- src/run.cpp:321-339 ------------------------------------------------------------- */
ORACLE_API void oracle_softmax(float* x, int size) {
    double max_val = x[0];
    for (int i = 1; i < size; i++) {
        if (x[i] > max_val) max_val = x[i];
    }
    double sum = 0.0;
    for (int i = 0; i < size; i++) {
        x[i] = expf((float)(x[i] - max_val));
        sum += x[i];
    }
    for (int i = 0; i < size; i++) {
        x[i] = (float)(x[i] / sum);
    }
}

/* ---- src/run.cpp:357-404 ------------------------------------------------------------- */
typedef struct {
    float value;
    int index;
} OraclePair;

static int oracle_compare_desc(const void* a, const void* b) {
    float diff = ((const OraclePair*)b)->value - ((const OraclePair*)a)->value;
    if (diff > 0) return 1;
    if (diff < 0) return -1;
    return 0;
}

ORACLE_API int oracle_topk(float* topk_values, int* topk_indices, const float* router_score,
                           int num_experts, int experts_per_token) {
    if (num_experts <= 0 || experts_per_token <= 0 || experts_per_token > num_experts) return -1;
    if (!router_score || !topk_values || !topk_indices) return -2;
    OraclePair* pairs = (OraclePair*)malloc((size_t)num_experts * sizeof(OraclePair));
    if (!pairs) return -3;
    /* stable insertion sort, descending by value: an element moves left only past strictly
     * smaller values, so equal values stay in ascending index order */
    for (int i = 0; i < num_experts; ++i) {
        OraclePair cur = {router_score[i], i};
        int j = i;
        while (j > 0 && oracle_compare_desc(&pairs[j - 1], &cur) > 0) {
            pairs[j] = pairs[j - 1];
            --j;
        }
        pairs[j] = cur;
    }
    for (int i = 0; i < experts_per_token; ++i) {
        topk_values[i] = pairs[i].value;
        topk_indices[i] = pairs[i].index;
    }
    free(pairs);
    return 0;
}

ORACLE_API int oracle_topk_qsort(float* topk_values, int* topk_indices, const float* router_score,
                                 int num_experts, int experts_per_token) {
    if (num_experts <= 0 || experts_per_token <= 0 || experts_per_token > num_experts) return -1;
    OraclePair* pairs = (OraclePair*)malloc((size_t)num_experts * sizeof(OraclePair));
    if (!pairs) return -3;
    for (int i = 0; i < num_experts; ++i) {
        pairs[i].value = router_score[i];
        pairs[i].index = i;
    }
    qsort(pairs, (size_t)num_experts, sizeof(OraclePair), oracle_compare_desc);
    for (int i = 0; i < experts_per_token; ++i) {
        topk_values[i] = pairs[i].value;
        topk_indices[i] = pairs[i].index;
    }
    free(pairs);
    return 0;
}

/* ---- src/run.cpp:666-689 ------------------------------------------------------------- */
ORACLE_API void oracle_swiglu(float* gate_up, const float* mlp1_out, int intermediate_dim,
                              float swiglu_limit) {
    const float alpha = 1.702f;
    for (int i = 0; i < intermediate_dim; i++) {
        float val = mlp1_out[2 * i];
        float up_val = mlp1_out[2 * i + 1];
        if (val > swiglu_limit) val = swiglu_limit;
        if (up_val > swiglu_limit) up_val = swiglu_limit;
        if (up_val < -swiglu_limit) up_val = -swiglu_limit;
        val *= (1.0f / (1.0f + expf(-alpha * val)));
        val *= (up_val + 1.0f);
        gate_up[i] = val;
    }
}

/* ---- src/run.cpp:628-707 ------------------------------------------------------------- *
 * One MoE block over T independent tokens (the reference handles one token per forward()
 * call; the outer loop is this file's only addition).
 *   t_in      [T,H]   block input (post-rmsnorm activations)
 *   w_router  [E,H]   b_router [E]
 *   w_mlp1    [E,2I,H] (gate/up rows interleaved)   b_mlp1 [E,2I]
 *   w_mlp2    [E,H,I]                                b_mlp2 [E,H]
 *   e_agg     [T,H]   block output
 *   topk_i    [T,K]   topk_v [T,K] (softmax weights, descending-logit order)
 *   router_score [T,E] optional (may be NULL)
 * The accumulate `e_agg += tb2 * w` is one fused multiply-add: the reference is built with
 * hipcc/clang, whose default floating-point contraction fuses a*b+c inside one statement.
 */
ORACLE_API int oracle_moe_block(int T, int H, int I, int E, int K, float swiglu_limit,
                                const float* t_in, const float* w_router, const float* b_router,
                                const float* w_mlp1, const float* b_mlp1, const float* w_mlp2,
                                const float* b_mlp2, float* e_agg, int* topk_i, float* topk_v,
                                float* router_score_out) {
    float* router_score = (float*)malloc(sizeof(float) * (size_t)E);
    float* mlp1_out = (float*)malloc(sizeof(float) * (size_t)(2 * I));
    float* gate_up = (float*)malloc(sizeof(float) * (size_t)I);
    float* tb2 = (float*)malloc(sizeof(float) * (size_t)H);
    if (!router_score || !mlp1_out || !gate_up || !tb2) return -3;
    for (int b = 0; b < T; ++b) {
        const float* t = t_in + (long long)b * H;
        float* agg = e_agg + (long long)b * H;
        int* ti = topk_i + (long long)b * K;
        float* tv = topk_v + (long long)b * K;
        oracle_matmul(router_score, t, w_router, H, E);
        for (int i = 0; i < E; i++) router_score[i] += b_router[i];
        if (router_score_out) memcpy(router_score_out + (long long)b * E, router_score, sizeof(float) * E);
        int rc = oracle_topk(tv, ti, router_score, E, K);
        if (rc) return rc;
        oracle_softmax(tv, K);
        memset(agg, 0, sizeof(float) * (size_t)H);
        for (int e = 0; e < E; e++) {
            float expert_w = 0;
            int in_topk = 0;
            for (int idx = 0; idx < K; idx++) {
                if (ti[idx] == e) {
                    in_topk = 1;
                    expert_w = tv[idx];
                    break;
                }
            }
            if (!in_topk) continue;
            const float* w1 = w_mlp1 + (long long)e * (2 * I) * H;
            const float* b1 = b_mlp1 + (long long)e * (2 * I);
            oracle_matmul(mlp1_out, t, w1, H, 2 * I);
            for (int i = 0; i < 2 * I; i++) mlp1_out[i] += b1[i];
            oracle_swiglu(gate_up, mlp1_out, I, swiglu_limit);
            const float* w2 = w_mlp2 + (long long)e * H * I;
            const float* b2 = b_mlp2 + (long long)e * H;
            oracle_matmul(tb2, gate_up, w2, I, H);
            for (int i = 0; i < H; i++) tb2[i] += b2[i];
            for (int i = 0; i < H; i++) agg[i] = fmaf(tb2[i], expert_w, agg[i]);
        }
    }
    free(router_score);
    free(mlp1_out);
    free(gate_up);
    free(tb2);
    return 0;
}

/* ---- src/run.cpp:626, 628-712 -------------------------------------------------------- *
 * x <- x + moe_block(rmsnorm(x, rms_w)); x is [T,H] and updated in place; t_scratch and
 * agg_scratch are [T,H].
 */
ORACLE_API int oracle_moe_layer(int T, int H, int I, int E, int K, float swiglu_limit, float* x,
                                const float* rms_w, const float* w_router, const float* b_router,
                                const float* w_mlp1, const float* b_mlp1, const float* w_mlp2,
                                const float* b_mlp2, float* t_scratch, float* agg_scratch,
                                int* topk_i, float* topk_v) {
    for (int b = 0; b < T; ++b)
        oracle_rmsnorm(t_scratch + (long long)b * H, x + (long long)b * H, rms_w, H);
    int rc = oracle_moe_block(T, H, I, E, K, swiglu_limit, t_scratch, w_router, b_router, w_mlp1,
                              b_mlp1, w_mlp2, b_mlp2, agg_scratch, topk_i, topk_v, NULL);
    if (rc) return rc;
    for (long long i = 0; i < (long long)T * H; ++i) x[i] += agg_scratch[i];
    return 0;
}

/* ---- tools/model_export/gpt-oss-20b/export_model_bin.py:75-133 ----------------------- *
 * One e2m1 code and one e8m0 scale byte to bf16 bits, in integer arithmetic.
 * LUT magnitudes are {0, .5, 1, 1.5, 2, 3, 4, 6} = (1 + f/2) * 2^(p-1) with (p,f) below, so
 * code * 2^(scale-127) has at most two significant bits and is exact in bf16 whenever it is
 * in range: biased exponent p + scale - 1; below 1 the result is a bf16 subnormal (still
 * exact: the shift never drops a set bit), at 255 and above it is infinity (what fp32
 * multiplication by 2^(scale-127) followed by rounding to bf16 gives).  Scale 255 means
 * 2^128 = +inf in fp32: non-zero codes become +-inf, zero codes NaN.
 */
ORACLE_API uint16_t oracle_mxfp4_to_bf16_bits(unsigned code, unsigned scale) {
    static const int P[8] = {0, 0, 1, 1, 2, 2, 3, 3};
    static const int F[8] = {0, 0, 0, 1, 0, 1, 0, 1};
    unsigned sign = (code >> 3) & 1u;
    unsigned mag = code & 7u;
    if (scale == 255u) return mag == 0 ? (uint16_t)0x7FC0u : (uint16_t)((sign << 15) | 0x7F80u);
    if (mag == 0) return (uint16_t)(sign << 15);
    int biased = P[mag] + (int)scale - 1;
    if (biased >= 255) return (uint16_t)((sign << 15) | 0x7F80u);
    if (biased >= 1) return (uint16_t)((sign << 15) | ((unsigned)biased << 7) | (F[mag] ? 0x40u : 0u));
    /* subnormal: value = (2+f) * 2^(biased-128); one bf16 subnormal unit is 2^-133 */
    unsigned units = (unsigned)(2 + F[mag]) << (biased + 5);
    return (uint16_t)((sign << 15) | units);
}

/* blocks [n_blocks,16] u8, scales [n_blocks] u8 -> out [n_blocks*32] bf16 bits */
ORACLE_API void oracle_dequant_mxfp4(const uint8_t* blocks, const uint8_t* scales, long long n_blocks,
                                     uint16_t* out) {
#pragma omp parallel for
    for (long long g = 0; g < n_blocks; ++g) {
        unsigned s = scales[g];
        for (int b = 0; b < 16; ++b) {
            unsigned byte = blocks[g * 16 + b];
            out[g * 32 + 2 * b] = oracle_mxfp4_to_bf16_bits(byte & 0xFu, s);
            out[g * 32 + 2 * b + 1] = oracle_mxfp4_to_bf16_bits(byte >> 4, s);
        }
    }
}

/* The same decoder widened to fp32 in one pass (bf16 -> fp32 is exact): fills the fp32 expert tensors the CPU
 * path holds without a bf16 copy in between. */
ORACLE_API void oracle_dequant_mxfp4_f32(const uint8_t* blocks, const uint8_t* scales, long long n_blocks,
                                         float* out) {
#pragma omp parallel for
    for (long long g = 0; g < n_blocks; ++g) {
        unsigned s = scales[g];
        for (int b = 0; b < 16; ++b) {
            unsigned byte = blocks[g * 16 + b];
            out[g * 32 + 2 * b] = moe_synth_bf16_bits_to_f32(oracle_mxfp4_to_bf16_bits(byte & 0xFu, s));
            out[g * 32 + 2 * b + 1] = moe_synth_bf16_bits_to_f32(oracle_mxfp4_to_bf16_bits(byte >> 4, s));
        }
    }
}

/* bf16 bits -> fp32 array (how the reference's CPU path holds every weight) */
ORACLE_API void oracle_bf16_to_f32(const uint16_t* in, long long n, float* out) {
#pragma omp parallel for
    for (long long i = 0; i < n; ++i) out[i] = moe_synth_bf16_bits_to_f32(in[i]);
}

ORACLE_API void oracle_f32_to_bf16(const float* in, long long n, uint16_t* out) {
#pragma omp parallel for
    for (long long i = 0; i < n; ++i) out[i] = moe_synth_f32_to_bf16_bits(in[i]);
}

/* ---- src/hip/scheduler.hip:11-61 ----------------------------------------------------- *
 * topk_i/topk_v [T,K] -> expert_offsets [E+1], tokens_flat [T*K], weights_flat [T*K],
 * slot_of [T*K] (position of assignment (t,k) inside tokens_flat).  Buckets are in ascending
 * expert id, tokens inside a bucket in ascending token id.
 */
ORACLE_API int oracle_bucket(const int* topk_i, const float* topk_v, int T, int K, int E,
                             int* expert_offsets, int* tokens_flat, float* weights_flat,
                             int* slot_of) {
    int* counts = (int*)calloc((size_t)E + 1, sizeof(int));
    if (!counts) return -3;
    for (long long a = 0; a < (long long)T * K; ++a) {
        int e = topk_i[a];
        if (e < 0 || e >= E) {
            free(counts);
            return -4;
        }
        counts[e]++;
    }
    int acc = 0;
    for (int e = 0; e < E; ++e) {
        expert_offsets[e] = acc;
        acc += counts[e];
        counts[e] = 0;
    }
    expert_offsets[E] = acc;
    for (int t = 0; t < T; ++t) {
        for (int k = 0; k < K; ++k) {
            int e = topk_i[(long long)t * K + k];
            int dst = expert_offsets[e] + counts[e]++;
            tokens_flat[dst] = t;
            weights_flat[dst] = topk_v[(long long)t * K + k];
            if (slot_of) slot_of[(long long)t * K + k] = dst;
        }
    }
    free(counts);
    return 0;
}

/* ---- src/hip/scheduler.hip:112-184 --------------------------------------------------- *
 * expert_offsets [E+1] -> wq_heavy / wq_light (triples expert, row_offset, row_count, ascending
 * expert id) and stats = {heavy_count, light_count, heavy_maxNe, active_experts, sumNe}.
 */
ORACLE_API void oracle_classify_queues(const int* expert_offsets, int E, int very_sparse_cutoff,
                                       float heavy_factor_sparse, float heavy_factor_default,
                                       int* wq_heavy, int* wq_light, long long* stats) {
    int active = 0;
    long long sum = 0;
    for (int e = 0; e < E; ++e) {
        int ne = expert_offsets[e + 1] - expert_offsets[e];
        if (ne > 0) {
            ++active;
            sum += ne;
        }
    }
    stats[0] = stats[1] = stats[2] = stats[3] = stats[4] = 0;
    if (active == 0) return;
    float avg = (float)sum / (float)active;
    float factor = heavy_factor_default;
    if (active <= very_sparse_cutoff)
        factor = 1.0f;
    else if (active <= 12)
        factor = heavy_factor_sparse;
    int thresh = (int)ceilf(factor * avg);
    int nh = 0, nl = 0, hmax = 0;
    for (int e = 0; e < E; ++e) {
        int off = expert_offsets[e];
        int ne = expert_offsets[e + 1] - off;
        if (ne <= 0) continue;
        if (active <= very_sparse_cutoff || ne >= thresh) {
            wq_heavy[3 * nh + 0] = e;
            wq_heavy[3 * nh + 1] = off;
            wq_heavy[3 * nh + 2] = ne;
            ++nh;
            if (ne > hmax) hmax = ne;
        } else {
            wq_light[3 * nl + 0] = e;
            wq_light[3 * nl + 1] = off;
            wq_light[3 * nl + 2] = ne;
            ++nl;
        }
    }
    stats[0] = nh;
    stats[1] = nl;
    stats[2] = hmax;
    stats[3] = active;
    stats[4] = sum;
}

/* ---- synthetic inputs (include/moe_synth.h), host side -------------------------------- */
ORACLE_API void oracle_synth_normal_table(float* table) { moe_synth_build_normal_table(table); }

/* every generator fills dst[0..n) with the stream elements start .. start+n-1 */
ORACLE_API void oracle_synth_normal_f32(float* dst, long long n, const float* table, float scale,
                                        unsigned seed, unsigned tensor_id, long long start) {
#pragma omp parallel for
    for (long long i = 0; i < n; ++i)
        dst[i] = moe_synth_normal_f32(table, scale, seed, tensor_id, (uint64_t)(start + i));
}

ORACLE_API void oracle_synth_normal_bf16(uint16_t* dst, long long n, const float* table, float scale,
                                         unsigned seed, unsigned tensor_id, long long start) {
#pragma omp parallel for
    for (long long i = 0; i < n; ++i)
        dst[i] = moe_synth_normal_bf16(table, scale, seed, tensor_id, (uint64_t)(start + i));
}

ORACLE_API void oracle_synth_bytes(uint8_t* dst, long long n, unsigned seed, unsigned tensor_id,
                                   long long start) {
#pragma omp parallel for
    for (long long i = 0; i < n; ++i) dst[i] = moe_synth_byte(seed, tensor_id, (uint64_t)(start + i));
}

ORACLE_API void oracle_synth_range_bytes(uint8_t* dst, long long n, unsigned seed, unsigned tensor_id,
                                         unsigned lo, unsigned span, long long start) {
#pragma omp parallel for
    for (long long i = 0; i < n; ++i)
        dst[i] = moe_synth_range_byte(seed, tensor_id, (uint64_t)(start + i), lo, span);
}
