/*
 * moe_abi.h — C ABI of libmoe_gfx950.so: the gpt-oss MoE expert block for one MI355X (gfx950).
 *
 * The reference (tuanlda78202/gpt-oss-amd) has no FFI boundary: its kernels are plain functions
 * in .hip files that src/forward.cpp includes textually (src/forward.cpp:2-16).  Each entry below
 * replaces one of those functions at its call site in the MoE section of the layer loop
 * (src/forward.cpp:317-514) and keeps that function's argument order and meaning; the citation
 * on each declaration names the function it stands in for.
 *
 * Conventions (all entries):
 *   - plain pointers and sizes only; every pointer is DEVICE memory unless named h_*;
 *   - the caller owns every buffer; nothing here allocates or frees device memory;
 *   - asynchronous: work is queued on `stream` (a hipStream_t passed as void*; NULL is the
 *     default stream) and the call returns without waiting;
 *   - returns 0 on success, a negative MOE_ERR_* for a rejected argument, or a positive
 *     hipError_t reported by the runtime.  Nothing exits the process or throws (the reference's
 *     CHECK_HIP prints and calls exit(1): include/model.hpp:8-17);
 *   - re-entrant per device: the library keeps no mutable global state, with one exception that
 *     says so where it is declared (moe_gemm_router_static: a fixed device array per GPU and its
 *     address, looked up once per device);
 *   - bf16 values cross the boundary as raw 16-bit patterns (moe_bf16_t); the reference's
 *     __hip_bfloat16 has the same size and bit layout.
 */
#ifndef MOE_ABI_H
#define MOE_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_ABI_VERSION 1

#define MOE_API __attribute__((visibility("default")))

typedef uint16_t moe_bf16_t;
typedef void* moe_stream_t;

enum {
    MOE_OK = 0,
    MOE_ERR_NULL = -1,       /* a required pointer is NULL */
    MOE_ERR_SHAPE = -2,      /* a dimension is non-positive or violates a documented multiple */
    MOE_ERR_LIMIT = -3,      /* a dimension exceeds a documented maximum */
    MOE_ERR_WORKSPACE = -4,  /* workspace missing, misaligned or too small */
    MOE_ERR_FORMAT = -5,     /* unknown weight format / flag */
    MOE_ERR_ALIGN = -6       /* a pointer does not have the documented alignment */
};

/* MXFP4: e2m1 codes, two per byte (low nibble = even element), one e8m0 scale byte per 32
 * consecutive elements along the input dimension; value = LUT[code] * 2^(scale-127)
 * (tools/model_export/gpt-oss-20b/export_model_bin.py:75-133). */
#define MOE_MXFP4_BLOCK_ELEMS 32
#define MOE_MXFP4_BLOCK_BYTES 16

enum {
    MOE_WEIGHTS_BF16 = 0,        /* [E, rows, K] bf16 row-major: the reference's device layout,
                                    include/model.hpp:109-117 */
    MOE_WEIGHTS_MXFP4_TILED = 1  /* output of moe_mxfp4_repack() */
};

MOE_API int moe_abi_version(void);
MOE_API const char* moe_error_string(int code);

/* ------------------------------------------------------------------------------------------
 * Router
 * ---------------------------------------------------------------------------------------- */

/* Replaces gemm_router (src/hip/gemms/gemm_router.hip:184-190; call site src/forward.cpp:321).
 * xout[n,m] = bias[m] + sum_k x_batch[n,k] * w[m,k], N tokens, K = hidden, M = experts.
 * Arithmetic follows the reference's CPU matmul (src/run.cpp:341-354): the product is an fp32
 * multiply of the fp32 activation with the widened bf16 weight, accumulated in fp64, rounded to
 * fp32, then the bias is added in fp32 (src/run.cpp:635-637).  Needs `scratch` of
 * moe_router_scratch_bytes(N, M) bytes (8-byte aligned).  M <= 1024, K % 8 == 0; x_batch and w
 * 16-byte aligned. */
MOE_API size_t moe_router_scratch_bytes(int N, int M);
MOE_API int moe_gemm_router(float* xout, const float* x_batch, const moe_bf16_t* w, const moe_bf16_t* bias,
                    int N, int K, int M, void* scratch, size_t scratch_bytes, moe_stream_t stream);

/* moe_gemm_router for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference;
 * its argument list is moe_gemm_router's without the scratch pair.  The fp64 partial sums live in a
 * fixed device array of
 * MOE_ROUTER_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held until the process
 * ends) instead of a caller buffer; the call allocates nothing.  Same arithmetic and same bits as
 * moe_gemm_router.  Returns MOE_ERR_LIMIT when the partial sums do not fit the array
 * (16 * N * M * 8 bytes always fit when N * M <= 131072: 4096 tokens x 32 experts,
 * 1024 x 128).  All calls on one GPU share the array: calls that overlap on one GPU (two streams,
 * two host threads) race, calls on one stream do not. */
#define MOE_ROUTER_STATIC_SCRATCH_BYTES (16u << 20)
MOE_API size_t moe_gemm_router_static_max_bytes(void);
MOE_API int moe_gemm_router_static(float* xout, const float* x_batch, const moe_bf16_t* w, const moe_bf16_t* bias,
                           int N, int K, int M, moe_stream_t stream);

/* The two-pass router that moe_block_forward uses for large batches, on its own and with its
 * intermediate results (no counterpart in the reference; same top-k and softmax weights as
 * moe_gemm_router + moe_topk + moe_softmax).  Pass 1 scores every expert approximately on the
 * matrix cores; pass 2 bounds the error of those scores per token, recomputes exactly (the
 * arithmetic of src/run.cpp:341-354) every expert whose approximate score is within twice the bound
 * of the K-th best, and selects among the exact scores.  Outputs besides topk_values / topk_indices
 * [N, experts_per_token], each optional: approx_scores [N, M] (pass 1, bias included), bound [N]
 * (the error bound pass 2 used), n_candidates [N] (experts rescored exactly).  A caller can thus
 * check the bound against exact scores of its own.  K % 32 == 0; scratch of
 * moe_router_two_pass_scratch_bytes(N, K, M) bytes, 16-byte aligned. */
MOE_API size_t moe_router_two_pass_scratch_bytes(int N, int K, int M);
MOE_API int moe_router_two_pass_report(const float* x_batch, const moe_bf16_t* w, const moe_bf16_t* bias, int N,
                               int K, int M, int experts_per_token, void* scratch, size_t scratch_bytes,
                               float* topk_values, int* topk_indices, float* approx_scores, float* bound,
                               int* n_candidates, moe_stream_t stream);

/* Replaces topk (src/hip/topk.hip:59-72; call site src/forward.cpp:325).  Per token the
 * experts_per_token largest scores in descending order with their indices; equal scores keep
 * the lower expert index first (the order the reference's CPU qsort yields, src/run.cpp:373-404).
 * num_experts <= 1024 (same limit as the reference), experts_per_token <= 8. */
MOE_API int moe_topk(float* topk_values, int* topk_indices, const float* router_scores, int batch_size,
             int num_experts, int experts_per_token, moe_stream_t stream);

/* Replaces softmax (src/hip/softmax.hip:46-51; call site src/forward.cpp:327): in place over the
 * last dimension of x [batch_size, size]; max and sum in fp64 as src/run.cpp:321-339.
 * size <= 64. */
MOE_API int moe_softmax(float* x, int batch_size, int size, moe_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Expert token bucketing
 * ---------------------------------------------------------------------------------------- */

/* Replaces the count / scan / compact sequence (src/hip/scheduler.hip:11-61; call sites
 * src/forward.cpp:333-349) with one launch and no atomics on the output order:
 *   expert_offsets [E+1]  exclusive prefix sum of tokens per expert
 *   tokens_flat    [B*K]  token ids grouped by expert, ascending token id inside a group
 *   weights_flat   [B*K]  the matching topk_v entry
 *   slot_of        [B*K]  optional: position of assignment (b,k) in tokens_flat
 * E <= 1024, K <= 8 (the limits of moe_topk).
 * Precondition (what moe_topk and the fused router write, and what the reference's kernels assume as
 * well): the K ids of one token are pairwise distinct and every id is in [0, E).  An id outside
 * [0, E) is dropped: it is counted in no bucket, expert_offsets[E] is then smaller than B*K, and its
 * slot_of entry is left as it was.  A token that names one expert twice gets one row in that bucket
 * (the first of the two k), while the bucket's count still says two: the last row of the expert's
 * range then holds whatever the buffer held before.  Neither case faults; neither is checked. */
MOE_API int moe_bucket_by_expert(const int* topk_i, const float* topk_v, int B, int K, int E,
                         int* expert_offsets, int* tokens_flat, float* weights_flat, int* slot_of,
                         moe_stream_t stream);

/* Replaces gather_rows / gather_rows_vec4 (src/hip/scheduler.hip:63-85; call site
 * src/forward.cpp:351-363): Y[row,:] = X[idx[row],:], fp32, H % 4 == 0. */
MOE_API int moe_gather_rows(const float* X, const int* idx, float* Y, int rows, int H, moe_stream_t stream);

/* The inverse of moe_gather_rows: X[idx[row],:] = Y[row,:] (idx without repeats).  No kernel of its
 * own in the reference, whose per-sequence state is the KV cache, written row by row at
 * batch_indices[row] inside split_qkv (call site src/forward.cpp:276-281); the decode loop of
 * host/moe_getp.hpp keeps one state row per sequence instead and returns a step's rows with this. */
MOE_API int moe_scatter_rows(const float* Y, const int* idx, float* X, int rows, int H, moe_stream_t stream);

/* The reference's bucketing steps one by one, each under the argument list of the kernel it replaces
 * plus the stream (the reference launches them inline with <<<grid, block, 0, stream>>>,
 * src/forward.cpp:333-376), for a host loop that keeps those call sites.  moe_bucket_by_expert above
 * does the first three in one launch.
 *
 * moe_count_tokens_per_expert: count_tokens_per_expert (src/hip/scheduler.hip:11-31).
 *   out_expert / out_token / out_w [B*K] = the assignments (b, k) flattened in b-major order: expert id,
 *   token b, routing weight; counts[e] += number of assignments to e (ids outside [0, E) are flattened
 *   but not counted).  counts must be zero on entry, as in the reference.
 * moe_exclusive_scan_expert_offsets: exclusive_scan_expert_offsets (:33-46).
 *   offsets[0] = 0, offsets[i+1] = counts[0] + .. + counts[i]; counts is zeroed.
 * moe_compact_by_expert: compact_by_expert_kernel (:48-61).
 *   tokens_flat / weights_flat [BK] = tokens / weights grouped by expert at offsets[e]; write_counters[e]
 *   grows by the bucket's size (zero on entry, as left by the scan).  Inside a bucket the entries keep
 *   ascending assignment index; the reference's order there is the order its atomic slot claims
 *   happen to finish.  One argument more than the reference kernel: E, the number of experts (the
 *   grid is one block per expert).  Every id must be in [0, E).
 * moe_classify_and_build_queues: classify_and_build_queues (:112-184), same decision rule, queues
 *   and statistics; moe_queue_stats is its MoEStats (:3-9).  wq_heavy / wq_light hold up to 3*E ints.
 * E <= 1024, B*K < 2^29. */
typedef struct moe_queue_stats {
    int heavy_count;
    int light_count;
    int heavy_maxNe;
    int active_experts;
    long long sumNe;
} moe_queue_stats;
MOE_API int moe_count_tokens_per_expert(const int* topk_i, const float* topk_v, int B, int K, int* out_expert,
                                int* out_token, float* out_w, int* counts, int E, moe_stream_t stream);
MOE_API int moe_exclusive_scan_expert_offsets(int* counts, int* offsets, int E, moe_stream_t stream);
MOE_API int moe_compact_by_expert(const int* expert_ids, const int* tokens, const float* weights, int BK,
                          const int* offsets, int* write_counters, int* tokens_flat, float* weights_flat, int E,
                          moe_stream_t stream);
MOE_API int moe_classify_and_build_queues(const int* expert_offsets, int E, int very_sparse_cutoff,
                                  float heavy_factor_sparse, float heavy_factor_default, int* wq_heavy,
                                  int* wq_light, moe_queue_stats* stats, moe_stream_t stream);

/* Replaces classify_and_build_queues (src/hip/scheduler.hip:112-184; call site
 * src/forward.cpp:373-376).  One queue of (expert, row_offset, row_count) triples for the
 * non-empty experts in ascending expert id; work_count[0] receives their number.  The
 * heavy/light split of the reference exists to feed two streams of different priority and is
 * not reproduced: the expert kernels here balance load themselves. */
MOE_API int moe_build_work_queue(const int* expert_offsets, int E, int* work_queue, int* work_count,
                         moe_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Expert GEMMs, reference data flow (fp32 rows gathered by expert)
 * ---------------------------------------------------------------------------------------- */

/* Replaces moe_mlp1_swiglu (src/hip/moe.hip:237-258; call sites src/forward.cpp:474, 492), same
 * argument list.  For each of the work_count queue entries (e, off, n) starting at entry
 * work_start: gate_by_expert[off+r, i] = swiglu(W1_e x_r + b1_e)[i] for the n rows
 * x_by_expert[off .. off+n).  W1 rows are interleaved gate, up, gate, up (src/run.cpp:667-670).
 * weights_base / bias_base point at the layer's first expert; strides are in elements.
 * maxNe is the largest row count in the queue (a smaller value is allowed: blocks then loop);
 * grid_cap is accepted for signature compatibility and ignored.  H % 64 == 0, I % 32 == 0. */
MOE_API int moe_mlp1_swiglu(const int* work_queue, int work_start, int work_count, const float* x_by_expert,
                    float* gate_by_expert, const moe_bf16_t* weights_base, const moe_bf16_t* bias_base,
                    int H, int I, long long expert_weight_stride, long long expert_bias_stride,
                    float alpha, float swiglu_limit, int maxNe, int grid_cap, moe_stream_t stream);

/* Replaces moe_mlp2_scatter (src/hip/moe.hip:514-536; call sites src/forward.cpp:481, 499), same
 * argument list.  For each queue entry:
 * e_agg[tokens_flat[off+r], :] += weights_flat[off+r] * (W2_e g_r + b2_e).
 * Like the reference this accumulates with fp32 atomics, so e_agg must be zero on entry and the
 * summation order over a token's experts is not fixed; moe_block_forward is the deterministic
 * path.  I % 64 == 0, H % 64 == 0. */
MOE_API int moe_mlp2_scatter(const int* work_queue, int work_start, int work_count, const float* gate_by_expert,
                     const int* tokens_flat, const float* weights_flat, float* e_agg,
                     const moe_bf16_t* weights_base, const moe_bf16_t* bias_base, int I, int H,
                     long long expert_weight_stride, long long expert_bias_stride, int maxNe,
                     int grid_cap, moe_stream_t stream);

/* MXFP4 siblings of the two entries above (no reference counterpart: the reference only ever
 * holds bf16 expert weights on the device).  tiled_blocks / tiled_scales are outputs of
 * moe_mxfp4_repack for the layer's [E, 2I, H] (mlp1) or [E, H, I] (mlp2) tensor. */
MOE_API int moe_mlp1_swiglu_mxfp4(const int* work_queue, int work_start, int work_count, const float* x_by_expert,
                          float* gate_by_expert, const uint8_t* tiled_blocks, const uint8_t* tiled_scales,
                          const moe_bf16_t* bias_base, int H, int I, long long expert_bias_stride,
                          float alpha, float swiglu_limit, int maxNe, int grid_cap, moe_stream_t stream);
MOE_API int moe_mlp2_scatter_mxfp4(const int* work_queue, int work_start, int work_count,
                           const float* gate_by_expert, const int* tokens_flat, const float* weights_flat,
                           float* e_agg, const uint8_t* tiled_blocks, const uint8_t* tiled_scales,
                           const moe_bf16_t* bias_base, int I, int H, long long expert_bias_stride,
                           int maxNe, int grid_cap, moe_stream_t stream);

/* Replaces vecadd_and_zero (src/hip/vecadd.hip:32-39; call site src/forward.cpp:514):
 * a += b * weight; b = 0. */
MOE_API int moe_vecadd_and_zero(float* a, float* b, float weight, int batch, int size, moe_stream_t stream);

/* FFN RMSNorm feeding the block (src/hip/rmsnorm.hip:3-45; call site src/forward.cpp:315;
 * arithmetic of src/run.cpp:306-319: fp64 sum of fp32 squares, eps 1e-5f). weight is bf16 as
 * the reference holds it on the device (include/model.hpp:93).  size % 4 == 0; o and x
 * 16-byte aligned, weight 8-byte aligned. */
MOE_API int moe_rmsnorm(float* o, const float* x, const moe_bf16_t* weight, int batch, int size,
                moe_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * MXFP4 (no counterpart at run time in the reference, which dequantises offline:
 * tools/model_export/gpt-oss-20b/export_model_bin.py:95-133)
 * ---------------------------------------------------------------------------------------- */

/* blocks [n_blocks,16] u8 + scales [n_blocks] u8 -> out [n_blocks*32] bf16, bit-exact with
 * dequantize_fp4 (export_model_bin.py:95-133) for every scale byte. */
MOE_API int moe_dequant_mxfp4(const uint8_t* blocks, const uint8_t* scales, long long n_blocks,
                      moe_bf16_t* out, moe_stream_t stream);

/* Load-time repack of one weight tensor from the checkpoint layout
 *   blocks [E, rows, K/32, 16] u8, scales [E, rows, K/32] u8
 * into the tiled layout the fused kernels stream with 128-bit loads.  K % 32 == 0.
 * moe_mxfp4_tiled_bytes gives the sizes of the two destination buffers for ONE expert; experts
 * are stored back to back.  moe_mxfp4_unpack is the exact inverse.  The tiled scale tensor is
 * padded to whole groups of four 128-element stages per row tile; moe_mxfp4_repack writes scale
 * byte 0 into the slots of MX blocks that do not exist (it clears the tensor first), and the
 * expert kernels rely on that byte: it converts to a factor of exactly 0 for whatever a lane past
 * the last block of a row has loaded.  A tiled tensor must therefore come from moe_mxfp4_repack
 * (or moe_ckpt_upload_layer, which calls it). */
MOE_API void moe_mxfp4_tiled_bytes(int rows, int K, size_t* block_bytes_per_expert,
                           size_t* scale_bytes_per_expert);
MOE_API int moe_mxfp4_repack(const uint8_t* blocks, const uint8_t* scales, int E, int rows, int K,
                     uint8_t* tiled_blocks, uint8_t* tiled_scales, moe_stream_t stream);
MOE_API int moe_mxfp4_unpack(const uint8_t* tiled_blocks, const uint8_t* tiled_scales, int E, int rows, int K,
                     uint8_t* blocks, uint8_t* scales, moe_stream_t stream);

/* Dequantise a tiled tensor back to row-major bf16 [E, rows, K] through the same device
 * routine the fused GEMM uses (so a bit-exact check of this output covers the fused path). */
MOE_API int moe_mxfp4_tiled_to_bf16(const uint8_t* tiled_blocks, const uint8_t* tiled_scales, int E, int rows,
                            int K, moe_bf16_t* out, moe_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * The whole block in one call: router -> top-k -> softmax -> bucketing -> gate/up GEMM + SwiGLU
 * -> down GEMM -> weighted combine in ascending expert id (src/forward.cpp:317-514 on the GPU,
 * src/run.cpp:628-707 on the CPU, whose arithmetic order it follows).
 * ---------------------------------------------------------------------------------------- */
typedef struct moe_block_params {
    uint32_t struct_bytes;   /* sizeof(moe_block_params) of the caller's header */
    int32_t n_tokens;        /* B <= 65535 */
    int32_t hidden_dim;      /* H, % 64 == 0 */
    int32_t intermediate_dim;/* I, % 64 == 0 */
    int32_t n_experts;       /* E <= 1024 */
    int32_t experts_per_token; /* K <= 8 */
    int32_t weight_format;   /* MOE_WEIGHTS_* for w_mlp1 / w_mlp2 */
    float swiglu_limit;      /* 7.0 */
    float alpha;             /* 1.702 */
    const float* t;          /* [B,H] block input (s->t) */
    const moe_bf16_t* w_router; /* [E,H] */
    const moe_bf16_t* b_router; /* [E] */
    const void* w_mlp1;      /* bf16 [E,2I,H] or tiled MXFP4 blocks */
    const void* w_mlp1_scales; /* tiled MXFP4 scales, else NULL */
    const moe_bf16_t* b_mlp1;/* [E,2I] */
    const void* w_mlp2;      /* bf16 [E,H,I] or tiled MXFP4 blocks */
    const void* w_mlp2_scales;
    const moe_bf16_t* b_mlp2;/* [E,H] */
    float* e_agg;            /* [B,H] output (overwritten, need not be zero) */
    int32_t* topk_i;         /* [B,K] output */
    float* topk_v;           /* [B,K] output (softmax weights) */
    float* router_score;     /* [B,E] optional output, may be NULL */
    float* residual_x;       /* optional: residual_x += e_agg (src/forward.cpp:514) */
    void* workspace;         /* moe_block_workspace_bytes(), 256-byte aligned */
    size_t workspace_bytes;
    uint32_t flags;          /* MOE_FLAG_* */
    /* Optional, both or neither; needs residual_x.  The RMSNorm that follows the residual add in
     * the layer loop (attention norm of the next layer, src/forward.cpp:262, or the final norm,
     * :997), done in the combine's pass over the row:
     *   next_norm_out = rmsnorm(residual_x after the add, next_norm_weight)   (as moe_rmsnorm)
     * A caller built against the struct without these two members (struct_bytes says so) gets
     * the behaviour of NULL. */
    const moe_bf16_t* next_norm_weight; /* [H] */
    float* next_norm_out;               /* [B,H] */
} moe_block_params;

enum {
    MOE_FLAG_ROUTER_STRICT_ORDER = 1u, /* accumulate each router dot product in one sequential
                                          pass over k, exactly the order of src/run.cpp:348-351 */
    MOE_FLAG_FORCE_STREAM = 2u,        /* always use the weight-streaming expert kernels */
    MOE_FLAG_FORCE_TILED = 4u,         /* always use the LDS-tiled expert kernels */
    MOE_FLAG_FORCE_DIRECT = 8u,        /* weight-streaming kernels: bucket inside the expert kernels whenever
                                          the batch allows it (n_tokens * experts_per_token <= 4096,
                                          n_tokens <= 2048), however long the buckets */
    MOE_FLAG_FORCE_BUCKET_LAUNCH = 16u, /* always run the bucketing kernel and its token-block map */
    MOE_FLAG_FUSED_GEMM_LAUNCH = 32u   /* decode-sized batches (those that bucket inside the expert kernels),
                                          n_experts <= 256: one launch for both expert GEMMs instead of one
                                          each; ignored for other batches */
};

MOE_API size_t moe_block_workspace_bytes(int n_tokens, int hidden_dim, int intermediate_dim, int n_experts,
                                 int experts_per_token);
MOE_API int moe_block_forward(const moe_block_params* params, moe_stream_t stream);

/* moe_block_forward for params[0 .. n_layers-1] in order on one stream: the MoE halves of a layer loop
 * (src/forward.cpp:258-514 runs one layer after the other the same way) issued by one call, for a host
 * language whose per-call cost would otherwise sit between the layers.  The array's stride is
 * params[0].struct_bytes (every element carries the same value).  Stops at the first error. */
MOE_API int moe_block_forward_layers(const moe_block_params* params, int n_layers, moe_stream_t stream);

/* Which kernels moe_block_forward would launch for these parameters (shapes, format, flags and
 * whether router_score / next_norm_out are set; pointers are not dereferenced and may be NULL), as
 * one line of text: "router=...; bucketing=...; gate_up=<kernel name as a profiler shows it>;
 * down=...; combine=...; compute_units=N".  For benchmarks and profile summaries that have to name
 * the kernel they measured.  text_bytes >= 64; MOE_ERR_LIMIT if the line does not fit. */
MOE_API int moe_block_describe(const moe_block_params* params, char* text, size_t text_bytes);

/* The down-projection GEMM of moe_block_forward on its own, on rows the caller provides (the
 * kernels that stand in for moe_mlp2_scatter_mfma_kernel, src/hip/moe.hip:261-512, without the
 * scatter): for every assignment (t, k), row t * K + k,
 *   y_by_assignment[t*K+k, :] = W2_e h_by_assignment[t*K+k, :] + b2_e,   e = params->topk_i[t, k].
 * params as for moe_block_forward with topk_i [B,K] as INPUT (distinct expert ids per token) and
 * t, w_router, b_router, w_mlp1, b_mlp1, e_agg unused; the same size rules and flags choose the
 * kernels, so a caller can put known rows (say unit vectors) through exactly the code the block
 * runs.  h_by_assignment: bf16 [B*K, I]; y_by_assignment: fp32 [B*K, H]; both 16-byte aligned. */
MOE_API int moe_block_down_gemm(const moe_block_params* params, const moe_bf16_t* h_by_assignment,
                        float* y_by_assignment, moe_stream_t stream);

/* Per-stage timing of moe_block_forward with HIP events on the caller's stream.  Stands in for
 * the reference's batch timing hooks, which its runtime calls but defines nowhere
 * (reset_batch_timings / print_batch_timing_summary, src/getp/run.cpp:322, 326).
 * Stages: 0 router partial dot products, 1 router finalise (top-k, softmax) + bf16 input copy,
 * 2 bucketing, 3 gate/up GEMM + SwiGLU, 4 down GEMM, 5 combine.
 * moe_block_forward_timed behaves like moe_block_forward and records MOE_N_STAGES + 1 events;
 * moe_stage_timer_read waits for the last event and returns the stage durations in ms. */
#define MOE_N_STAGES 6
typedef struct moe_stage_timer moe_stage_timer;
MOE_API int moe_stage_timer_create(moe_stage_timer** out);
MOE_API void moe_stage_timer_destroy(moe_stage_timer* timer);
MOE_API int moe_block_forward_timed(const moe_block_params* params, moe_stream_t stream, moe_stage_timer* timer);
MOE_API int moe_stage_timer_read(moe_stage_timer* timer, float* stage_ms);

/* ------------------------------------------------------------------------------------------
 * Synthetic workload generator (include/moe_synth.h), device side: fills device buffers with
 * the same values the host generator produces for (seed, tensor_id, index).
 * ---------------------------------------------------------------------------------------- */
/* Host side: the 65536-entry table of N(0,1) quantiles the normal generators index
 * (moe_synth_build_normal_table of include/moe_synth.h); h_table has room for 65536 floats. */
MOE_API void moe_synth_normal_table(float* h_table);
MOE_API int moe_synth_normal_f32(float* dst, long long n, const float* table_d, float scale, unsigned seed,
                         unsigned tensor_id, moe_stream_t stream);
MOE_API int moe_synth_normal_bf16(moe_bf16_t* dst, long long n, const float* table_d, float scale,
                          unsigned seed, unsigned tensor_id, moe_stream_t stream);
MOE_API int moe_synth_bytes(uint8_t* dst, long long n, unsigned seed, unsigned tensor_id, moe_stream_t stream);
MOE_API int moe_synth_range_bytes(uint8_t* dst, long long n, unsigned seed, unsigned tensor_id, unsigned lo,
                          unsigned span, moe_stream_t stream);

/* Checksum of a device buffer: out_d[0] = sum of its 32-bit little-endian words modulo 2^64.  n_bytes is a positive
 * multiple of 16, src is 16-byte aligned, out_d points to MOE_SYNTH_CHECKSUM_WORDS 64-bit words of device memory
 * (word 0 is the result, the rest per-block partial sums).  The launch only reads src, each byte once, so timed over
 * a buffer far larger than the caches it measures the read rate the device's memory sustains; the host generator
 * gives the expected value for a buffer filled by the moe_synth_* entries above.  No counterpart in the reference. */
#define MOE_SYNTH_CHECKSUM_WORDS 2049
MOE_API int moe_synth_checksum(const void* src, long long n_bytes, unsigned long long* out_d, moe_stream_t stream);

/* What the current device reports about itself (hipDeviceGetAttribute): compute units, engine clock and memory
 * clock in kHz, memory bus width in bits, L2 size in bytes.  Any pointer may be NULL.  No counterpart in the
 * reference; the benchmark prints these beside the published peaks it prices against. */
MOE_API int moe_device_attributes(int* compute_units, int* clock_khz, int* memory_clock_khz, int* memory_bus_bits,
                                  int* l2_bytes);

#ifdef __cplusplus
}
#endif
#endif /* MOE_ABI_H */
