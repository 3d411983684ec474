// Drop-in replacements, under the reference's own function names and argument lists, for the
// kernels the MoE section of its layer loop calls (src/forward.cpp:317-514).  Including this header
// instead of src/hip/gemms/gemm_router.hip, topk.hip, softmax.hip, scheduler.hip, moe.hip and
// vecadd.hip routes those calls through the C ABI of libmoe_gfx950.so (include/moe_abi.h).
//
// Differences a caller sees:
//   * errors come back as return codes (0 = ok) instead of exit(1) inside CHECK_HIP
//     (include/model.hpp:8-17);
//   * gemm_router needs a scratch buffer (fp64 partial sums): register one per host thread through
//     moe_router_scratch(), sized by moe_router_scratch_bytes(); without one the call returns
//     MOE_ERR_WORKSPACE.  A caller that cannot provide one (graph capture, no allocation allowed) may opt
//     into the fixed array inside the library with moe_router_scratch().use_static_array = true: that
//     array is one per GPU, so only ONE stream of ONE host thread per GPU may then run gemm_router at a
//     time (two calls that overlap on a GPU mix their partial sums and return wrong logits, silently);
//   * bucketing is one call (bucket_by_expert) instead of memset + three kernels
//     (src/forward.cpp:333-349), and there is one work queue instead of a heavy and a light one;
//   * __hip_bfloat16 pointers are passed as moe_bf16_t* (same size and bit layout).
#pragma once
#include "../../include/moe_abi.h"

namespace moe_dropin {

struct RouterScratch {
    void* ptr = nullptr;
    size_t bytes = 0;
    bool use_static_array = false;  // no buffer: fall back to moe_gemm_router_static (one call per GPU at a time!)
};
// one scratch registration per host thread, matching the reference's thread-per-GPU model
// (src/getp/run.cpp:680-692); the library itself keeps no state
inline RouterScratch& moe_router_scratch() {
    thread_local RouterScratch s;
    return s;
}

// src/hip/gemms/gemm_router.hip:184-185
inline int gemm_router(float* xout, const float* x_batch, const moe_bf16_t* w, const moe_bf16_t* bias, int N, int K,
                       int M, moe_stream_t stream = nullptr) {
    RouterScratch& s = moe_router_scratch();
    if (s.ptr) return moe_gemm_router(xout, x_batch, w, bias, N, K, M, s.ptr, s.bytes, stream);
    // no registered buffer: an error, unless the caller asked for the library's fixed array (see above)
    if (!s.use_static_array) return MOE_ERR_WORKSPACE;
    return moe_gemm_router_static(xout, x_batch, w, bias, N, K, M, stream);
}

// src/hip/topk.hip:59-60
inline int topk(float* topk_values, int* topk_indices, float* router_scores, int batch_size, int num_experts,
                int experts_per_token, moe_stream_t stream = nullptr) {
    return moe_topk(topk_values, topk_indices, router_scores, batch_size, num_experts, experts_per_token, stream);
}

// src/hip/softmax.hip:46
inline int softmax(float* x, int batch_size, int size, moe_stream_t stream = nullptr) {
    return moe_softmax(x, batch_size, size, stream);
}

// src/hip/scheduler.hip:11-61 (count_tokens_per_expert + exclusive_scan_expert_offsets +
// compact_by_expert_kernel), launched at src/forward.cpp:333-349
inline int bucket_by_expert(const int* topk_i, const float* topk_v, int B, int K, int E, int* expert_offsets,
                            int* tokens_flat, float* weights_flat, moe_stream_t stream = nullptr) {
    return moe_bucket_by_expert(topk_i, topk_v, B, K, E, expert_offsets, tokens_flat, weights_flat, nullptr, stream);
}

// The same three steps one by one, under the kernels' own names and argument lists + the stream
// (src/hip/scheduler.hip:11, 33, 48): `k<<<grid, block, 0, s>>>(args)` becomes `k(args, s)`;
// compact_by_expert_kernel also takes the number of experts.
using MoEStats = moe_queue_stats;  // src/hip/scheduler.hip:3-9
inline int count_tokens_per_expert(const int* topk_i, const float* topk_v, int B, int K, int* out_expert,
                                   int* out_token, float* out_w, int* counts, int E, moe_stream_t stream = nullptr) {
    return moe_count_tokens_per_expert(topk_i, topk_v, B, K, out_expert, out_token, out_w, counts, E, stream);
}
inline int exclusive_scan_expert_offsets(int* counts, int* offsets, int E, moe_stream_t stream = nullptr) {
    return moe_exclusive_scan_expert_offsets(counts, offsets, E, stream);
}
inline int compact_by_expert_kernel(const int* expert_ids, const int* tokens, const float* weights, int BK,
                                    const int* offsets, int* write_counters, int* tokens_flat, float* weights_flat,
                                    int E, moe_stream_t stream = nullptr) {
    return moe_compact_by_expert(expert_ids, tokens, weights, BK, offsets, write_counters, tokens_flat, weights_flat, E,
                                 stream);
}
// src/hip/scheduler.hip:112-119
inline int classify_and_build_queues(const int* expert_offsets, int E, int very_sparse_cutoff,
                                     float heavy_factor_sparse, float heavy_factor_default, int* wq_heavy,
                                     int* wq_light, MoEStats* stats_out, moe_stream_t stream = nullptr) {
    return moe_classify_and_build_queues(expert_offsets, E, very_sparse_cutoff, heavy_factor_sparse,
                                         heavy_factor_default, wq_heavy, wq_light, stats_out, stream);
}

// src/hip/scheduler.hip:63-85, launched at src/forward.cpp:351-363
inline int gather_rows(const float* X, const int* idx, float* Y, int BK, int H, moe_stream_t stream = nullptr) {
    return moe_gather_rows(X, idx, Y, BK, H, stream);
}

// src/hip/scheduler.hip:112-184, launched at src/forward.cpp:373-376
inline int build_work_queue(const int* expert_offsets, int E, int* work_queue, int* work_count_d,
                            moe_stream_t stream = nullptr) {
    return moe_build_work_queue(expert_offsets, E, work_queue, work_count_d, stream);
}

// src/hip/moe.hip:237-242
inline int moe_mlp1_swiglu(const int* work_queue, int work_start, int work_count, const float* x_by_expert,
                           float* gate_by_expert, const moe_bf16_t* weights_base, const moe_bf16_t* bias_base, int H,
                           int I, long long expert_weight_stride, long long expert_bias_stride, float alpha,
                           float swiglu_limit, int maxNe, int grid_cap, moe_stream_t stream = nullptr) {
    return ::moe_mlp1_swiglu(work_queue, work_start, work_count, x_by_expert, gate_by_expert, weights_base, bias_base,
                             H, I, expert_weight_stride, expert_bias_stride, alpha, swiglu_limit, maxNe, grid_cap,
                             stream);
}

// src/hip/moe.hip:514-520
inline int moe_mlp2_scatter(const int* work_queue, int work_start, int work_count, const float* gate_by_expert,
                            const int* tokens_flat, const float* weights_flat, float* e_agg,
                            const moe_bf16_t* weights_base, const moe_bf16_t* bias_base, int I, int H,
                            long long expert_weight_stride, long long expert_bias_stride, int maxNe, int grid_cap,
                            moe_stream_t stream = nullptr) {
    return ::moe_mlp2_scatter(work_queue, work_start, work_count, gate_by_expert, tokens_flat, weights_flat, e_agg,
                              weights_base, bias_base, I, H, expert_weight_stride, expert_bias_stride, maxNe, grid_cap,
                              stream);
}

// src/hip/vecadd.hip:32-33
inline int vecadd_and_zero(float* a, float* b, float weight, int batch_size, int size,
                           moe_stream_t stream = nullptr) {
    return moe_vecadd_and_zero(a, b, weight, batch_size, size, stream);
}

// src/hip/rmsnorm.hip:39 (the FFN norm that produces the block input, src/forward.cpp:315)
inline int rmsnorm(float* o, const float* x, const moe_bf16_t* weight, int batch_size, int size,
                   moe_stream_t stream = nullptr) {
    return moe_rmsnorm(o, x, weight, batch_size, size, stream);
}

}  // namespace moe_dropin
