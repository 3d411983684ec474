// extern "C" entry points of libmoe_gfx950.so (declared in include/moe_abi.h): argument checks,
// workspace carving and launch sequencing.  No entry allocates, synchronises or exits.
#include "../../include/moe_checkpoint.h"
#include "../../include/moe_synth.h"
#include "common.h"
#include "kernels.h"

#include <algorithm>
#include <atomic>
#include <cstddef>
#include <cstdio>
#include <cstring>
#include <new>

using namespace moe;

namespace {

constexpr size_t kAlign = 256;
inline size_t align_up(size_t v) { return (v + kAlign - 1) / kAlign * kAlign; }
inline hipStream_t as_stream(moe_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Token-block sizes of the expert kernels' tile map: decode-sized buckets / prefill-sized buckets.
constexpr int kStreamTileTokens = 64;
constexpr int kPrefillTileTokens = 128;

// Which family runs the expert GEMMs, by average bucket size T*K/E (measured crossovers, 20b
// shapes, token counts 256..4096).  MXFP4: the 128-token-block kernels win as soon as buckets start
// to overflow one 64-token block (the streaming kernel then reads an expert's weights once per
// block of its bucket).  bf16: the same (E = 32: 350 against 428 us at 48 rows per expert, 572 against
// 437 us at 64).
inline bool use_prefill_kernels(int T, int K, int E, int format, unsigned flags) {
    if (flags & MOE_FLAG_FORCE_STREAM) return false;
    if (flags & MOE_FLAG_FORCE_TILED) return true;
    const long long rows = (long long)T * K;
    return format == MOE_WEIGHTS_MXFP4_TILED ? rows >= 52LL * E : rows >= 56LL * E;
}

// Bucketing inside the expert kernels instead of a launch of its own: for the weight-streaming
// kernels, while the assignment list is short enough for one block to scan and buckets mostly fit one
// 64-token block (a block runs its bucket's token blocks one after the other).
inline bool use_direct_bucketing(int T, int K, int E, bool prefill, unsigned flags) {
    if (prefill || (flags & MOE_FLAG_FORCE_BUCKET_LAUNCH)) return false;
    const long long A = (long long)T * K;
    if (A > expert_direct_max_assignments() || T > 2048) return false;
    if (flags & MOE_FLAG_FORCE_DIRECT) return true;
    return A <= 48LL * E;
}

// Both expert GEMMs in one launch: on request, when the bucketing is done inside the expert kernels and
// the experts fit the kernel's per-XCD tables.  Measured at the 20b decode shape it ties with the two
// launches for bf16 weights (what it saves in launch boundaries it pays for emptying and refilling its
// pipeline where a down item has to wait for its expert's gate/up items) and is slower for MXFP4,
// whose stages are a quarter as long; so it is not the default.
inline bool use_fused_experts(int E, bool direct, unsigned flags) {
    return direct && (flags & MOE_FLAG_FUSED_GEMM_LAUNCH) && E <= expert_fused_max_experts();
}

// Carves the caller's workspace for moe_block_forward; with base == nullptr only sizes it.
struct BlockWorkspace {
    double* router_partial;
    uint16_t* t_bf16;      // [T,H] bf16 copy of the block input
    int* expert_offsets;   // [E+1]
    int* tokens_flat;      // [A]
    float* weights_flat;   // [A]
    int* slot_of;          // [A]
    int* tile_expert;      // [2][max_tiles]: the token-block map in two orders (bucket.hip)
    int* tile_row0;
    int* tile_rows;
    int* n_tiles;          // [1]
    int* fused_ctr;        // counters of the one-launch expert kernel (experts_fused.hip)
    uint16_t* h_by_slot;   // [A, I] bf16 SwiGLU outputs
    float* y_by_slot;      // [A, H] fp32 down-projection rows
    int max_tiles;
    size_t bytes;

    BlockWorkspace(void* base, int T, int H, int I, int E, int K) {
        const size_t A = (size_t)T * K;
        size_t off = 0;
        auto take = [&](size_t n) {
            void* p = base ? static_cast<char*>(base) + off : nullptr;
            off += align_up(n);
            return p;
        };
        const int S = router_segments(T, E, H, false);
        router_partial = static_cast<double*>(
            take(std::max((size_t)S * T * E * sizeof(double), router_two_pass(T, E, H) ? router_screen_bytes(T, E, H) : 0)));
        t_bf16 = static_cast<uint16_t*>(take((size_t)T * H * 2));
        expert_offsets = static_cast<int*>(take((size_t)(E + 1) * 4));
        tokens_flat = static_cast<int*>(take(A * 4));
        weights_flat = static_cast<float*>(take(A * 4));
        slot_of = static_cast<int*>(take(A * 4));
        max_tiles = tile_map_capacity((int)A, E, kStreamTileTokens);
        tile_expert = static_cast<int*>(take((size_t)2 * max_tiles * 4));
        tile_row0 = static_cast<int*>(take((size_t)2 * max_tiles * 4));
        tile_rows = static_cast<int*>(take((size_t)2 * max_tiles * 4));
        n_tiles = static_cast<int*>(take(4));
        fused_ctr = static_cast<int*>(take((size_t)expert_fused_ctr_words(E) * 4));
        h_by_slot = static_cast<uint16_t*>(take(A * I * 2));
        y_by_slot = static_cast<float*>(take(A * H * 4));
        bytes = off;
    }
};

int check_dims(int T, int H, int I, int E, int K) {
    if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || K <= 0) return MOE_ERR_SHAPE;
    if (H % 64 != 0 || I % 64 != 0) return MOE_ERR_SHAPE;
    if (K > E) return MOE_ERR_SHAPE;
    if (E > 1024 || K > 8) return MOE_ERR_LIMIT;
    if (T > 65535) return MOE_ERR_LIMIT;  // one grid row per token in the combine kernel
    return MOE_OK;
}

}  // namespace

extern "C" {

int moe_abi_version(void) { return MOE_ABI_VERSION; }

const char* moe_error_string(int code) {
    switch (code) {
        case MOE_OK: return "ok";
        case MOE_ERR_NULL: return "a required pointer is NULL";
        case MOE_ERR_SHAPE: return "a dimension is non-positive or not a documented multiple";
        case MOE_ERR_LIMIT: return "a dimension exceeds a documented maximum";
        case MOE_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case MOE_ERR_FORMAT: return "unknown weight format or flag";
        case MOE_ERR_ALIGN: return "a pointer does not have the documented alignment";
        case MOE_ERR_IO: return "the file cannot be opened, sized or mapped";
        case MOE_ERR_PARSE: return "malformed checkpoint header";
        case MOE_ERR_MISSING: return "a tensor the call needs is not in the file";
        default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}

// ---- router ----------------------------------------------------------------------------------
size_t moe_router_scratch_bytes(int N, int M) {
    if (N <= 0 || M <= 0) return 0;
    return (size_t)16 * N * M * sizeof(double);
}

int moe_gemm_router(float* xout, const float* x_batch, const moe_bf16_t* w, const moe_bf16_t* bias, int N,
                    int K, int M, void* scratch, size_t scratch_bytes, moe_stream_t stream) {
    if (!xout || !x_batch || !w || !bias) return MOE_ERR_NULL;
    if (N <= 0 || K <= 0 || M <= 0 || K % 8 != 0) return MOE_ERR_SHAPE;
    if (M > 1024) return MOE_ERR_LIMIT;
    if (((uintptr_t)x_batch | (uintptr_t)w) & 15u) return MOE_ERR_ALIGN;
    const int S = router_segments(N, M, K, false);
    if (!scratch || ((uintptr_t)scratch & 7u) || scratch_bytes < (size_t)S * N * M * sizeof(double))
        return MOE_ERR_WORKSPACE;
    double* partial = static_cast<double*>(scratch);
    int rc = launch_router_partial(x_batch, w, partial, nullptr, N, K, M, S, as_stream(stream));
    if (rc) return rc;
    return launch_router_finalize(partial, S, nullptr, bias, xout, nullptr, nullptr, N, M, 0, 0, 0, as_stream(stream));
}

size_t moe_router_two_pass_scratch_bytes(int N, int K, int M) {
    if (N <= 0 || K <= 0 || M <= 0 || K % 32 != 0) return 0;
    return router_screen_bytes(N, M, K);
}

int moe_router_two_pass_report(const float* x_batch, const moe_bf16_t* w, const moe_bf16_t* bias, int N, int K, int M,
                               int experts_per_token, void* scratch, size_t scratch_bytes, float* topk_values,
                               int* topk_indices, float* approx_scores, float* bound, int* n_candidates,
                               moe_stream_t stream) {
    if (!x_batch || !w || !bias || !topk_values || !topk_indices) return MOE_ERR_NULL;
    if (N <= 0 || K <= 0 || M <= 0 || K % 32 != 0 || experts_per_token <= 0 || experts_per_token > M)
        return MOE_ERR_SHAPE;
    if (M > 1024 || experts_per_token > 8) return MOE_ERR_LIMIT;
    if (((uintptr_t)x_batch | (uintptr_t)w) & 15u) return MOE_ERR_ALIGN;
    if (!scratch || ((uintptr_t)scratch & 15u) || scratch_bytes < router_screen_bytes(N, M, K)) return MOE_ERR_WORKSPACE;
    return launch_router_two_pass(x_batch, w, bias, scratch, nullptr, topk_values, topk_indices, N, K, M,
                                  experts_per_token, 1, as_stream(stream), nullptr, approx_scores, bound, n_candidates);
}

int moe_topk(float* topk_values, int* topk_indices, const float* router_scores, int batch_size, int num_experts,
             int experts_per_token, moe_stream_t stream) {
    if (!topk_values || !topk_indices || !router_scores) return MOE_ERR_NULL;
    if (batch_size <= 0 || num_experts <= 0 || experts_per_token <= 0 || experts_per_token > num_experts)
        return MOE_ERR_SHAPE;
    if (num_experts > 1024 || experts_per_token > 8) return MOE_ERR_LIMIT;
    return launch_router_finalize(nullptr, 0, router_scores, nullptr, nullptr, topk_values, topk_indices, batch_size,
                                  num_experts, experts_per_token, 1, 0, as_stream(stream));
}

int moe_softmax(float* x, int batch_size, int size, moe_stream_t stream) {
    if (!x) return MOE_ERR_NULL;
    if (batch_size <= 0 || size <= 0) return MOE_ERR_SHAPE;
    if (size > 64) return MOE_ERR_LIMIT;
    return launch_softmax_rows(x, batch_size, size, as_stream(stream));
}

// ---- bucketing -------------------------------------------------------------------------------
int moe_bucket_by_expert(const int* topk_i, const float* topk_v, int B, int K, int E, int* expert_offsets,
                         int* tokens_flat, float* weights_flat, int* slot_of, moe_stream_t stream) {
    if (!topk_i || !topk_v || !expert_offsets || !tokens_flat || !weights_flat) return MOE_ERR_NULL;
    if (B <= 0 || K <= 0 || E <= 0) return MOE_ERR_SHAPE;
    if (E > 1024 || K > 8 || (long long)B * K > 0x7FFFFFFFll / 4) return MOE_ERR_LIMIT;
    TileMap none{nullptr, nullptr, nullptr, nullptr, 0, 0, 0};
    return launch_bucket(topk_i, topk_v, B, K, E, expert_offsets, tokens_flat, weights_flat, slot_of, none,
                         as_stream(stream));
}

int moe_gather_rows(const float* X, const int* idx, float* Y, int rows, int H, moe_stream_t stream) {
    if (!X || !idx || !Y) return MOE_ERR_NULL;
    if (rows <= 0 || H <= 0 || H % 4 != 0) return MOE_ERR_SHAPE;
    return launch_gather_rows(X, idx, Y, rows, H, as_stream(stream));  // slabs of 65535 rows inside
}

int moe_scatter_rows(const float* Y, const int* idx, float* X, int rows, int H, moe_stream_t stream) {
    if (!X || !idx || !Y) return MOE_ERR_NULL;
    if (rows <= 0 || H <= 0 || H % 4 != 0) return MOE_ERR_SHAPE;
    return launch_scatter_rows(Y, idx, X, rows, H, as_stream(stream));  // slabs of 65535 rows inside
}

int moe_count_tokens_per_expert(const int* topk_i, const float* topk_v, int B, int K, int* out_expert, int* out_token,
                                float* out_w, int* counts, int E, moe_stream_t stream) {
    if (!topk_i || !topk_v || !out_expert || !out_token || !out_w || !counts) return MOE_ERR_NULL;
    if (B <= 0 || K <= 0 || E <= 0) return MOE_ERR_SHAPE;
    if (E > 1024 || (long long)B * K >= (1LL << 29)) return MOE_ERR_LIMIT;
    return launch_count_tokens_per_expert(topk_i, topk_v, B, K, out_expert, out_token, out_w, counts, E,
                                          as_stream(stream));
}

int moe_exclusive_scan_expert_offsets(int* counts, int* offsets, int E, moe_stream_t stream) {
    if (!counts || !offsets) return MOE_ERR_NULL;
    if (E <= 0) return MOE_ERR_SHAPE;
    if (E > 1024) return MOE_ERR_LIMIT;
    return launch_exclusive_scan_expert_offsets(counts, offsets, E, as_stream(stream));
}

int moe_compact_by_expert(const int* expert_ids, const int* tokens, const float* weights, int BK, const int* offsets,
                          int* write_counters, int* tokens_flat, float* weights_flat, int E, moe_stream_t stream) {
    if (!expert_ids || !tokens || !weights || !offsets || !write_counters || !tokens_flat || !weights_flat)
        return MOE_ERR_NULL;
    if (BK <= 0 || E <= 0) return MOE_ERR_SHAPE;
    if (E > 1024 || BK >= (1 << 29)) return MOE_ERR_LIMIT;
    return launch_compact_by_expert(expert_ids, tokens, weights, BK, offsets, write_counters, tokens_flat, weights_flat,
                                    E, as_stream(stream));
}

int moe_classify_and_build_queues(const int* expert_offsets, int E, int very_sparse_cutoff, float heavy_factor_sparse,
                                  float heavy_factor_default, int* wq_heavy, int* wq_light, moe_queue_stats* stats,
                                  moe_stream_t stream) {
    if (!expert_offsets || !wq_heavy || !wq_light || !stats) return MOE_ERR_NULL;
    if (E <= 0) return MOE_ERR_SHAPE;
    if (E > 1024) return MOE_ERR_LIMIT;
    return launch_classify_and_build_queues(expert_offsets, E, very_sparse_cutoff, heavy_factor_sparse,
                                            heavy_factor_default, wq_heavy, wq_light, stats, as_stream(stream));
}

int moe_build_work_queue(const int* expert_offsets, int E, int* work_queue, int* work_count, moe_stream_t stream) {
    if (!expert_offsets || !work_queue || !work_count) return MOE_ERR_NULL;
    if (E <= 0) return MOE_ERR_SHAPE;
    return launch_build_work_queue(expert_offsets, E, work_queue, work_count, as_stream(stream));
}

// ---- expert GEMMs, reference data flow ---------------------------------------------------------
static int queue_gemm(int epi, int format, const int* work_queue, int work_start, int work_count,
                      const float* act, void* out, const int* tokens_flat, const float* weights_flat,
                      const void* w, const uint8_t* w_scales, const moe_bf16_t* bias, int rows, int Kdim,
                      long long w_stride, long long s_stride, long long bias_stride, float alpha, float limit,
                      int maxNe, moe_stream_t stream) {
    if (!work_queue || !act || !out || !w || !bias) return MOE_ERR_NULL;
    if (format == MOE_WEIGHTS_MXFP4_TILED && !w_scales) return MOE_ERR_NULL;
    if (work_count < 0 || work_start < 0 || rows <= 0 || Kdim <= 0) return MOE_ERR_SHAPE;
    if (work_count > 65535) return MOE_ERR_LIMIT;
    ExpertGemmArgs a{};
    a.w = w;
    a.w_scales = w_scales;
    a.bias = bias;
    a.act_f32 = act;
    a.tokens_flat = tokens_flat;
    a.weights_flat = weights_flat;
    a.work_queue = work_queue;
    a.work_start = work_start;
    a.work_count = work_count;
    a.max_rows_hint = maxNe < 64 ? 64 : (maxNe > 64 * 1024 ? 64 * 1024 : maxNe);
    a.out = out;
    a.rows = rows;
    a.K = Kdim;
    a.w_expert_stride = w_stride;
    a.s_expert_stride = s_stride;
    a.bias_expert_stride = bias_stride;
    a.alpha = alpha;
    a.limit = limit;
    a.format = format;
    a.waves_per_block = 4;
    return launch_expert_stream(a, epi, as_stream(stream));
}

int moe_mlp1_swiglu(const int* work_queue, int work_start, int work_count, const float* x_by_expert,
                    float* gate_by_expert, const moe_bf16_t* weights_base, const moe_bf16_t* bias_base, int H, int I,
                    long long expert_weight_stride, long long expert_bias_stride, float alpha, float swiglu_limit,
                    int maxNe, int grid_cap, moe_stream_t stream) {
    (void)grid_cap;
    if (H % 64 != 0 || I % 32 != 0) return MOE_ERR_SHAPE;
    return queue_gemm(2, MOE_WEIGHTS_BF16, work_queue, work_start, work_count, x_by_expert, gate_by_expert, nullptr,
                      nullptr, weights_base, nullptr, bias_base, 2 * I, H, expert_weight_stride, 0,
                      expert_bias_stride, alpha, swiglu_limit, maxNe, stream);
}

int moe_mlp2_scatter(const int* work_queue, int work_start, int work_count, const float* gate_by_expert,
                     const int* tokens_flat, const float* weights_flat, float* e_agg,
                     const moe_bf16_t* weights_base, const moe_bf16_t* bias_base, int I, int H,
                     long long expert_weight_stride, long long expert_bias_stride, int maxNe, int grid_cap,
                     moe_stream_t stream) {
    (void)grid_cap;
    if (!tokens_flat || !weights_flat) return MOE_ERR_NULL;
    if (H % 64 != 0 || I % 64 != 0) return MOE_ERR_SHAPE;
    return queue_gemm(3, MOE_WEIGHTS_BF16, work_queue, work_start, work_count, gate_by_expert, e_agg, tokens_flat,
                      weights_flat, weights_base, nullptr, bias_base, H, I, expert_weight_stride, 0,
                      expert_bias_stride, 0.f, 0.f, maxNe, stream);
}

int moe_mlp1_swiglu_mxfp4(const int* work_queue, int work_start, int work_count, const float* x_by_expert,
                          float* gate_by_expert, const uint8_t* tiled_blocks, const uint8_t* tiled_scales,
                          const moe_bf16_t* bias_base, int H, int I, long long expert_bias_stride, float alpha,
                          float swiglu_limit, int maxNe, int grid_cap, moe_stream_t stream) {
    (void)grid_cap;
    if (H % 32 != 0 || I % 32 != 0 || H <= 0 || I <= 0) return MOE_ERR_SHAPE;
    size_t bb, sb;
    mxfp4_tiled_bytes(2 * I, H, &bb, &sb);
    return queue_gemm(2, MOE_WEIGHTS_MXFP4_TILED, work_queue, work_start, work_count, x_by_expert, gate_by_expert,
                      nullptr, nullptr, tiled_blocks, tiled_scales, bias_base, 2 * I, H, (long long)bb, (long long)sb,
                      expert_bias_stride, alpha, swiglu_limit, maxNe, stream);
}

int moe_mlp2_scatter_mxfp4(const int* work_queue, int work_start, int work_count, const float* gate_by_expert,
                           const int* tokens_flat, const float* weights_flat, float* e_agg,
                           const uint8_t* tiled_blocks, const uint8_t* tiled_scales, const moe_bf16_t* bias_base,
                           int I, int H, long long expert_bias_stride, int maxNe, int grid_cap, moe_stream_t stream) {
    (void)grid_cap;
    if (!tokens_flat || !weights_flat) return MOE_ERR_NULL;
    if (H % 64 != 0 || I % 32 != 0 || H <= 0 || I <= 0) return MOE_ERR_SHAPE;
    size_t bb, sb;
    mxfp4_tiled_bytes(H, I, &bb, &sb);
    return queue_gemm(3, MOE_WEIGHTS_MXFP4_TILED, work_queue, work_start, work_count, gate_by_expert, e_agg,
                      tokens_flat, weights_flat, tiled_blocks, tiled_scales, bias_base, H, I, (long long)bb,
                      (long long)sb, expert_bias_stride, 0.f, 0.f, maxNe, stream);
}

int moe_vecadd_and_zero(float* a, float* b, float weight, int batch, int size, moe_stream_t stream) {
    if (!a || !b) return MOE_ERR_NULL;
    if (batch <= 0 || size <= 0) return MOE_ERR_SHAPE;
    return launch_vecadd_and_zero(a, b, weight, batch, size, as_stream(stream));
}

int moe_rmsnorm(float* o, const float* x, const moe_bf16_t* weight, int batch, int size, moe_stream_t stream) {
    if (!o || !x || !weight) return MOE_ERR_NULL;
    if (batch <= 0 || size <= 0 || size % 4 != 0) return MOE_ERR_SHAPE;
    if ((((uintptr_t)o | (uintptr_t)x) & 15u) || ((uintptr_t)weight & 7u)) return MOE_ERR_ALIGN;
    return launch_rmsnorm(o, x, weight, batch, size, as_stream(stream));
}

// ---- MXFP4 -----------------------------------------------------------------------------------
int moe_dequant_mxfp4(const uint8_t* blocks, const uint8_t* scales, long long n_blocks, moe_bf16_t* out,
                      moe_stream_t stream) {
    if (!blocks || !scales || !out) return MOE_ERR_NULL;
    if (n_blocks <= 0) return MOE_ERR_SHAPE;
    if (n_blocks > 0x7FFFFFFFll * 256) return MOE_ERR_LIMIT;
    if (((uintptr_t)blocks | (uintptr_t)out) & 15u) return MOE_ERR_ALIGN;
    return launch_dequant_mxfp4(blocks, scales, n_blocks, out, as_stream(stream));
}

void moe_mxfp4_tiled_bytes(int rows, int K, size_t* block_bytes_per_expert, size_t* scale_bytes_per_expert) {
    if (rows <= 0 || K <= 0 || rows % 64 != 0 || K % 32 != 0) {
        if (block_bytes_per_expert) *block_bytes_per_expert = 0;
        if (scale_bytes_per_expert) *scale_bytes_per_expert = 0;
        return;
    }
    mxfp4_tiled_bytes(rows, K, block_bytes_per_expert, scale_bytes_per_expert);
}

static int repack_common(const uint8_t* blocks, const uint8_t* scales, int E, int rows, int K, uint8_t* tiled_blocks,
                         uint8_t* tiled_scales, bool inverse, moe_stream_t stream) {
    if (!blocks || !scales || !tiled_blocks || !tiled_scales) return MOE_ERR_NULL;
    if (E <= 0 || rows <= 0 || K <= 0 || rows % 64 != 0 || K % 32 != 0) return MOE_ERR_SHAPE;
    if (((uintptr_t)blocks | (uintptr_t)tiled_blocks) & 15u) return MOE_ERR_ALIGN;
    if ((uintptr_t)tiled_scales & 3u) return MOE_ERR_ALIGN;
    if ((long long)E * rows * (K / 32) > 0x7FFFFFFFll * 256) return MOE_ERR_LIMIT;
    return launch_mxfp4_repack(blocks, scales, E, rows, K, tiled_blocks, tiled_scales, inverse, as_stream(stream));
}

int moe_mxfp4_repack(const uint8_t* blocks, const uint8_t* scales, int E, int rows, int K, uint8_t* tiled_blocks,
                     uint8_t* tiled_scales, moe_stream_t stream) {
    return repack_common(blocks, scales, E, rows, K, tiled_blocks, tiled_scales, false, stream);
}

int moe_mxfp4_unpack(const uint8_t* tiled_blocks, const uint8_t* tiled_scales, int E, int rows, int K,
                     uint8_t* blocks, uint8_t* scales, moe_stream_t stream) {
    return repack_common(blocks, scales, E, rows, K, const_cast<uint8_t*>(tiled_blocks),
                         const_cast<uint8_t*>(tiled_scales), true, stream);
}

int moe_mxfp4_tiled_to_bf16(const uint8_t* tiled_blocks, const uint8_t* tiled_scales, int E, int rows, int K,
                            moe_bf16_t* out, moe_stream_t stream) {
    if (!tiled_blocks || !tiled_scales || !out) return MOE_ERR_NULL;
    if (E <= 0 || rows <= 0 || K <= 0 || rows % 64 != 0 || K % 32 != 0) return MOE_ERR_SHAPE;
    if (((uintptr_t)tiled_blocks | (uintptr_t)out) & 15u) return MOE_ERR_ALIGN;
    return launch_mxfp4_tiled_to_bf16(tiled_blocks, tiled_scales, E, rows, K, out, as_stream(stream));
}

// ---- whole block -----------------------------------------------------------------------------
size_t moe_block_workspace_bytes(int n_tokens, int hidden_dim, int intermediate_dim, int n_experts,
                                 int experts_per_token) {
    if (check_dims(n_tokens, hidden_dim, intermediate_dim, n_experts, experts_per_token) != MOE_OK) return 0;
    return BlockWorkspace(nullptr, n_tokens, hidden_dim, intermediate_dim, n_experts, experts_per_token).bytes;
}

struct moe_stage_timer {
    hipEvent_t ev[MOE_N_STAGES + 1];
};

// Compute units of the current device, asked once per device (the kernel choices below count rounds
// of blocks over them).
static int device_cu_count() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// Launch parameters of the two expert GEMMs of one block.
struct ExpertPlan {
    const moe_block_params* p;
    ExpertGemmArgs g{};
    bool prefill, direct;
    int est_tiles, n_cus;
    int second_map;  // index of the token-block map in bucket order inside the map arrays

    ExpertPlan(const moe_block_params* p_, const BlockWorkspace& ws, bool prefill_, bool direct_, int tile_tokens,
               int max_tiles)
        : p(p_), prefill(prefill_), direct(direct_) {
        const int T = p->n_tokens, E = p->n_experts, K = p->experts_per_token;
        g.tokens_flat = ws.tokens_flat;
        g.tile_expert = ws.tile_expert;
        g.tile_row0 = ws.tile_row0;
        g.tile_rows = ws.tile_rows;
        g.n_tiles = ws.n_tiles;
        g.max_tiles = max_tiles;
        g.alpha = p->alpha;
        g.limit = p->swiglu_limit;
        g.format = p->weight_format;
        if (direct) {
            g.topk_i = p->topk_i;
            g.n_assign = T * K;
            g.assign_div = K;
            g.n_experts = E;
        }
        est_tiles = direct ? E : std::max(ceil_div(T * K, tile_tokens), std::min(E, T * K));
        n_cus = device_cu_count();
        second_map = ws.max_tiles;
    }
    // Decode-sized buckets (producer/consumer kernel, one block per CU): 10 or 12 consumer waves of
    // 32 rows each.  Blocks run in rounds of one per CU, so the cheaper choice is the one with the
    // smaller rounds x rows-per-block product; more rows per block also re-read the activations less.
    int pick_kernel(int rows) const {
        if (prefill) {  // bf16 weights, buckets of 80 rows and more on average: the one-block-a-CU kernel
            const bool big = (long long)p->n_tokens * p->experts_per_token >= 80LL * p->n_experts;
            return p->weight_format == MOE_WEIGHTS_BF16 && big ? 17 : 16;
        }
        const int cost10 = ceil_div(ceil_div(rows / 32, 10) * est_tiles, n_cus) * 10;
        const int cost12 = ceil_div(ceil_div(rows / 32, 12) * est_tiles, n_cus) * 12;
        return cost12 <= cost10 ? 1 : 0;
    }
    // one row block more than necessary when that makes the block count a whole number of rounds
    int pick_row_blocks(int rows, int kernel) const {
        if (prefill) return 0;
        const int n = ceil_div(rows / 32, kernel == 1 ? 12 : 10);
        return ((n * est_tiles) % n_cus != 0 && ((n + 1) * est_tiles) % n_cus == 0) ? n + 1 : n;
    }
    // MXFP4 with the bucketing inside the kernel: a block may cover up to two passes of CONS row units
    // (the second pass starts with its weights already in flight), so fewer, longer blocks pay fewer
    // pipeline fills.  Time of a round of blocks ~ one fill + passes x stages x consumers / 12; all
    // (consumers, row blocks) choices that keep every compute unit busy are priced.
    void pick_two_pass(int rows, int* kernel, int* row_blocks) const {
        const int units = rows / 32;
        double best = 1e30;
        for (int k = 0; k < 2; ++k) {
            const int cons = k == 1 ? 12 : 10;
            for (int n = ceil_div(units, 2 * cons); n <= ceil_div(units, cons); ++n) {
                const int per_block = ceil_div(units, n);
                const int passes = ceil_div(per_block, cons);
                const int rounds = ceil_div(n * est_tiles, n_cus);
                const double cost = rounds * (6.0 + passes * 25.0 * cons / 12.0);
                if (cost < best - 1e-9) {
                    best = cost;
                    *kernel = k;
                    *row_blocks = n;
                }
            }
        }
    }
    // One launch for both GEMMs: row blocks per expert (n1 gate/up, n2 down, at most the kernel's consumer
    // waves in row units each).  A block's time is its number of items (an item's ticks take about the same
    // time whatever its rows), so: as few rounds of items over an XCD's compute units as possible, and among
    // those the split that leaves the fewest compute units without an item in the last round.
    void pick_fused(int* n1, int* n2, int* drain_slack) const {
        const int cons = expert_fused_consumers();
        const int U1 = 2 * p->intermediate_dim / 32, U2 = p->hidden_dim / 32;
        const int per_xcd = std::max(1, ceil_div(p->n_experts, 8)), cus = std::max(1, n_cus / 8);
        long long best = -1;
        for (int a = ceil_div(U1, cons); a <= ceil_div(U1, cons) + 4; ++a)
            for (int b = ceil_div(U2, cons); b <= ceil_div(U2, cons) + 4; ++b) {
                const int items = per_xcd * (a + b), rounds = ceil_div(items, cus);
                const long long cost = (long long)rounds * 1000000 + (long long)(rounds * cus - items) * 100 + a + b;
                if (best < 0 || cost < best) {
                    best = cost;
                    *n1 = a;
                    *n2 = b;
                }
            }
        *drain_slack = 2 * cus;  // two rounds of items
    }
    void set_weights(ExpertGemmArgs& a, const void* w, const void* scales, int rows, int Kdim) const {
        a.w = w;
        a.w_scales = static_cast<const uint8_t*>(scales);
        a.rows = rows;
        a.K = Kdim;
        a.bias_expert_stride = rows;
        if (direct && p->weight_format == MOE_WEIGHTS_MXFP4_TILED) {
            pick_two_pass(rows, &a.waves_per_block, &a.row_blocks);
        } else {
            a.waves_per_block = pick_kernel(rows);
            a.row_blocks = pick_row_blocks(rows, a.waves_per_block);
        }
        if (p->weight_format == MOE_WEIGHTS_BF16) {
            a.w_expert_stride = (long long)rows * Kdim;
        } else {
            size_t bb, sb;
            mxfp4_tiled_bytes(rows, Kdim, &bb, &sb);
            a.w_expert_stride = (long long)bb;
            a.s_expert_stride = (long long)sb;
        }
    }
    // act: bf16 [T, H] rows gathered by token; out: bf16 SwiGLU rows [A, I]
    ExpertGemmArgs gate_up(const uint16_t* act, uint16_t* out) const {
        ExpertGemmArgs a = g;
        set_weights(a, p->w_mlp1, p->w_mlp1_scales, 2 * p->intermediate_dim, p->hidden_dim);
        a.bias = p->b_mlp1;
        a.act = act;
        a.gather = 1;
        a.out = out;
        // measured with the bucketing inside the kernel (one block per expert and row block): keeping an expert's
        // row blocks on one XCD takes 1 % off the bf16 launch (its token rows enter one L2 instead of eight) and
        // leaves the MXFP4 launch as it is; with token blocks from the tile map it cost up to 2 %
        a.xcd_tiles = direct ? 1 : 0;
        return a;
    }
    // act: bf16 [A, I] rows (by slot, or by assignment when bucketing is done in the kernel); out: fp32 [A, H]
    ExpertGemmArgs down(const uint16_t* act, float* out) const {
        ExpertGemmArgs a = g;
        set_weights(a, p->w_mlp2, p->w_mlp2_scales, p->hidden_dim, p->intermediate_dim);
        a.bias = p->b_mlp2;
        a.act = act;
        a.gather = 0;
        a.out = out;
        // Measured at 4096 tokens: the gate/up GEMM is up to 9 % faster with the partial token blocks last
        // (largest first: the launch's tail is made of short blocks); the down GEMM is 2 % faster in bucket
        // order, where a partial block runs next to full blocks of its expert and finds the expert's weights
        // on their way through the caches.
        if (!direct) {
            a.tile_expert += second_map;
            a.tile_row0 += second_map;
            a.tile_rows += second_map;
        }
        // measured: the down GEMM gains 4-10 % from keeping a token block on one XCD (its input rows were
        // written by the gate/up launch just before)
        a.xcd_tiles = 1;
        return a;
    }
};

static int block_forward_impl(const moe_block_params* caller, moe_stream_t stream_, moe_stage_timer* timer) {
    if (!caller) return MOE_ERR_NULL;
    // the struct as it was before next_norm_weight / next_norm_out were appended is still accepted
    constexpr size_t kOldBytes = offsetof(moe_block_params, next_norm_weight);
    if (caller->struct_bytes != sizeof(moe_block_params) && caller->struct_bytes != kOldBytes) return MOE_ERR_FORMAT;
    moe_block_params local{};
    memcpy(&local, caller, caller->struct_bytes);
    const moe_block_params* p = &local;
    if ((p->next_norm_weight != nullptr) != (p->next_norm_out != nullptr)) return MOE_ERR_NULL;
    if (p->next_norm_out && !p->residual_x) return MOE_ERR_NULL;
    if (((uintptr_t)p->next_norm_out & 15u) || ((uintptr_t)p->next_norm_weight & 7u)) return MOE_ERR_ALIGN;
    const int T = p->n_tokens, H = p->hidden_dim, I = p->intermediate_dim, E = p->n_experts,
              K = p->experts_per_token;
    int rc = check_dims(T, H, I, E, K);
    if (rc) return rc;
    if (!p->t || !p->w_router || !p->b_router || !p->w_mlp1 || !p->b_mlp1 || !p->w_mlp2 || !p->b_mlp2 ||
        !p->e_agg || !p->topk_i || !p->topk_v)
        return MOE_ERR_NULL;
    const int fmt = p->weight_format;
    if (fmt != MOE_WEIGHTS_BF16 && fmt != MOE_WEIGHTS_MXFP4_TILED) return MOE_ERR_FORMAT;
    if (fmt == MOE_WEIGHTS_MXFP4_TILED && (!p->w_mlp1_scales || !p->w_mlp2_scales)) return MOE_ERR_NULL;
    if (((uintptr_t)p->t | (uintptr_t)p->e_agg | (uintptr_t)p->w_mlp1 | (uintptr_t)p->w_mlp2 |
         (uintptr_t)p->w_router | (uintptr_t)p->residual_x) & 15u)
        return MOE_ERR_ALIGN;
    if (!p->workspace || ((uintptr_t)p->workspace & (kAlign - 1))) return MOE_ERR_WORKSPACE;
    BlockWorkspace ws(p->workspace, T, H, I, E, K);
    if (p->workspace_bytes < ws.bytes) return MOE_ERR_WORKSPACE;
    hipStream_t stream = as_stream(stream_);
    int stage = 0;
    auto mark = [&]() -> int {
        if (!timer) return MOE_OK;
        return (int)hipEventRecord(timer->ev[stage++], stream);
    };
    if ((rc = mark())) return rc;

    // 1. router logits -> top-k -> softmax  (src/forward.cpp:318-327; src/run.cpp:630-642)
    // Large batches without a request for the full score matrix take the two-pass router (same
    // indices and weights); everything else the single exact pass.
    const bool strict = (p->flags & MOE_FLAG_ROUTER_STRICT_ORDER) != 0;
    if (!strict && !p->router_score && router_two_pass(T, E, H)) {
        rc = launch_router_two_pass(p->t, p->w_router, p->b_router, ws.router_partial, ws.t_bf16, p->topk_v, p->topk_i, T,
                                    H, E, K, 1, stream, timer ? timer->ev[stage++] : nullptr);
        if (rc) return rc;
    } else if (!strict && router_fused_fits(H)) {
        // one launch, block per token: the exact pass of the two-pass router applied to every expert
        rc = launch_router_fused(p->t, p->w_router, p->b_router, ws.t_bf16, p->router_score, p->topk_v, p->topk_i, T, H,
                                 E, K, 1, stream);
        if (rc) return rc;
        if ((rc = mark())) return rc;
    } else {
        const int S = router_segments(T, E, H, strict);
        rc = launch_router_partial(p->t, p->w_router, ws.router_partial, ws.t_bf16, T, H, E, S, stream);
        if (rc) return rc;
        if ((rc = mark())) return rc;
        rc = launch_router_finalize(ws.router_partial, S, nullptr, p->b_router, p->router_score, p->topk_v, p->topk_i, T,
                                    E, K, 1, 1, stream);
        if (rc) return rc;
    }
    if ((rc = mark())) return rc;

    // 2. bucketing + token-block map  (src/forward.cpp:329-376)
    // Small batches need no bucketing launch: each block of the expert kernels finds its expert's
    // bucket in topk_i itself and rows are addressed by assignment id (token * K + k).
    const bool prefill = use_prefill_kernels(T, K, E, p->weight_format, p->flags);
    const bool direct = use_direct_bucketing(T, K, E, prefill, p->flags);
    const int tile_tokens = prefill ? kPrefillTileTokens : kStreamTileTokens;
    const int max_tiles = tile_map_capacity(T * K, E, tile_tokens);  // <= ws.max_tiles (sized for 64)
    if (!direct) {
        TileMap map{ws.tile_expert, ws.tile_row0, ws.tile_rows, ws.n_tiles, tile_tokens, max_tiles, ws.max_tiles};
        rc = launch_bucket(p->topk_i, p->topk_v, T, K, E, ws.expert_offsets, ws.tokens_flat, ws.weights_flat,
                           ws.slot_of, map, stream);
        if (rc) return rc;
    }
    if ((rc = mark())) return rc;

    // 3. gate/up GEMM + SwiGLU  (src/forward.cpp:474-479; src/run.cpp:657-689)
    // 4. down GEMM  (src/forward.cpp:481-487; src/run.cpp:691-700)
    const ExpertPlan plan(p, ws, prefill, direct, tile_tokens, max_tiles);
    const ExpertGemmArgs a1 = plan.gate_up(ws.t_bf16, ws.h_by_slot);
    const ExpertGemmArgs a2 = plan.down(ws.h_by_slot, ws.y_by_slot);
    if (use_fused_experts(E, direct, p->flags)) {
        // one launch for both (its stage time is reported as the gate/up stage, the down stage is empty)
        ExpertFusedArgs f{};
        f.gu = a1;
        f.dn = a2;
        f.ctr = ws.fused_ctr;
        f.spin_limit = 1 << 20;
        plan.pick_fused(&f.n1, &f.n2, &f.drain_slack);
        rc = launch_fill_zero(reinterpret_cast<uint32_t*>(ws.fused_ctr), expert_fused_ctr_words(E), stream);
        if (rc) return rc;
        rc = launch_expert_fused(f, plan.n_cus, stream);
        if (rc) return rc;
        if ((rc = mark())) return rc;
    } else {
        rc = launch_expert_stream(a1, 0, stream);
        if (rc) return rc;
        if ((rc = mark())) return rc;
        rc = launch_expert_stream(a2, 1, stream);
        if (rc) return rc;
    }
    if ((rc = mark())) return rc;

    // 5. weighted combine in ascending expert id (+ residual)  (src/run.cpp:702-712)
    const int* slot_of = direct ? nullptr : ws.slot_of;  // direct: the row of assignment (t, k) is t * K + k
    if (p->next_norm_out) {
        rc = launch_combine_norm(ws.y_by_slot, slot_of, p->topk_i, p->topk_v, p->e_agg, p->residual_x,
                                 p->next_norm_weight, p->next_norm_out, T, K, H, stream);
        if (rc != MOE_ERR_LIMIT) return rc ? rc : mark();
    }
    rc = launch_combine(ws.y_by_slot, slot_of, p->topk_i, p->topk_v, p->e_agg, p->residual_x, T, K, H, stream);
    if (rc) return rc;
    if (p->next_norm_out) {  // rows too long for the fused kernel
        rc = launch_rmsnorm(p->next_norm_out, p->residual_x, p->next_norm_weight, T, H, stream);
        if (rc) return rc;
    }
    return mark();
}


int moe_block_forward(const moe_block_params* p, moe_stream_t stream) { return block_forward_impl(p, stream, nullptr); }

int moe_block_forward_layers(const moe_block_params* params, int n_layers, moe_stream_t stream) {
    if (!params) return MOE_ERR_NULL;
    if (n_layers <= 0) return MOE_ERR_SHAPE;
    const uint8_t* p = reinterpret_cast<const uint8_t*>(params);
    for (int l = 0; l < n_layers; ++l) {
        const moe_block_params* q = reinterpret_cast<const moe_block_params*>(p);
        if (q->struct_bytes < offsetof(moe_block_params, next_norm_weight)) return MOE_ERR_FORMAT;
        const int rc = block_forward_impl(q, stream, nullptr);
        if (rc) return rc;
        p += q->struct_bytes;  // the array's stride is the caller's struct size
    }
    return MOE_OK;
}

int moe_block_describe(const moe_block_params* p, char* text, size_t text_bytes) {
    if (!p || !text) return MOE_ERR_NULL;
    if (text_bytes < 64) return MOE_ERR_LIMIT;
    if (p->struct_bytes != sizeof(moe_block_params) && p->struct_bytes != offsetof(moe_block_params, next_norm_weight))
        return MOE_ERR_FORMAT;
    const int T = p->n_tokens, H = p->hidden_dim, I = p->intermediate_dim, E = p->n_experts,
              K = p->experts_per_token;
    int rc = check_dims(T, H, I, E, K);
    if (rc) return rc;
    const int fmt = p->weight_format;
    if (fmt != MOE_WEIGHTS_BF16 && fmt != MOE_WEIGHTS_MXFP4_TILED) return MOE_ERR_FORMAT;
    // the same decisions, in the same order, as block_forward_impl
    const bool strict = (p->flags & MOE_FLAG_ROUTER_STRICT_ORDER) != 0;
    const char* router = (!strict && !p->router_score && router_two_pass(T, E, H))
                             ? "router_screen_kernel + router_refine_kernel"
                             : (!strict && router_fused_fits(H)) ? "router_fused_kernel"
                                                                 : "router_partial_kernel + router_finalize_kernel";
    const bool prefill = use_prefill_kernels(T, K, E, fmt, p->flags);
    const bool direct = use_direct_bucketing(T, K, E, prefill, p->flags);
    const int tile_tokens = prefill ? kPrefillTileTokens : kStreamTileTokens;
    BlockWorkspace ws(nullptr, T, H, I, E, K);
    const ExpertPlan plan(p, ws, prefill, direct, tile_tokens, tile_map_capacity(T * K, E, tile_tokens));
    auto gemm_name = [&](int rows, int epi, char* out, size_t n) {
        int kernel = plan.pick_kernel(rows), row_blocks = plan.pick_row_blocks(rows, kernel);
        if (direct && fmt == MOE_WEIGHTS_MXFP4_TILED) plan.pick_two_pass(rows, &kernel, &row_blocks);
        const int cons = kernel == 1 ? 12 : 10;
        if (prefill && kernel == 17) {
            snprintf(out, n, "expert_prefill_bf16_kernel<%d>", epi);
        } else if (prefill) {
            snprintf(out, n, "expert_prefill_kernel<%d, %d, 4>", fmt, epi);
        } else if (direct) {
            // as the launcher: at least enough row blocks for one (bf16) or two (MXFP4) passes of `cons` row units
            const int units = rows / 32;
            const int rb = std::max(row_blocks, ceil_div(units, (fmt == MOE_WEIGHTS_MXFP4_TILED ? 2 : 1) * cons));
            const bool two = fmt == MOE_WEIGHTS_MXFP4_TILED && ceil_div(units, rb) > cons;
            snprintf(out, n, "expert_stream_direct_kernel<%d, %d, %d, 2, %s>", fmt, epi, cons, two ? "true" : "false");
        } else {
            snprintf(out, n, "expert_stream_ws_kernel<%d, %d, %d, 2>", fmt, epi, cons);
        }
    };
    char g1[96], g2[96];
    if (use_fused_experts(E, direct, p->flags)) {
        snprintf(g1, sizeof(g1), "expert_fused_kernel<%d>", fmt);
        snprintf(g2, sizeof(g2), "expert_fused_kernel<%d>", fmt);
    } else {
        gemm_name(2 * I, 0, g1, sizeof(g1));
        gemm_name(H, 1, g2, sizeof(g2));
    }
    const int n = snprintf(text, text_bytes, "router=%s; bucketing=%s; gate_up=%s; down=%s; combine=%s; compute_units=%d",
                           router, direct ? "in the expert kernels" : "bucket_kernel", g1, g2,
                           p->next_norm_out ? "combine_norm_kernel" : "combine_kernel", plan.n_cus);
    return (n < 0 || (size_t)n >= text_bytes) ? MOE_ERR_LIMIT : MOE_OK;
}

void moe_synth_normal_table(float* h_table) {
#if !defined(__HIP_DEVICE_COMPILE__)  // the builder exists in the host pass only (libm)
    if (h_table) moe_synth_build_normal_table(h_table);
#endif
}

int moe_block_down_gemm(const moe_block_params* caller, const moe_bf16_t* h_by_assignment, float* y_by_assignment,
                        moe_stream_t stream_) {
    if (!caller || !h_by_assignment || !y_by_assignment) return MOE_ERR_NULL;
    // as moe_block_forward: the struct as it was before next_norm_weight / next_norm_out is still accepted
    constexpr size_t kOldBytes = offsetof(moe_block_params, next_norm_weight);
    if (caller->struct_bytes != sizeof(moe_block_params) && caller->struct_bytes != kOldBytes) return MOE_ERR_FORMAT;
    moe_block_params local{};
    memcpy(&local, caller, caller->struct_bytes);
    const moe_block_params* p = &local;
    const int T = p->n_tokens, H = p->hidden_dim, I = p->intermediate_dim, E = p->n_experts,
              K = p->experts_per_token;
    int rc = check_dims(T, H, I, E, K);
    if (rc) return rc;
    if (!p->w_mlp2 || !p->b_mlp2 || !p->topk_i || !p->topk_v) return MOE_ERR_NULL;
    const int fmt = p->weight_format;
    if (fmt != MOE_WEIGHTS_BF16 && fmt != MOE_WEIGHTS_MXFP4_TILED) return MOE_ERR_FORMAT;
    if (fmt == MOE_WEIGHTS_MXFP4_TILED && !p->w_mlp2_scales) return MOE_ERR_NULL;
    if (((uintptr_t)h_by_assignment | (uintptr_t)y_by_assignment | (uintptr_t)p->w_mlp2) & 15u) return MOE_ERR_ALIGN;
    if (!p->workspace || ((uintptr_t)p->workspace & (kAlign - 1))) return MOE_ERR_WORKSPACE;
    BlockWorkspace ws(p->workspace, T, H, I, E, K);
    if (p->workspace_bytes < ws.bytes) return MOE_ERR_WORKSPACE;
    hipStream_t stream = as_stream(stream_);
    const bool prefill = use_prefill_kernels(T, K, E, fmt, p->flags);
    const bool direct = use_direct_bucketing(T, K, E, prefill, p->flags);
    const int tile_tokens = prefill ? kPrefillTileTokens : kStreamTileTokens;
    const int max_tiles = tile_map_capacity(T * K, E, tile_tokens);
    const ExpertPlan plan(p, ws, prefill, direct, tile_tokens, max_tiles);
    if (direct) return launch_expert_stream(plan.down(h_by_assignment, y_by_assignment), 1, stream);
    // rows by slot: bucket, bring the caller's rows into slot order, multiply, bring the result back
    TileMap map{ws.tile_expert, ws.tile_row0, ws.tile_rows, ws.n_tiles, tile_tokens, max_tiles, ws.max_tiles};
    rc = launch_bucket(p->topk_i, p->topk_v, T, K, E, ws.expert_offsets, ws.tokens_flat, ws.weights_flat, ws.slot_of,
                       map, stream);
    if (rc) return rc;
    // a bf16 row of I values is moved as I/2 floats
    rc = launch_scatter_rows(reinterpret_cast<const float*>(h_by_assignment), ws.slot_of,
                             reinterpret_cast<float*>(ws.h_by_slot), T * K, I / 2, stream);
    if (rc) return rc;
    rc = launch_expert_stream(plan.down(ws.h_by_slot, ws.y_by_slot), 1, stream);
    if (rc) return rc;
    return launch_gather_rows(ws.y_by_slot, ws.slot_of, y_by_assignment, T * K, H, stream);
}

int moe_block_forward_timed(const moe_block_params* p, moe_stream_t stream, moe_stage_timer* timer) {
    if (!timer) return MOE_ERR_NULL;
    return block_forward_impl(p, stream, timer);
}

int moe_stage_timer_create(moe_stage_timer** out) {
    if (!out) return MOE_ERR_NULL;
    moe_stage_timer* t = new (std::nothrow) moe_stage_timer();
    if (!t) return (int)hipErrorOutOfMemory;
    for (int i = 0; i <= MOE_N_STAGES; ++i) {
        hipError_t e = hipEventCreate(&t->ev[i]);
        if (e != hipSuccess) {
            for (int j = 0; j < i; ++j) (void)hipEventDestroy(t->ev[j]);
            delete t;
            return (int)e;
        }
    }
    *out = t;
    return MOE_OK;
}

void moe_stage_timer_destroy(moe_stage_timer* t) {
    if (!t) return;
    for (int i = 0; i <= MOE_N_STAGES; ++i) (void)hipEventDestroy(t->ev[i]);
    delete t;
}

int moe_stage_timer_read(moe_stage_timer* t, float* stage_ms) {
    if (!t || !stage_ms) return MOE_ERR_NULL;
    MOE_RETURN_IF_HIP(hipEventSynchronize(t->ev[MOE_N_STAGES]));
    for (int i = 0; i < MOE_N_STAGES; ++i) MOE_RETURN_IF_HIP(hipEventElapsedTime(&stage_ms[i], t->ev[i], t->ev[i + 1]));
    return MOE_OK;
}

// ---- synthetic workloads ----------------------------------------------------------------------
int moe_synth_normal_f32(float* dst, long long n, const float* table_d, float scale, unsigned seed,
                         unsigned tensor_id, moe_stream_t stream) {
    if (!dst || !table_d) return MOE_ERR_NULL;
    if (n <= 0) return MOE_ERR_SHAPE;
    return launch_synth(0, dst, n, table_d, scale, seed, tensor_id, 0, 0, as_stream(stream));
}
int moe_synth_normal_bf16(moe_bf16_t* dst, long long n, const float* table_d, float scale, unsigned seed,
                          unsigned tensor_id, moe_stream_t stream) {
    if (!dst || !table_d) return MOE_ERR_NULL;
    if (n <= 0) return MOE_ERR_SHAPE;
    return launch_synth(1, dst, n, table_d, scale, seed, tensor_id, 0, 0, as_stream(stream));
}
int moe_synth_bytes(uint8_t* dst, long long n, unsigned seed, unsigned tensor_id, moe_stream_t stream) {
    if (!dst) return MOE_ERR_NULL;
    if (n <= 0) return MOE_ERR_SHAPE;
    if ((uintptr_t)dst & 3u) return MOE_ERR_ALIGN;
    return launch_synth(2, dst, n, nullptr, 0.f, seed, tensor_id, 0, 0, as_stream(stream));
}
int moe_synth_range_bytes(uint8_t* dst, long long n, unsigned seed, unsigned tensor_id, unsigned lo, unsigned span,
                          moe_stream_t stream) {
    if (!dst) return MOE_ERR_NULL;
    if (n <= 0 || span == 0 || lo + span > 256) return MOE_ERR_SHAPE;
    if ((uintptr_t)dst & 3u) return MOE_ERR_ALIGN;
    return launch_synth(3, dst, n, nullptr, 0.f, seed, tensor_id, lo, span, as_stream(stream));
}

int moe_device_attributes(int* compute_units, int* clock_khz, int* memory_clock_khz, int* memory_bus_bits,
                          int* l2_bytes) {
    int dev = 0;
    MOE_RETURN_IF_HIP(hipGetDevice(&dev));
    const struct { int* out; hipDeviceAttribute_t attr; } want[] = {
        {compute_units, hipDeviceAttributeMultiprocessorCount}, {clock_khz, hipDeviceAttributeClockRate},
        {memory_clock_khz, hipDeviceAttributeMemoryClockRate}, {memory_bus_bits, hipDeviceAttributeMemoryBusWidth},
        {l2_bytes, hipDeviceAttributeL2CacheSize}};
    for (const auto& w : want)
        if (w.out) MOE_RETURN_IF_HIP(hipDeviceGetAttribute(w.out, w.attr, dev));
    return MOE_OK;
}

int moe_synth_checksum(const void* src, long long n_bytes, unsigned long long* out_d, moe_stream_t stream) {
    if (!src || !out_d) return MOE_ERR_NULL;
    if (n_bytes <= 0 || (n_bytes & 15)) return MOE_ERR_SHAPE;
    if (((uintptr_t)src & 15u) || ((uintptr_t)out_d & 7u)) return MOE_ERR_ALIGN;
    return launch_synth_checksum(src, n_bytes, out_d, MOE_SYNTH_CHECKSUM_WORDS - 1, as_stream(stream));
}

}  // extern "C"
