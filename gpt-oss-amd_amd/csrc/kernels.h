// Internal launcher declarations shared by the translation units of libmoe_gfx950.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

struct moe_queue_stats;  // include/moe_abi.h

namespace moe {

// ---- router.hip -------------------------------------------------------------------------------
int router_segments(int T, int E, int H, bool strict);
int launch_router_partial(const float* x, const uint16_t* w, double* partial, uint16_t* x_bf16, int T, int H,
                          int E, int S, hipStream_t stream);
int launch_router_finalize(const double* partial, int S, const float* scores_in, const uint16_t* bias,
                           float* scores_out, float* topk_v, int* topk_i, int T, int E, int K, int do_topk,
                           int do_softmax, hipStream_t stream);
int launch_softmax_rows(float* x, int B, int size, hipStream_t stream);
// Whole router in one launch (block per token): logits as the exact pass of the two-pass router,
// top-k, softmax, the bf16 activation copy and, if scores_out is not NULL, the score matrix.
bool router_fused_fits(int H);
int launch_router_fused(const float* x, const uint16_t* w, const uint16_t* bias, uint16_t* x_bf16, float* scores_out,
                        float* topk_v, int* topk_i, int T, int H, int E, int K, int do_softmax, hipStream_t stream);
// Two-pass router (fp32 screening of all experts, exact scores of the candidates): same top-k and
// softmax as partial + finalize.  `scratch` holds router_screen_bytes(); `between`, if not NULL, is
// recorded after the first pass.
bool router_two_pass(int T, int E, int H);
size_t router_screen_bytes(int T, int E, int H);
int launch_router_two_pass(const float* x, const uint16_t* w, const uint16_t* bias, void* scratch, uint16_t* x_bf16,
                           float* topk_v, int* topk_i, int T, int H, int E, int K, int do_softmax,
                           hipStream_t stream, hipEvent_t between, float* approx_out = nullptr,
                           float* delta_out = nullptr, int* n_cand_out = nullptr);

// ---- bucket.hip -------------------------------------------------------------------------------
// Token-block map consumed by the expert kernels: tile i covers rows
// [tile_row0[i], tile_row0[i] + tile_rows[i]) of tokens_flat, all routed to tile_expert[i].
struct TileMap {
    int* tile_expert;
    int* tile_row0;
    int* tile_rows;
    int* n_tiles;   // device scalar
    int tile_tokens;  // rows per tile (NB); 0 = no map requested
    int max_tiles;    // capacity = upper bound used as grid dimension
    int second;       // the same tiles in bucket order start at this index of the three arrays (0: not wanted)
};
inline int tile_map_capacity(int A, int E, int tile_tokens) { return (A + tile_tokens - 1) / tile_tokens + E; }

int launch_bucket(const int* topk_i, const float* topk_v, int T, int K, int E, int* expert_offsets,
                  int* tokens_flat, float* weights_flat, int* slot_of, TileMap map, hipStream_t stream);
int launch_gather_rows(const float* X, const int* idx, float* Y, int rows, int H, hipStream_t stream);
int launch_scatter_rows(const float* Y, const int* idx, float* X, int rows, int H, hipStream_t stream);
int launch_build_work_queue(const int* expert_offsets, int E, int* work_queue, int* work_count,
                            hipStream_t stream);

// ---- scheduler_ref.hip: the reference's bucketing steps under their own argument lists ------------
int launch_count_tokens_per_expert(const int* topk_i, const float* topk_v, int B, int K, int* out_expert,
                                   int* out_token, float* out_w, int* counts, int E, hipStream_t stream);
int launch_exclusive_scan_expert_offsets(int* counts, int* offsets, int E, hipStream_t stream);
int launch_compact_by_expert(const int* expert_ids, const int* tokens, const float* weights, int BK, const int* offsets,
                             int* write_counters, int* tokens_flat, float* weights_flat, int E, hipStream_t stream);
int launch_classify_and_build_queues(const int* expert_offsets, int E, int very_sparse_cutoff,
                                     float heavy_factor_sparse, float heavy_factor_default, int* wq_heavy,
                                     int* wq_light, ::moe_queue_stats* stats, hipStream_t stream);

// ---- experts_stream.hip ------------------------------------------------------------------------
struct ExpertGemmArgs {
    const void* w;              // bf16 [E, rows, K] or tiled MXFP4 blocks
    const uint8_t* w_scales;    // tiled MXFP4 scales or nullptr
    const uint16_t* bias;       // bf16 [E, rows]
    const uint16_t* act;        // bf16 activations: [T, K] (gathered through tokens_flat) or [A, K]
    const float* act_f32;       // queue entries only: fp32 activations [A, K] indexed by slot row
    const int* tokens_flat;     // slot row -> token id
    const float* weights_flat;  // slot row -> router weight (scatter epilogue)
    int gather;                 // 1: activation row = tokens_flat[slot row]; 0: slot row itself
    const int* topk_i;          // non-null: no tile map, the kernel buckets the [n_assign] expert ids itself and
                                // addresses rows by assignment id (token * experts_per_token + k)
    int n_assign;               // tokens x experts per token
    int assign_div;             // activation row of assignment s: s / assign_div when gather, else s
    int n_experts;
    const int* work_queue;      // non-null: (expert, row_offset, row_count) triples instead of the tile map
    int work_start, work_count, max_rows_hint;
    const int* tile_expert;
    const int* tile_row0;
    const int* tile_rows;
    const int* n_tiles;
    void* out;                  // see launch_expert_stream
    int rows;                   // weight rows per expert (2I or H)
    int K;                      // contraction length (H or I)
    long long w_expert_stride;  // bf16: elements; MXFP4: bytes of blocks per expert
    long long s_expert_stride;  // MXFP4: bytes of scales per expert
    long long bias_expert_stride;
    float alpha, limit;
    int max_tiles;
    int format;
    int row_blocks;             // row blocks per token block (producer-consumer kernel: 0 = as few as fit;
                                // prefill kernel: set by the launcher)
    int xcd_tiles;              // producer-consumer kernel: all row blocks of a token block on one XCD
    int waves_per_block;        // kernel choice of the fused block: 0 / 1 producer-consumer kernel with 10 / 12
                                // consumer waves (+ 2 producers), 64-token blocks; 16 prefill kernel (4 waves,
                                // 128-token blocks, two blocks a CU); 17 bf16 weights only: prefill kernel with
                                // one block a CU and a register ring of weights (MXFP4: as 16).  Ignored by the
                                // work-queue entries.
};
int launch_expert_stream(const ExpertGemmArgs& a, int epi, hipStream_t stream);
int expert_direct_max_assignments();

// ---- experts_fused.hip: both expert GEMMs of a block in one launch (bucketing inside the kernel) --
struct ExpertFusedArgs {
    ExpertGemmArgs gu, dn;  // the gate/up and the down GEMM as launch_expert_stream would get them
    int* ctr;               // expert_fused_ctr_words() ints, all zero at launch: [0..7] item queue heads per XCD,
                            // [8] set when a bounded wait ran out, [16 + e] finished gate/up items of expert e
    int n1, n2;             // row blocks per expert of the gate/up and of the down GEMM
    int drain_slack;        // a gate/up item is counted as finished at once when fewer queue positions than this lie
                            // between its expert's last gate/up item and first down item
    int spin_limit;         // quads a block keeps looking for a finished-items count before it gives up
};
inline int expert_fused_ctr_words(int n_experts) { return 16 + n_experts; }
int expert_fused_max_assignments();
int expert_fused_max_experts();
int expert_fused_consumers();
int launch_expert_fused(const ExpertFusedArgs& f, int n_blocks, hipStream_t stream);

// ---- combine.hip -------------------------------------------------------------------------------
int launch_combine(const float* y_by_slot, const int* slot_of, const int* topk_i, const float* topk_v,
                   float* e_agg, float* residual_x, int T, int K, int H, hipStream_t stream);
// combine + residual add + the RMSNorm that follows; MOE_ERR_LIMIT if H is too long for one pass
int launch_combine_norm(const float* y_by_slot, const int* slot_of, const int* topk_i, const float* topk_v,
                        float* e_agg, float* residual_x, const uint16_t* norm_weight, float* norm_out, int T, int K,
                        int H, hipStream_t stream);
int launch_vecadd_and_zero(float* a, float* b, float weight, int batch, int size, hipStream_t stream);
int launch_rmsnorm(float* o, const float* x, const uint16_t* weight, int batch, int size, hipStream_t stream);

// ---- mxfp4.hip ---------------------------------------------------------------------------------
void mxfp4_tiled_bytes(int rows, int K, size_t* block_bytes, size_t* scale_bytes);
int launch_fill_zero(uint32_t* words, size_t n, hipStream_t stream);
int launch_dequant_mxfp4(const uint8_t* blocks, const uint8_t* scales, long long n_blocks, uint16_t* out,
                         hipStream_t stream);
int launch_mxfp4_repack(const uint8_t* blocks, const uint8_t* scales, int E, int rows, int K,
                        uint8_t* tiled_blocks, uint8_t* tiled_scales, bool inverse, hipStream_t stream);
int launch_mxfp4_tiled_to_bf16(const uint8_t* tiled_blocks, const uint8_t* tiled_scales, int E, int rows, int K,
                               uint16_t* out, hipStream_t stream);

// ---- synth.hip ---------------------------------------------------------------------------------
int launch_synth(int kind, void* dst, long long n, const float* table, float scale, unsigned seed,
                 unsigned tensor_id, unsigned lo, unsigned span, hipStream_t stream);
// out[0] = sum of the n_bytes / 16 * 4 32-bit words at src modulo 2^64; out[1 .. max_partials] is scratch.
int launch_synth_checksum(const void* src, long long n_bytes, unsigned long long* out, int max_partials,
                          hipStream_t stream);

}  // namespace moe
