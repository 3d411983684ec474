// The reference's per-step entry of the GPU path,
//   float* forward(OssTransformerHybrid*, OssExpertParallelGroup*, int* tokens, const int* pos_per_token_h,
//                  int batch_size, const int* batch_indices_h, int B_stride)      (src/forward.cpp:202-204),
// for the part of the model this library covers: the MoE half of every layer on one GPU.  Both forms
// exist: the reference's own seven arguments, where the expert-parallel group must describe this one GPU
// (NULL, or ep_size 1: one GPU, no peers; anything else is MOE_ERR_FORMAT), so that the call in the decode
// loop of the getp runtime (src/getp/run.cpp:588) compiles and runs unchanged; and the same without the
// group.
//
// What it runs, for l = 0 .. n_layers-1 on the compact batch of `batch_size` rows of s->x:
//   t = rmsnorm(x, rms_ffn_w[l]);  e_agg = moe(t);  x += e_agg          (src/forward.cpp:315-514)
// with the residual add and the next layer's norm folded into the block's last kernel.  The attention
// half (src/forward.cpp:260-312) is not part of this library: a caller that has one runs it per layer
// through forward_layer() instead; `tokens`, `pos_per_token_h`, `batch_indices_h` and `B_stride` only
// address the embedding table and the KV cache there, and are checked but not read here.
// Returns the device pointer of the residual stream (s->x, [batch_size, hidden_dim]); the reference
// returns its logits buffer, which sits behind a head this library does not have.  NULL on error, with
// the code in transformer->last_error (the reference prints and exits instead).
#pragma once
#include "moe_layer.hpp"

namespace moe_host {

// include/model.hpp:217-239 (OssTransformerHybrid) reduced to the MoE members
struct OssMoeTransformer {
    OssMoeConfig config;
    OssMoeWeights weights;
    OssMoeRunState state;
    int device_id = 0;
    moe_stream_t stream = nullptr;  // the reference's tls.compute (src/forward.cpp:92-113)
    unsigned flags = 0;             // MOE_FLAG_* passed to every block
    int last_error = MOE_OK;
};

// The MoE half of layers [first, last) on rows [0, batch_size) of s->x.  `norm_ready` says that s->t
// already holds rmsnorm(x, rms_ffn_w[first]) (left there by the previous call's fused norm).
inline int forward_layers(OssMoeTransformer* tr, int batch_size, int first, int last, bool norm_ready = false) {
    const OssMoeConfig& p = tr->config;
    const OssMoeWeights& w = tr->weights;
    const OssMoeRunState& s = tr->state;
    if (batch_size <= 0 || batch_size > p.batch_size || first < 0 || last > p.n_layers || first > last)
        return MOE_ERR_SHAPE;
    const long long H = p.hidden_dim;
    for (int l = first; l < last; ++l) {
        if (l == first && !norm_ready) {
            const int rc = moe_rmsnorm(s.t, s.x, w.rms_ffn_w + l * H, batch_size, p.hidden_dim, tr->stream);
            if (rc) return rc;
        }
        moe_block_params bp;
        moe_fill_block_params(p, w, s, l, batch_size, tr->flags, &bp);
        if (l + 1 < last) {  // the next layer's FFN norm, written by this block's last kernel
            bp.next_norm_weight = w.rms_ffn_w + (l + 1) * H;
            bp.next_norm_out = s.t;
        }
        const int rc = moe_block_forward(&bp, tr->stream);
        if (rc) return rc;
    }
    return MOE_OK;
}

// One layer, for a caller that runs its own attention half between the MoE halves.
inline int forward_layer(OssMoeTransformer* tr, int l, int batch_size) { return forward_layers(tr, batch_size, l, l + 1); }

// include/model.hpp:264-269: what forward() reads of the reference's expert-parallel context.  This
// library runs every expert on the caller's GPU, so a group can only name that one GPU.
struct OssExpertParallelGroup {
    void** shards = nullptr;       // the reference's shard descriptors; never read here
    int dp_rank = 0;
    int ep_size = 1;               // number of shards: must be 1
    int primary_shard_index = 0;
};

// src/forward.cpp:202-204 without the expert-parallel group.
inline float* forward(OssMoeTransformer* transformer, int* tokens, const int* pos_per_token_h, int batch_size,
                      const int* batch_indices_h, int B_stride) {
    if (!transformer) return nullptr;
    transformer->last_error = MOE_OK;
    if (!tokens || !pos_per_token_h || !batch_indices_h) {
        transformer->last_error = MOE_ERR_NULL;
        return nullptr;
    }
    // the reference asserts batch_size <= staging capacity (src/forward.cpp:236) and addresses the
    // KV cache of sequence batch_indices_h[i] inside a B_stride-sized table (src/forward.cpp:276-281)
    if (batch_size <= 0 || batch_size > transformer->config.batch_size || B_stride < batch_size) {
        transformer->last_error = MOE_ERR_SHAPE;
        return nullptr;
    }
    for (int i = 0; i < batch_size; ++i) {
        if (batch_indices_h[i] < 0 || batch_indices_h[i] >= B_stride || pos_per_token_h[i] < 0) {
            transformer->last_error = MOE_ERR_SHAPE;
            return nullptr;
        }
    }
    const int rc = forward_layers(transformer, batch_size, 0, transformer->config.n_layers);
    if (rc) {
        transformer->last_error = rc;
        return nullptr;
    }
    return transformer->state.x;
}

// src/forward.cpp:202-204, argument for argument.
inline float* forward(OssMoeTransformer* transformer, OssExpertParallelGroup* ep_group, int* tokens,
                      const int* pos_per_token_h, int batch_size, const int* batch_indices_h, int B_stride) {
    if (!transformer) return nullptr;
    if (ep_group && ep_group->ep_size != 1) {  // the reference exits on an invalid context (:209-212)
        transformer->last_error = MOE_ERR_FORMAT;
        return nullptr;
    }
    return forward(transformer, tokens, pos_per_token_h, batch_size, batch_indices_h, B_stride);
}

}  // namespace moe_host
