// The reference's per-step entry of the GPU path,
//   float* forward(OssTransformerHybrid*, OssExpertParallelGroup*, int* tokens, const int* pos_per_token_h,
//                  int batch_size, const int* batch_indices_h, int B_stride)      (src/forward.cpp:202-204),
// for the part of the model this library covers: the MoE half of every layer on one GPU.  The
// expert-parallel group is gone (one GPU, no peers); every other argument keeps its place and meaning,
// so the decode loop of the getp runtime (src/getp/run.cpp:573-588) can call it unchanged.
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
    const long long H = p.hidden_dim, I = p.intermediate_dim, E = p.n_experts;
    size_t b1 = 0, s1 = 0, b2 = 0, s2 = 0;
    if (w.w_mlp1_blocks) {
        moe_mxfp4_tiled_bytes(2 * p.intermediate_dim, p.hidden_dim, &b1, &s1);
        moe_mxfp4_tiled_bytes(p.hidden_dim, p.intermediate_dim, &b2, &s2);
    }
    for (int l = first; l < last; ++l) {
        if (l == first && !norm_ready) {
            const int rc = moe_rmsnorm(s.t, s.x, w.rms_ffn_w + l * H, batch_size, p.hidden_dim, tr->stream);
            if (rc) return rc;
        }
        moe_block_params bp{};
        bp.struct_bytes = sizeof(bp);
        bp.n_tokens = batch_size;
        bp.hidden_dim = p.hidden_dim;
        bp.intermediate_dim = p.intermediate_dim;
        bp.n_experts = p.n_experts;
        bp.experts_per_token = p.experts_per_token;
        bp.swiglu_limit = p.swiglu_limit;
        bp.alpha = 1.702f;  // literal in the reference: src/run.cpp:673, src/forward.cpp:467
        bp.t = s.t;
        bp.w_router = w.w_router + l * E * H;
        bp.b_router = w.b_router + l * E;
        bp.b_mlp1 = w.b_mlp1 + l * E * 2 * I;
        bp.b_mlp2 = w.b_mlp2 + l * E * H;
        if (w.w_mlp1_blocks) {
            bp.weight_format = MOE_WEIGHTS_MXFP4_TILED;
            bp.w_mlp1 = w.w_mlp1_blocks + (size_t)l * E * b1;
            bp.w_mlp1_scales = w.w_mlp1_scales + (size_t)l * E * s1;
            bp.w_mlp2 = w.w_mlp2_blocks + (size_t)l * E * b2;
            bp.w_mlp2_scales = w.w_mlp2_scales + (size_t)l * E * s2;
        } else {
            bp.weight_format = MOE_WEIGHTS_BF16;
            bp.w_mlp1 = w.w_mlp1 + l * E * 2 * I * H;
            bp.w_mlp2 = w.w_mlp2 + l * E * H * I;
        }
        bp.e_agg = s.e_agg;
        bp.topk_i = s.topk_i;
        bp.topk_v = s.topk_v;
        bp.router_score = s.router_score;
        bp.residual_x = s.x;
        bp.workspace = s.workspace;
        bp.workspace_bytes = s.workspace_bytes;
        bp.flags = tr->flags;
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

}  // namespace moe_host
