// Host side of the MoE section of the reference's layer loop (src/forward.cpp:315-514), written
// against the C ABI of libmoe_gfx950.so.  Field names and tensor shapes follow the reference's
// structs (include/model.hpp: OssConfig :25-48, OssTransformerWeightsBFloat16 :109-117,
// OssRunState :132-139 and :164-180); only the MoE members are kept, and MXFP4 members are added.
// Plain C++17, no HIP headers: streams are passed as void*.
#pragma once
#include <cstddef>
#include <cstdint>

#include "../../include/moe_abi.h"
#include "../../include/moe_checkpoint.h"

namespace moe_host {

// include/model.hpp:25-48 (MoE-related members)
struct OssMoeConfig {
    int hidden_dim;
    int n_experts;
    int experts_per_token;
    int intermediate_dim;
    int n_layers;
    float swiglu_limit;
    int batch_size;
};

// include/model.hpp:93, 109-117: all layers back to back, layer l at offset l * per-layer size.
// Expert weights are either bf16 (the reference's device format) or tiled MXFP4 (moe_mxfp4_repack).
struct OssMoeWeights {
    const moe_bf16_t* rms_ffn_w;  // (n_layers, hidden_dim)
    const moe_bf16_t* w_router;   // (n_layers, n_experts, hidden_dim)  (out, in)
    const moe_bf16_t* b_router;   // (n_layers, n_experts)
    const moe_bf16_t* w_mlp1;     // (n_layers, n_experts, 2*intermediate_dim, hidden_dim), gate/up rows interleaved
    const moe_bf16_t* w_mlp2;     // (n_layers, n_experts, hidden_dim, intermediate_dim)
    const moe_bf16_t* b_mlp1;     // (n_layers, n_experts, 2*intermediate_dim)
    const moe_bf16_t* b_mlp2;     // (n_layers, n_experts, hidden_dim)
    // MXFP4 alternative to w_mlp1 / w_mlp2 (NULL when the bf16 tensors are used)
    const uint8_t* w_mlp1_blocks;  // n_layers * n_experts * block bytes per expert (moe_mxfp4_tiled_bytes)
    const uint8_t* w_mlp1_scales;
    const uint8_t* w_mlp2_blocks;
    const uint8_t* w_mlp2_scales;
};

// include/model.hpp:132-139, 164-180: the buffers the block reads and writes, plus one workspace
// that replaces the reference's per-purpose scratch arrays (assign_*, expert_counts, x_by_expert,
// gate_by_expert, d_wq_*).
struct OssMoeRunState {
    float* x;             // (B, hidden_dim) residual stream
    float* t;             // (B, hidden_dim) rmsnorm output = block input
    float* router_score;  // (B, n_experts), may be NULL
    float* topk_v;        // (B, experts_per_token)
    int* topk_i;          // (B, experts_per_token)
    float* e_agg;         // (B, hidden_dim) block output
    void* workspace;      // moe_block_workspace_bytes(batch_size, ...), 256-byte aligned
    size_t workspace_bytes;
};

// Config of an open checkpoint (src/run.cpp:26-46) reduced to the MoE members.
inline int moe_config_from_checkpoint(const moe_ckpt* ck, int batch_size, OssMoeConfig* out) {
    moe_ckpt_config c;
    const int rc = moe_ckpt_get_config(ck, &c);
    if (rc) return rc;
    *out = OssMoeConfig{c.hidden_dim,  c.n_experts,    c.experts_per_token, c.intermediate_dim,
                        c.n_layers,    c.swiglu_limit, batch_size};
    return MOE_OK;
}

// Fills the stacked device tensors of `w` (the caller allocated them, sized for every layer) from an
// open checkpoint, layer by layer: the MoE part of copy_transformer_to_device (src/model.cpp:363-460).
// MXFP4 files go to the w_mlp*_blocks / w_mlp*_scales members, dense files to w_mlp1 / w_mlp2.
inline int moe_upload_weights(const moe_ckpt* ck, const OssMoeConfig& p, const OssMoeWeights& w, void* d_staging,
                              size_t staging_bytes, moe_stream_t stream) {
    const long long H = p.hidden_dim, I = p.intermediate_dim, E = p.n_experts;
    const bool tiled = w.w_mlp1_blocks != nullptr;
    size_t b1 = 0, s1 = 0, b2 = 0, s2 = 0;
    if (tiled) {
        moe_mxfp4_tiled_bytes(2 * p.intermediate_dim, p.hidden_dim, &b1, &s1);
        moe_mxfp4_tiled_bytes(p.hidden_dim, p.intermediate_dim, &b2, &s2);
    }
    for (int l = 0; l < p.n_layers; ++l) {
        moe_layer_device d{};
        d.struct_bytes = sizeof(d);
        d.weight_format = tiled ? MOE_WEIGHTS_MXFP4_TILED : MOE_WEIGHTS_BF16;
        d.rms_ffn_w = const_cast<moe_bf16_t*>(w.rms_ffn_w) + l * H;
        d.w_router = const_cast<moe_bf16_t*>(w.w_router) + l * E * H;
        d.b_router = const_cast<moe_bf16_t*>(w.b_router) + l * E;
        d.b_mlp1 = const_cast<moe_bf16_t*>(w.b_mlp1) + l * E * 2 * I;
        d.b_mlp2 = const_cast<moe_bf16_t*>(w.b_mlp2) + l * E * H;
        if (tiled) {
            d.w_mlp1 = const_cast<uint8_t*>(w.w_mlp1_blocks) + (size_t)l * E * b1;
            d.w_mlp1_scales = const_cast<uint8_t*>(w.w_mlp1_scales) + (size_t)l * E * s1;
            d.w_mlp2 = const_cast<uint8_t*>(w.w_mlp2_blocks) + (size_t)l * E * b2;
            d.w_mlp2_scales = const_cast<uint8_t*>(w.w_mlp2_scales) + (size_t)l * E * s2;
        } else {
            d.w_mlp1 = const_cast<moe_bf16_t*>(w.w_mlp1) + l * E * 2 * I * H;
            d.w_mlp2 = const_cast<moe_bf16_t*>(w.w_mlp2) + l * E * H * I;
        }
        const int rc = moe_ckpt_upload_layer(ck, l, &d, d_staging, staging_bytes, stream);
        if (rc) return rc;
    }
    return MOE_OK;
}

inline size_t moe_workspace_bytes(const OssMoeConfig& p) {
    return moe_block_workspace_bytes(p.batch_size, p.hidden_dim, p.intermediate_dim, p.n_experts, p.experts_per_token);
}

// The argument block of moe_block_forward for layer l: one layer's slices of the stacked tensors
// (src/forward.cpp:317-514 addresses them the same way: base + l * per-layer size).
inline void moe_fill_block_params(const OssMoeConfig& p, const OssMoeWeights& w, const OssMoeRunState& s, int l,
                                  int batch_size, unsigned flags, moe_block_params* out) {
    const long long H = p.hidden_dim, I = p.intermediate_dim, E = p.n_experts;
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
        size_t b1 = 0, s1 = 0, b2 = 0, s2 = 0;
        moe_mxfp4_tiled_bytes(2 * p.intermediate_dim, p.hidden_dim, &b1, &s1);
        moe_mxfp4_tiled_bytes(p.hidden_dim, p.intermediate_dim, &b2, &s2);
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
    bp.flags = flags;
    *out = bp;
}

// One layer's FFN half, the counterpart of src/forward.cpp:315-514 on a single GPU:
//   t = rmsnorm(x, rms_ffn_w[l]);  e_agg = moe(t);  x += e_agg
// Everything is queued on `stream`; nothing waits for the device (the reference blocks on a D2H copy
// of the expert offsets once per layer, src/forward.cpp:340-345, 381).
inline int moe_forward_layer(const OssMoeConfig& p, const OssMoeWeights& w, const OssMoeRunState& s, int l,
                             int batch_size, moe_stream_t stream, unsigned flags = 0) {
    const int rc = moe_rmsnorm(s.t, s.x, w.rms_ffn_w + (long long)l * p.hidden_dim, batch_size, p.hidden_dim, stream);
    if (rc) return rc;
    moe_block_params bp;
    moe_fill_block_params(p, w, s, l, batch_size, flags, &bp);
    return moe_block_forward(&bp, stream);
}

}  // namespace moe_host
