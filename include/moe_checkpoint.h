/*
 * moe_checkpoint.h — reads the MoE tensors of a gpt-oss checkpoint from disk and puts one layer
 * at a time into the device layouts moe_block_forward() consumes (include/moe_abi.h).
 *
 * Two on-disk formats:
 *
 *  (1) the reference's packed .bin.  Header = the Config struct (src/run.cpp:26-46), fifteen
 *      little-endian 4-byte fields written by write_config_header
 *      (tools/model_export/gpt-oss-20b/export_model_bin.py:33-49, 232-241), followed by every
 *      tensor back to back in the order of memory_map_weights (src/run.cpp:196-238; the writer
 *      orders them by CATEGORIES and layer index, export_model_bin.py:51-71, 203-227).  The
 *      payload is fp32 (default) or raw bf16 (--dtype bfloat16, export_model_bin.py:244-268);
 *      the reference's own reader (load_checkpoint, src/run.cpp:240-283) only takes fp32.
 *      Expert weights in this file were dequantised offline to bf16 values, so the fp32 -> bf16
 *      conversion at upload (round to nearest even) is exact for them.
 *
 *  (2) a .safetensors file that still holds the experts as MXFP4: `X.blocks` u8
 *      [E, rows, K/32, 16] + `X.scales` u8 [E, rows, K/32] pairs, the input of the reference's
 *      exporter (collect_effective_keys, export_model_bin.py:150-196).  Tensor names end in the
 *      exporter's category suffixes and carry `block.<layer>.` (export_model_bin.py:51-71, 200).
 *      Nothing is dequantised: blocks and scales go through moe_mxfp4_repack() into the tiled
 *      layout, 4.25 bits per weight in HBM instead of 16.
 *
 * The reference has no counterpart of (2) at run time (it expands to fp32 on the host and to
 * bf16 on upload: src/model.cpp:363-400).
 *
 * Conventions: a moe_ckpt is a read-only memory map owned by the library between open and
 * close; h_* pointers point into that map and die with it.  Upload calls copy through a device
 * staging buffer the CALLER provides (the library allocates no device memory) and queue their
 * copies and kernels on `stream`; keep the checkpoint open and the staging buffer alive until
 * the stream has drained.  Return codes as in moe_abi.h plus the MOE_ERR_* below.
 */
#ifndef MOE_CHECKPOINT_H
#define MOE_CHECKPOINT_H

#include "moe_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

enum {
    MOE_ERR_IO = -7,      /* the file cannot be opened, sized or mapped */
    MOE_ERR_PARSE = -8,   /* malformed header (config fields, safetensors JSON, data offsets) */
    MOE_ERR_MISSING = -9  /* a tensor the call needs is not in the file */
};

/* Config of src/run.cpp:26-46, field for field (same order, same 4-byte types). */
typedef struct moe_ckpt_config {
    int32_t vocab_size;
    int32_t hidden_dim;
    int32_t n_experts;
    int32_t experts_per_token;
    int32_t intermediate_dim;
    int32_t n_layers;
    int32_t head_dim;
    int32_t n_attn_heads;
    int32_t n_kv_heads;
    int32_t seq_len;
    int32_t initial_context_length;
    float rope_theta;
    float rope_scaling_factor;
    int32_t sliding_window;
    float swiglu_limit;
} moe_ckpt_config;

enum { MOE_DTYPE_F32 = 0, MOE_DTYPE_BF16 = 1, MOE_DTYPE_U8 = 2, MOE_DTYPE_OTHER = 3 };

/* The per-layer tensors of the MoE half of a layer (TransformerWeights, src/run.cpp:48-84). */
enum {
    MOE_T_RMS_FFN = 0,      /* mlp.norm.scale   [H]        */
    MOE_T_W_ROUTER = 1,     /* mlp.gate.weight  [E, H]     */
    MOE_T_B_ROUTER = 2,     /* mlp.gate.bias    [E]        */
    MOE_T_W_MLP1 = 3,       /* mlp.mlp1_weight  [E, 2I, H]  (.blocks [E, 2I, H/32, 16] when MXFP4) */
    MOE_T_B_MLP1 = 4,       /* mlp.mlp1_bias    [E, 2I]    */
    MOE_T_W_MLP2 = 5,       /* mlp.mlp2_weight  [E, H, I]   (.blocks [E, H, I/32, 16] when MXFP4)  */
    MOE_T_B_MLP2 = 6,       /* mlp.mlp2_bias    [E, H]     */
    MOE_T_W_MLP1_SCALES = 7,/* mlp.mlp1_weight.scales [E, 2I, H/32], MXFP4 files only */
    MOE_T_W_MLP2_SCALES = 8,/* mlp.mlp2_weight.scales [E, H, I/32],  MXFP4 files only */
    MOE_T_COUNT = 9
};

typedef struct moe_ckpt moe_ckpt;

/* Opens a reference .bin (load_checkpoint, src/run.cpp:240-283).  payload_dtype is
 * MOE_DTYPE_F32 or MOE_DTYPE_BF16; the file size must equal header + every tensor of the
 * config at that width, else MOE_ERR_SHAPE. */
MOE_API int moe_ckpt_open_bin(const char* path, int payload_dtype, moe_ckpt** out);

/* Opens a .safetensors file.  cfg supplies what the file does not record (experts_per_token,
 * swiglu_limit, ...: the exporter reads them from config.json, export_model_bin.py:302-304);
 * hidden_dim, intermediate_dim, n_experts and n_layers are checked against the tensor shapes
 * found, and may be passed as 0 to have them filled in from the file.  cfg may be NULL. */
MOE_API int moe_ckpt_open_safetensors(const char* path, const moe_ckpt_config* cfg, moe_ckpt** out);

MOE_API void moe_ckpt_close(moe_ckpt* ck);

MOE_API int moe_ckpt_get_config(const moe_ckpt* ck, moe_ckpt_config* cfg);

/* 1 when the expert weights are MXFP4 blocks/scales, 0 when they are dense. */
MOE_API int moe_ckpt_is_mxfp4(const moe_ckpt* ck);

/* Host view of one tensor of one layer: pointer into the map, size and element type.
 * MOE_ERR_MISSING when the file does not hold it. */
MOE_API int moe_ckpt_layer_tensor(const moe_ckpt* ck, int layer, int which, const void** h_data,
                                  size_t* bytes, int* dtype);

/* Generic listing (safetensors files: every tensor; .bin files: the MoE tensors of all layers).
 * shape must have room for 8 entries. */
MOE_API int moe_ckpt_n_tensors(const moe_ckpt* ck);
MOE_API int moe_ckpt_tensor_info(const moe_ckpt* ck, int index, const char** name, int* dtype, int* rank,
                                 long long* shape, const void** h_data, size_t* bytes);

/* Device destinations of one layer.  NULL members are skipped.  weight_format tells what
 * w_mlp1 / w_mlp2 receive:
 *   MOE_WEIGHTS_BF16         bf16 [E,2I,H] / [E,H,I]  (dense files; MXFP4 files are dequantised
 *                            with moe_dequant_mxfp4's arithmetic)
 *   MOE_WEIGHTS_MXFP4_TILED  tiled blocks + scales of moe_mxfp4_repack (MXFP4 files only;
 *                            sizes from moe_mxfp4_tiled_bytes x E) */
typedef struct moe_layer_device {
    uint32_t struct_bytes;      /* sizeof(moe_layer_device) */
    int32_t weight_format;      /* MOE_WEIGHTS_* */
    moe_bf16_t* rms_ffn_w;      /* [H] */
    moe_bf16_t* w_router;       /* [E,H] */
    moe_bf16_t* b_router;       /* [E] */
    void* w_mlp1;
    void* w_mlp1_scales;        /* tiled format only */
    moe_bf16_t* b_mlp1;         /* [E,2I] */
    void* w_mlp2;
    void* w_mlp2_scales;        /* tiled format only */
    moe_bf16_t* b_mlp2;         /* [E,H] */
} moe_layer_device;

/* Smallest staging buffer moe_ckpt_upload_layer accepts: one expert's largest tensor as stored in
 * the file (256-byte aligned device memory).  A larger buffer means fewer, larger copies. */
MOE_API size_t moe_ckpt_staging_bytes(const moe_ckpt* ck);

/* Copies layer `layer` to the device: dense fp32 payloads are converted to bf16 (round to nearest
 * even) on the device, bf16 payloads are copied, MXFP4 payloads are repacked (or dequantised, see
 * weight_format).  Replaces the per-layer part of copy_transformer_to_device
 * (src/model.cpp:363-400, 411-460). */
MOE_API int moe_ckpt_upload_layer(const moe_ckpt* ck, int layer, const moe_layer_device* dst, void* d_staging,
                                  size_t staging_bytes, moe_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_CHECKPOINT_H */
