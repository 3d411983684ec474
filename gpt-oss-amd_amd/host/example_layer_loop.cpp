// Compile-and-link check for the host headers, and a template for wiring the block into a layer
// loop shaped like the reference's (src/forward.cpp:260-514).  Device buffers are the caller's
// business; this program only resolves the library and prints the workspace a 20b-shaped layer needs.
#include <cstdio>
#include <string>

#include "moe_kernels.hpp"
#include "moe_layer.hpp"

// With a path: opens a reference .bin (fp32 payload) or a .safetensors file and prints what the
// MoE half of the model needs; the upload itself needs device buffers (moe_host::moe_upload_weights).
static int describe_checkpoint(const char* path) {
    const std::string p(path);
    const bool st = p.size() > 12 && p.compare(p.size() - 12, 12, ".safetensors") == 0;
    moe_ckpt* ck = nullptr;
    const int rc = st ? moe_ckpt_open_safetensors(path, nullptr, &ck) : moe_ckpt_open_bin(path, MOE_DTYPE_F32, &ck);
    if (rc) {
        std::printf("open %s -> %d (%s)\n", path, rc, moe_error_string(rc));
        return 2;
    }
    moe_host::OssMoeConfig cfg{};
    moe_host::moe_config_from_checkpoint(ck, 256, &cfg);
    std::printf("%s: %d layers, %d experts, H=%d, I=%d, %s experts, staging %zu bytes, %d tensors indexed\n", path,
                cfg.n_layers, cfg.n_experts, cfg.hidden_dim, cfg.intermediate_dim,
                moe_ckpt_is_mxfp4(ck) ? "MXFP4" : "dense", moe_ckpt_staging_bytes(ck), moe_ckpt_n_tensors(ck));
    moe_ckpt_close(ck);
    return 0;
}

int main(int argc, char** argv) {
    if (argc > 1) return describe_checkpoint(argv[1]);
    moe_host::OssMoeConfig cfg{2880, 32, 4, 2880, 24, 7.0f, 256};
    std::printf("abi %d, workspace for B=%d: %zu bytes\n", moe_abi_version(), cfg.batch_size,
                moe_host::moe_workspace_bytes(cfg));
    // argument checks run before anything touches the device
    moe_host::OssMoeWeights w{};
    moe_host::OssMoeRunState s{};
    const int rc = moe_host::moe_forward_layer(cfg, w, s, 0, cfg.batch_size, nullptr);
    std::printf("forward with null buffers -> %d (%s)\n", rc, moe_error_string(rc));
    const int rc2 = moe_dropin::topk(nullptr, nullptr, nullptr, 1, 32, 4);
    return (rc == MOE_ERR_NULL && rc2 == MOE_ERR_NULL) ? 0 : 1;
}
