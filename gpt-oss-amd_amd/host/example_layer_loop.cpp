// Compile-and-link check for the host headers, and a template for wiring the block into a layer
// loop shaped like the reference's (src/forward.cpp:260-514).  Device buffers are the caller's
// business; this program only resolves the library and prints the workspace a 20b-shaped layer needs.
#include <cstdio>

#include "moe_kernels.hpp"
#include "moe_layer.hpp"

int main() {
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
