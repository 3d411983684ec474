// Runs the C++ host side of the library on the device: a checkpoint file goes through
// moe_host::moe_upload_weights into stacked device tensors, then either
//   layers  the MoE half of every layer is applied to a batch of rows with moe_host::forward_layers,
//           the residual stream being written out after each layer, or
//   getp    a request file goes through moe_getp::inference (the decode loop with its live-batch
//           compaction) and the generated tokens are written in the reference's output format.
// Usage:
//   moe_stack_main layers <ckpt> <bin_f32|bin_bf16|safetensors:K> <x.f32> <T> <out.f32> [flags]
//   moe_stack_main getp   <ckpt> <bin_f32|bin_bf16|safetensors:K> <in.txt> <out.txt> <steps> <batch> <vocab> <eos>
//                         [<final_states.f32> [<step_sizes.txt> [<trace.bin>]]]   (trace: DecodeOptions::trace)
//   moe_stack_main dropin <ckpt> <bin_f32|bin_bf16> <x.f32> <T> <out.f32> <scratch: own|static|none>
//           every layer's MoE half issued call by call, in the reference's order (src/forward.cpp:315-514),
//           through the reference-named wrappers of moe_kernels.hpp; residual stream written out per layer
//   moe_stack_main synth  <T> <H> <I> <E> <K> <layers> <steps> <warmup> [flags]
//           a synthetic MXFP4 stack generated on the device, forward() timed over <steps> calls (one JSON line)
//   moe_stack_main requests <in.txt> <out.txt> <max_seq_len> [truncate]     (file formats only, no device)
//   moe_stack_main verify <generated.txt> <ground_truth.txt>
// MXFP4 files stay MXFP4 on the device (tiled layout); dense files are uploaded as bf16.
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "moe_getp.hpp"
#include "moe_kernels.hpp"

#define CHECK_RC(expr)                                                                      \
    do {                                                                                    \
        const long long rc_ = (long long)(expr);                                            \
        if (rc_ != 0) {                                                                     \
            std::fprintf(stderr, "%s -> %lld (%s)\n", #expr, rc_, moe_error_string((int)rc_)); \
            return 3;                                                                       \
        }                                                                                   \
    } while (0)

static double now_ms() {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

template <typename T>
static int dev_alloc(T** p, size_t count) {
    return (int)hipMalloc((void**)p, sizeof(T) * (count ? count : 1));
}

struct Model {
    moe_host::OssMoeTransformer tr;
    std::vector<void*> owned;
    ~Model() {
        for (void* p : owned) (void)hipFree(p);
    }
};

// Stacked device tensors of every layer for m->tr.config (bf16 experts, or tiled MXFP4 ones), owned by `m`.
static int alloc_weights(bool tiled, Model* m) {
    const moe_host::OssMoeConfig& c = m->tr.config;
    int rc;
    const size_t L = c.n_layers, E = c.n_experts, H = c.hidden_dim, I = c.intermediate_dim;
    moe_host::OssMoeWeights& w = m->tr.weights;
    w = moe_host::OssMoeWeights{};
    moe_bf16_t *rms, *wr, *br, *b1, *b2, *w1 = nullptr, *w2 = nullptr;
    uint8_t *q1 = nullptr, *s1 = nullptr, *q2 = nullptr, *s2 = nullptr;
    if ((rc = dev_alloc(&rms, L * H)) || (rc = dev_alloc(&wr, L * E * H)) || (rc = dev_alloc(&br, L * E)) ||
        (rc = dev_alloc(&b1, L * E * 2 * I)) || (rc = dev_alloc(&b2, L * E * H)))
        return rc;
    m->owned.insert(m->owned.end(), {rms, wr, br, b1, b2});
    if (tiled) {
        size_t bb1, sb1, bb2, sb2;
        moe_mxfp4_tiled_bytes((int)(2 * I), (int)H, &bb1, &sb1);
        moe_mxfp4_tiled_bytes((int)H, (int)I, &bb2, &sb2);
        if ((rc = dev_alloc(&q1, L * E * bb1)) || (rc = dev_alloc(&s1, L * E * sb1)) || (rc = dev_alloc(&q2, L * E * bb2)) ||
            (rc = dev_alloc(&s2, L * E * sb2)))
            return rc;
        m->owned.insert(m->owned.end(), {q1, s1, q2, s2});
    } else {
        if ((rc = dev_alloc(&w1, L * E * 2 * I * H)) || (rc = dev_alloc(&w2, L * E * H * I))) return rc;
        m->owned.insert(m->owned.end(), {w1, w2});
    }
    w.rms_ffn_w = rms;
    w.w_router = wr;
    w.b_router = br;
    w.b_mlp1 = b1;
    w.b_mlp2 = b2;
    w.w_mlp1 = w1;
    w.w_mlp2 = w2;
    w.w_mlp1_blocks = q1;
    w.w_mlp1_scales = s1;
    w.w_mlp2_blocks = q2;
    w.w_mlp2_scales = s2;
    return MOE_OK;
}

// The run-state buffers for config.batch_size rows, owned by `m`.
static int alloc_state(Model* m) {
    const moe_host::OssMoeConfig& c = m->tr.config;
    moe_host::OssMoeRunState& s = m->tr.state;
    const size_t B = c.batch_size, H = c.hidden_dim;
    int rc;
    s.workspace_bytes = moe_host::moe_workspace_bytes(c);
    uint8_t* ws;
    if ((rc = dev_alloc(&s.x, B * H)) || (rc = dev_alloc(&s.t, B * H)) || (rc = dev_alloc(&s.e_agg, B * H)) ||
        (rc = dev_alloc(&s.topk_v, B * c.experts_per_token)) || (rc = dev_alloc(&s.topk_i, B * c.experts_per_token)) ||
        (rc = dev_alloc(&ws, s.workspace_bytes)))
        return rc;
    s.workspace = ws;
    s.router_score = nullptr;
    m->owned.insert(m->owned.end(), {s.x, s.t, s.e_agg, s.topk_v, s.topk_i, ws});
    return MOE_OK;
}

// kind: bin_f32 | bin_bf16 | safetensors:<experts per token> (a safetensors file does not record it; the
// reference's exporter takes it from config.json, tools/model_export/gpt-oss-20b/export_model_bin.py:302-304)
static int load_model(const char* path, const std::string& kind, int batch_size, Model* m) {
    moe_ckpt* ck = nullptr;
    int rc;
    if (kind.rfind("safetensors", 0) == 0) {
        moe_ckpt_config want{};  // shapes come from the file
        want.experts_per_token = kind.size() > 12 ? std::atoi(kind.c_str() + 12) : 4;
        want.swiglu_limit = 7.0f;
        rc = moe_ckpt_open_safetensors(path, &want, &ck);
    } else {
        rc = moe_ckpt_open_bin(path, kind == "bin_bf16" ? MOE_DTYPE_BF16 : MOE_DTYPE_F32, &ck);
    }
    if (rc) return rc;
    moe_host::OssMoeConfig& c = m->tr.config;
    rc = moe_host::moe_config_from_checkpoint(ck, batch_size, &c);
    if (rc) return rc;
    const bool tiled = moe_ckpt_is_mxfp4(ck) != 0;
    if ((rc = alloc_weights(tiled, m))) return rc;
    moe_host::OssMoeWeights& w = m->tr.weights;
    const size_t staging_bytes = moe_ckpt_staging_bytes(ck);
    uint8_t* staging;
    if ((rc = dev_alloc(&staging, staging_bytes))) return rc;
    rc = moe_host::moe_upload_weights(ck, c, w, staging, staging_bytes, nullptr);
    if (!rc) rc = (int)hipDeviceSynchronize();
    (void)hipFree(staging);
    moe_ckpt_close(ck);
    if (rc) return rc;

    return alloc_state(m);
}

static int read_floats(const char* path, std::vector<float>* out, size_t count) {
    FILE* f = std::fopen(path, "rb");
    if (!f) return MOE_ERR_IO;
    out->resize(count);
    const size_t got = std::fread(out->data(), sizeof(float), count, f);
    std::fclose(f);
    return got == count ? MOE_OK : MOE_ERR_IO;
}

static int run_layers(int argc, char** argv) {
    if (argc < 7) return 2;
    const int T = std::atoi(argv[5]);
    Model m;
    CHECK_RC(load_model(argv[2], argv[3], T, &m));
    if (argc > 7) m.tr.flags = (unsigned)std::atoi(argv[7]);
    const moe_host::OssMoeConfig& c = m.tr.config;
    const size_t n = (size_t)T * c.hidden_dim;
    std::vector<float> x;
    CHECK_RC(read_floats(argv[4], &x, n));
    CHECK_RC(hipMemcpy(m.tr.state.x, x.data(), n * sizeof(float), hipMemcpyHostToDevice));
    FILE* out = std::fopen(argv[6], "wb");
    if (!out) return 3;
    std::printf("layers: %d layers, %d experts, top-%d, H=%d, I=%d, T=%d, %s experts\n", c.n_layers, c.n_experts,
                c.experts_per_token, c.hidden_dim, c.intermediate_dim, T, m.tr.weights.w_mlp1_blocks ? "MXFP4" : "bf16");
    // layer by layer, so that every layer's residual stream can be checked
    for (int l = 0; l < c.n_layers; ++l) {
        CHECK_RC(moe_host::forward_layer(&m.tr, l, T));
        CHECK_RC(hipDeviceSynchronize());
        CHECK_RC(hipMemcpy(x.data(), m.tr.state.x, n * sizeof(float), hipMemcpyDeviceToHost));
        std::fwrite(x.data(), sizeof(float), n, out);
    }
    std::fclose(out);
    // the whole stack again through forward() itself (every norm but the first folded into the block
    // before it), from the same input: must equal the last dump
    std::vector<float> x0;
    CHECK_RC(read_floats(argv[4], &x0, n));
    CHECK_RC(hipMemcpy(m.tr.state.x, x0.data(), n * sizeof(float), hipMemcpyHostToDevice));
    std::vector<int> tokens(T, 0), pos(T, 0), idx(T);
    for (int i = 0; i < T; ++i) idx[i] = i;
    float* y = moe_host::forward(&m.tr, tokens.data(), pos.data(), T, idx.data(), T);
    if (!y) CHECK_RC(m.tr.last_error);
    CHECK_RC(hipDeviceSynchronize());
    CHECK_RC(hipMemcpy(x0.data(), y, n * sizeof(float), hipMemcpyDeviceToHost));
    if (std::memcmp(x0.data(), x.data(), n * sizeof(float)) != 0) {
        std::fprintf(stderr, "forward() differs from the layer-by-layer result\n");
        return 4;
    }
    std::printf("forward() equals the layer-by-layer result bit for bit\n");
    // the reference's seven-argument form: a group of one shard runs, a group of two is refused
    moe_host::OssExpertParallelGroup one, two;
    two.ep_size = 2;
    if (moe_host::forward(&m.tr, &two, tokens.data(), pos.data(), T, idx.data(), T) != nullptr ||
        m.tr.last_error != MOE_ERR_FORMAT) {
        std::fprintf(stderr, "forward() accepted an expert-parallel group of two shards\n");
        return 4;
    }
    std::vector<float> x1;
    CHECK_RC(read_floats(argv[4], &x1, n));
    CHECK_RC(hipMemcpy(m.tr.state.x, x1.data(), n * sizeof(float), hipMemcpyHostToDevice));
    y = moe_host::forward(&m.tr, &one, tokens.data(), pos.data(), T, idx.data(), T);
    if (!y) CHECK_RC(m.tr.last_error);
    CHECK_RC(hipDeviceSynchronize());
    CHECK_RC(hipMemcpy(x1.data(), y, n * sizeof(float), hipMemcpyDeviceToHost));
    if (std::memcmp(x1.data(), x.data(), n * sizeof(float)) != 0) {
        std::fprintf(stderr, "the seven-argument forward() differs\n");
        return 4;
    }
    std::printf("forward() with the reference's seven arguments: same bits; a group of two shards is refused\n");
    return 0;
}

// synth <T> <H> <I> <E> <K> <layers> <steps> <warmup> [flags]: a stack of MXFP4 layers filled on the device by the
// library's synthetic generator (include/moe_synth.h; stream ids of layer l: 2..9 + 16 l for router weight, router
// bias, gate/up blocks, gate/up bias, down blocks, down bias, gate/up scales, down scales; input rows: id 1; seed 0;
// unit FFN norm weights), then <warmup> + <steps> calls of forward() on the evolving residual stream.  Prints one
// JSON line: wall-clock and HIP-event time per forward() call and the checksum (moe_synth_checksum) of the residual
// stream after the first call, which a caller that builds the same stack can compare with its own.
static int run_synth(int argc, char** argv) {
    if (argc < 10) return 2;
    const int T = std::atoi(argv[2]), H = std::atoi(argv[3]), I = std::atoi(argv[4]), E = std::atoi(argv[5]),
              K = std::atoi(argv[6]), L = std::atoi(argv[7]), steps = std::atoi(argv[8]), warmup = std::atoi(argv[9]);
    if (T < 1 || H < 32 || I < 32 || E < 1 || K < 1 || L < 1 || steps < 1 || warmup < 0) return 2;
    Model m;
    m.tr.config = moe_host::OssMoeConfig{H, E, K, I, L, 7.0f, T};
    if (argc > 10) m.tr.flags = (unsigned)std::atoi(argv[10]);
    CHECK_RC(alloc_weights(true, &m));
    CHECK_RC(alloc_state(&m));
    const moe_host::OssMoeWeights& w = m.tr.weights;
    const unsigned seed = 0;
    std::vector<float> table(65536);
    moe_synth_normal_table(table.data());
    float* table_d;
    CHECK_RC(dev_alloc(&table_d, table.size()));
    m.owned.push_back(table_d);
    CHECK_RC(hipMemcpy(table_d, table.data(), table.size() * sizeof(float), hipMemcpyHostToDevice));
    std::vector<uint16_t> ones((size_t)L * H, 0x3F80);  // bf16 1.0
    CHECK_RC(hipMemcpy(const_cast<moe_bf16_t*>(w.rms_ffn_w), ones.data(), ones.size() * 2, hipMemcpyHostToDevice));
    size_t bb1, sb1, bb2, sb2;
    moe_mxfp4_tiled_bytes(2 * I, H, &bb1, &sb1);
    moe_mxfp4_tiled_bytes(H, I, &bb2, &sb2);
    const long long nb1 = (long long)E * 2 * I * (H / 32), nb2 = (long long)E * H * (I / 32);  // 32-value groups
    uint8_t *blocks, *scales;
    CHECK_RC(dev_alloc(&blocks, (size_t)(nb1 > nb2 ? nb1 : nb2) * 16));
    CHECK_RC(dev_alloc(&scales, (size_t)(nb1 > nb2 ? nb1 : nb2)));
    for (int l = 0; l < L; ++l) {
        const unsigned o = 16u * (unsigned)l;
        const size_t sl = (size_t)l;
        CHECK_RC(moe_synth_normal_bf16(const_cast<moe_bf16_t*>(w.w_router) + sl * E * H, (long long)E * H, table_d, 0.02f,
                                       seed, 2 + o, nullptr));
        CHECK_RC(moe_synth_normal_bf16(const_cast<moe_bf16_t*>(w.b_router) + sl * E, E, table_d, 0.02f, seed, 3 + o, nullptr));
        CHECK_RC(moe_synth_normal_bf16(const_cast<moe_bf16_t*>(w.b_mlp1) + sl * E * 2 * I, (long long)E * 2 * I, table_d,
                                       0.02f, seed, 5 + o, nullptr));
        CHECK_RC(moe_synth_normal_bf16(const_cast<moe_bf16_t*>(w.b_mlp2) + sl * E * H, (long long)E * H, table_d, 0.02f,
                                       seed, 7 + o, nullptr));
        CHECK_RC(moe_synth_bytes(blocks, nb1 * 16, seed, 4 + o, nullptr));
        CHECK_RC(moe_synth_range_bytes(scales, nb1, seed, 8 + o, 119, 9, nullptr));
        CHECK_RC(moe_mxfp4_repack(blocks, scales, E, 2 * I, H, const_cast<uint8_t*>(w.w_mlp1_blocks) + sl * E * bb1,
                                  const_cast<uint8_t*>(w.w_mlp1_scales) + sl * E * sb1, nullptr));
        CHECK_RC(moe_synth_bytes(blocks, nb2 * 16, seed, 6 + o, nullptr));
        CHECK_RC(moe_synth_range_bytes(scales, nb2, seed, 9 + o, 119, 9, nullptr));
        CHECK_RC(moe_mxfp4_repack(blocks, scales, E, H, I, const_cast<uint8_t*>(w.w_mlp2_blocks) + sl * E * bb2,
                                  const_cast<uint8_t*>(w.w_mlp2_scales) + sl * E * sb2, nullptr));
    }
    CHECK_RC(hipDeviceSynchronize());
    (void)hipFree(blocks);
    (void)hipFree(scales);
    CHECK_RC(moe_synth_normal_f32(m.tr.state.x, (long long)T * H, table_d, 1.0f, seed, 1, nullptr));

    std::vector<int> tokens(T, 0), pos(T, 0), idx(T);
    for (int i = 0; i < T; ++i) idx[i] = i;
    moe_host::OssExpertParallelGroup group;  // one shard: this GPU
    unsigned long long* sum_d;
    CHECK_RC(dev_alloc(&sum_d, MOE_SYNTH_CHECKSUM_WORDS));
    m.owned.push_back(sum_d);
    unsigned long long first_sum = 0;
    hipEvent_t e0, e1;
    CHECK_RC(hipEventCreate(&e0));
    CHECK_RC(hipEventCreate(&e1));
    double wall_ms = 0;
    float event_ms = 0;
    for (int it = 0; it < warmup + steps; ++it) {
        if (it == warmup) {
            CHECK_RC(hipDeviceSynchronize());
            CHECK_RC(hipEventRecord(e0, nullptr));
            wall_ms = -now_ms();
        }
        if (!moe_host::forward(&m.tr, &group, tokens.data(), pos.data(), T, idx.data(), T)) CHECK_RC(m.tr.last_error);
        if (it == 0) {
            if (((size_t)T * H * 4) % 16 == 0) {
                CHECK_RC(moe_synth_checksum(m.tr.state.x, (long long)T * H * 4, sum_d, nullptr));
                CHECK_RC(hipMemcpy(&first_sum, sum_d, 8, hipMemcpyDeviceToHost));
            }
        }
    }
    CHECK_RC(hipEventRecord(e1, nullptr));
    CHECK_RC(hipDeviceSynchronize());
    wall_ms += now_ms();
    CHECK_RC(hipEventElapsedTime(&event_ms, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    std::printf("{\"mode\": \"synth\", \"T\": %d, \"H\": %d, \"I\": %d, \"E\": %d, \"K\": %d, \"layers\": %d, "
                "\"steps\": %d, \"warmup\": %d, \"flags\": %u, \"ms_per_forward_wall\": %.6f, "
                "\"ms_per_forward_events\": %.6f, \"x_checksum_after_first_forward\": %llu}\n",
                T, H, I, E, K, L, steps, warmup, m.tr.flags, wall_ms / steps, (double)event_ms / steps, first_sum);
    return 0;
}

// The MoE half of every layer the way the reference's layer loop issues it (src/forward.cpp:315-514):
// rmsnorm, gemm_router, topk, softmax, the three bucketing kernels, gather_rows, the work queue, the two
// expert GEMMs, vecadd_and_zero — each through its reference-named wrapper.  `scratch`: "own" registers a
// router scratch buffer for this thread, "static" opts into the library's fixed array, "none" does neither
// (gemm_router must then refuse with MOE_ERR_WORKSPACE).
static int run_dropin(int argc, char** argv) {
    if (argc < 8) return 2;
    const int T = std::atoi(argv[5]);
    const std::string scratch = argv[7];
    Model m;
    CHECK_RC(load_model(argv[2], argv[3], T, &m));
    const moe_host::OssMoeConfig& c = m.tr.config;
    const moe_host::OssMoeWeights& w = m.tr.weights;
    const moe_host::OssMoeRunState& s = m.tr.state;
    if (w.w_mlp1_blocks) {
        std::fprintf(stderr, "dropin: the reference-named wrappers take bf16 experts\n");
        return 2;
    }
    const long long H = c.hidden_dim, I = c.intermediate_dim, E = c.n_experts, K = c.experts_per_token;
    const size_t A = (size_t)T * K, n = (size_t)T * H;
    float *router_score, *x_by_expert, *gate_by_expert, *assign_w, *weights_flat;
    int *assign_expert, *assign_token, *expert_counts, *expert_offsets, *tokens_flat, *work_queue, *work_count;
    void* router_scratch = nullptr;
    CHECK_RC(dev_alloc(&router_score, (size_t)T * E));
    CHECK_RC(dev_alloc(&x_by_expert, A * H));
    CHECK_RC(dev_alloc(&gate_by_expert, A * I));
    CHECK_RC(dev_alloc(&assign_w, A));
    CHECK_RC(dev_alloc(&weights_flat, A));
    CHECK_RC(dev_alloc(&assign_expert, A));
    CHECK_RC(dev_alloc(&assign_token, A));
    CHECK_RC(dev_alloc(&expert_counts, (size_t)E));
    CHECK_RC(dev_alloc(&expert_offsets, (size_t)E + 1));
    CHECK_RC(dev_alloc(&tokens_flat, A));
    CHECK_RC(dev_alloc(&work_queue, (size_t)3 * E));
    CHECK_RC(dev_alloc(&work_count, 1));
    m.owned.insert(m.owned.end(), {router_score, x_by_expert, gate_by_expert, assign_w, weights_flat, assign_expert,
                                   assign_token, expert_counts, expert_offsets, tokens_flat, work_queue, work_count});
    if (scratch == "own") {
        const size_t bytes = moe_router_scratch_bytes(T, (int)E);
        CHECK_RC(hipMalloc(&router_scratch, bytes));
        m.owned.push_back(router_scratch);
        moe_dropin::moe_router_scratch().ptr = router_scratch;
        moe_dropin::moe_router_scratch().bytes = bytes;
    } else if (scratch == "static") {
        moe_dropin::moe_router_scratch().use_static_array = true;
    }
    std::vector<float> x;
    CHECK_RC(read_floats(argv[4], &x, n));
    CHECK_RC(hipMemcpy(s.x, x.data(), n * sizeof(float), hipMemcpyHostToDevice));
    CHECK_RC(hipMemset(s.e_agg, 0, n * sizeof(float)));          // zero on entry, re-zeroed by vecadd_and_zero
    CHECK_RC(hipMemset(expert_counts, 0, sizeof(int) * E));      // zero on entry, reset by the scan
    FILE* out = std::fopen(argv[6], "wb");
    if (!out) return 3;
    using namespace moe_dropin;
    for (int l = 0; l < c.n_layers; ++l) {
        CHECK_RC(rmsnorm(s.t, s.x, w.rms_ffn_w + l * H, T, (int)H));
        const int rc = gemm_router(router_score, s.t, w.w_router + l * E * H, w.b_router + l * E, T, (int)H, (int)E);
        if (scratch == "none") {
            std::printf("gemm_router without a scratch buffer -> %d (%s)\n", rc, moe_error_string(rc));
            std::fclose(out);
            return rc == MOE_ERR_WORKSPACE ? 0 : 4;
        }
        CHECK_RC(rc);
        CHECK_RC(topk(s.topk_v, s.topk_i, router_score, T, (int)E, (int)K));
        CHECK_RC(softmax(s.topk_v, T, (int)K));
        CHECK_RC(count_tokens_per_expert(s.topk_i, s.topk_v, T, (int)K, assign_expert, assign_token, assign_w,
                                         expert_counts, (int)E));
        CHECK_RC(exclusive_scan_expert_offsets(expert_counts, expert_offsets, (int)E));
        CHECK_RC(compact_by_expert_kernel(assign_expert, assign_token, assign_w, (int)A, expert_offsets, expert_counts,
                                          tokens_flat, weights_flat, (int)E));
        // the compaction counted its writes in expert_counts; the reference zeroes them again for the next layer
        CHECK_RC(hipMemsetAsync(expert_counts, 0, sizeof(int) * E, nullptr));
        CHECK_RC(gather_rows(s.t, tokens_flat, x_by_expert, (int)A, (int)H));
        CHECK_RC(build_work_queue(expert_offsets, (int)E, work_queue, work_count));
        int n_work = 0;
        CHECK_RC(hipMemcpy(&n_work, work_count, sizeof(int), hipMemcpyDeviceToHost));  // the reference's one D2H copy
        CHECK_RC(moe_dropin::moe_mlp1_swiglu(work_queue, 0, n_work, x_by_expert, gate_by_expert, w.w_mlp1 + l * E * 2 * I * H,
                                             w.b_mlp1 + l * E * 2 * I, (int)H, (int)I, 2 * I * H, 2 * I, 1.702f,
                                             c.swiglu_limit, T, 0));
        CHECK_RC(moe_dropin::moe_mlp2_scatter(work_queue, 0, n_work, gate_by_expert, tokens_flat, weights_flat, s.e_agg,
                                              w.w_mlp2 + l * E * H * I, w.b_mlp2 + l * E * H, (int)I, (int)H, H * I, H, T,
                                              0));
        CHECK_RC(vecadd_and_zero(s.x, s.e_agg, 1.0f, T, (int)H));
        CHECK_RC(hipDeviceSynchronize());
        CHECK_RC(hipMemcpy(x.data(), s.x, n * sizeof(float), hipMemcpyDeviceToHost));
        std::fwrite(x.data(), sizeof(float), n, out);
    }
    std::fclose(out);
    std::printf("dropin: %d layers through the reference-named wrappers, router scratch: %s\n", c.n_layers, scratch.c_str());
    return 0;
}

static int run_getp(int argc, char** argv) {
    if (argc < 10) return 2;
    const int steps = std::atoi(argv[6]), batch = std::atoi(argv[7]);
    moe_getp::DecodeOptions opt;
    opt.vocab = std::atoi(argv[8]);
    opt.eos_token = std::atoi(argv[9]);
    moe_host::OssExpertParallelGroup group;  // one GPU: a group of one shard
    opt.ep_group = &group;
    Model m;
    CHECK_RC(load_model(argv[2], argv[3], batch, &m));
    moe_getp::Requests reqs;
    CHECK_RC(moe_getp::read_inputfile(argv[4], /*max_token_len=*/8, steps, &reqs, 0));
    if (argc > 12) {
        opt.trace = std::fopen(argv[12], "wb");
        if (!opt.trace) return 3;
    }
    moe_getp::DecodeBuffers buffers;
    std::vector<int> step_sizes;
    std::vector<float> finals((size_t)reqs.num_reqs * m.tr.config.hidden_dim);
    const long long n_tokens = moe_getp::inference(&m.tr, &buffers, &reqs, steps, opt, &step_sizes, finals.data());
    if (opt.trace) std::fclose(opt.trace);
    if (n_tokens < 0) CHECK_RC(-n_tokens);
    CHECK_RC(moe_getp::write_outputfile(argv[5], &reqs));
    std::printf("getp: %d requests, batch %d, %lld tokens generated, %zu steps\n", reqs.num_reqs, batch, n_tokens,
                step_sizes.size());
    if (argc > 10) {
        FILE* f = std::fopen(argv[10], "wb");
        if (!f) return 3;
        std::fwrite(finals.data(), sizeof(float), finals.size(), f);
        std::fclose(f);
    }
    if (argc > 11) {
        FILE* f = std::fopen(argv[11], "w");
        if (!f) return 3;
        for (int s : step_sizes) std::fprintf(f, "%d\n", s);
        std::fclose(f);
    }
    moe_getp::free_decode_buffers(&buffers);
    moe_getp::free_requests(&reqs);
    return 0;
}

// requests <in.txt> <out.txt> <max_seq_len> [truncate]: reads a request file, gives request i the
// "generated" tokens len(request i), i, i + 1, ... (len % 7 + 1 of them) and writes them out: the two
// file formats without a device.
static int run_requests(int argc, char** argv) {
    if (argc < 5) return 2;
    moe_getp::Requests reqs;
    const int rc = moe_getp::read_inputfile(argv[2], 8, std::atoi(argv[4]), &reqs, argc > 5 ? std::atoi(argv[5]) : 0);
    if (rc) {
        std::printf("read_inputfile -> %d (%s)\n", rc, moe_error_string(rc));
        return 3;
    }
    std::printf("num requests: %d\n", reqs.num_reqs);
    for (int i = 0; i < reqs.num_reqs; ++i) {
        const int len = (int)std::strlen(moe_getp::get_str_req_ptr(&reqs, i));
        int* out = moe_getp::get_tok_gen_ptr(&reqs, i);
        int n = len % 7 + 1;
        if (n > reqs.max_seq_len) n = reqs.max_seq_len;
        out[0] = len;
        for (int j = 1; j < n; ++j) out[j] = i + j - 1;
        out[n] = -1;
    }
    CHECK_RC(moe_getp::write_outputfile(argv[3], &reqs));
    moe_getp::free_requests(&reqs);
    return 0;
}

// verify <generated> <ground truth>: exit code 0 match, 1 mismatch, 255 unreadable
static int run_verify(int argc, char** argv) {
    if (argc < 4) return 2;
    int mismatches = 0;
    const int rc = moe_getp::verify_output(argv[2], argv[3], &mismatches, stdout);
    std::printf("mismatches: %d\n", mismatches);
    return rc < 0 ? 255 : rc;
}

int main(int argc, char** argv) {
    if (argc >= 2 && std::string(argv[1]) == "requests") return run_requests(argc, argv);
    if (argc >= 2 && std::string(argv[1]) == "verify") return run_verify(argc, argv);
    if (argc >= 2 && std::string(argv[1]) == "layers") return run_layers(argc, argv);
    if (argc >= 2 && std::string(argv[1]) == "dropin") return run_dropin(argc, argv);
    if (argc >= 2 && std::string(argv[1]) == "getp") return run_getp(argc, argv);
    if (argc >= 2 && std::string(argv[1]) == "synth") return run_synth(argc, argv);
    std::fprintf(stderr, "usage: %s layers|dropin|getp|synth|requests|verify ... (see the head of moe_stack_main.cpp)\n", argv[0]);
    return 2;
}
