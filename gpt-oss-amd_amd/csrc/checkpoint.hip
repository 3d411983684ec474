// Checkpoint reader: the reference's packed .bin (src/run.cpp:196-283, written by
// tools/model_export/gpt-oss-20b/export_model_bin.py:232-268) and safetensors files with MXFP4
// experts (the exporter's input, export_model_bin.py:150-196).  Host code except for the
// fp32 -> bf16 conversion kernel used at upload.
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <new>
#include <initializer_list>
#include <string>
#include <vector>

#include "../../include/moe_checkpoint.h"
#include "common.h"
#include "kernels.h"

struct moe_ckpt_entry {
    std::string name;
    int dtype = MOE_DTYPE_OTHER;
    int rank = 0;
    long long shape[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    size_t offset = 0;  // from the start of the map
    size_t bytes = 0;
};

struct moe_ckpt {
    int fd = -1;
    const uint8_t* map = nullptr;
    size_t map_bytes = 0;
    bool mxfp4 = false;
    moe_ckpt_config cfg;
    std::vector<moe_ckpt_entry> tensors;
    std::vector<int> layer_index;  // [n_layers * MOE_T_COUNT] -> index into tensors, -1 if absent
};

namespace moe {
namespace {

static_assert(sizeof(moe_ckpt_config) == 60, "Config is fifteen 4-byte fields (src/run.cpp:26-46)");

inline hipStream_t as_stream(moe_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

size_t dtype_bytes(int dtype) { return dtype == MOE_DTYPE_F32 ? 4 : dtype == MOE_DTYPE_BF16 ? 2 : 1; }

size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }

int map_file(const char* path, moe_ckpt* ck) {
    ck->fd = open(path, O_RDONLY);
    if (ck->fd < 0) return MOE_ERR_IO;
    struct stat st;
    if (fstat(ck->fd, &st) != 0 || st.st_size <= 0) return MOE_ERR_IO;
    ck->map_bytes = (size_t)st.st_size;
    void* p = mmap(nullptr, ck->map_bytes, PROT_READ, MAP_PRIVATE, ck->fd, 0);
    if (p == MAP_FAILED) return MOE_ERR_IO;
    ck->map = static_cast<const uint8_t*>(p);
    return MOE_OK;
}

void release(moe_ckpt* ck) {
    if (!ck) return;
    if (ck->map) munmap(const_cast<uint8_t*>(ck->map), ck->map_bytes);
    if (ck->fd >= 0) close(ck->fd);
    delete ck;
}

// Suffixes of the MoE tensor names, indexed by MOE_T_* (export_model_bin.py:51-71).
const char* const kSuffix[MOE_T_COUNT] = {
    "mlp.norm.scale", "mlp.gate.weight", "mlp.gate.bias",          "mlp.mlp1_weight",       "mlp.mlp1_bias",
    "mlp.mlp2_weight", "mlp.mlp2_bias",  "mlp.mlp1_weight.scales", "mlp.mlp2_weight.scales"};

// ---- reference .bin ---------------------------------------------------------------------------
// Element offsets follow memory_map_weights (src/run.cpp:196-238) term by term.
int index_bin(moe_ckpt* ck, int payload_dtype) {
    const moe_ckpt_config& c = ck->cfg;
    const long long V = c.vocab_size, H = c.hidden_dim, E = c.n_experts, I = c.intermediate_dim, L = c.n_layers;
    const long long hd = c.head_dim, nq = c.n_attn_heads, nkv = c.n_kv_heads;
    if (V <= 0 || H <= 0 || E <= 0 || I <= 0 || L <= 0 || hd <= 0 || nq <= 0 || nkv <= 0) return MOE_ERR_PARSE;
    if (c.experts_per_token <= 0 || c.experts_per_token > E) return MOE_ERR_PARSE;
    if (V > (1ll << 24) || H > (1ll << 20) || E > 4096 || I > (1ll << 20) || L > 4096 || hd > 4096 || nq > 4096 ||
        nkv > 4096)
        return MOE_ERR_PARSE;
    const long long qkv = hd * nq + 2 * hd * nkv;  // at most 3 * 2^24 under the limits above
    // The header's fields come from the file: every product and the running sum are checked, so a
    // header whose sizes do not fit 63 bits is a parse error instead of a wrapped offset.
    bool overflow = false;
    long long pos = 0;
    auto take = [&](std::initializer_list<long long> factors) {  // returns the offset of the tensor it appends
        const long long at = pos;
        long long n = 1;
        for (const long long f : factors) overflow |= __builtin_mul_overflow(n, f, &n);
        overflow |= __builtin_add_overflow(pos, n, &pos);
        return at;
    };
    take({V, H});                                     // token_embedding_table
    take({V, H});                                     // out (unembedding)
    take({L, H});                                     // rms_attn_w
    const long long rms_ffn = take({L, H});           // rms_ffn_w
    take({H});                                        // rms_out_w
    take({L, H, qkv});                                // w_qkv
    take({L, qkv});                                   // b_qkv
    take({L, hd * nq, H});                            // w_o
    take({L, H});                                     // b_o
    take({L, nq});                                    // attn_sinks
    const long long w_router = take({L, H, E});
    const long long b_router = take({L, E});
    const long long w_mlp1 = take({L, E, 2 * I, H});
    const long long b_mlp1 = take({L, E, 2 * I});
    const long long w_mlp2 = take({L, E, H, I});
    const long long b_mlp2 = take({L, E, H});
    const size_t eb = dtype_bytes(payload_dtype);
    long long payload_bytes = 0, file_bytes = 0;
    overflow |= __builtin_mul_overflow(pos, (long long)eb, &payload_bytes);
    overflow |= __builtin_add_overflow(payload_bytes, (long long)sizeof(moe_ckpt_config), &file_bytes);
    if (overflow) return MOE_ERR_PARSE;
    if (ck->map_bytes != (size_t)file_bytes) return MOE_ERR_SHAPE;

    struct Slot {
        int which;
        long long base, per_layer;
        int rank;
        long long shape[3];
    };
    const Slot slots[7] = {
        {MOE_T_RMS_FFN, rms_ffn, H, 1, {H, 0, 0}},          {MOE_T_W_ROUTER, w_router, E * H, 2, {E, H, 0}},
        {MOE_T_B_ROUTER, b_router, E, 1, {E, 0, 0}},        {MOE_T_W_MLP1, w_mlp1, E * 2 * I * H, 3, {E, 2 * I, H}},
        {MOE_T_B_MLP1, b_mlp1, E * 2 * I, 2, {E, 2 * I, 0}}, {MOE_T_W_MLP2, w_mlp2, E * H * I, 3, {E, H, I}},
        {MOE_T_B_MLP2, b_mlp2, E * H, 2, {E, H, 0}}};
    ck->layer_index.assign((size_t)L * MOE_T_COUNT, -1);
    for (int l = 0; l < (int)L; ++l) {
        for (const Slot& s : slots) {
            moe_ckpt_entry t;
            t.name = "block." + std::to_string(l) + "." + kSuffix[s.which];
            t.dtype = payload_dtype;
            t.rank = s.rank;
            for (int i = 0; i < s.rank; ++i) t.shape[i] = s.shape[i];
            t.offset = sizeof(moe_ckpt_config) + (size_t)(s.base + l * s.per_layer) * eb;
            t.bytes = (size_t)s.per_layer * eb;
            if (t.offset > ck->map_bytes || t.bytes > ck->map_bytes - t.offset) return MOE_ERR_SHAPE;
            ck->layer_index[(size_t)l * MOE_T_COUNT + s.which] = (int)ck->tensors.size();
            ck->tensors.push_back(t);
        }
    }
    return MOE_OK;
}

// ---- safetensors header: u64 length + JSON ------------------------------------------------------
struct Json {
    const char* p;
    const char* end;
    bool ok = true;
    int depth = 0;

    void ws() {
        while (p < end && (*p == ' ' || *p == '\n' || *p == '\r' || *p == '\t')) ++p;
    }
    bool eat(char c) {
        ws();
        if (p < end && *p == c) {
            ++p;
            return true;
        }
        return false;
    }
    bool expect(char c) {
        if (!eat(c)) ok = false;
        return ok;
    }
    bool string(std::string* out) {
        ws();
        if (p >= end || *p != '"') return ok = false;
        ++p;
        while (p < end && *p != '"') {
            char c = *p++;
            if (c == '\\') {
                if (p >= end) return ok = false;
                const char e = *p++;
                switch (e) {
                    case 'n': c = '\n'; break;
                    case 't': c = '\t'; break;
                    case 'r': c = '\r'; break;
                    case 'b': c = '\b'; break;
                    case 'f': c = '\f'; break;
                    case 'u':  // names here are ASCII; anything else becomes '?'
                        if (end - p < 4) return ok = false;
                        p += 4;
                        c = '?';
                        break;
                    default: c = e;  // \" \\ \/
                }
            }
            if (out) out->push_back(c);
        }
        if (p >= end) return ok = false;
        ++p;
        return true;
    }
    bool integer(long long* out) {
        ws();
        const char* s = p;
        if (p < end && *p == '-') ++p;
        if (p >= end || *p < '0' || *p > '9') return ok = false;
        long long v = 0;
        while (p < end && *p >= '0' && *p <= '9') {
            if (v > (0x7FFFFFFFFFFFFFFFll - 9) / 10) return ok = false;
            v = v * 10 + (*p++ - '0');
        }
        *out = (*s == '-') ? -v : v;
        return true;
    }
    bool int_array(long long* out, int cap, int* n) {
        *n = 0;
        if (!expect('[')) return false;
        if (eat(']')) return true;
        do {
            long long v;
            if (!integer(&v) || *n >= cap) return ok = false;
            out[(*n)++] = v;
        } while (eat(','));
        return expect(']');
    }
    bool skip_value() {
        ws();
        if (p >= end || ++depth > 32) return ok = false;
        bool r = true;
        if (*p == '"') {
            r = string(nullptr);
        } else if (*p == '{') {
            ++p;
            if (!eat('}')) {
                do {
                    if (!string(nullptr) || !expect(':') || !skip_value()) return ok = false;
                } while (eat(','));
                r = expect('}');
            }
        } else if (*p == '[') {
            ++p;
            if (!eat(']')) {
                do {
                    if (!skip_value()) return ok = false;
                } while (eat(','));
                r = expect(']');
            }
        } else {  // number, true, false, null
            const char* s = p;
            while (p < end && *p != ',' && *p != '}' && *p != ']' && *p != ' ' && *p != '\n' && *p != '\r' &&
                   *p != '\t')
                ++p;
            r = p > s;
        }
        --depth;
        return ok = ok && r;
    }
};

int dtype_of(const std::string& s, size_t* width) {
    if (s == "F32") return *width = 4, MOE_DTYPE_F32;
    if (s == "BF16") return *width = 2, MOE_DTYPE_BF16;
    if (s == "U8") return *width = 1, MOE_DTYPE_U8;
    *width = s == "F64" || s == "I64" || s == "U64" ? 8
             : s == "I32" || s == "U32"             ? 4
             : s == "F16" || s == "I16" || s == "U16" ? 2
                                                      : 1;  // I8, BOOL, F8_*
    return MOE_DTYPE_OTHER;
}

bool ends_with(const std::string& s, const std::string& suffix) {
    return s.size() >= suffix.size() && s.compare(s.size() - suffix.size(), suffix.size(), suffix) == 0;
}

// `block.<n>.` anywhere in the name (export_model_bin.py:200); -1 if absent.
int layer_of(const std::string& name) {
    size_t at = 0;
    while ((at = name.find("block.", at)) != std::string::npos) {
        size_t q = at + 6;
        long long v = 0;
        const size_t q0 = q;
        while (q < name.size() && name[q] >= '0' && name[q] <= '9' && v < 100000) v = v * 10 + (name[q++] - '0');
        if (q > q0 && q < name.size() && name[q] == '.') return (int)v;
        at = q0;
    }
    return -1;
}

int parse_safetensors(moe_ckpt* ck) {
    if (ck->map_bytes < 8) return MOE_ERR_PARSE;
    uint64_t n = 0;
    memcpy(&n, ck->map, 8);
    if (n < 2 || n > ck->map_bytes - 8 || n > (100u << 20)) return MOE_ERR_PARSE;
    const size_t data0 = 8 + (size_t)n;
    const size_t data_bytes = ck->map_bytes - data0;
    Json j{reinterpret_cast<const char*>(ck->map) + 8, reinterpret_cast<const char*>(ck->map) + data0};
    if (!j.expect('{')) return MOE_ERR_PARSE;
    if (!j.eat('}')) {
        do {
            moe_ckpt_entry t;
            if (!j.string(&t.name) || !j.expect(':')) return MOE_ERR_PARSE;
            if (t.name == "__metadata__") {
                if (!j.skip_value()) return MOE_ERR_PARSE;
                continue;
            }
            if (!j.expect('{')) return MOE_ERR_PARSE;
            bool have_dtype = false, have_shape = false, have_off = false;
            size_t width = 1;
            long long off[2] = {0, 0};
            if (!j.eat('}')) {
                do {
                    std::string key;
                    if (!j.string(&key) || !j.expect(':')) return MOE_ERR_PARSE;
                    if (key == "dtype") {
                        std::string d;
                        if (!j.string(&d)) return MOE_ERR_PARSE;
                        t.dtype = dtype_of(d, &width);
                        have_dtype = true;
                    } else if (key == "shape") {
                        if (!j.int_array(t.shape, 8, &t.rank)) return MOE_ERR_PARSE;
                        have_shape = true;
                    } else if (key == "data_offsets") {
                        int cnt = 0;
                        if (!j.int_array(off, 2, &cnt) || cnt != 2) return MOE_ERR_PARSE;
                        have_off = true;
                    } else if (!j.skip_value()) {
                        return MOE_ERR_PARSE;
                    }
                } while (j.eat(','));
                if (!j.expect('}')) return MOE_ERR_PARSE;
            }
            if (!have_dtype || !have_shape || !have_off) return MOE_ERR_PARSE;
            if (off[0] < 0 || off[1] < off[0] || (size_t)off[1] > data_bytes) return MOE_ERR_PARSE;
            unsigned long long elems = 1;
            for (int i = 0; i < t.rank; ++i) {
                if (t.shape[i] < 0) return MOE_ERR_PARSE;
                if (t.shape[i] != 0 && elems > (1ull << 48) / (unsigned long long)t.shape[i]) return MOE_ERR_PARSE;
                elems *= (unsigned long long)t.shape[i];
            }
            t.offset = data0 + (size_t)off[0];
            t.bytes = (size_t)(off[1] - off[0]);
            if (t.dtype != MOE_DTYPE_OTHER && elems * width != t.bytes) return MOE_ERR_PARSE;
            ck->tensors.push_back(t);
        } while (j.eat(','));
        if (!j.expect('}')) return MOE_ERR_PARSE;
    }
    j.ws();
    return j.ok ? MOE_OK : MOE_ERR_PARSE;
}

// Sorts the tensors found into the per-layer table and derives / checks H, I, E and the layer count.
int index_safetensors(moe_ckpt* ck, const moe_ckpt_config* want) {
    int n_layers = 0;
    for (const moe_ckpt_entry& t : ck->tensors) n_layers = std::max(n_layers, layer_of(t.name) + 1);
    if (n_layers <= 0) return MOE_ERR_MISSING;
    ck->layer_index.assign((size_t)n_layers * MOE_T_COUNT, -1);
    for (size_t i = 0; i < ck->tensors.size(); ++i) {
        const moe_ckpt_entry& t = ck->tensors[i];
        const int l = layer_of(t.name);
        if (l < 0) continue;
        int which = -1;
        for (int w = 0; w < MOE_T_COUNT; ++w)
            if (ends_with(t.name, kSuffix[w])) which = w;
        if (ends_with(t.name, "mlp.mlp1_weight.blocks")) which = MOE_T_W_MLP1, ck->mxfp4 = true;
        if (ends_with(t.name, "mlp.mlp2_weight.blocks")) which = MOE_T_W_MLP2, ck->mxfp4 = true;
        if (which >= 0) ck->layer_index[(size_t)l * MOE_T_COUNT + which] = (int)i;
    }
    long long H = 0, I = 0, E = 0;
    for (int l = 0; l < n_layers; ++l) {
        const int* idx = &ck->layer_index[(size_t)l * MOE_T_COUNT];
        const int need_dense[] = {MOE_T_W_ROUTER, MOE_T_B_ROUTER, MOE_T_W_MLP1, MOE_T_B_MLP1, MOE_T_W_MLP2, MOE_T_B_MLP2};
        for (int w : need_dense)
            if (idx[w] < 0) return MOE_ERR_MISSING;
        if (ck->mxfp4 && (idx[MOE_T_W_MLP1_SCALES] < 0 || idx[MOE_T_W_MLP2_SCALES] < 0)) return MOE_ERR_MISSING;
        const moe_ckpt_entry& wr = ck->tensors[idx[MOE_T_W_ROUTER]];
        const moe_ckpt_entry& w1 = ck->tensors[idx[MOE_T_W_MLP1]];
        const moe_ckpt_entry& w2 = ck->tensors[idx[MOE_T_W_MLP2]];
        if (wr.rank != 2) return MOE_ERR_SHAPE;
        const long long e = wr.shape[0], h = wr.shape[1];
        long long i2, hh, ii, h1;
        if (ck->mxfp4) {
            if (w1.rank != 4 || w2.rank != 4 || w1.shape[3] != MOE_MXFP4_BLOCK_BYTES ||
                w2.shape[3] != MOE_MXFP4_BLOCK_BYTES || w1.dtype != MOE_DTYPE_U8 || w2.dtype != MOE_DTYPE_U8)
                return MOE_ERR_SHAPE;
            i2 = w1.shape[1], h1 = w1.shape[2] * MOE_MXFP4_BLOCK_ELEMS;
            hh = w2.shape[1], ii = w2.shape[2] * MOE_MXFP4_BLOCK_ELEMS;
            const moe_ckpt_entry& s1 = ck->tensors[idx[MOE_T_W_MLP1_SCALES]];
            const moe_ckpt_entry& s2 = ck->tensors[idx[MOE_T_W_MLP2_SCALES]];
            if (s1.dtype != MOE_DTYPE_U8 || s2.dtype != MOE_DTYPE_U8 || s1.rank != 3 || s2.rank != 3) return MOE_ERR_SHAPE;
            for (int d = 0; d < 3; ++d)
                if (s1.shape[d] != w1.shape[d] || s2.shape[d] != w2.shape[d]) return MOE_ERR_SHAPE;
        } else {
            if (w1.rank != 3 || w2.rank != 3) return MOE_ERR_SHAPE;
            i2 = w1.shape[1], h1 = w1.shape[2], hh = w2.shape[1], ii = w2.shape[2];
        }
        if (w1.shape[0] != e || w2.shape[0] != e || h1 != h || hh != h || i2 != 2 * ii) return MOE_ERR_SHAPE;
        const moe_ckpt_entry& br = ck->tensors[idx[MOE_T_B_ROUTER]];
        const moe_ckpt_entry& b1 = ck->tensors[idx[MOE_T_B_MLP1]];
        const moe_ckpt_entry& b2 = ck->tensors[idx[MOE_T_B_MLP2]];
        if (br.rank != 1 || br.shape[0] != e || b1.rank != 2 || b1.shape[0] != e || b1.shape[1] != i2 || b2.rank != 2 ||
            b2.shape[0] != e || b2.shape[1] != h)
            return MOE_ERR_SHAPE;
        if (idx[MOE_T_RMS_FFN] >= 0) {
            const moe_ckpt_entry& rn = ck->tensors[idx[MOE_T_RMS_FFN]];
            if (rn.rank != 1 || rn.shape[0] != h) return MOE_ERR_SHAPE;
        }
        for (int w = 0; w < MOE_T_W_MLP1_SCALES; ++w) {
            if (idx[w] < 0) continue;
            const int dt = ck->tensors[idx[w]].dtype;
            const bool packed = ck->mxfp4 && (w == MOE_T_W_MLP1 || w == MOE_T_W_MLP2);
            if (!packed && dt != MOE_DTYPE_F32 && dt != MOE_DTYPE_BF16) return MOE_ERR_FORMAT;
        }
        if (l == 0) H = h, I = ii, E = e;
        if (h != H || ii != I || e != E) return MOE_ERR_SHAPE;
    }
    if (H > 0x7FFFFFFF || I > 0x7FFFFFFF || E > 0x7FFFFFFF) return MOE_ERR_LIMIT;
    memset(&ck->cfg, 0, sizeof(ck->cfg));
    if (want) ck->cfg = *want;
    moe_ckpt_config& c = ck->cfg;
    if ((c.hidden_dim && c.hidden_dim != H) || (c.intermediate_dim && c.intermediate_dim != I) ||
        (c.n_experts && c.n_experts != E) || (c.n_layers && c.n_layers != n_layers))
        return MOE_ERR_SHAPE;
    c.hidden_dim = (int32_t)H;
    c.intermediate_dim = (int32_t)I;
    c.n_experts = (int32_t)E;
    c.n_layers = n_layers;
    return MOE_OK;
}

// ---- upload -----------------------------------------------------------------------------------
__global__ void f32_to_bf16_kernel(const float* __restrict__ src, uint16_t* __restrict__ dst, long long n) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long k = i; k < n; k += stride) dst[k] = f32_to_bf16_bits(src[k]);
}

int upload_dense(const moe_ckpt* ck, int layer, int which, uint16_t* d_dst, void* d_staging, size_t staging_bytes,
                 hipStream_t stream) {
    if (!d_dst) return MOE_OK;
    const int ti = ck->layer_index[(size_t)layer * MOE_T_COUNT + which];
    if (ti < 0) return MOE_ERR_MISSING;
    const moe_ckpt_entry& t = ck->tensors[ti];
    const uint8_t* h = ck->map + t.offset;
    if (t.dtype == MOE_DTYPE_BF16) {
        MOE_RETURN_IF_HIP(hipMemcpyAsync(d_dst, h, t.bytes, hipMemcpyHostToDevice, stream));
        return MOE_OK;
    }
    if (t.dtype != MOE_DTYPE_F32) return MOE_ERR_FORMAT;
    const long long n = (long long)(t.bytes / 4);
    const long long chunk = (long long)(staging_bytes / 4);
    for (long long at = 0; at < n; at += chunk) {
        const long long c = std::min(chunk, n - at);
        MOE_RETURN_IF_HIP(hipMemcpyAsync(d_staging, h + (size_t)at * 4, (size_t)c * 4, hipMemcpyHostToDevice, stream));
        const int blocks = (int)std::min<long long>(ceil_div<long long>(c, 256), 4096);
        hipLaunchKernelGGL(f32_to_bf16_kernel, dim3(blocks), dim3(256), 0, stream,
                           static_cast<const float*>(d_staging), d_dst + at, c);
        const int rc = launch_status();
        if (rc != MOE_OK) return rc;
    }
    return MOE_OK;
}

// One MXFP4 weight tensor: whole experts through the staging buffer, as many at a time as fit.
int upload_mxfp4(const moe_ckpt* ck, int layer, int which_blocks, int which_scales, int format, void* d_w,
                 void* d_scales, void* d_staging, size_t staging_bytes, hipStream_t stream) {
    if (!d_w) return MOE_OK;
    const int bi = ck->layer_index[(size_t)layer * MOE_T_COUNT + which_blocks];
    const int si = ck->layer_index[(size_t)layer * MOE_T_COUNT + which_scales];
    if (bi < 0 || si < 0) return MOE_ERR_MISSING;
    const moe_ckpt_entry& tb = ck->tensors[bi];
    const moe_ckpt_entry& ts = ck->tensors[si];
    const long long E = tb.shape[0], rows = tb.shape[1], G = tb.shape[2];
    const long long K = G * MOE_MXFP4_BLOCK_ELEMS;
    if (rows > 0x7FFFFFFF || K > 0x7FFFFFFF) return MOE_ERR_LIMIT;
    const size_t blk_e = (size_t)rows * G * MOE_MXFP4_BLOCK_BYTES, scl_e = (size_t)rows * G;
    size_t tiled_b = 0, tiled_s = 0;
    if (format == MOE_WEIGHTS_MXFP4_TILED) {
        if (!d_scales) return MOE_ERR_NULL;
        if (rows % 64 != 0) return MOE_ERR_SHAPE;
        mxfp4_tiled_bytes((int)rows, (int)K, &tiled_b, &tiled_s);
    }
    long long per = (long long)E;
    while (per > 1 && align256(per * blk_e) + per * scl_e > staging_bytes) --per;
    if (align256(per * blk_e) + per * scl_e > staging_bytes) return MOE_ERR_WORKSPACE;
    uint8_t* stg_b = static_cast<uint8_t*>(d_staging);
    for (long long e0 = 0; e0 < E; e0 += per) {
        const long long n = std::min(per, E - e0);
        uint8_t* stg_s = stg_b + align256(n * blk_e);
        MOE_RETURN_IF_HIP(hipMemcpyAsync(stg_b, ck->map + tb.offset + e0 * blk_e, n * blk_e, hipMemcpyHostToDevice, stream));
        MOE_RETURN_IF_HIP(hipMemcpyAsync(stg_s, ck->map + ts.offset + e0 * scl_e, n * scl_e, hipMemcpyHostToDevice, stream));
        int rc;
        if (format == MOE_WEIGHTS_MXFP4_TILED) {
            rc = launch_mxfp4_repack(stg_b, stg_s, (int)n, (int)rows, (int)K, static_cast<uint8_t*>(d_w) + e0 * tiled_b,
                                     static_cast<uint8_t*>(d_scales) + e0 * tiled_s, false, stream);
        } else {
            rc = launch_dequant_mxfp4(stg_b, stg_s, n * rows * G, static_cast<uint16_t*>(d_w) + e0 * rows * K, stream);
        }
        if (rc != MOE_OK) return rc;
    }
    return MOE_OK;
}

}  // namespace
}  // namespace moe

using namespace moe;

extern "C" {

int moe_ckpt_open_bin(const char* path, int payload_dtype, moe_ckpt** out) {
    if (!path || !out) return MOE_ERR_NULL;
    *out = nullptr;
    if (payload_dtype != MOE_DTYPE_F32 && payload_dtype != MOE_DTYPE_BF16) return MOE_ERR_FORMAT;
    moe_ckpt* ck = new (std::nothrow) moe_ckpt();
    if (!ck) return MOE_ERR_IO;
    int rc = map_file(path, ck);
    if (rc == MOE_OK && ck->map_bytes < sizeof(moe_ckpt_config)) rc = MOE_ERR_PARSE;
    if (rc == MOE_OK) {
        memcpy(&ck->cfg, ck->map, sizeof(moe_ckpt_config));
        rc = index_bin(ck, payload_dtype);
    }
    if (rc != MOE_OK) {
        release(ck);
        return rc;
    }
    *out = ck;
    return MOE_OK;
}

int moe_ckpt_open_safetensors(const char* path, const moe_ckpt_config* cfg, moe_ckpt** out) {
    if (!path || !out) return MOE_ERR_NULL;
    *out = nullptr;
    moe_ckpt* ck = new (std::nothrow) moe_ckpt();
    if (!ck) return MOE_ERR_IO;
    int rc = map_file(path, ck);
    if (rc == MOE_OK) rc = parse_safetensors(ck);
    if (rc == MOE_OK) rc = index_safetensors(ck, cfg);
    if (rc != MOE_OK) {
        release(ck);
        return rc;
    }
    *out = ck;
    return MOE_OK;
}

void moe_ckpt_close(moe_ckpt* ck) { release(ck); }

int moe_ckpt_get_config(const moe_ckpt* ck, moe_ckpt_config* cfg) {
    if (!ck || !cfg) return MOE_ERR_NULL;
    *cfg = ck->cfg;
    return MOE_OK;
}

int moe_ckpt_is_mxfp4(const moe_ckpt* ck) { return ck && ck->mxfp4 ? 1 : 0; }

int moe_ckpt_layer_tensor(const moe_ckpt* ck, int layer, int which, const void** h_data, size_t* bytes, int* dtype) {
    if (!ck) return MOE_ERR_NULL;
    if (layer < 0 || layer >= ck->cfg.n_layers || which < 0 || which >= MOE_T_COUNT) return MOE_ERR_SHAPE;
    const int ti = ck->layer_index[(size_t)layer * MOE_T_COUNT + which];
    if (ti < 0) return MOE_ERR_MISSING;
    const moe_ckpt_entry& t = ck->tensors[ti];
    if (h_data) *h_data = ck->map + t.offset;
    if (bytes) *bytes = t.bytes;
    if (dtype) *dtype = t.dtype;
    return MOE_OK;
}

int moe_ckpt_n_tensors(const moe_ckpt* ck) { return ck ? (int)ck->tensors.size() : 0; }

int moe_ckpt_tensor_info(const moe_ckpt* ck, int index, const char** name, int* dtype, int* rank, long long* shape,
                         const void** h_data, size_t* bytes) {
    if (!ck) return MOE_ERR_NULL;
    if (index < 0 || index >= (int)ck->tensors.size()) return MOE_ERR_SHAPE;
    const moe_ckpt_entry& t = ck->tensors[index];
    if (name) *name = t.name.c_str();
    if (dtype) *dtype = t.dtype;
    if (rank) *rank = t.rank;
    if (shape)
        for (int i = 0; i < 8; ++i) shape[i] = t.shape[i];
    if (h_data) *h_data = ck->map + t.offset;
    if (bytes) *bytes = t.bytes;
    return MOE_OK;
}

size_t moe_ckpt_staging_bytes(const moe_ckpt* ck) {
    if (!ck) return 0;
    const moe_ckpt_config& c = ck->cfg;
    if (ck->mxfp4) {
        const size_t g1 = (size_t)2 * c.intermediate_dim * (c.hidden_dim / MOE_MXFP4_BLOCK_ELEMS);
        const size_t g2 = (size_t)c.hidden_dim * (c.intermediate_dim / MOE_MXFP4_BLOCK_ELEMS);
        const size_t g = g1 > g2 ? g1 : g2;
        return align256(g * MOE_MXFP4_BLOCK_BYTES) + align256(g);
    }
    return align256((size_t)2 * c.intermediate_dim * c.hidden_dim * sizeof(float));
}

int moe_ckpt_upload_layer(const moe_ckpt* ck, int layer, const moe_layer_device* dst, void* d_staging,
                          size_t staging_bytes, moe_stream_t stream) {
    if (!ck || !dst || !d_staging) return MOE_ERR_NULL;
    if (dst->struct_bytes != sizeof(moe_layer_device)) return MOE_ERR_FORMAT;
    if (layer < 0 || layer >= ck->cfg.n_layers) return MOE_ERR_SHAPE;
    if ((uintptr_t)d_staging & 255u) return MOE_ERR_ALIGN;
    if (staging_bytes < moe_ckpt_staging_bytes(ck)) return MOE_ERR_WORKSPACE;
    const int fmt = dst->weight_format;
    if (fmt != MOE_WEIGHTS_BF16 && fmt != MOE_WEIGHTS_MXFP4_TILED) return MOE_ERR_FORMAT;
    if (fmt == MOE_WEIGHTS_MXFP4_TILED && !ck->mxfp4) return MOE_ERR_FORMAT;
    hipStream_t s = as_stream(stream);
    int rc = MOE_OK;
    const struct {
        int which;
        uint16_t* d;
    } small[] = {{MOE_T_W_ROUTER, dst->w_router}, {MOE_T_B_ROUTER, dst->b_router}, {MOE_T_B_MLP1, dst->b_mlp1},
                 {MOE_T_B_MLP2, dst->b_mlp2}};
    for (const auto& t : small)
        if ((rc = upload_dense(ck, layer, t.which, t.d, d_staging, staging_bytes, s)) != MOE_OK) return rc;
    if (dst->rms_ffn_w && (rc = upload_dense(ck, layer, MOE_T_RMS_FFN, dst->rms_ffn_w, d_staging, staging_bytes, s)) != MOE_OK)
        return rc;
    if (ck->mxfp4) {
        rc = upload_mxfp4(ck, layer, MOE_T_W_MLP1, MOE_T_W_MLP1_SCALES, fmt, dst->w_mlp1, dst->w_mlp1_scales, d_staging,
                          staging_bytes, s);
        if (rc != MOE_OK) return rc;
        return upload_mxfp4(ck, layer, MOE_T_W_MLP2, MOE_T_W_MLP2_SCALES, fmt, dst->w_mlp2, dst->w_mlp2_scales, d_staging,
                            staging_bytes, s);
    }
    rc = upload_dense(ck, layer, MOE_T_W_MLP1, static_cast<uint16_t*>(dst->w_mlp1), d_staging, staging_bytes, s);
    if (rc != MOE_OK) return rc;
    return upload_dense(ck, layer, MOE_T_W_MLP2, static_cast<uint16_t*>(dst->w_mlp2), d_staging, staging_bytes, s);
}

}  // extern "C"
