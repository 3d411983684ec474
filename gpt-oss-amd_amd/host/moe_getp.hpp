// The batch runtime around forward(), for the part one GPU and the MoE half of the model can show:
//   * the request file formats and the exact-match verifier of src/getp/eval.cpp (:18-100, :109-206),
//     same layouts and same text, with return codes instead of exit();
//   * the decode loop of generate() (src/getp/run.cpp:467-659): per step the sequences that are still
//     running are compacted to the front of the batch (valid_batch_size, batch_indices, B_stride,
//     :573-588), forward() runs on that compact batch, and each sequence then takes its next prompt
//     token or a sampled one and may finish (commit_generation, :545-571);
//   * inference() (src/getp/run.cpp:661-736) as one worker that takes the requests batch by batch.
// The library has no tokenizer, embedding, attention or logits head.  Their places are taken by the
// smallest stand-ins that keep the loop's data flow: a request's prompt tokens are its bytes, every
// sequence owns one row of a [B_stride, hidden_dim] state table on the device (where the reference
// keeps a KV cache slot per sequence, addressed by the same batch_indices), a step gathers the running
// sequences' rows into the compact batch, runs forward() and scatters the rows back, and the "logits"
// of a sequence at position p are `vocab` consecutive values of its output row, starting at
// (p * vocab) % (hidden_dim - vocab + 1) (greedy argmax over them, as the reference's temperature-0
// path, src/getp/run.cpp:619-637).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <string>
#include <vector>

#include "moe_forward.hpp"

namespace moe_getp {

// ---- request management (src/getp/eval.cpp:9-40) -------------------------------------------------
struct Requests {
    int num_reqs = 0;       // number of requests
    int max_token_len = 0;  // maximum size of token
    int max_seq_len = 0;    // maximum number of sequence
    char* str_reqs = nullptr;  // buffer for requested strings
    int* tok_gens = nullptr;   // buffer for generated tokens
};

inline size_t str_req_stride(const Requests* r) { return (size_t)r->max_token_len * (r->max_seq_len + 1); }

inline int build_requests(Requests* reqs, int num_reqs, int max_token_len, int max_seq_len) {
    if (num_reqs < 0 || max_token_len <= 0 || max_seq_len <= 0) return MOE_ERR_SHAPE;
    reqs->num_reqs = num_reqs;
    reqs->max_token_len = max_token_len;
    reqs->max_seq_len = max_seq_len;
    reqs->str_reqs = (char*)calloc((size_t)num_reqs * str_req_stride(reqs) + 1, sizeof(char));
    reqs->tok_gens = (int*)calloc((size_t)num_reqs * (max_seq_len + 1) + 1, sizeof(int));
    if (!reqs->str_reqs || !reqs->tok_gens) return (int)hipErrorOutOfMemory;
    return MOE_OK;
}

inline void free_requests(Requests* reqs) {
    free(reqs->str_reqs);
    free(reqs->tok_gens);
    reqs->str_reqs = nullptr;
    reqs->tok_gens = nullptr;
}

inline char* get_str_req_ptr(Requests* reqs, int idx) { return reqs->str_reqs + (size_t)idx * str_req_stride(reqs); }
inline int* get_tok_gen_ptr(Requests* reqs, int idx) { return reqs->tok_gens + (size_t)idx * (reqs->max_seq_len + 1); }

// src/getp/eval.cpp:42-79.  First line: the number of requests; then one request per line.  A line
// longer than a request slot is cut to the slot (the reference copies it whole).
inline int read_inputfile(const char* input_filename, int max_token_len, int max_seq_len, Requests* reqs,
                          int truncate_lines) {
    std::ifstream in(input_filename);
    if (!in.is_open()) return MOE_ERR_IO;
    std::string line;
    std::getline(in, line);
    int num_reqs = atoi(line.c_str());
    if (num_reqs < 0) return MOE_ERR_PARSE;
    if (truncate_lines > 0 && truncate_lines < num_reqs) num_reqs = truncate_lines;
    const int rc = build_requests(reqs, num_reqs, max_token_len, max_seq_len);
    if (rc) return rc;
    int idx = 0;
    while (idx < num_reqs && std::getline(in, line)) {
        const size_t n = line.size() < str_req_stride(reqs) - 1 ? line.size() : str_req_stride(reqs) - 1;
        memcpy(get_str_req_ptr(reqs, idx), line.c_str(), n);
        idx++;
    }
    return MOE_OK;
}

// src/getp/eval.cpp:81-100.  One line per request: its generated tokens up to the first negative
// entry, separated by single spaces.  A request's slot holds max_seq_len + 1 entries: the walk stops
// there even without a terminator (the reference walks on into the next request's slot).
inline int write_outputfile(const char* output_filename, Requests* reqs) {
    std::ofstream out(output_filename);
    if (!out.is_open()) return MOE_ERR_IO;
    for (int i = 0; i < reqs->num_reqs; i++) {
        const int* output_tokens = get_tok_gen_ptr(reqs, i);
        for (int j = 0; j <= reqs->max_seq_len && output_tokens[j] >= 0; j++) {
            if (j > 0) out << ' ';
            out << output_tokens[j];
        }
        out << '\n';
    }
    return MOE_OK;
}

// src/getp/eval.cpp:109-206.  0: every line of the ground truth matches; 1: mismatches (their number
// in *mismatches); -1: a file cannot be opened.  `log` (may be NULL) receives the reference's messages.
inline int verify_output(const char* generated_filename, const char* ground_truth_filename, int* mismatches = nullptr,
                         FILE* log = nullptr) {
    std::ifstream generated_file(generated_filename);
    std::ifstream gt_file(ground_truth_filename);
    if (!generated_file.is_open() || !gt_file.is_open()) return -1;
    std::string gen_line, gt_line;
    int line_num = 1, total_mismatches = 0, total_lines = 0;
    while (std::getline(gt_file, gt_line)) {
        total_lines++;
        if (!std::getline(generated_file, gen_line)) {
            if (log) fprintf(log, "Output has fewer lines than GT at line %d\n", line_num);
            total_mismatches++;
            break;
        }
        if (gt_line.empty() && gen_line.empty()) {
            line_num++;
            continue;
        }
        std::vector<int> gt_tokens, gen_tokens;
        std::istringstream gt_stream(gt_line), gen_stream(gen_line);
        int token;
        while (gt_stream >> token) gt_tokens.push_back(token);
        while (gen_stream >> token) gen_tokens.push_back(token);
        bool line_matches = true;
        if (gt_tokens.size() != gen_tokens.size()) {
            if (log)
                fprintf(log, "Request #%d: Length mismatch (GT: %zu tokens, Generated: %zu tokens)\n", line_num,
                        gt_tokens.size(), gen_tokens.size());
            line_matches = false;
        } else {
            for (size_t i = 0; i < gt_tokens.size(); i++) {
                if (gt_tokens[i] != gen_tokens[i]) {
                    if (log)
                        fprintf(log, "Request %d: Token mismatch at position %zu (GT: %d, Generated: %d)\n", line_num, i,
                                gt_tokens[i], gen_tokens[i]);
                    line_matches = false;
                    break;
                }
            }
        }
        if (!line_matches) total_mismatches++;
        line_num++;
    }
    if (std::getline(generated_file, gen_line)) {
        if (log) fprintf(log, "Output file has more lines than GT\n");
        total_mismatches++;
    }
    if (log)
        fprintf(log, "Total requests checked: %d\nRequests with mismatches: %d\nRequests matching: %d\n", total_lines,
                total_mismatches, total_lines - total_mismatches);
    if (mismatches) *mismatches = total_mismatches;
    return total_mismatches == 0 ? 0 : 1;
}

// ---- decode loop -----------------------------------------------------------------------------------
struct DecodeOptions {
    int vocab = 64;       // that many consecutive values of an output row stand in for the logits
    int eos_token = -1;   // a sampled token equal to this ends its sequence (the reference: 199999, 200002)
    bool record_steps = false;
    // If not NULL, every step is appended as: int32 {valid_batch_size, window}, int32 indices[valid],
    // int32 tokens_in[valid], float rows_in[valid, hidden], float rows_out[valid, hidden],
    // int32 tokens_out[valid] (the token each sequence takes next), so that a test can follow the loop
    // step by step.  Costs two device-to-host copies per step.
    FILE* trace = nullptr;
    // the reference's thread-local expert-parallel group (src/getp/run.cpp:136), handed to forward() as there;
    // NULL or a group of one shard
    moe_host::OssExpertParallelGroup* ep_group = nullptr;
};

// Device and pinned host buffers of one worker (the reference's ThreadLocalBatchBuffers,
// src/getp/run.cpp:330-420): allocated once for the transformer's batch_size.
struct DecodeBuffers {
    int capacity = 0, hidden = 0, vocab = 0;
    int *tokens = nullptr, *positions = nullptr, *indices = nullptr;  // pinned host, [capacity]
    int* indices_d = nullptr;                                          // device, [capacity]
    float* x_seq_d = nullptr;                                          // device, [capacity, hidden]: one row per sequence
    float* logits_h = nullptr;                                         // pinned host, [capacity, vocab]
};

inline void free_decode_buffers(DecodeBuffers* b) {
    if (b->tokens) (void)hipHostFree(b->tokens);
    if (b->positions) (void)hipHostFree(b->positions);
    if (b->indices) (void)hipHostFree(b->indices);
    if (b->logits_h) (void)hipHostFree(b->logits_h);
    if (b->indices_d) (void)hipFree(b->indices_d);
    if (b->x_seq_d) (void)hipFree(b->x_seq_d);
    *b = DecodeBuffers();
}

inline int ensure_decode_buffers(DecodeBuffers* b, int capacity, int hidden, int vocab) {
    if (b->capacity >= capacity && b->hidden == hidden && b->vocab >= vocab) return MOE_OK;
    free_decode_buffers(b);
    hipError_t e;
    if ((e = hipHostMalloc((void**)&b->tokens, sizeof(int) * capacity)) != hipSuccess) return (int)e;
    if ((e = hipHostMalloc((void**)&b->positions, sizeof(int) * capacity)) != hipSuccess) return (int)e;
    if ((e = hipHostMalloc((void**)&b->indices, sizeof(int) * capacity)) != hipSuccess) return (int)e;
    if ((e = hipHostMalloc((void**)&b->logits_h, sizeof(float) * capacity * vocab)) != hipSuccess) return (int)e;
    if ((e = hipMalloc((void**)&b->indices_d, sizeof(int) * capacity)) != hipSuccess) return (int)e;
    if ((e = hipMalloc((void**)&b->x_seq_d, sizeof(float) * (size_t)capacity * hidden)) != hipSuccess) return (int)e;
    b->capacity = capacity;
    b->hidden = hidden;
    b->vocab = vocab;
    return MOE_OK;
}

// Stand-in for the embedding of a prompt: the initial state row of a sequence, a pure function of the
// request's bytes (FNV-1a of the string seeds a 32-bit xorshift; values in [-1, 1)).
inline void initial_state_row(const char* request, int hidden, float* row) {
    uint32_t h = 2166136261u;
    for (const char* c = request; *c; ++c) h = (h ^ (uint8_t)*c) * 16777619u;
    if (h == 0) h = 1;
    for (int i = 0; i < hidden; ++i) {
        h ^= h << 13;
        h ^= h >> 17;
        h ^= h << 5;
        row[i] = (float)(int32_t)h * (1.0f / 2147483648.0f);
    }
}

// One batch of requests through the decode loop (generate(), src/getp/run.cpp:467-659).
// input_seqs / output_tokens_batch as in the reference: output_tokens_batch[b] receives the generated
// tokens of request b, terminated by -1.  Returns the number of generated tokens, or a negative
// MOE_ERR_* / minus a hipError_t.  step_sizes (may be NULL) receives valid_batch_size of every step.
// final_rows_h (may be NULL): [batch_size, hidden_dim], the state row of every sequence after its last step.
inline long long generate(moe_host::OssMoeTransformer* t_d, DecodeBuffers* buffers, const char** input_seqs,
                          int** output_tokens_batch, int batch_size, int steps, const DecodeOptions& opt,
                          std::vector<int>* step_sizes = nullptr, float* final_rows_h = nullptr) {
    const int H = t_d->config.hidden_dim;
    if (batch_size <= 0 || batch_size > t_d->config.batch_size || opt.vocab <= 0 || opt.vocab > H) return MOE_ERR_SHAPE;
    int rc = ensure_decode_buffers(buffers, t_d->config.batch_size, H, opt.vocab);
    if (rc) return -(long long)rc;
    hipStream_t stream = reinterpret_cast<hipStream_t>(t_d->stream);
    long long total_tokens_out = 0;

    // prompt tokens = the request's bytes (the reference tokenises here, :497-510); at least one
    std::vector<std::vector<int>> prompt_tokens(batch_size);
    std::vector<float> rows((size_t)batch_size * H);
    for (int b = 0; b < batch_size; b++) {
        const char* input_seq = input_seqs[b] ? input_seqs[b] : "";
        for (const char* c = input_seq; *c; ++c) prompt_tokens[b].push_back((uint8_t)*c);
        if (prompt_tokens[b].empty()) prompt_tokens[b].push_back(0);
        initial_state_row(input_seq, H, rows.data() + (size_t)b * H);
    }
    if (hipMemcpyAsync(buffers->x_seq_d, rows.data(), sizeof(float) * rows.size(), hipMemcpyHostToDevice, stream) !=
        hipSuccess)
        return -(long long)hipGetLastError();
    if (hipStreamSynchronize(stream) != hipSuccess) return -(long long)hipGetLastError();

    std::vector<int> current_tokens(batch_size), pos(batch_size, 0);
    std::vector<char> finished(batch_size, 0);
    int active_sequences = batch_size;
    for (int b = 0; b < batch_size; b++) current_tokens[b] = prompt_tokens[b][0];

    auto commit_generation = [&](int b_idx, int next_token, bool counted) {  // :545-571
        const int n_prompt = (int)prompt_tokens[b_idx].size();
        if (counted && output_tokens_batch[b_idx]) {
            const int output_idx = pos[b_idx] - n_prompt;
            if (output_idx >= 0) output_tokens_batch[b_idx][output_idx] = next_token;
        }
        if (counted) total_tokens_out++;
        if ((next_token == opt.eos_token || pos[b_idx] + 1 >= steps) && !finished[b_idx]) {
            finished[b_idx] = 1;
            active_sequences--;
            if (output_tokens_batch[b_idx]) {
                // a sequence that runs out of steps inside its prompt has generated nothing: the terminator
                // goes to entry 0 (the reference writes none then, and its writer walks past the slot)
                const int end_idx = pos[b_idx] - n_prompt + 1;
                output_tokens_batch[b_idx][end_idx >= 0 ? end_idx : 0] = -1;
            }
        }
        current_tokens[b_idx] = next_token;
    };

    int iteration = 0;
    while (active_sequences > 0) {
        // the sequences still running, compacted to the front of the batch (:573-583)
        int valid_batch_size = 0;
        for (int b = 0; b < batch_size && valid_batch_size < batch_size; b++) {
            if (!finished[b] && pos[b] + 1 < steps) {
                buffers->tokens[valid_batch_size] = current_tokens[b];
                buffers->positions[valid_batch_size] = pos[b];
                buffers->indices[valid_batch_size] = b;
                valid_batch_size++;
            }
        }
        if (valid_batch_size == 0) break;
        if (step_sizes) step_sizes->push_back(valid_batch_size);

        // state rows of the running sequences -> compact batch; forward; rows back to their sequences
        if (hipMemcpyAsync(buffers->indices_d, buffers->indices, sizeof(int) * valid_batch_size, hipMemcpyHostToDevice,
                           stream) != hipSuccess)
            return -(long long)hipGetLastError();
        if ((rc = moe_gather_rows(buffers->x_seq_d, buffers->indices_d, t_d->state.x, valid_batch_size, H, t_d->stream)))
            return -(long long)rc;
        std::vector<float> trace_rows;
        if (opt.trace) {
            trace_rows.resize((size_t)2 * valid_batch_size * H);
            if (hipMemcpyAsync(trace_rows.data(), t_d->state.x, sizeof(float) * (size_t)valid_batch_size * H,
                               hipMemcpyDeviceToHost, stream) != hipSuccess ||
                hipStreamSynchronize(stream) != hipSuccess)
                return -(long long)hipGetLastError();
        }
        float* out = moe_host::forward(t_d, opt.ep_group, buffers->tokens, buffers->positions, valid_batch_size,
                                       buffers->indices, t_d->config.batch_size);  // :588
        if (!out) return -(long long)t_d->last_error;
        if ((rc = moe_scatter_rows(out, buffers->indices_d, buffers->x_seq_d, valid_batch_size, H, t_d->stream)))
            return -(long long)rc;
        // the stand-in logits: a window of `vocab` values of every output row that moves with the position
        // (every sequence of a batch is at the same position: all started together, one step each per pass)
        const int window = (int)(((long long)iteration * opt.vocab) % (H - opt.vocab + 1));
        iteration++;
        if (hipMemcpy2DAsync(buffers->logits_h, sizeof(float) * opt.vocab, out + window, sizeof(float) * H,
                             sizeof(float) * opt.vocab, valid_batch_size, hipMemcpyDeviceToHost, stream) != hipSuccess)
            return -(long long)hipGetLastError();
        if (hipStreamSynchronize(stream) != hipSuccess) return -(long long)hipGetLastError();
        if (opt.trace) {
            if (hipMemcpy(trace_rows.data() + (size_t)valid_batch_size * H, out, sizeof(float) * (size_t)valid_batch_size * H,
                          hipMemcpyDeviceToHost) != hipSuccess)
                return -(long long)hipGetLastError();
            const int head[2] = {valid_batch_size, window};
            fwrite(head, sizeof(int), 2, opt.trace);
            fwrite(buffers->indices, sizeof(int), valid_batch_size, opt.trace);
            fwrite(buffers->tokens, sizeof(int), valid_batch_size, opt.trace);
            fwrite(trace_rows.data(), sizeof(float), trace_rows.size(), opt.trace);
        }

        for (int i = 0; i < valid_batch_size; i++) {  // :603-617
            const int b_idx = buffers->indices[i];
            pos[b_idx]++;
            if (pos[b_idx] < (int)prompt_tokens[b_idx].size()) {
                commit_generation(b_idx, prompt_tokens[b_idx][pos[b_idx]], false);
            } else {
                const float* logits = buffers->logits_h + (size_t)i * opt.vocab;
                int next_token = 0;  // greedy: first maximum
                for (int v = 1; v < opt.vocab; ++v)
                    if (logits[v] > logits[next_token]) next_token = v;
                commit_generation(b_idx, next_token, true);
            }
        }
        if (opt.trace) {
            std::vector<int> taken(valid_batch_size);
            for (int i = 0; i < valid_batch_size; i++) taken[i] = current_tokens[buffers->indices[i]];
            fwrite(taken.data(), sizeof(int), valid_batch_size, opt.trace);
        }
    }
    if (final_rows_h) {
        if (hipMemcpyAsync(final_rows_h, buffers->x_seq_d, sizeof(float) * (size_t)batch_size * H, hipMemcpyDeviceToHost,
                           stream) != hipSuccess ||
            hipStreamSynchronize(stream) != hipSuccess)
            return -(long long)hipGetLastError();
    }
    return total_tokens_out;
}

// All requests, batch_size at a time, by one worker (inference(), src/getp/run.cpp:661-736, whose
// OpenMP workers pull batches from a shared counter; one GPU, one worker here).
inline long long inference(moe_host::OssMoeTransformer* t_d, DecodeBuffers* buffers, Requests* requests, int steps,
                           const DecodeOptions& opt, std::vector<int>* step_sizes = nullptr,
                           float* final_rows_h = nullptr) {
    const int batch_size = t_d->config.batch_size;
    long long num_token_out = 0;
    std::vector<const char*> input_seqs(batch_size);
    std::vector<int*> output_tokens(batch_size);
    for (int start = 0; start < requests->num_reqs; start += batch_size) {
        const int n = requests->num_reqs - start < batch_size ? requests->num_reqs - start : batch_size;
        for (int i = 0; i < n; ++i) {
            input_seqs[i] = get_str_req_ptr(requests, start + i);
            output_tokens[i] = get_tok_gen_ptr(requests, start + i);
        }
        const long long got = generate(t_d, buffers, input_seqs.data(), output_tokens.data(), n, steps, opt, step_sizes,
                                       final_rows_h ? final_rows_h + (size_t)start * t_d->config.hidden_dim : nullptr);
        if (got < 0) return got;
        num_token_out += got;
    }
    return num_token_out;
}

}  // namespace moe_getp
