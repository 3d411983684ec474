// Expert GEMMs of the MoE block: y = W x + b per expert over its bucket of token rows, with the
// SwiGLU (gate/up launch) or the per-slot row store (down launch) in the epilogue.
// Replaces moe_mlp1_swiglu_mfma_kernel (src/hip/moe.hip:9-235) and moe_mlp2_scatter_mfma_kernel
// (src/hip/moe.hip:261-512); the arithmetic contract is the CPU path's (src/run.cpp:657-705).
//
// Common to all kernels here: every weight byte is loaded from HBM once per token block, straight
// into the MFMA A-operand registers with 128-bit loads (no LDS for weights: a weight element is
// used by one wave only); the bucket's activation rows are the B operand and are shared by the
// waves of a block through LDS, 128 contraction elements (one stage) at a time, one barrier per
// stage; fp32 accumulation in v_mfma_f32_16x16x32_bf16.  A wave owns R MFMA row tiles (16 R weight
// rows) over the whole contraction length and up to NT*16 tokens.
//
// The contraction index is a dummy index, so lanes are free to pick which k each of their eight
// operand elements stands for as long as A and B agree.  Inside a stage, k-step j (0..3) and lane
// group g = lane/16 take
//   bf16, uniform-wave kernel    : elements 32j + 8g .. +8
//   bf16, producer/consumer      : elements 64(j/2) + 16g + 8(j%2) .. +8  (a lane's two loads of a
//                                  pair of steps are adjacent: whole 128-byte lines per row)
//   MXFP4                        : elements 32g + 8j .. +8  (lane group g owns MX block g of the
//                                  stage: one 128-bit load + one scale byte per row tile and stage,
//                                  dequantised in registers to four A operands)
//
// Kernels: expert_stream_ws_kernel (decode-sized buckets, producer and consumer waves) and
// expert_prefill_kernel (128-token blocks, 64 x 128 tile per wave) are what the fused block uses;
// expert_stream_queue_kernel (uniform waves, fp32 activations staged through registers) serves the
// entries that keep the reference's signatures and work queue.
#include <type_traits>

#include "expert_tiles.h"

namespace moe {

namespace {


MOE_DEVICE u32x4 pack_f32x8_to_bf16x8(const float4& lo, const float4& hi) {
    return u32x4{pack_bf16x2(lo.x, lo.y), pack_bf16x2(lo.z, lo.w), pack_bf16x2(hi.x, hi.y), pack_bf16x2(hi.z, hi.w)};
}


// One (row unit, token block) of one expert.  ACT_F32: activations are fp32 rows indexed by slot
// (the reference's x_by_expert / gate_by_expert buffers) and are rounded to bf16 while staged.
// `active` is false for the waves of a ragged last block that own no rows: they still stage
// activations and take part in every barrier.
template <int FMT, int R, int NT, int EPI, bool ACT_F32, int WAVES, int NTMAX = kNTMax>
MOE_DEVICE void stream_body(const ExpertGemmArgs& a, uint8_t* lds, int e, int row0, int nrows, int unit,
                            bool active) {
    static_assert(WAVES == 4 || WAVES == 8, "a block has 4 or 8 waves");
    constexpr int kStagers = WAVES / 4;                       // waves that stage the same k-step
    constexpr int TS = (NT + kStagers - 1) / kStagers;        // token tiles staged per wave
    constexpr int kUnitsPerGroup = 4 / R;
    constexpr int kStageBytes = kStageSteps * NTMAX * 1024;  // one LDS stage buffer
    static_assert(NT <= NTMAX && TS * kStagers <= NTMAX, "token tiles must fit the LDS stage");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane & 15;
    const int g = lane >> 4;
    const int group = unit / kUnitsPerGroup;
    const int r0 = (unit % kUnitsPerGroup) * R;
    const int K = a.K;
    const int n_stages = ceil_div(K, kStageElems);

    // ---- A operand addressing ----
    const uint8_t* a_ptr[R];
    const uint8_t* s_ptr[R];
    if constexpr (FMT == FMT_BF16) {
        const uint16_t* wbase = reinterpret_cast<const uint16_t*>(a.w) + (size_t)e * a.w_expert_stride;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = active ? group * 64 + tile_row_in_group(r0 + r, q) : 0;
            a_ptr[r] = reinterpret_cast<const uint8_t*>(wbase + (size_t)row * K + 8 * g);
            s_ptr[r] = nullptr;
        }
    } else {
        const int G = K / 32;
        const size_t tile_bytes = (size_t)G * 256;
        const size_t stile_bytes = (size_t)ceil_div(ceil_div(G, 4), 4) * 256;
        const uint8_t* wbase = reinterpret_cast<const uint8_t*>(a.w) + (size_t)e * a.w_expert_stride;
        const uint8_t* sbase = a.w_scales + (size_t)e * a.s_expert_stride;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const size_t tile = active ? (size_t)group * 4 + (r0 + r) : 0;
            a_ptr[r] = wbase + tile * tile_bytes + (size_t)lane * 16;
            s_ptr[r] = sbase + tile * stile_bytes + (size_t)lane * 4;
        }
    }

    // ---- B staging: wave w stages k-step w%4 of every stage, for token tiles w/4, w/4 + WAVES/4, ...
    // (a tile index past NT-1 stages a clamped copy into an LDS slot nobody reads) ----
    const int step_w = wave & 3;
    const int half_w = wave >> 2;
    // element offset inside an activation row of this lane's eight elements at stage 0
    const int k_lane = (FMT == FMT_BF16) ? (32 * step_w + 8 * g) : (32 * g + 8 * step_w);
    const uint8_t* b_src[TS];
#pragma unroll
    for (int i = 0; i < TS; ++i) {
        const int t = half_w + kStagers * i;
        const int idx = min(t * 16 + q, nrows - 1);
        if constexpr (ACT_F32) {
            b_src[i] = reinterpret_cast<const uint8_t*>(a.act_f32 + (size_t)(row0 + idx) * K + k_lane);
        } else {
            const int src = a.gather ? a.tokens_flat[row0 + idx] : row0 + idx;
            b_src[i] = reinterpret_cast<const uint8_t*>(a.act + (size_t)src * K + k_lane);
        }
    }
    uint8_t* const lds_wr = lds + (size_t)(step_w * NTMAX + half_w) * 1024 + (size_t)lane * 16;
    const uint8_t* const lds_rd = lds + (size_t)lane * 16;

    // Everything inside the stage loops is branch-free (clamped addresses + selects instead of
    // guards), so the compiler can count outstanding loads exactly and keep the prefetches in flight.
    u32x4 stg[TS];
    auto stage_load = [&](int s) {
        // s may point past the last stage (prefetch of a stage that does not exist): stage zeros
        const bool live = (s * kStageElems + k_lane) < K;  // false in a ragged or non-existent stage
        const size_t off = live ? (size_t)s * kStageElems : 0;
#pragma unroll
        for (int t = 0; t < TS; ++t) {
            u32x4 v;
            if constexpr (ACT_F32) {
                const float4* p = reinterpret_cast<const float4*>(b_src[t] + off * 4 - (live ? 0 : k_lane * 4));
                v = pack_f32x8_to_bf16x8(p[0], p[1]);
            } else {
                v = *reinterpret_cast<const u32x4*>(b_src[t] + off * 2 - (live ? 0 : k_lane * 2));
            }
            stg[t] = live ? v : u32x4{0u, 0u, 0u, 0u};
        }
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int t = 0; t < TS; ++t)
            *reinterpret_cast<u32x4*>(lds_wr + (size_t)buf * kStageBytes + t * kStagers * 1024) = stg[t];
    };
    auto b_frag = [&](int buf, int j, int t) {
        return *reinterpret_cast<const u32x4*>(lds_rd + (size_t)buf * kStageBytes + (j * NTMAX + t) * 1024);
    };

    if (!active) {
        // no rows to compute: keep the block's staging and barrier sequence going
        const int n_iter = (FMT == FMT_BF16) ? n_stages : ceil_div(n_stages, 4) * 4;
        stage_load(0);
        stage_store(0);
        __syncthreads();
        for (int s = 0; s < n_iter; ++s) {
            stage_load(s + 1);
            stage_store((s & 1) ^ 1);
            __syncthreads();
        }
        return;
    }

    f32x4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    if constexpr (FMT == FMT_BF16) {
        // A ring of four k-steps, loads issued three steps ahead of their use
        const int n_steps = K / 32;
        const int n_full = K / kStageElems;  // stages with all four k-steps
        u32x4 ar[4][R];
        auto load_a = [&](int slot, int n) {
            const size_t off = (size_t)min(n, n_steps - 1) * 64;  // past the end: reload the last step
#pragma unroll
            for (int r = 0; r < R; ++r) ar[slot][r] = *reinterpret_cast<const u32x4*>(a_ptr[r] + off);
        };
        auto step = [&](int buf, int j) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const u32x4 b = b_frag(buf, j, t);
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r][t] = mfma_16x16x32(ar[j][r], b, acc[r][t]);
            }
        };
        stage_load(0);
        load_a(0, 0);
        load_a(1, 1);
        load_a(2, 2);
        stage_store(0);
        __syncthreads();
        for (int s = 0; s < n_full; ++s) {
            const int buf = s & 1;
            stage_load(s + 1);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                load_a((j + 3) & 3, 4 * s + j + 3);
                step(buf, j);
            }
            stage_store(buf ^ 1);
            __syncthreads();
        }
        if (n_full < n_stages) {  // ragged last stage: K % 128 in {32, 64, 96}
            const int buf = n_full & 1;
            const int left = n_steps - 4 * n_full;
            step(buf, 0);
            if (left > 1) step(buf, 1);
            if (left > 2) step(buf, 2);
            __syncthreads();
        }
    } else {
        // A ring of D stages (one 128-bit load per row tile and stage), loads issued D-1 stages ahead
        // of their use; one scale word per row tile covers four stages and is fetched one quad
        // ahead.  The stage count is padded to a multiple of four with all-zero stages (zero
        // weights against zero activations) to keep the loop uniform.
        constexpr int D = (R >= 4) ? 2 : 4;
        const int rem_groups = (K / 32) & 3;  // MX blocks in a ragged last stage (0 = none)
        const int n_quads = ceil_div(n_stages, 4);
        u32x4 araw[D][R];
        uint32_t sw_cur[R], sw_nxt[R];
        auto load_a = [&](int slot, int s) {
            const bool live = s < n_stages && !(rem_groups != 0 && s == n_stages - 1 && g >= rem_groups);
            // a dead lane group re-reads a block that exists and drops it
            const size_t off = live ? (size_t)s * 1024 : 0;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(a_ptr[r] + off);
                araw[slot][r] = live ? v : u32x4{0u, 0u, 0u, 0u};
            }
        };
        auto load_scales = [&](uint32_t (&dst)[R], int quad) {
            const size_t off = (size_t)min(quad, n_quads - 1) * 256;
#pragma unroll
            for (int r = 0; r < R; ++r) dst[r] = *reinterpret_cast<const uint32_t*>(s_ptr[r] + off);
        };
        auto do_stage = [&](int slot, int qpos, int s) {
            const int buf = s & 1;
            stage_load(s + 1);
            load_a((slot + D - 1) % D, s + D - 1);
            float sc[R];
#pragma unroll
            for (int r = 0; r < R; ++r) sc[r] = mxfp4_scale_to_f32((sw_cur[r] >> (8 * qpos)) & 0xFFu);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32x4 av[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    uint32_t d[4];
                    mxfp4_dword_to_bf16x8(araw[slot][r][j], sc[r], d);
                    av[r] = u32x4{d[0], d[1], d[2], d[3]};
                }
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const u32x4 b = b_frag(buf, j, t);
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[r][t] = mfma_16x16x32(av[r], b, acc[r][t]);
                }
            }
            stage_store(buf ^ 1);
            __syncthreads();
        };
        stage_load(0);
        load_scales(sw_cur, 0);
#pragma unroll
        for (int i = 0; i < D - 1; ++i) load_a(i, i);
        stage_store(0);
        __syncthreads();
        for (int qd = 0; qd < n_quads; ++qd) {
            load_scales(sw_nxt, qd + 1);
#pragma unroll
            for (int i = 0; i < 4; ++i) do_stage(i % D, i, 4 * qd + i);
#pragma unroll
            for (int r = 0; r < R; ++r) sw_cur[r] = sw_nxt[r];
        }
    }

    uint2 bias_raw[R];
    load_bias<R>(a, e, group, r0, bias_raw);
    stream_epilogue<R, NT, EPI>(a, acc, e, [&](int i) { return row0 + i; }, nrows, group, r0, bias_raw);
}

// ---------------------------------------------------------------------------------------------
// Producer/consumer variant used by the fused block: a block has CONS consumer waves (R = 2 row
// tiles each, 32 CONS weight rows per block) and two producer waves.  Producers move the bucket's
// activation rows global -> LDS with direct-to-LDS 128-bit loads (no registers, a ring of four
// 16 KiB stage slots, three stages ahead of the consumers); consumers only have weight loads in
// their memory queue.  One barrier per stage; every wave of the block executes exactly
// 1 + ceil(K / 128) barriers.
// Positions of the contraction range that do not exist (ragged last stage, padding stages) carry
// a weight operand of exact zeros; the activation operand there is a clamped re-read of real data.
// ---------------------------------------------------------------------------------------------


// The same load in assembly, the LDS address given as a wave-uniform integer (held in a scalar register
// by the caller), for a wave that issues these loads several stages ahead and also reads LDS fragments
// itself: the compiler puts a wait for every direct-to-LDS load it knows of in front of the wave's next
// LDS read, so a ring of such loads must be invisible to it.  The load does count in vmcnt; the caller
// waits for it itself.  Writes M0: a kernel that uses this must not use the builtin form as well.
MOE_DEVICE void dma16_asm(const void* gsrc, uint32_t lds_addr_uniform) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gsrc), "s"(lds_addr_uniform)
                 : "memory");
}


// act_row(i): row of a.act that holds bucket row i of the token block (i < nrows).
// The stages of the bucket's rows are streamed `passes` times over (once per pass of the consumers
// over their row units), without a break in between.
template <int FMT, int NT, int PROD, class RowFn>
MOE_DEVICE void ws_producer(const ExpertGemmArgs& a, uint8_t* lds, RowFn act_row, int nrows, int p, int passes) {
    constexpr int BP = 4 / PROD;  // four-row blocks of a token tile moved by this wave
    constexpr int Q = BP * NT;    // direct-to-LDS loads per stage issued by this wave
    const int lane = threadIdx.x & 63;
    const int pos = lane & 15;   // chunk position inside the row's LDS image
    const int sub = lane >> 4;   // row inside the instruction's block of four
    const int K = a.K;
    const int n_stages = ceil_div(K, kStageElems);
    // this wave moves row blocks BP*p .. BP*p + BP-1 of every token tile; in the bucket's last token
    // tile only those that hold a row of the bucket (n_last of them), and of those only the lanes whose row
    // exists.  The places of the rows past the bucket's end are cleared once, below, in every ring slot, and no
    // load ever writes them.  The accumulator columns they feed are never stored, so any value would do for
    // the result; zeros are what the matrix pipe spends least on (measured on a synthetic kernel of this shape:
    // a token tile of zeros costs a stage 0.0-0.1 us, a tile of arbitrary values 0.15-0.25 us, at the same
    // instruction count), and a bucket of 33 rows has 15 such columns in its third tile.
    int n_last = 0;
#pragma unroll
    for (int ii = 0; ii < BP; ++ii) n_last += (16 * (NT - 1) + 4 * (BP * p + ii) < nrows) ? 1 : 0;
    const uint8_t* row[NT][BP];
    int chunk[BP];
    bool last_live[BP];  // this lane's row of the last token tile exists
#pragma unroll
    for (int ii = 0; ii < BP; ++ii) {
        const int q = 4 * (BP * p + ii) + sub;
        chunk[ii] = ws_chunk_at<FMT>(pos ^ q);
        last_live[ii] = 16 * (NT - 1) + q < nrows;
        if (!last_live[ii]) {
#pragma unroll
            for (int slot = 0; slot < kWsRing; ++slot)
                *reinterpret_cast<u32x4*>(lds + (size_t)slot * kLdsStageBytes + (NT - 1) * 4096 + (BP * p + ii) * 1024 +
                                          lane * 16) = u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int idx = min(t * 16 + q, nrows - 1);
            row[t][ii] = reinterpret_cast<const uint8_t*>(a.act + (size_t)act_row(idx) * K);
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the clearing stores, before this wave's first barrier
    // stage st of the rows into ring slot gs % 4 (gs counts stages over all passes)
    auto issue = [&](int gs, int st) {
        uint8_t* slot = lds + (size_t)(gs & (kWsRing - 1)) * kLdsStageBytes;
#pragma unroll
        for (int ii = 0; ii < BP; ++ii) {
            const int k = st * kStageElems + 8 * chunk[ii];
            const size_t off = (k < K) ? (size_t)k * 2 : 0;  // a position past the row re-reads its start
#pragma unroll
            for (int t = 0; t < NT - 1; ++t) dma16(row[t][ii] + off, slot + t * 4096 + (BP * p + ii) * 1024);
            // the last tile: a block without a row is skipped (wave-uniform, the waits below count on it); in a block
            // with rows the lanes without one sit the instruction out (it is issued, and counted, all the same)
            if (ii < n_last && last_live[ii]) dma16(row[NT - 1][ii] + off, slot + (NT - 1) * 4096 + (BP * p + ii) * 1024);
        }
    };
    // stage s has landed once only the loads of the two stages issued after it are outstanding
    auto wait_two_stages = [&]() {
        static_assert(BP == 2, "three possible load counts per stage");
        if (n_last == 2) wait_vmcnt<2 * Q>();
        else if (n_last == 1) wait_vmcnt<2 * Q - 2>();
        else wait_vmcnt<2 * Q - 4>();
    };
    // Bare s_barrier, not __syncthreads(): the fence of __syncthreads() makes the compiler wait for
    // every outstanding direct-to-LDS load (vmcnt(0)) in front of each barrier, i.e. also for the
    // stages issued just now, and the ring would hide nothing.  The explicit wait above each barrier
    // is the guarantee the consumers need: the stage they read next has been written to LDS.
    int st = 0;  // stage (inside a pass) issued next
    auto next_stage = [&]() { st = (st + 1 == n_stages) ? 0 : st + 1; };
    for (int gs = 0; gs < 3; ++gs) {
        issue(gs, st);
        next_stage();
    }
    wait_two_stages();  // stage 0 has landed
    __builtin_amdgcn_s_barrier();
    const int total = passes * n_stages;
    for (int i = 0; i < total; ++i) {
        issue(i + 3, st);  // past the last stage of the last pass: a re-read nobody consumes
        next_stage();
        wait_two_stages();  // stage i+1 has landed
        __builtin_amdgcn_s_barrier();
    }
    wait_vmcnt<0>();  // nothing may still be writing this block's LDS when the wave ends
}

// slot_of_row(i): output row of bucket row i.  PRE: one more barrier comes first, right after the
// first weight loads have been issued (the kernel that finds the bucket itself completes the bucket
// list behind that barrier; the consumers need the list only in their epilogue, so their weights are
// already on the way while the producers read it).
// tile0: the first of the wave's R row tiles of 16 weight rows (R = 2: a row unit, tile0 even; R = 1: a single
// tile, for blocks whose range of tiles starts or ends inside a unit).
template <int FMT, int NT, int EPI, bool PRE = false, int R = 2, class SlotFn>
MOE_DEVICE void ws_consumer(const ExpertGemmArgs& a, const uint8_t* lds, int e, SlotFn slot_of_row, int nrows, int tile0,
                            bool active) {
    static_assert(R == 1 || R == 2, "one or two row tiles per wave");
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4;
    const int q = lane & 15;
    const int K = a.K;
    const int n_stages = ceil_div(K, kStageElems);
    if (!active) {
        for (int i = 0; i <= n_stages + (PRE ? 1 : 0); ++i) __syncthreads();
        return;
    }
    const int group = tile0 >> 2;
    const int r0 = tile0 & 3;
    uint2 bias_raw[R];  // fetched now, used by the epilogue
    load_bias<R>(a, e, group, r0, bias_raw);
    const uint8_t* const lds_rd = lds + (size_t)q * 256;
    auto b_frag = [&](int s, int j, int t) {
        return *reinterpret_cast<const u32x4*>(lds_rd + (size_t)(s & (kWsRing - 1)) * kLdsStageBytes + t * 4096 +
                                               ((ws_pos<FMT>(ws_chunk<FMT>(j, g)) ^ q) << 4));
    };
    f32x4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};

    if constexpr (FMT == FMT_BF16) {
        // The contraction range is walked in pairs of MFMA steps (64 elements = one 128-byte line of a
        // weight row).  A pair of a row tile is fetched by two instructions that each take WHOLE lines:
        // instruction i holds tile rows 8i .. 8i+7, its lane (g, q) the 16-byte chunk 2g + (q >> 3) of tile
        // row 8i + (q & 7).  Every line is then requested by one instruction only, which is what lets the
        // loads be non-temporal (a line shared by two instructions is fetched twice under that hint) and
        // takes the stream from the plain-load rate to the streaming rate of the memory system.  The MFMA
        // operand of step h wants lane (g, q) to hold chunk 2g + h of tile row q: lanes 8..15 of every
        // 16-lane row of instruction 0 and lanes 0..7 of instruction 1 trade places (row_ror:8 under a bank
        // mask, in the stage that consumes the pair).  Ring of four pairs, loads issued three pairs (one
        // and a half stages) ahead of their use; nothing touches a loaded value before that pair.
        constexpr int DP = 4;
        const int n_pairs = K / 64;
        // Buffer loads: the expert's matrix is the buffer, the wave-uniform part of an address (row tile, pair,
        // instruction) is the scalar offset and the lane's part a 32-bit register that never changes, so a load
        // costs no vector arithmetic (and a read past the matrix would return zeros instead of faulting).
        const uint16_t* wbase = reinterpret_cast<const uint16_t*>(a.w) + (size_t)e * a.w_expert_stride;
        const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t*>(wbase), 0, (int)((uint32_t)a.rows * (uint32_t)K * 2u), 0x00020000);
        uint32_t a_tile[R];  // wave-uniform byte offset of the row tile's first row
#pragma unroll
        for (int r = 0; r < R; ++r) a_tile[r] = (uint32_t)(group * 64 + tile_row_in_group(r0 + r, 0)) * (uint32_t)K * 2u;
        const uint32_t a_lane = (uint32_t)(tile_row_in_group(0, q & 7) * K + 8 * (2 * g + (q >> 3))) * 2u;
        const uint32_t second_half = 32u * (uint32_t)K * 2u;  // tile row q + 8 is weight row + 32 (tile_row_in_group)
        u32x4 ar[DP][2][R];
        auto load_a = [&](int slot, int pair) {
            const uint32_t off = (uint32_t)(pair < n_pairs ? pair : 0) * 128u;  // a padding pair re-reads pair 0 (unused)
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int r = 0; r < R; ++r)
                    ar[slot][i][r] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)a_lane,
                                                                           (int)(a_tile[r] + off + second_half * i), 2 /* nt */);
        };
#pragma unroll
        for (int i = 0; i < DP - 1; ++i) load_a(i, i);
        if constexpr (PRE) __syncthreads();
        __syncthreads();
        // one stage = two pairs; `ss` (stage parity) fixes the ring slots at compile time.  HALF: the ragged
        // last stage of a K that is an odd number of pairs runs its first pair only.
        auto stage = [&](auto ss_tag, auto half_tag, int st) {
            constexpr int ss = decltype(ss_tag)::value;
            constexpr bool HALF = decltype(half_tag)::value;
#pragma unroll
            for (int pp = 0; pp < (HALF ? 1 : 2); ++pp) {
                constexpr int kSlots = DP;
                const int u = 2 * ss + pp;  // ring slot of this pair
                const int pair = 2 * st + pp;
                load_a((u + kSlots - 1) % kSlots, pair + kSlots - 1);
                __builtin_amdgcn_sched_barrier(0);  // the loads are issued here, three pairs ahead of their use
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    u32x4 av[R];
#pragma unroll
                    for (int r = 0; r < R; ++r)
#pragma unroll
                        for (int d = 0; d < 4; ++d)
                            av[r][d] = h == 0 ? (uint32_t)__builtin_amdgcn_update_dpp((int)ar[u][0][r][d], (int)ar[u][1][r][d],
                                                                                      0x128, 0xF, 0xC, false)
                                              : (uint32_t)__builtin_amdgcn_update_dpp((int)ar[u][1][r][d], (int)ar[u][0][r][d],
                                                                                      0x128, 0xF, 0x3, false);
                    if constexpr (NT == 4) {
                        // four token tiles: one activation operand at a time, for both row tiles (the four of them
                        // held at once cost the registers that keep this loop free of spills; a spill access in
                        // here waits for every weight load in flight, since it counts in the same counter)
#pragma unroll
                        for (int t = 0; t < NT; ++t) {
                            const u32x4 b = b_frag(st, 2 * pp + h, t);
#pragma unroll
                            for (int r = 0; r < R; ++r) acc[r][t] = mfma_16x16x32(av[r], b, acc[r][t]);
                        }
                    } else {
                        u32x4 b[NT];
#pragma unroll
                        for (int t = 0; t < NT; ++t) b[t] = b_frag(st, 2 * pp + h, t);
#pragma unroll
                        for (int r = 0; r < R; ++r)
#pragma unroll
                            for (int t = 0; t < NT; ++t) acc[r][t] = mfma_16x16x32(av[r], b[t], acc[r][t]);
                    }
                }
            }
            __syncthreads();
        };
        const int full_stages = n_pairs >> 1;
        const int n_even = full_stages & ~1;
        for (int s0 = 0; s0 < n_even; s0 += 2) {
            stage(std::integral_constant<int, 0>{}, std::false_type{}, s0);
            stage(std::integral_constant<int, 1>{}, std::false_type{}, s0 + 1);
        }
        if (full_stages & 1) {
            stage(std::integral_constant<int, 0>{}, std::false_type{}, n_even);
            if (n_pairs & 1) stage(std::integral_constant<int, 1>{}, std::true_type{}, n_even + 1);
        } else if (n_pairs & 1) {
            stage(std::integral_constant<int, 0>{}, std::true_type{}, n_even);
        }
    } else {
        // Weights: a ring of four stages (one 128-bit load per row tile and stage, issued three
        // stages ahead of its use); scales: one word per row tile covers four stages and is
        // fetched one group of four ahead.  Addresses are a wave-uniform base (scalar registers)
        // plus a per-lane 32-bit offset that never changes, so a stage costs scalar arithmetic
        // only.  Nothing touches a loaded value before the stage that consumes it: an instruction
        // on it at load time would pin the wait for the load to the stage that issued it.
        constexpr int D = 4;
        const int G = K / 32;
        const uint32_t tile_bytes = (uint32_t)G * 256u;
        const uint32_t stile_bytes = (uint32_t)ceil_div(ceil_div(G, 4), 4) * 256u;
        // Buffer loads: the expert's tiled blocks (scales) are the buffer, the wave-uniform part of an address
        // (row tile, stage) is the scalar offset and the lane's part a constant register.  A read past the
        // buffer returns zeros instead of faulting, and a read past the tile inside it returns another tile's
        // bytes: both only ever happen in lanes or stages whose values are dropped (scale 0) or never used,
        // so no address needs a guard.
        const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t*>(reinterpret_cast<const uint8_t*>(a.w) + (size_t)e * a.w_expert_stride), 0,
            (int)a.w_expert_stride, 0x00020000);
        const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t*>(a.w_scales + (size_t)e * a.s_expert_stride), 0, (int)a.s_expert_stride, 0x00020000);
        uint32_t wtile[R], stile[R];  // wave-uniform byte offsets inside the expert
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t tile = (uint32_t)(group * 4 + (r0 + r));
            wtile[r] = tile * tile_bytes;
            stile[r] = tile * stile_bytes;
        }
        const int voff_w = lane * 16;
        const int voff_s = lane * 4;
        u32x4 araw[D][R];
        uint32_t sw_cur[R], sw_nxt[R];
        auto load_a = [&](int slot, int s) {  // s may lie past the last stage: padding that nobody consumes
#pragma unroll
            for (int r = 0; r < R; ++r)
                // non-temporal: a 1 KiB chunk is read once, by this instruction alone, so keeping its
                // lines in L1/L2 only evicts the activation rows (measured: -5 % kernel time; the prefill
                // kernel, where neighbouring token blocks re-read the weights, is slower with it)
                araw[slot][r] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, voff_w, (int)(wtile[r] + (uint32_t)s * 1024u),
                                                                      2 /* nt */);
        };
        auto load_scales = [&](uint32_t (&dst)[R], int quad) {
#pragma unroll
            for (int r = 0; r < R; ++r)
                dst[r] = __builtin_amdgcn_raw_buffer_load_b32(s_rsrc, voff_s, (int)(stile[r] + (uint32_t)quad * 256u), 0);
        };
        load_scales(sw_cur, 0);
#pragma unroll
        for (int i = 0; i < D - 1; ++i) load_a(i, i);
        if constexpr (PRE) __syncthreads();
        __syncthreads();
        // stage st, the i-th of its group of four (i fixes ring slot and scale byte at compile time)
        auto stage = [&](auto i_tag, int st) {
            constexpr int i = decltype(i_tag)::value;
            load_a((i + D - 1) % D, st + D - 1);
            __builtin_amdgcn_sched_barrier(0);  // the loads are issued here, three stages ahead of their use
            // In a ragged last stage the lane groups past the last MX block hold another tile's bytes (or zeros);
            // the tiled scale tensor has scale byte 0 in the slots of blocks that do not exist (moe_mxfp4_repack
            // clears the tensor before it scatters), which converts to a factor of exactly 0: no select needed.
            float sc[R];
#pragma unroll
            for (int r = 0; r < R; ++r) sc[r] = mxfp4_scale_to_f32((sw_cur[r] >> (8 * i)) & 0xFFu);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                u32x4 b[NT];
#pragma unroll
                for (int t = 0; t < NT; ++t) b[t] = b_frag(st, j, t);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    uint32_t d[4];
                    mxfp4_dword_to_bf16x8(araw[i][r][j], sc[r], d);
                    const u32x4 av = {d[0], d[1], d[2], d[3]};
#pragma unroll
                    for (int t = 0; t < NT; ++t) acc[r][t] = mfma_16x16x32(av, b[t], acc[r][t]);
                }
            }
            __syncthreads();
        };
        const int full_quads = n_stages / 4;
        for (int qd = 0; qd < full_quads; ++qd) {
            load_scales(sw_nxt, qd + 1);
            stage(std::integral_constant<int, 0>{}, 4 * qd + 0);
            stage(std::integral_constant<int, 1>{}, 4 * qd + 1);
            stage(std::integral_constant<int, 2>{}, 4 * qd + 2);
            stage(std::integral_constant<int, 3>{}, 4 * qd + 3);
#pragma unroll
            for (int r = 0; r < R; ++r) sw_cur[r] = sw_nxt[r];
        }
        // the last, partial group of four (wave-uniform conditions; its weights are already in the ring)
        const int tail = n_stages - 4 * full_quads;
        if (tail > 0) stage(std::integral_constant<int, 0>{}, 4 * full_quads + 0);
        if (tail > 1) stage(std::integral_constant<int, 1>{}, 4 * full_quads + 1);
        if (tail > 2) stage(std::integral_constant<int, 2>{}, 4 * full_quads + 2);
    }
    stream_epilogue<R, NT, EPI>(a, acc, e, slot_of_row, nrows, group, r0, bias_raw);
}

// ws_consumer for blocks that cover up to 2 CONS row units.
// The wave takes row units unit0 and, with two passes, unit0 + unit_step (each if < unit_end), one per
// pass over the bucket's activation stages (which the producers stream `passes` <= 2 times); in a pass
// without a unit of its own it only takes part in the barriers.  The weight ring runs on across passes: the loads that the last
// stages of a pass issue are the first stages of the next pass's unit, so only the first pass of a
// block starts from an empty pipeline, and a pass's epilogue runs while those loads are in flight.
// Kept apart from ws_consumer: the second pass's code costs registers even when it does not run, so
// blocks that make one pass use the single-pass function.
template <int FMT, int NT, int EPI, bool PRE = false, class SlotFn>
MOE_DEVICE void ws_consumer_two(const ExpertGemmArgs& a, const uint8_t* lds, int e, SlotFn slot_of_row, int nrows, int unit0,
                            int unit_end, int unit_step, int passes) {
    constexpr int R = 2;
    constexpr bool TWO = true;
    const int lane = threadIdx.x & 63;
    const int g = lane >> 4;
    const int q = lane & 15;
    const int K = a.K;
    const int n_stages = ceil_div(K, kStageElems);
    if (unit0 >= unit_end) {  // no unit at all: barriers only
        for (int i = 0; i < 1 + (PRE ? 1 : 0) + passes * n_stages; ++i) __syncthreads();
        return;
    }
    const uint8_t* const lds_rd = lds + (size_t)q * 256;
    // gs: stage counted over all passes (the producers' ring slot)
    auto b_frag = [&](int gs, int j, int t) {
        return *reinterpret_cast<const u32x4*>(lds_rd + (size_t)(gs & (kWsRing - 1)) * kLdsStageBytes + t * 4096 +
                                               ((ws_pos<FMT>(ws_chunk<FMT>(j, g)) ^ q) << 4));
    };
    f32x4 acc[R][NT];
    uint2 bias_raw[R];

    // MXFP4 only: the bf16 stage loops have no registers to spare for a second pass's addresses at 128 registers a
    // lane (built and measured: 390 spilled registers, gate/up launch 206 against 190 us), so bf16 blocks make one pass.
    static_assert(FMT == FMT_MXFP4, "two-pass blocks exist for MXFP4 weights only");
    {
        // Weights: a ring of four stages (one 128-bit load per row tile and stage, issued three
        // stages ahead of its use); scales: one word per row tile covers four stages and is
        // fetched one group of four ahead.  Addresses are a wave-uniform base (scalar registers)
        // plus a per-lane 32-bit offset that never changes, so a stage costs scalar arithmetic
        // only.  Nothing touches a loaded value before the stage that consumes it: an instruction
        // on it at load time would pin the wait for the load to the stage that issued it.
        // Stage numbers at or past n_pad (the stage count rounded up to whole groups of four) mean the
        // next pass's unit; those in between are never used and re-read stage 0 with scale 0.
        constexpr int D = 4;
        const int G = K / 32;
        const uint32_t tile_bytes = (uint32_t)G * 256u;
        const uint32_t stile_bytes = (uint32_t)ceil_div(ceil_div(G, 4), 4) * 256u;
        // Buffer loads: the expert's tiled blocks (scales) are the buffer, the wave-uniform part of an address
        // (row tile, stage) is the scalar offset and the lane's part a constant register.  A read past the
        // buffer returns zeros instead of faulting, and a read past the tile inside it returns another tile's
        // bytes: both only ever happen in lanes or stages whose values are dropped (scale 0) or never used,
        // so no address needs a guard.
        const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t*>(reinterpret_cast<const uint8_t*>(a.w) + (size_t)e * a.w_expert_stride), 0,
            (int)a.w_expert_stride, 0x00020000);
        const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint8_t*>(a.w_scales + (size_t)e * a.s_expert_stride), 0, (int)a.s_expert_stride, 0x00020000);
        uint32_t wtile[R], stile[R], wnext[R], snext[R];  // wave-uniform byte offsets inside the expert
        const int voff_w = lane * 16;
        const int voff_s = lane * 4;
        const int n_quads = ceil_div(n_stages, 4);
        const int n_pad = 4 * n_quads;
        u32x4 araw[D][R];
        uint32_t sw_cur[R], sw_nxt[R];
        // stage s of the current pass, or (s >= n_pad) stage s - n_pad of the next pass's unit; a stage number in
        // between is padding that nobody consumes
        auto load_a = [&](int slot, int s) {
            const bool nxt = TWO && s >= n_pad;  // wave-uniform
            const uint32_t so = (uint32_t)(nxt ? s - n_pad : s) * 1024u;
#pragma unroll
            for (int r = 0; r < R; ++r)
                // non-temporal: a 1 KiB chunk is read once, by this instruction alone, so keeping its
                // lines in L1/L2 only evicts the activation rows (measured: -5 % kernel time; the prefill
                // kernel, where neighbouring token blocks re-read the weights, is slower with it)
                araw[slot][r] = __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, voff_w, (int)((nxt ? wnext[r] : wtile[r]) + so),
                                                                      2 /* nt */);
        };
        auto load_scales = [&](uint32_t (&dst)[R], int quad) {  // quad n_quads = the next pass's first
            const bool nxt = TWO && quad >= n_quads;
#pragma unroll
            for (int r = 0; r < R; ++r)
                dst[r] = __builtin_amdgcn_raw_buffer_load_b32(
                    s_rsrc, voff_s, (int)(nxt ? snext[r] : stile[r] + (uint32_t)quad * 256u), 0);
        };
        // one pass; written out once per pass instead of looped (see the bf16 branch)
        auto do_pass = [&](auto first_tag, int unit, bool more, int gs0) {
            constexpr bool first = decltype(first_tag)::value;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t tile = (uint32_t)((unit >> 1) * 4 + ((unit & 1) * R + r));
                const uint32_t tile_n = more ? (uint32_t)(((unit + unit_step) >> 1) * 4 + (((unit + unit_step) & 1) * R + r)) : tile;
                wtile[r] = tile * tile_bytes;
                stile[r] = tile * stile_bytes;
                if constexpr (TWO) {
                    wnext[r] = tile_n * tile_bytes;
                    snext[r] = tile_n * stile_bytes;
                }
            }
            load_bias<R>(a, e, unit >> 1, (unit & 1) * R, bias_raw);  // fetched now, used by the epilogue
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int t = 0; t < NT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
            if constexpr (first) {
                load_scales(sw_cur, 0);
#pragma unroll
                for (int i = 0; i < D - 1; ++i) load_a(i, i);
                if constexpr (PRE) __syncthreads();
                __syncthreads();
            }
            // stage st, the i-th of its group of four (i fixes ring slot and scale byte at compile time)
            // In a ragged last stage the lane groups past the last MX block hold another tile's bytes (or zeros); the
            // tiled scale tensor has scale byte 0 in the slots of blocks that do not exist (moe_mxfp4_repack clears
            // the tensor before it scatters), which converts to a factor of exactly 0, so their products vanish
            // without a select.
            auto stage = [&](auto i_tag, int st) {
                constexpr int i = decltype(i_tag)::value;
                load_a((i + D - 1) % D, st + D - 1);
                __builtin_amdgcn_sched_barrier(0);  // the loads are issued here, three stages ahead of their use
                float sc[R];
#pragma unroll
                for (int r = 0; r < R; ++r) sc[r] = mxfp4_scale_to_f32((sw_cur[r] >> (8 * i)) & 0xFFu);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    u32x4 b[NT];
#pragma unroll
                    for (int t = 0; t < NT; ++t) b[t] = b_frag(gs0 + st, j, t);
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        uint32_t d[4];
                        mxfp4_dword_to_bf16x8(araw[i][r][j], sc[r], d);
                        const u32x4 av = {d[0], d[1], d[2], d[3]};
#pragma unroll
                        for (int t = 0; t < NT; ++t) acc[r][t] = mfma_16x16x32(av, b[t], acc[r][t]);
                    }
                }
                __syncthreads();
            };
            const int full_quads = n_stages / 4;
            for (int qd = 0; qd < full_quads; ++qd) {
                load_scales(sw_nxt, qd + 1);
                stage(std::integral_constant<int, 0>{}, 4 * qd + 0);
                stage(std::integral_constant<int, 1>{}, 4 * qd + 1);
                stage(std::integral_constant<int, 2>{}, 4 * qd + 2);
                stage(std::integral_constant<int, 3>{}, 4 * qd + 3);
#pragma unroll
                for (int r = 0; r < R; ++r) sw_cur[r] = sw_nxt[r];
            }
            // the last, partial group of four (wave-uniform conditions; its weights are already in the
            // ring); the stages it lacks still issue their loads, which belong to the next pass
            const int tail = n_stages - 4 * full_quads;
            if constexpr (TWO) {
                if (tail > 0) {
                    load_scales(sw_nxt, n_quads);
                    stage(std::integral_constant<int, 0>{}, 4 * full_quads + 0);
                    if (tail > 1) stage(std::integral_constant<int, 1>{}, 4 * full_quads + 1);
                    else load_a(0, 4 * full_quads + 4);
                    if (tail > 2) stage(std::integral_constant<int, 2>{}, 4 * full_quads + 2);
                    else load_a(1, 4 * full_quads + 5);
                    load_a(2, 4 * full_quads + 6);
#pragma unroll
                    for (int r = 0; r < R; ++r) sw_cur[r] = sw_nxt[r];
                }
            } else {
                if (tail > 0) stage(std::integral_constant<int, 0>{}, 4 * full_quads + 0);
                if (tail > 1) stage(std::integral_constant<int, 1>{}, 4 * full_quads + 1);
                if (tail > 2) stage(std::integral_constant<int, 2>{}, 4 * full_quads + 2);
            }
            stream_epilogue<R, NT, EPI>(a, acc, e, slot_of_row, nrows, unit >> 1, (unit & 1) * R, bias_raw);
        };
        if constexpr (TWO) {
            const int unit1 = unit0 + unit_step;
            do_pass(std::true_type{}, unit0, passes > 1 && unit1 < unit_end, 0);
            if (passes > 1) {
                if (unit1 < unit_end) do_pass(std::false_type{}, unit1, false, n_stages);
                else for (int i = 0; i < n_stages; ++i) __syncthreads();  // wave-uniform: no unit left for this wave
            }
        } else {
            do_pass(std::true_type{}, unit0, false, 0);
        }
    }
}

template <int FMT, int NT, int EPI, bool PRE, bool TWO, class SlotFn>
MOE_DEVICE void ws_consume_units(const ExpertGemmArgs& a, const uint8_t* lds, int e, SlotFn slot_of_row, int nrows,
                                 int unit0, int unit_end, int unit_step, int passes) {
    if constexpr (TWO) ws_consumer_two<FMT, NT, EPI, PRE>(a, lds, e, slot_of_row, nrows, unit0, unit_end, unit_step, passes);
    else ws_consumer<FMT, NT, EPI, PRE>(a, lds, e, slot_of_row, nrows, 2 * unit0, unit0 < unit_end);
}

// The same for a block whose rows are a range of row TILES [t0, t1) that need not start or end on a unit: a
// tile in front of the first whole unit goes to wave 0 and one behind the last whole unit to the wave after the
// last whole unit, each as a single tile; the launch sees to it that CONS waves are enough.
template <int FMT, int NT, int EPI, bool PRE, class SlotFn>
MOE_DEVICE void ws_consume_tiles(const ExpertGemmArgs& a, const uint8_t* lds, int e, SlotFn slot_of_row, int nrows,
                                 int t0, int t1, int wave) {
    const int lead = (t0 & 1) && t0 < t1;  // an empty range has no waves at work
    const int first = (wave == 0 || !lead) ? t0 + 2 * wave : t0 + 2 * wave - 1;  // wave-uniform
    if (lead && wave == 0) {
        ws_consumer<FMT, NT, EPI, PRE, 1>(a, lds, e, slot_of_row, nrows, t0, true);
    } else if (first + 1 == t1) {
        ws_consumer<FMT, NT, EPI, PRE, 1>(a, lds, e, slot_of_row, nrows, first, true);
    } else {
        ws_consumer<FMT, NT, EPI, PRE, 2>(a, lds, e, slot_of_row, nrows, first, first + 1 < t1);
    }
}

// One token block: the producer or consumer role of this wave, for the block's token-tile count.
// u0, u1: the block's row units [u0, u1), walked in passes of CONS units; with TILES its row tiles [u0, u1)
// (one pass, see ws_consume_tiles).
template <int FMT, int EPI, int CONS, int PROD, bool PRE = false, bool TWO = false, bool TILES = false, class RowFn,
          class SlotFn>
MOE_DEVICE void ws_token_block(const ExpertGemmArgs& a, uint8_t* lds, int wave, int u0, int u1, int e, RowFn act_row,
                               SlotFn slot_of_row, int nrows) {
    const int nt = (nrows + 15) >> 4;  // block-uniform
    const int passes = TWO ? min(2, max(1, ceil_div(u1 - u0, CONS))) : 1;
    if (wave >= CONS) {
        const int p = wave - CONS;
        if constexpr (PRE) __syncthreads();  // no direct-to-LDS load is in flight yet
        if (nt == 4) ws_producer<FMT, 4, PROD>(a, lds, act_row, nrows, p, passes);
        else if (nt == 3) ws_producer<FMT, 3, PROD>(a, lds, act_row, nrows, p, passes);
        else if (nt == 2) ws_producer<FMT, 2, PROD>(a, lds, act_row, nrows, p, passes);
        else ws_producer<FMT, 1, PROD>(a, lds, act_row, nrows, p, passes);
    } else if constexpr (TILES) {
        static_assert(!TWO, "a range of tiles is walked in one pass");
        if (nt == 4) ws_consume_tiles<FMT, 4, EPI, PRE>(a, lds, e, slot_of_row, nrows, u0, u1, wave);
        else if (nt == 3) ws_consume_tiles<FMT, 3, EPI, PRE>(a, lds, e, slot_of_row, nrows, u0, u1, wave);
        else if (nt == 2) ws_consume_tiles<FMT, 2, EPI, PRE>(a, lds, e, slot_of_row, nrows, u0, u1, wave);
        else ws_consume_tiles<FMT, 1, EPI, PRE>(a, lds, e, slot_of_row, nrows, u0, u1, wave);
    } else {
        if (nt == 4) ws_consume_units<FMT, 4, EPI, PRE, TWO>(a, lds, e, slot_of_row, nrows, u0 + wave, u1, CONS, passes);
        else if (nt == 3) ws_consume_units<FMT, 3, EPI, PRE, TWO>(a, lds, e, slot_of_row, nrows, u0 + wave, u1, CONS, passes);
        else if (nt == 2) ws_consume_units<FMT, 2, EPI, PRE, TWO>(a, lds, e, slot_of_row, nrows, u0 + wave, u1, CONS, passes);
        else ws_consume_units<FMT, 1, EPI, PRE, TWO>(a, lds, e, slot_of_row, nrows, u0 + wave, u1, CONS, passes);
    }
}

// Linear block index -> (token block or expert, row block).  Workgroups go to the eight XCDs
// round-robin by linear index; with xcd_tiles all row blocks of an item run on one XCD (its
// activations enter one L2 once), otherwise they are spread over all of them.
MOE_DEVICE void ws_block_coords(const ExpertGemmArgs& a, int& item, int& rb) {
    const int n_rb = a.row_blocks;
    item = a.xcd_tiles ? ((blockIdx.x >> 3) / n_rb) * 8 + (blockIdx.x & 7) : blockIdx.x / n_rb;
    rb = a.xcd_tiles ? (blockIdx.x >> 3) % n_rb : blockIdx.x % n_rb;
}

// the row units of the weight matrix are spread evenly over the row blocks (sizes differ by at most one unit):
// block rb takes [u0, u1)
MOE_DEVICE void ws_row_units(const ExpertGemmArgs& a, int rb, int& u0, int& u1) {
    const int units = a.rows / 32;
    // the blocks with one unit more come first in the launch order: when the blocks take more than one round
    // over the compute units, the second-round blocks are handed out in that order to the units as they finish,
    // so a unit whose first block was a long one ends with a short one (measured: bf16 gate/up launch at 256
    // tokens, 512 blocks of 11 or 12 units, -3 %)
    const int q = units / a.row_blocks, rem = units - q * a.row_blocks;
    u0 = rb * q + min(rb, rem);
    u1 = u0 + q + (rb < rem ? 1 : 0);
}

// The same split in row tiles of 16 rows (two per unit), for blocks that make one pass: block sizes then differ
// by half a unit at most.  A block whose range starts or ends inside a unit needs a wave for each of those single
// tiles, so this split is only used while a block stays below 2 CONS tiles; otherwise the unit split, in tiles.
template <int CONS>
MOE_DEVICE void ws_row_tiles(const ExpertGemmArgs& a, int rb, int& t0, int& t1) {
    const int tiles = a.rows / 16;
    const int q = tiles / a.row_blocks, rem = tiles - q * a.row_blocks;
    if (q + (rem ? 1 : 0) <= 2 * CONS - 1) {
        t0 = rb * q + min(rb, rem);
        t1 = t0 + q + (rb < rem ? 1 : 0);
    } else {
        ws_row_units(a, rb, t0, t1);
        t0 *= 2;
        t1 *= 2;
    }
}

// Token blocks from the tile map written by the bucketing kernel.
// grid = row blocks x token blocks (padded to a multiple of 8), block = 64 (CONS + PROD); one block per CU: twelve
// waves leave 168 registers per lane, fourteen leave 128.
template <int FMT, int EPI, int CONS, int PROD>
__global__ __launch_bounds__((CONS + PROD) * 64, (CONS + PROD > 12) ? 4 : 3) void expert_stream_ws_kernel(ExpertGemmArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[kWsRing * kLdsStageBytes];
    int tile, rb;
    ws_block_coords(a, tile, rb);
    if (tile >= *a.n_tiles) return;  // block-uniform
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int e = a.tile_expert[tile];
    const int row0 = a.tile_row0[tile];
    const int nrows = a.tile_rows[tile];
    int u0, u1;
    ws_row_units(a, rb, u0, u1);
    ws_token_block<FMT, EPI, CONS, PROD>(
        a, lds, wave, u0, u1, e, [&](int i) { return a.gather ? a.tokens_flat[row0 + i] : row0 + i; },
        [&](int i) { return row0 + i; }, nrows);
}

// ---------------------------------------------------------------------------------------------
// The same expert GEMM without a bucketing launch in front of it, for batches of at most
// kDirectMaxAssign assignments (tokens x experts per token).  A block is one (expert, row block)
// pair, known from the block index alone, and finds the expert's bucket itself: every wave compares
// chunks of 64 consecutive assignments of topk_i with the expert id, the per-chunk match counts go
// through LDS, one wave-wide prefix sum gives every chunk its offset, and the matching assignment
// ids (token * experts_per_token + k, ascending: the bucket order of bucket_kernel) land in an LDS
// list.  The block then runs the bucket's token blocks of up to 64 rows one after the other.
// Rows are addressed by assignment id: the activation row of assignment s is s / assign_div (gate/up
// launch: the token's row) or s itself (down launch), and the output row is s.
// grid = row blocks x experts (padded to a multiple of 8), block = 64 (CONS + PROD).
// ---------------------------------------------------------------------------------------------
constexpr int kDirectMaxAssign = 4096;  // 64 chunks of 64: one lane per chunk in the prefix sum
constexpr int kDirectMaxRows = 2048;    // longest bucket the LDS list holds

// TWO: blocks cover up to 2 CONS row units, in two passes over the bucket's activations.
template <int FMT, int EPI, int CONS, int PROD, bool TWO>
__global__ __launch_bounds__((CONS + PROD) * 64, (CONS + PROD > 12) ? 4 : 3) void expert_stream_direct_kernel(ExpertGemmArgs a) {
    constexpr int WAVES = CONS + PROD;
    constexpr int P = (64 + WAVES - 1) / WAVES;  // chunks per wave
    __shared__ __attribute__((aligned(16))) uint8_t lds[kWsRing * kLdsStageBytes];
    __shared__ int bucket[kDirectMaxRows];
    __shared__ int chunk_cnt[64];
    int e, rb;
    ws_block_coords(a, e, rb);
    if (e >= a.n_experts) return;  // block-uniform (grid padding)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_chunks = (a.n_assign + 63) >> 6;
    // bf16 blocks make one pass over their rows and take them as a range of row tiles; MXFP4 blocks make up to two
    // passes of CONS units each, whose time does not depend on how many units a pass holds
    constexpr bool TILES = !TWO && FMT == FMT_BF16;
    int u0, u1;
    if constexpr (TILES) ws_row_tiles<CONS>(a, rb, u0, u1);
    else ws_row_units(a, rb, u0, u1);
    int n_bucket;
    {
        // this wave's chunks of the assignment list
        int ids[P];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int s = (p * WAVES + wave) * 64 + lane;
            ids[p] = s < a.n_assign ? a.topk_i[s] : -1;
        }
        unsigned long long match[P];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int c = p * WAVES + wave;
            match[p] = __ballot(ids[p] == e);
            if (lane == 0 && c < n_chunks) chunk_cnt[c] = __popcll(match[p]);
        }
        __syncthreads();
        // inclusive prefix sum of the chunk counts over the wave's lanes
        uint32_t incl = lane < n_chunks ? (uint32_t)chunk_cnt[lane] : 0u;
#define MOE_STEP(C, M) incl += dpp_move<C, M>(0u, incl);
        MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
        n_bucket = min((int)__builtin_amdgcn_readlane(incl, 63), kDirectMaxRows);
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const int c = p * WAVES + wave;
            if (c < n_chunks) {  // wave-uniform
                const int base = (int)__builtin_amdgcn_readlane(incl, c) - __popcll(match[p]);
                const int dst = base + __popcll(match[p] & ((1ull << lane) - 1ull));
                if (ids[p] == e && dst < kDirectMaxRows) bucket[dst] = c * 64 + lane;
            }
        }
        // the barrier that completes the list is the first one of the token block below
    }
    if (n_bucket == 0) return;
    // token of assignment s = s / assign_div, as a float multiplication (exact for s < 4096, assign_div <= 8)
    const float inv_div = 1.0f / (float)a.assign_div;
    auto token_of = [&](int s) { return (int)(((float)s + 0.5f) * inv_div); };
    // The first token block takes the bucket's remainder (1..64 rows, any tile count) in straight-line
    // code; what is left are whole blocks of 64 rows, run by a loop that holds the four-tile variant
    // only (a loop around all tile-count variants costs every variant 30 registers per lane).
    const int first = n_bucket - ((n_bucket - 1) & ~63);
    ws_token_block<FMT, EPI, CONS, PROD, true, TWO, TILES>(
        a, lds, wave, u0, u1, e, [&](int i) { return a.gather ? token_of(bucket[i]) : bucket[i]; },
        [&](int i) { return bucket[i]; }, first);
    const int passes = TWO ? min(2, max(1, ceil_div(u1 - u0, CONS))) : 1;
    for (int row0 = first; row0 < n_bucket; row0 += 64) {
        auto act_row = [&](int i) { return a.gather ? token_of(bucket[row0 + i]) : bucket[row0 + i]; };
        auto slot_of_row = [&](int i) { return bucket[row0 + i]; };
        if (wave >= CONS) ws_producer<FMT, 4, PROD>(a, lds, act_row, 64, wave - CONS, passes);
        else if constexpr (TILES) ws_consume_tiles<FMT, 4, EPI, false>(a, lds, e, slot_of_row, 64, u0, u1, wave);
        else ws_consume_units<FMT, 4, EPI, false, TWO>(a, lds, e, slot_of_row, 64, u0 + wave, u1, CONS, passes);
    }
}

template <int FMT, int R, int EPI, bool ACT_F32, int WAVES>
MOE_DEVICE void stream_dispatch(const ExpertGemmArgs& a, uint8_t* lds, int e, int row0, int nrows, int unit,
                                bool active) {
    const int nt = (nrows + 15) >> 4;  // block-uniform
    if (nt == 4) {
        stream_body<FMT, R, 4, EPI, ACT_F32, WAVES>(a, lds, e, row0, nrows, unit, active);
    } else if (nt == 3) {
        stream_body<FMT, R, 3, EPI, ACT_F32, WAVES>(a, lds, e, row0, nrows, unit, active);
    } else if (nt == 2) {
        stream_body<FMT, R, 2, EPI, ACT_F32, WAVES>(a, lds, e, row0, nrows, unit, active);
    } else if (nt == 1) {
        stream_body<FMT, R, 1, EPI, ACT_F32, WAVES>(a, lds, e, row0, nrows, unit, active);
    }
}

// Token blocks from a queue of (expert, row_offset, row_count) triples (entry format of
// src/hip/scheduler.hip:163-166).  grid = (ceil(row units / 4), token blocks per entry, entries).
template <int FMT, int R, int EPI>
__global__ __launch_bounds__(256) void expert_stream_queue_kernel(ExpertGemmArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kLdsStageBytes];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = blockIdx.x * 4 + wave;
    const bool active = unit < (a.rows / 64) * (4 / R);
    const int* entry = a.work_queue + 3 * (a.work_start + blockIdx.z);
    const int e = entry[0], off = entry[1], n = entry[2];
    for (int tb = blockIdx.y; tb * 64 < n; tb += gridDim.y) {
        stream_dispatch<FMT, R, EPI, true, 4>(a, lds, e, off + tb * 64, min(64, n - tb * 64), unit, active);
        __syncthreads();  // the next token block restages both LDS buffers
    }
}

// ---------------------------------------------------------------------------------------------
// Prefill-sized buckets: a 64-row x 128-token tile per wave (R = 4 row tiles, up to 8 token tiles),
// so a weight operand — for MXFP4 dequantised once in registers — feeds eight MFMAs, and the LDS
// holds the 128-token activation stage (2 x 32 KiB).  MXFP4 weights: activations are moved
// global -> LDS by direct-to-LDS loads issued one stage ahead by all eight waves (no staging
// registers), weights are fetched one stage ahead into registers.  bf16 weights reuse
// stream_body with the same tile.
// grid = (ceil(rows / (64 WAVES)), max_tiles), token blocks of up to 128 rows.
// ---------------------------------------------------------------------------------------------
template <int NT, int EPI, int WAVES>
MOE_DEVICE void prefill_body_mxfp4(const ExpertGemmArgs& a, uint8_t* lds, int e, int row0, int nrows, int unit,
                                   bool active) {
    constexpr int R = 4;
    constexpr int NTMAX = 8;
    constexpr int kStageBytes = kStageSteps * NTMAX * 1024;
    constexpr int kStagers = WAVES / 4;                 // waves that stage the same k-step
    constexpr int TS = (NT + kStagers - 1) / kStagers;  // token tiles staged per wave
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane & 15;
    const int g = lane >> 4;
    const int K = a.K;
    const int G = K / 32;
    const int n_stages = ceil_div(K, kStageElems);
    const int n_quads = ceil_div(n_stages, 4);
    const int rem_groups = G & 3;

    // activation staging, LDS image as in the producer/consumer kernel (token tile t at t*4096, row
    // q at q*256, 16-byte chunk c at position c ^ q): this wave moves the four-row block wave%4
    // (256 contiguous bytes per row, whole cache lines) of token tiles wave/4, wave/4 + WAVES/4, ...
    const int blk_w = wave & 3;
    const int half_w = wave >> 2;
    const int q_dma = 4 * blk_w + (lane >> 4);     // row of the token tile this lane moves
    const int chunk_dma = ws_chunk_at<FMT_MXFP4>((lane & 15) ^ q_dma);  // chunk of the stage it fetches
    const uint8_t* b_row[TS];
#pragma unroll
    for (int i = 0; i < TS; ++i) {
        const int idx = min((half_w + kStagers * i) * 16 + q_dma, nrows - 1);
        const int src = a.gather ? a.tokens_flat[row0 + idx] : row0 + idx;
        b_row[i] = reinterpret_cast<const uint8_t*>(a.act + (size_t)src * K);
    }
    auto issue_b = [&](int s) {
        const int k = s * kStageElems + 8 * chunk_dma;
        const size_t off = (k < K) ? (size_t)k * 2 : 0;  // past the row: re-read its start (weights are 0 there)
        uint8_t* dst = lds + (size_t)(s & 1) * kStageBytes + (size_t)half_w * 4096 + blk_w * 1024;
#pragma unroll
        for (int i = 0; i < TS; ++i) dma16(b_row[i] + off, dst + i * kStagers * 4096);
    };
    const uint8_t* const lds_rd = lds + (size_t)q * 256;
    auto b_frag = [&](int s, int j, int t) {  // lane group g owns MX block g of a stage: chunk 4g + j
        return *reinterpret_cast<const u32x4*>(lds_rd + (size_t)(s & 1) * kStageBytes + t * 4096 +
                                               ((ws_pos<FMT_MXFP4>(4 * g + j) ^ q) << 4));
    };

    if (!active) {
        issue_b(0);
        wait_vmcnt<0>();
        __syncthreads();
        for (int s = 0; s < n_stages; ++s) {
            issue_b(s + 1);
            wait_vmcnt<0>();
            __syncthreads();
        }
        return;
    }

    const size_t tile_bytes = (size_t)G * 256;
    const size_t stile_bytes = (size_t)ceil_div(ceil_div(G, 4), 4) * 256;
    // wave-uniform bases (scalar registers) + per-lane 32-bit offsets that never change
    const uint8_t* const a_base = reinterpret_cast<const uint8_t*>(a.w) + (size_t)e * a.w_expert_stride +
                                  (size_t)unit * 4 * tile_bytes;
    const uint8_t* const s_base = a.w_scales + (size_t)e * a.s_expert_stride + (size_t)unit * 4 * stile_bytes;
    const uint32_t voff_w = (uint32_t)lane * 16;
    // ragged last stage: a lane group past the last MX block re-reads block 0 and gets scale 0
    const uint32_t voff_w_ragged = (uint32_t)((g < rem_groups ? lane : q) * 16);
    const uint32_t voff_s = (uint32_t)lane * 4;
    f32x4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    u32x4 araw[2][R];
    uint32_t sw_cur[R], sw_nxt[R];
    // Nothing touches a loaded weight before the stage that consumes it (an instruction on it at
    // load time would make the wave wait for the load right there): a stage or MX block that does
    // not exist re-reads one that does and is multiplied by scale 0.
    auto load_a = [&](int slot, int s) {
        const int su = s < n_stages ? s : 0;
        const bool ragged = rem_groups != 0 && su == n_stages - 1;
        const uint32_t vo = ragged ? voff_w_ragged : voff_w;
#pragma unroll
        for (int r = 0; r < R; ++r)
            araw[slot][r] = *reinterpret_cast<const u32x4*>(a_base + r * tile_bytes + (size_t)su * 1024 + vo);
    };
    auto load_scales = [&](uint32_t (&dst)[R], int quad) {
        const size_t off = (size_t)min(quad, n_quads - 1) * 256;
#pragma unroll
        for (int r = 0; r < R; ++r)
            dst[r] = *reinterpret_cast<const uint32_t*>(s_base + r * stile_bytes + off + voff_s);
    };
    auto do_stage = [&](int slot, int qpos, int s) {
        issue_b(s + 1);
        load_a(slot ^ 1, s + 1);
        __builtin_amdgcn_sched_barrier(0);  // next stage's loads are issued here, before this stage's MFMAs
        const bool live = s < n_stages && !(rem_groups != 0 && s == n_stages - 1 && g >= rem_groups);
        float sc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) sc[r] = live ? mxfp4_scale_to_f32((sw_cur[r] >> (8 * qpos)) & 0xFFu) : 0.0f;
        u32x4 bq[2];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            u32x4 av[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t d[4];
                mxfp4_dword_to_bf16x8(araw[slot][r][j], sc[r], d);
                av[r] = u32x4{d[0], d[1], d[2], d[3]};
            }
            // activation operands are read from LDS two token tiles ahead of the MFMAs that use
            // them, across the k-steps of the stage (NT is even, so the buffer parity carries over)
            if (j == 0) {
                bq[0] = b_frag(s, 0, 0);
                bq[1] = b_frag(s, 0, 1);
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const u32x4 b = bq[t & 1];
                if (t + 2 < NT) bq[t & 1] = b_frag(s, j, t + 2);
                else if (j + 1 < 4) bq[t & 1] = b_frag(s, j + 1, t + 2 - NT);
                __builtin_amdgcn_sched_barrier(0);  // keep the read above ahead of the MFMAs below
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r][t] = mfma_16x16x32(av[r], b, acc[r][t]);
            }
        }
        wait_vmcnt<0>();  // next stage's activations (direct-to-LDS) and weights have landed
        __syncthreads();
    };
    // weights, scales and biases first: their addresses need the tile's expert only, while the activation
    // loads wait for the token ids of the tile's rows (one memory round trip more)
    load_scales(sw_cur, 0);
    load_a(0, 0);
    uint2 bias_raw[R];  // fetched with the first stage: its latency stays off the block's tail
    load_bias<R>(a, e, unit, 0, bias_raw);
    __builtin_amdgcn_sched_barrier(0);
    issue_b(0);
    wait_vmcnt<0>();
    __syncthreads();
    for (int qd = 0; qd < n_quads; ++qd) {
        load_scales(sw_nxt, qd + 1);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (4 * qd + i < n_stages) do_stage(i & 1, i, 4 * qd + i);  // block-uniform: the last group may be partial
#pragma unroll
        for (int r = 0; r < R; ++r) sw_cur[r] = sw_nxt[r];
    }
    stream_epilogue<R, NT, EPI>(a, acc, e, [&](int i) { return row0 + i; }, nrows, unit, 0, bias_raw);
}

// ---------------------------------------------------------------------------------------------
// Prefill-sized buckets, bf16 weights.  A 128-token block needs its expert's rows from HBM (2 bytes a
// weight, 128 flops a byte: the launch is bound by that stream), so everything here serves keeping
// loads far ahead: ONE block of four waves per CU, i.e. one wave per SIMD with the whole register file
// (128 accumulator registers for the 64 x 128 tile + a ring of three stages of weight registers, 192, so
// weights are requested two stages = 256 contraction elements ahead) and 96 KiB of LDS (a ring of
// three 128-token activation stages, moved global -> LDS two stages ahead by direct-to-LDS loads).
// Order of issue in stage s: the weights of stage s + 2 (ordinary loads), the first MFMA group of stage
// s (in front of which the compiler puts its wait for the weights of s: it knows of the 32 ordinary
// loads issued since and not of the direct-to-LDS loads between them, so its wait also covers the
// activations of stage s + 1), then the direct-to-LDS loads of stage s + 2 in assembly.  The stage
// ends with an explicit wait for the activations of stage s + 1 (everything but the 16 + NT loads
// issued after them) and the barrier.  The one or two stages after the last whole turn of the ring
// request nothing and wait for every load: a count of younger loads holds only where those loads are
// in the code, and the compiler removes weight loads whose registers no later stage reads.  Weight elements of k-step j (0..3) and lane group g: 64 (j/2) + 16 g + 8 (j%2)
// .. +8, as in the producer/consumer kernel (a lane's two loads of a pair of steps are adjacent).
// ---------------------------------------------------------------------------------------------
constexpr int kBf16PrefillRing = 3;

template <int NT, int EPI>
MOE_DEVICE void prefill_body_bf16(const ExpertGemmArgs& a, uint8_t* lds, int e, int row0, int nrows, int unit,
                                  bool active) {
    constexpr int R = 4;
    constexpr int D = kBf16PrefillRing;
    constexpr int kSlotBytes = kStageSteps * 8 * 1024;  // 128 tokens x 128 elements x 2 bytes
    constexpr int kYounger = (D - 2) * (4 * R + NT);    // loads of the stages requested after the next one
    static_assert(kYounger <= 63, "vmcnt holds six bits");
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int q = lane & 15;
    const int g = lane >> 4;
    const int K = a.K;
    const int n_stages = ceil_div(K, kStageElems);

    // activation staging: this wave moves the four-row block `wave` of every token tile, 256 contiguous
    // bytes per row (chunk c of row q stored at position c ^ q)
    const int q_dma = 4 * wave + (lane >> 4);
    const int chunk_dma = (lane & 15) ^ q_dma;
    const uint8_t* b_row[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const int idx = min(i * 16 + q_dma, nrows - 1);
        const int src = a.gather ? a.tokens_flat[row0 + idx] : row0 + idx;
        b_row[i] = reinterpret_cast<const uint8_t*>(a.act + (size_t)src * K);
    }
    const uint32_t lds_dma0 = __builtin_amdgcn_readfirstlane(
        (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)(lds + wave * 1024));
    auto issue_b = [&](int s) {
        const int k = s * kStageElems + 8 * chunk_dma;
        const size_t off = (k < K) ? (size_t)k * 2 : 0;  // past the row (or the last stage): re-read its start
        const uint32_t dst = lds_dma0 + (uint32_t)(s % D) * kSlotBytes;
#pragma unroll
        for (int i = 0; i < NT; ++i) dma16_asm(b_row[i] + off, dst + i * 4096);
    };
    const uint8_t* const lds_rd = lds + (size_t)q * 256;
    // slot: ring slot of the stage (compile-time in the stage code)
    auto b_frag = [&](int slot, int j, int t) {
        return *reinterpret_cast<const u32x4*>(lds_rd + (size_t)slot * kSlotBytes + t * 4096 +
                                               ((ws_chunk<FMT_BF16>(j, g) ^ q) << 4));
    };

    if (!active) {  // no row unit: this wave only moves its share of the activations
#pragma unroll
        for (int s = 0; s < D - 1; ++s) issue_b(s);
        wait_vmcnt<(D - 2) * NT>();
        __syncthreads();
        for (int s = 0; s < n_stages; ++s) {
            if (s < D * (n_stages / D)) {  // as the waves with rows: the stages of whole ring turns request
                issue_b(s + D - 1);
                wait_vmcnt<(D - 2) * NT>();
            } else {
                wait_vmcnt<0>();
            }
            __syncthreads();
        }
        wait_vmcnt<0>();  // nothing may still be writing this block's LDS when the wave ends
        return;
    }

    const uint16_t* wbase = reinterpret_cast<const uint16_t*>(a.w) + (size_t)e * a.w_expert_stride;
    const uint8_t* a_ptr[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        a_ptr[r] = reinterpret_cast<const uint8_t*>(wbase + (size_t)(unit * 64 + tile_row_in_group(r, q)) * K);
    // byte offset inside a row of this lane's eight elements of k-step j at stage 0
    const int k_lane0 = 16 * g;
    f32x4 acc[R][NT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
    u32x4 araw[D][kStageSteps][R];
    auto load_a = [&](int slot, int s) {
#pragma unroll
        for (int j = 0; j < kStageSteps; ++j) {
            const int k = s * kStageElems + 64 * (j >> 1) + k_lane0 + 8 * (j & 1);
            const size_t off = (k < K) ? (size_t)k * 2 : 0;  // past the row: re-read its start (zeroed at use)
#pragma unroll
            for (int r = 0; r < R; ++r) araw[slot][j][r] = *reinterpret_cast<const u32x4*>(a_ptr[r] + off);
        }
    };
    // stage s in ring slot i (compile-time).  AHEAD: the loop's stages request stage s + 2; the last
    // stages, after the loop, request nothing and wait for everything (a count of younger loads is only
    // right where those loads are certain to be in the code: the compiler drops loads whose registers
    // no later stage reads).
    auto do_stage = [&](auto i_tag, auto ahead_tag, int s) {
        constexpr int i = decltype(i_tag)::value;
        constexpr bool AHEAD = decltype(ahead_tag)::value;
        if constexpr (AHEAD) load_a((i + D - 1) % D, s + D - 1);
        __builtin_amdgcn_sched_barrier(0);
        u32x4 bq[2];
        bq[0] = b_frag(i, 0, 0);
        bq[1] = b_frag(i, 0, 1);
#pragma unroll
        for (int j = 0; j < kStageSteps; ++j) {
            // elements past the contraction length (ragged last stage) multiply as zeros
            const bool live = s * kStageElems + 64 * (j >> 1) + k_lane0 + 8 * (j & 1) < K;
            u32x4 av[R];
#pragma unroll
            for (int r = 0; r < R; ++r) av[r] = live ? araw[i][j][r] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const u32x4 b = bq[t & 1];
                if (t + 2 < NT) bq[t & 1] = b_frag(i, j, t + 2);
                else if (j + 1 < kStageSteps) bq[t & 1] = b_frag(i, j + 1, t + 2 - NT);
                __builtin_amdgcn_sched_barrier(0);  // keep the read above ahead of the MFMAs below
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r][t] = mfma_16x16x32(av[r], b, acc[r][t]);
                if (AHEAD && j == 0 && t == 0) {
                    __builtin_amdgcn_sched_barrier(0);  // this stage's weights have been waited for: now the
                    issue_b(s + D - 1);                 // direct-to-LDS loads two stages ahead
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        wait_vmcnt<AHEAD ? kYounger : 0>();  // the activations of stage s + 1 have landed (and everything older)
        __syncthreads();
    };
    uint2 bias_raw[R];
    load_bias<R>(a, e, unit, 0, bias_raw);
    static_assert(D == 3, "the stage loop below walks the ring in threes");
    load_a(0, 0);
    issue_b(0);
    load_a(1, 1);
    issue_b(1);
    wait_vmcnt<kYounger>();  // stage 0's activations
    __syncthreads();
    // whole turns of the ring in the loop (when nothing is left over, its last requests re-read the rows'
    // starts into slots nobody reads again), then the one or two stages left over
    const int full_turns = n_stages / D;
    using std::integral_constant;
    for (int tr = 0; tr < full_turns; ++tr) {
        do_stage(integral_constant<int, 0>{}, std::true_type{}, D * tr + 0);
        do_stage(integral_constant<int, 1>{}, std::true_type{}, D * tr + 1);
        do_stage(integral_constant<int, 2>{}, std::true_type{}, D * tr + 2);
    }
    const int tail = n_stages - D * full_turns;  // block-uniform
    if (tail > 0) do_stage(integral_constant<int, 0>{}, std::false_type{}, D * full_turns + 0);
    if (tail > 1) do_stage(integral_constant<int, 1>{}, std::false_type{}, D * full_turns + 1);
    wait_vmcnt<0>();  // nothing may still be writing this block's LDS when the wave ends
    stream_epilogue<R, NT, EPI>(a, acc, e, [&](int i) { return row0 + i; }, nrows, unit, 0, bias_raw);
}

// One block of four waves per CU (one wave per SIMD: 512 registers a lane, 128 KiB of LDS).  Block
// index -> (token block, row block) as in expert_prefill_kernel.
template <int EPI>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void expert_prefill_bf16_kernel(ExpertGemmArgs a) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[kBf16PrefillRing * kStageSteps * 8 * 1024];
    const int n_rb = a.row_blocks;
    const int xcd = blockIdx.x & 7;
    const int m = blockIdx.x >> 3;
    const int tile = (m / n_rb) * 8 + xcd;
    const int row_block = m % n_rb;
    if (tile >= *a.n_tiles) return;  // block-uniform
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = row_block * 4 + wave;
    const bool active = unit < a.rows / 64;
    const int e = a.tile_expert[tile];
    const int row0 = a.tile_row0[tile];
    const int nrows = a.tile_rows[tile];
    const int nt = (nrows + 15) >> 4;  // block-uniform
    if (nt > 6) prefill_body_bf16<8, EPI>(a, lds, e, row0, nrows, unit, active);
    else if (nt > 4) prefill_body_bf16<6, EPI>(a, lds, e, row0, nrows, unit, active);
    else if (nt > 2) prefill_body_bf16<4, EPI>(a, lds, e, row0, nrows, unit, active);
    else prefill_body_bf16<2, EPI>(a, lds, e, row0, nrows, unit, active);
}

template <int FMT, int NT, int EPI, int WAVES>
MOE_DEVICE void prefill_body(const ExpertGemmArgs& a, uint8_t* lds, int e, int row0, int nrows, int unit, bool active) {
    if constexpr (FMT == FMT_MXFP4) {
        prefill_body_mxfp4<NT, EPI, WAVES>(a, lds, e, row0, nrows, unit, active);
    } else {
        stream_body<FMT, 4, NT, EPI, false, WAVES, 8>(a, lds, e, row0, nrows, unit, active);
    }
}

// Two blocks of WAVES = 4 waves per CU: their barriers are independent, so one block's stage
// hand-over overlaps the other's MFMAs (one block of eight waves measured slower).
template <int FMT, int EPI, int WAVES>
__global__ __launch_bounds__(WAVES * 64, 2) void expert_prefill_kernel(ExpertGemmArgs a) {
    constexpr int NTMAX = 8;
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * kStageSteps * NTMAX * 1024];
    // Row block fastest: neighbouring blocks share one token block's activations, which measured
    // faster than the order that keeps an expert's token blocks (same weights) together on one XCD.
    // Workgroups go to the eight XCDs round-robin by linear index, and each XCD has its own L2.
    // All row blocks of a token block run on ONE XCD, back to back in that XCD's sequence, so the
    // block's activations are fetched into that L2 once instead of once per XCD (measured: 40 %
    // less traffic into the L2s, -3 % time; sharing the weights between neighbouring token blocks
    // as well cut the traffic further but ran slower).
    const int n_rb = a.row_blocks;
    const int xcd = blockIdx.x & 7;
    const int m = blockIdx.x >> 3;
    const int tile = (m / n_rb) * 8 + xcd;
    const int row_block = m % n_rb;
    if (tile >= *a.n_tiles) return;  // block-uniform
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int unit = row_block * WAVES + wave;
    const bool active = unit < a.rows / 64;
    const int e = a.tile_expert[tile];
    const int row0 = a.tile_row0[tile];
    const int nrows = a.tile_rows[tile];
    const int nt = (nrows + 15) >> 4;  // block-uniform
    if (nt > 6) {
        prefill_body<FMT, 8, EPI, WAVES>(a, lds, e, row0, nrows, unit, active);
    } else if (nt > 4) {
        prefill_body<FMT, 6, EPI, WAVES>(a, lds, e, row0, nrows, unit, active);
    } else if (nt > 2) {
        prefill_body<FMT, 4, EPI, WAVES>(a, lds, e, row0, nrows, unit, active);
    } else {
        prefill_body<FMT, 2, EPI, WAVES>(a, lds, e, row0, nrows, unit, active);
    }
}

template <int FMT, int EPI>
int launch_cfg(const ExpertGemmArgs& a, hipStream_t stream) {
    constexpr int R = 2;
    const int units = (a.rows / 64) * (4 / R);
    if (a.work_queue) {
        if (a.work_count <= 0) return MOE_OK;
        dim3 grid(ceil_div(units, 4), max(1, ceil_div(a.max_rows_hint, 64)), a.work_count);
        hipLaunchKernelGGL((expert_stream_queue_kernel<FMT, R, EPI>), grid, dim3(256), 0, stream, a);
    } else if constexpr (EPI == EPI_SWIGLU_BF16 || EPI == EPI_ROWS_F32) {
        if (a.topk_i) {  // bucketing inside the expert kernel
            if (a.n_assign > kDirectMaxAssign || a.assign_div <= 0 || a.assign_div > 8 || a.n_experts <= 0) return MOE_ERR_LIMIT;
            ExpertGemmArgs b = a;
            const int cons = a.waves_per_block == 1 ? 12 : 10;
            // a block covers at most `cons` row units per pass; MXFP4 blocks may make two passes (the
            // second pass's code would cost the bf16 stage loops registers they do not have)
            const int units = a.rows / 32;
            b.row_blocks = max(a.row_blocks, ceil_div(units, (FMT == FMT_MXFP4 ? 2 : 1) * cons));
            const bool two = ceil_div(units, b.row_blocks) > cons;
            dim3 grid(ceil_div(a.n_experts, 8) * 8 * b.row_blocks);
            if constexpr (FMT == FMT_MXFP4) {
                if (two && cons == 12) {
                    hipLaunchKernelGGL((expert_stream_direct_kernel<FMT, EPI, 12, 2, true>), grid, dim3(896), 0, stream, b);
                    return launch_status();
                }
                if (two) {
                    hipLaunchKernelGGL((expert_stream_direct_kernel<FMT, EPI, 10, 2, true>), grid, dim3(768), 0, stream, b);
                    return launch_status();
                }
            }
            if (cons == 12) {
                hipLaunchKernelGGL((expert_stream_direct_kernel<FMT, EPI, 12, 2, false>), grid, dim3(896), 0, stream, b);
            } else {
                hipLaunchKernelGGL((expert_stream_direct_kernel<FMT, EPI, 10, 2, false>), grid, dim3(768), 0, stream, b);
            }
        } else if (a.waves_per_block == 16 || a.waves_per_block == 17) {
            ExpertGemmArgs b = a;
            b.row_blocks = ceil_div(a.rows / 64, 4);
            dim3 grid(ceil_div(a.max_tiles, 8) * 8 * b.row_blocks);  // every XCD gets whole token blocks
            if constexpr (FMT == FMT_BF16) {
                if (a.waves_per_block == 17) {
                    hipLaunchKernelGGL((expert_prefill_bf16_kernel<EPI>), grid, dim3(256), 0, stream, b);
                    return launch_status();
                }
            }
            hipLaunchKernelGGL((expert_prefill_kernel<FMT, EPI, 4>), grid, dim3(256), 0, stream, b);
        } else if (a.waves_per_block == 0) {
            ExpertGemmArgs b = a;
            b.row_blocks = max(a.row_blocks, ceil_div(a.rows / 32, 10));
            dim3 grid(ceil_div(a.max_tiles, 8) * 8 * b.row_blocks);
            hipLaunchKernelGGL((expert_stream_ws_kernel<FMT, EPI, 10, 2>), grid, dim3(768), 0, stream, b);
        } else if (a.waves_per_block == 1) {
            ExpertGemmArgs b = a;
            b.row_blocks = max(a.row_blocks, ceil_div(a.rows / 32, 12));
            dim3 grid(ceil_div(a.max_tiles, 8) * 8 * b.row_blocks);
            hipLaunchKernelGGL((expert_stream_ws_kernel<FMT, EPI, 12, 2>), grid, dim3(896), 0, stream, b);
        } else {
            return MOE_ERR_FORMAT;
        }
    } else {
        return MOE_ERR_FORMAT;
    }
    return launch_status();
}

template <int FMT>
int launch_fmt(const ExpertGemmArgs& a, int epi, hipStream_t stream) {
    switch (epi) {
        case EPI_SWIGLU_BF16: return launch_cfg<FMT, EPI_SWIGLU_BF16>(a, stream);
        case EPI_ROWS_F32: return launch_cfg<FMT, EPI_ROWS_F32>(a, stream);
        case EPI_SWIGLU_F32: return launch_cfg<FMT, EPI_SWIGLU_F32>(a, stream);
        case EPI_SCATTER: return launch_cfg<FMT, EPI_SCATTER>(a, stream);
    }
    return MOE_ERR_FORMAT;
}

}  // namespace

int expert_direct_max_assignments() { return kDirectMaxAssign; }

// epi: 0 fused gate/up (bf16 SwiGLU out), 1 fused down (fp32 rows per slot), 2 gate/up with fp32
// in/out, 3 down with fp32 in and atomic scatter.  Token blocks hold at most 64 rows.
int launch_expert_stream(const ExpertGemmArgs& a, int epi, hipStream_t stream) {
    if (a.rows % 64 != 0 || a.K % 32 != 0) return MOE_ERR_SHAPE;
    const bool queue = a.work_queue != nullptr;
    if (queue != (epi == EPI_SWIGLU_F32 || epi == EPI_SCATTER)) return MOE_ERR_FORMAT;
    if (a.format == FMT_BF16) {
        // the streaming consumers address an expert's matrix through a buffer descriptor: 32-bit byte offsets
        if ((unsigned long long)a.rows * (unsigned long long)a.K * 2ull > 0x7fffffffull) return MOE_ERR_LIMIT;
        return launch_fmt<FMT_BF16>(a, epi, stream);
    }
    if (a.format == FMT_MXFP4) {
        if (a.w_expert_stride > 0x7fffffffll || a.s_expert_stride > 0x7fffffffll) return MOE_ERR_LIMIT;
        return launch_fmt<FMT_MXFP4>(a, epi, stream);
    }
    return MOE_ERR_FORMAT;
}

}  // namespace moe
