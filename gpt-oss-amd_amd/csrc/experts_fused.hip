// Gate/up GEMM + SwiGLU and down GEMM of one MoE block in ONE launch, for decode-sized batches (at most
// kFusedMaxAssign assignments, at most kFusedMaxLocal experts per XCD).  Replaces the two launches of
// moe_mlp1_swiglu / moe_mlp2_scatter (src/forward.cpp:474-487, src/hip/moe.hip:9-235, :261-512) and the
// bucketing launches in front of them (src/hip/scheduler.hip); arithmetic as src/run.cpp:657-700.
//
// grid = one block per compute unit.  A block asks the hardware which XCD (L2 cache) it runs under and
// serves that XCD's experts e = xcd, xcd + 8, ...: their buckets (lists of assignment ids, ascending)
// are built once, in LDS, at the start.  Work comes in items taken from the XCD's queue (a counter in
// global memory): first the gate/up items of all the XCD's experts (n1 row blocks each), then their down
// items (n2 row blocks each).  An item is (expert, up to kFusedCons row units of 32 weight rows) over the
// expert's whole bucket, in passes of up to 64 rows.
//
// A block is one pipeline that never drains between items.  Time is cut into ticks (one 128-element
// stage of the contraction, one block barrier each) and quads of four ticks; a pass takes whole quads.
// Three kinds of waves:
//   * the planner wave writes, two quads ahead, what each quad is (a descriptor in LDS): which pass of
//     which item, or nothing.  It takes the items from the queue, and for a down item it first looks
//     (without waiting) whether all gate/up items of that expert have been counted as finished; if not,
//     the quad stays empty and it looks again a quad later.
//   * two producer waves move the activation rows of the quad's pass global -> LDS with direct-to-LDS
//     loads, three ticks ahead, into a ring of four stage slots (the image of expert_tiles.h);
//   * kFusedCons consumer waves stream the weights of their row unit HBM -> registers (three ticks ahead
//     for MXFP4, one for bf16), multiply (v_mfma_f32_16x16x32_bf16) and, in a pass's last quad, run the
//     epilogue.  Lookahead loads cross pass and item boundaries: the first stages of the next pass are
//     requested while the current one finishes, and its epilogue runs with those loads in flight.
//
// Hand-over of the SwiGLU rows inside the launch: a down item reads rows that gate/up items of the same
// expert wrote earlier.  Those items ran under the same L2 (the queue is per XCD), so the rows go
// through that L2 and nothing is written back or invalidated.  A consumer wave's row stores are known
// to have reached the L2 once the wave has waited for loads it issued after them (vector memory
// operations complete in order): the wave does that wait, explicitly, at the end of the quad after the
// epilogue; the barrier that opens the quad after that orders all consumer waves, and then the planner
// counts the item in done[e].  Readers load the rows past their own L1 (device-scope loads).  Every
// item a down item waits for was taken from the queue before it, by a block that is running and never
// waits for anything itself, so the launch cannot deadlock; the looking is bounded all the same, and a
// block that gives up sets the error word and carries on with whatever it reads.
#include <type_traits>

#include "expert_tiles.h"

namespace moe {

namespace {

constexpr int kFusedCons = 12;
constexpr int kFusedProd = 2;
constexpr int kFusedWaves = kFusedCons + kFusedProd + 1;
constexpr int kFusedMaxAssign = 4096;  // 64 chunks of 64 assignments
constexpr int kFusedMaxLocal = 32;     // experts per XCD

struct QuadDesc {
    int valid;   // 0: nothing is computed or moved in this quad
    int stop;    // 1: every wave leaves at the start of this quad
    int phase;   // 0 gate/up, 1 down
    int e;
    int u0, u1;  // the item's row units
    int s0;      // first stage of the quad inside the pass (a multiple of 4; 0 = the pass starts here)
    int list0;   // index of the pass's first row in the LDS list
    int nrows;   // rows of the pass (1..64)
    int last;    // the pass ends in this quad
    int drain;   // gate/up item, last pass: finished-item count wanted at once (see the planner)
    int wait;    // down item, first quad: the producers hold the pass's first load until done[e] is complete
    int pad[4];
};

MOE_DEVICE int hw_xcd_id() {
    // hardware register 20 (XCC_ID), bits 3:0
    return (int)(__builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & 7u);
}

MOE_DEVICE int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

// s_waitcnt vmcnt(n) for a wave-uniform n known only at run time
MOE_DEVICE void wait_vmcnt_dyn(int n) {
    switch (n) {
        case 0: wait_vmcnt<0>(); break;
        case 1: wait_vmcnt<1>(); break;
        case 2: wait_vmcnt<2>(); break;
        case 3: wait_vmcnt<3>(); break;
        case 4: wait_vmcnt<4>(); break;
        case 5: wait_vmcnt<5>(); break;
        case 6: wait_vmcnt<6>(); break;
        case 7: wait_vmcnt<7>(); break;
        case 8: wait_vmcnt<8>(); break;
        case 9: wait_vmcnt<9>(); break;
        case 10: wait_vmcnt<10>(); break;
        case 11: wait_vmcnt<11>(); break;
        case 12: wait_vmcnt<12>(); break;
        case 13: wait_vmcnt<13>(); break;
        case 14: wait_vmcnt<14>(); break;
        case 15: wait_vmcnt<15>(); break;
        default: wait_vmcnt<16>(); break;
    }
}

// LDS writes of this wave visible to the block, then the tick's barrier (no fence: a fence would make a
// wave with direct-to-LDS loads in flight wait for all of them)
MOE_DEVICE void tick_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

struct PhaseDims {
    int K, n_stages, rem_groups, n_pairs;
    long long tile_bytes, stile_bytes;
};

MOE_DEVICE PhaseDims phase_dims(const ExpertGemmArgs& a) {
    PhaseDims d;
    d.K = a.K;
    d.n_stages = ceil_div(a.K, kStageElems);
    const int G = a.K / 32;
    d.rem_groups = G & 3;
    d.n_pairs = a.K / 64;
    d.tile_bytes = (long long)G * 256;
    d.stile_bytes = (long long)ceil_div(ceil_div(G, 4), 4) * 256;
    return d;
}

template <int FMT>
__global__ __launch_bounds__(kFusedWaves * 64, 4) void expert_fused_kernel(ExpertFusedArgs f) {
    constexpr int R = 2;
    constexpr int W = kFusedWaves;
    // more than half of a compute unit's LDS, so that two blocks never share one
    __shared__ __attribute__((aligned(16))) uint8_t lds[kWsRing * kLdsStageBytes + 12 * 1024];
    __shared__ uint16_t list[kFusedMaxAssign];
    __shared__ uint16_t cnt[kFusedMaxLocal][64];
    __shared__ int list_off[kFusedMaxLocal + 1];
    __shared__ QuadDesc desc[4];
    __shared__ int drained;  // consumer waves whose row stores of a draining item have been acknowledged

    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
    const int q = lane & 15;
    const int g = lane >> 4;
    const int xcd = hw_xcd_id();
    const int E = f.gu.n_experts;
    const int n_mine = max(0, (E - xcd + 7) >> 3);  // experts xcd, xcd + 8, ...
    const int n_gu = n_mine * f.n1;
    const int n_items = n_gu + n_mine * f.n2;
    int* const head = f.ctr + xcd;
    int* const err = f.ctr + 8;
    int* const done = f.ctr + 16;
    const PhaseDims dims_gu = phase_dims(f.gu), dims_dn = phase_dims(f.dn);
    auto dims_of = [&](int phase) { return phase ? dims_dn : dims_gu; };  // selects, not an indexed array

    // ---- the buckets of this XCD's experts, as one list in LDS --------------------------------------
    {
        const int n_assign = f.gu.n_assign;
        const int n_chunks = (n_assign + 63) >> 6;
        const int* __restrict__ topk_i = f.gu.topk_i;
        for (int c = wave; c < n_chunks; c += W) {
            const int s = c * 64 + lane;
            const int id = s < n_assign ? topk_i[s] : -1;
            const bool mine = id >= 0 && (id & 7) == xcd;
            const int m = id >> 3;
            for (int mm = 0; mm < n_mine; ++mm) {
                const unsigned long long b = __ballot(mine && m == mm);
                if (lane == 0) cnt[mm][c] = (uint16_t)__popcll(b);
            }
        }
        __syncthreads();
        for (int mm = wave; mm < n_mine; mm += W) {  // exclusive prefix over the chunks, total of the expert
            const uint32_t v = lane < n_chunks ? (uint32_t)cnt[mm][lane] : 0u;
            uint32_t incl = v;
#define MOE_STEP(C, M) incl += dpp_move<C, M>(0u, incl);
            MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
            cnt[mm][lane] = (uint16_t)(incl - v);
            if (lane == 63) list_off[mm + 1] = (int)incl;
        }
        __syncthreads();
        if (wave == 0) {  // prefix over the experts
            const uint32_t v = (lane < n_mine) ? (uint32_t)list_off[lane + 1] : 0u;
            uint32_t incl = v;
#define MOE_STEP(C, M) incl += dpp_move<C, M>(0u, incl);
            MOE_DPP_STEPS(MOE_STEP)
#undef MOE_STEP
            if (lane < n_mine) list_off[lane + 1] = (int)incl;
            if (lane == 0) list_off[0] = 0;
        }
        __syncthreads();
        for (int c = wave; c < n_chunks; c += W) {
            const int s = c * 64 + lane;
            const int id = s < n_assign ? topk_i[s] : -1;
            const bool mine = id >= 0 && (id & 7) == xcd;
            const int m = id >> 3;
            for (int mm = 0; mm < n_mine; ++mm) {
                const unsigned long long b = __ballot(mine && m == mm);
                if (mine && m == mm)
                    list[list_off[mm] + cnt[mm][c] + __popcll(b & ((1ull << lane) - 1ull))] = (uint16_t)s;
            }
        }
        __syncthreads();
    }

    // one quad descriptor, wave-uniform
    auto read_desc = [&](int Q) {
        QuadDesc d;
        const QuadDesc& s = desc[Q & 3];
        d.valid = uniform(s.valid);
        d.stop = uniform(s.stop);
        d.phase = uniform(s.phase);
        d.e = uniform(s.e);
        d.u0 = uniform(s.u0);
        d.u1 = uniform(s.u1);
        d.s0 = uniform(s.s0);
        d.list0 = uniform(s.list0);
        d.nrows = uniform(s.nrows);
        d.last = uniform(s.last);
        d.drain = uniform(s.drain);
        d.wait = uniform(s.wait);
        return d;
    };

    if (wave == W - 1) {
        // =========================== planner ===========================================================
        // Requests to global memory (the next item, a finished-items count) are sent when they become
        // known and read a quad or more later, so the planner never keeps a tick's barrier waiting.
        auto pull = [&]() {
            int v = 0;
            if (lane == 0) v = __hip_atomic_fetch_add(head, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return v;  // lane 0 holds the value; uniform() it where it is used
        };
        auto count_done = [&](int e) {
            if (lane == 0) __hip_atomic_fetch_add(done + e, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        };
        auto decode = [&](int item, int& down, int& m, int& rb) {
            down = item >= n_gu ? 1 : 0;
            const int idx = down ? item - n_gu : item;
            const int n_rb = down ? f.n2 : f.n1;
            m = idx / n_rb;
            rb = idx - m * n_rb;
        };
        bool have = false;
        int ph = 0, e = 0, u0 = 0, u1 = 0, l0 = 0, left = 0, s = 0, ns = 0, spins = 0;
        int sig_e[4] = {0, 0, 0, 0}, sig_q[4] = {0, 0, 0, 0};
        int sig_n = 0;  // pending finished-item counts, oldest first
        // A gate/up item whose expert's down items come up soon in the queue is counted as soon as its row
        // stores have been acknowledged (its consumer waves wait for exactly that and then add to `drained`;
        // the planner spins on that LDS word).  The other gate/up items finish long before anybody asks, and
        // are counted two quads later without that wait.
        int fast_q = -1, fast_e = 0, fast_n = 0;  // quad whose epilogue drains, its expert, its consumer waves
        int cur_m = 0;
        bool last_valid = false, must_wait = false;  // the descriptor written last; the item accepted last
        if (lane == 0) drained = 0;
        int pulled = uniform(pull());  // the item that comes next
        int pulled_v = pull();         // the one after it (in flight)
        int done_v = 0;                // count asked for the item `pulled`, if it is a down item (in flight)
        auto ask_done = [&]() {
            done_v = 0;
            if (pulled < n_items && pulled >= n_gu) {
                int down, m, rb;
                decode(pulled, down, m, rb);
                if (lane == 0) done_v = __hip_atomic_load(done + xcd + 8 * m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        };
        auto advance = [&]() {  // `pulled` has been dealt with
            pulled = uniform(pulled_v);
            pulled_v = pull();
            ask_done();
        };
        ask_done();
        auto plan = [&](int Qt) {
            if (!have) {
                while (pulled < n_items) {
                    int down, m, rb;
                    decode(pulled, down, m, rb);
                    const int n_rb = down ? f.n2 : f.n1;
                    const int e_ = xcd + 8 * m;
                    const int rows = uniform(list_off[m + 1] - list_off[m]);
                    if (rows == 0) {  // nobody routed here: a gate/up item is finished as it stands
                        if (!down) count_done(e_);
                        advance();
                        continue;
                    }
                    must_wait = false;
                    if (down && uniform(done_v) < f.n1) {
                        // Not all gate/up items of this expert have been counted.  With nothing of this block's own
                        // in the pipeline (the quad before is empty, every count of its own items sent by then) the
                        // item starts all the same, its weights on their way, and the producers hold its first load
                        // until the count is complete; otherwise the quad stays empty and the planner looks again.
                        const bool clear = !last_valid && sig_n == 0 && (fast_q < 0 || fast_q <= Qt - 2);
                        if (!clear) {
                            if (++spins <= f.spin_limit) {
                                ask_done();
                                break;
                            }
                            if (lane == 0) __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        } else {
                            must_wait = true;
                        }
                    }
                    spins = 0;
                    const int units = (down ? f.dn.rows : f.gu.rows) / 32;
                    have = true;
                    cur_m = m;
                    ph = down;
                    e = e_;
                    u0 = (int)((long long)rb * units / n_rb);
                    u1 = (int)((long long)(rb + 1) * units / n_rb);
                    l0 = uniform(list_off[m]);
                    left = rows;
                    s = 0;
                    ns = dims_of(ph).n_stages;
                    advance();
                    break;
                }
            }
            QuadDesc d{};
            if (have) {
                d.valid = 1;
                d.phase = ph;
                d.e = e;
                d.u0 = u0;
                d.u1 = u1;
                d.s0 = s;
                d.list0 = l0;
                d.nrows = min(64, left);
                d.last = (s + 4 >= ns) ? 1 : 0;
                d.wait = (must_wait && s == 0 && l0 == uniform(list_off[cur_m])) ? 1 : 0;
                s += 4;
                if (d.last) {
                    left -= d.nrows;
                    l0 += d.nrows;
                    s = 0;
                    if (left == 0) {
                        have = false;
                        // queue positions between this expert's last gate/up item and its first down item
                        if (ph == 0 && n_gu + cur_m * f.n2 - (cur_m + 1) * f.n1 < f.drain_slack) {
                            d.drain = 1;
                            fast_q = Qt;
                            fast_e = e;
                            fast_n = min(u1 - u0, kFusedCons);
                        } else if (ph == 0 && sig_n < 4) {  // counted two quads after the one with the epilogue
                            sig_e[sig_n] = e;
                            sig_q[sig_n] = Qt + 2;
                            ++sig_n;
                        }
                    }
                }
            } else if (pulled >= n_items && sig_n == 0 && fast_q < 0) {
                d.stop = 1;
            }
            last_valid = d.valid != 0;
            if (lane == 0) desc[Qt & 3] = d;
        };
        if (lane == 0) desc[0] = QuadDesc{};
        plan(1);
        tick_barrier();  // the descriptors of quads 0 and 1 are there
        for (int Q = 0;; ++Q) {
            if (uniform(desc[Q & 3].stop)) break;
            if (fast_q >= 0 && fast_q == Q - 1) {  // the quad before ended with a draining epilogue
                int spins = 0, v = 0;
                do {
                    v = uniform(__hip_atomic_load(&drained, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
                } while (v < fast_n && ++spins < (1 << 20));
                if (v < fast_n && lane == 0) __hip_atomic_store(err, 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                count_done(fast_e);
                if (lane == 0) drained = 0;
                fast_q = -1;
            }
            tick_barrier();
            // A gate/up item cannot end while four counts are pending: a pass takes at least one quad and a
            // count is due two quads after the pass's last, so there are at most three.
            while (sig_n > 0 && sig_q[0] <= Q) {
                count_done(sig_e[0]);
                sig_e[0] = sig_e[1]; sig_q[0] = sig_q[1];
                sig_e[1] = sig_e[2]; sig_q[1] = sig_q[2];
                sig_e[2] = sig_e[3]; sig_q[2] = sig_q[3];
                --sig_n;
            }
            plan(Q + 2);  // read by the other waves at the start of quad Q + 1
            tick_barrier();
            tick_barrier();
            tick_barrier();
        }
        return;
    }

    if (wave >= kFusedCons) {
        // =========================== producers =========================================================
        const int p = wave - kFusedCons;
        const int pos = lane & 15;  // chunk position inside the row's LDS image
        const int sub = lane >> 4;  // row inside the instruction's block of four
        int chunk[2];
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) chunk[ii] = ws_chunk_at<FMT>(pos ^ (4 * (2 * p + ii) + sub));
        struct Rows {
            const uint8_t* row[kNTMax][2];
            int nt, n_last, phase;
        };
        Rows cur{}, nxt{};
        auto set_rows = [&](Rows& r, const QuadDesc& d) {
            const ExpertGemmArgs& a = d.phase ? f.dn : f.gu;
            const float inv_div = 1.0f / (float)a.assign_div;
            r.nt = (d.nrows + 15) >> 4;
            r.phase = d.phase;
            r.n_last = 0;
#pragma unroll
            for (int ii = 0; ii < 2; ++ii) {
                const int qq = 4 * (2 * p + ii) + sub;
                r.n_last += (16 * (r.nt - 1) + 4 * (2 * p + ii) < d.nrows) ? 1 : 0;
#pragma unroll
                for (int t = 0; t < kNTMax; ++t) {
                    const int idx = min(t * 16 + qq, d.nrows - 1);
                    const int s = (int)list[d.list0 + idx];
                    // token of assignment s = s / assign_div, as a float multiplication (exact for s < 4096)
                    const int src = a.gather ? (int)(((float)s + 0.5f) * inv_div) : s;
                    r.row[t][ii] = reinterpret_cast<const uint8_t*>(a.act + (size_t)src * a.K);
                }
            }
        };
        // the loads of stage st of the pass into ring slot `slot`; returns how many were issued
        auto issue = [&](const Rows& r, int st, int slot) {
            const int K = dims_of(r.phase).K;
            uint8_t* dst = lds + (size_t)slot * kLdsStageBytes;
#pragma unroll
            for (int ii = 0; ii < 2; ++ii) {
                const int k = st * kStageElems + 8 * chunk[ii];
                const size_t off = (k < K) ? (size_t)k * 2 : 0;  // a position past the row re-reads its start
#pragma unroll
                for (int t = 0; t < kNTMax; ++t) {
                    if (t < r.nt - 1 || (t == r.nt - 1 && ii < r.n_last)) {  // wave-uniform
                        // gate/up: rows of the block input; down: rows written earlier in this launch
                        if (r.phase) dma16<16>(r.row[t][ii] + off, dst + t * 4096 + (2 * p + ii) * 1024);
                        else dma16<0>(r.row[t][ii] + off, dst + t * 4096 + (2 * p + ii) * 1024);
                    }
                }
            }
            return 2 * (r.nt - 1) + r.n_last;
        };
        int l_prev = 0;  // loads issued in the tick before
        tick_barrier();
        for (int Q = 0;; ++Q) {
            const QuadDesc d0 = read_desc(Q), d1 = read_desc(Q + 1);
            if (d0.stop) break;
            const bool d1_first = d1.valid && d1.s0 == 0;
            if (d1_first) set_rows(nxt, d1);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // this tick requests the stage of tick 4Q + i + 3
                int l_now = 0;
                if (i == 0) {
                    if (d0.valid && d0.s0 + 3 < dims_of(d0.phase).n_stages) l_now = issue(cur, d0.s0 + 3, 3);
                } else {
                    if (i == 1 && d1_first && d1.wait) {  // rows written in this launch: all of them must be there
                        int spins = 0, v = 0;
                        do {
                            if (lane == 0) v = __hip_atomic_load(done + d1.e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                            v = uniform(v);
                        } while (v < f.n1 && ++spins < f.spin_limit);
                        if (v < f.n1 && lane == 0) __hip_atomic_store(err, 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    const int st = d1.s0 + i - 1;
                    if (d1.valid && st < dims_of(d1.phase).n_stages) l_now = d1_first ? issue(nxt, st, i - 1) : issue(cur, st, i - 1);
                }
                wait_vmcnt_dyn(l_prev + l_now);  // the stage of tick 4Q + i + 1 has landed
                l_prev = l_now;
                tick_barrier();
            }
            if (d1_first) cur = nxt;
        }
        wait_vmcnt<0>();  // nothing may still be writing this block's LDS when the wave ends
        return;
    }

    // =============================== consumers =========================================================
    // per-lane LDS offsets of the four fragment reads of a stage (token tile 0, ring slot 0)
    uint32_t frag_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) frag_off[j] = (uint32_t)(q * 256 + ((ws_pos<FMT>(ws_chunk<FMT>(j, g)) ^ q) << 4));
    auto b_frag = [&](int slot, int j, int t) {
        return *reinterpret_cast<const u32x4*>(lds + frag_off[j] + slot * kLdsStageBytes + t * 4096);
    };
    // weights of a pass as seen by this wave: wave-uniform bases, the lane's part is added at the load
    struct Unit {
        const uint8_t* w[R];
        const uint8_t* s[R];
        int phase, e, unit, active;
    };
    const uint8_t* const dummy = reinterpret_cast<const uint8_t*>(f.gu.w);
    auto set_unit = [&](Unit& u, const QuadDesc& d) {
        const ExpertGemmArgs& a = d.phase ? f.dn : f.gu;
        const PhaseDims pd = dims_of(d.phase);
        u.phase = d.phase;
        u.e = d.e;
        u.unit = d.u0 + wave;
        u.active = (u.unit < d.u1) ? 1 : 0;
        const int unit = u.active ? u.unit : d.u0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if constexpr (FMT == FMT_MXFP4) {
                const long long tile = (long long)(unit >> 1) * 4 + ((unit & 1) * R + r);
                u.w[r] = reinterpret_cast<const uint8_t*>(a.w) + (long long)d.e * a.w_expert_stride + tile * pd.tile_bytes;
                u.s[r] = a.w_scales + (long long)d.e * a.s_expert_stride + tile * pd.stile_bytes;
            } else {
                const long long row = (long long)(unit >> 1) * 64 + ((unit & 1) * R + r) * 4;
                u.w[r] = reinterpret_cast<const uint8_t*>(a.w) + ((long long)d.e * a.w_expert_stride + row * pd.K) * 2;
                u.s[r] = nullptr;
            }
        }
    };
    Unit cur{}, nxt{};
    uint2 bias_raw[R] = {};
    int need_store_wait = 0;
    int Q = 0;
    QuadDesc d0{}, d1{};

    // The quads of one pass are run by code specialised for the pass's tile count NT (0: a quad without
    // work), with the accumulators local to it: the ring of weight registers is all that lives from one
    // pass to the next.  (One body with the tile count as a run-time value, or a switch per tick, costs
    // the register allocator more registers than there are.)
    if constexpr (FMT == FMT_MXFP4) {
        constexpr int D = 4;
        const uint32_t voff_w = (uint32_t)lane * 16;
        const uint32_t voff_s = (uint32_t)lane * 4;
        u32x4 araw[D][R];
        uint32_t sw_cur[R] = {}, sw_nxt[R] = {};
        // the weights of stage st of unit u into ring slot `slot`; a stage that does not exist (or a wave
        // without a unit) reads the start of the weights instead, so that every tick issues R loads
        auto load_a = [&](int slot, const Unit& u, bool valid, int st) {
            const PhaseDims pd = dims_of(u.phase);
            const bool real = valid && u.active && st < pd.n_stages;
            const bool ragged = real && pd.rem_groups != 0 && st == pd.n_stages - 1;
            // ragged last stage: a lane group past the last MX block re-reads block 0 (and gets scale 0)
            const uint32_t vo = ragged ? (uint32_t)((g < pd.rem_groups ? lane : q) * 16) : voff_w;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint8_t* base = real ? u.w[r] + (size_t)st * 1024 : dummy;
                // non-temporal: a 1 KiB chunk is read once, by this instruction alone
                araw[slot][r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(base + vo));
            }
        };
        auto load_scales = [&](uint32_t (&dst)[R], const Unit& u, bool valid, int st0) {
            const bool real = valid && u.active;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint8_t* base = real ? u.s[r] + (size_t)(st0 >> 2) * 256 : dummy;
                dst[r] = *reinterpret_cast<const uint32_t*>(base + voff_s);
            }
        };
        auto run_pass = [&](auto nt_tag) {
            constexpr int NT = decltype(nt_tag)::value;
            constexpr int NA = NT > 0 ? NT : 1;
            f32x4 acc[R][NA];
            auto tick = [&](auto i_tag, bool d1_first) {
                constexpr int i = decltype(i_tag)::value;
                // requests for tick 4Q + i + 3
                if constexpr (i == 0) {
                    load_a(3, cur, d0.valid != 0, d0.s0 + 3);
                    load_scales(sw_nxt, d1_first ? nxt : cur, d1.valid != 0, d1.s0);
                } else {
                    load_a(i - 1, d1_first ? nxt : cur, d1.valid != 0, d1.s0 + i - 1);
                }
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (NT > 0) {
                    const int st = d0.s0 + i;
                    const PhaseDims pd = dims_of(cur.phase);
                    if (cur.active && st < pd.n_stages) {  // wave-uniform
                        const bool live = !(pd.rem_groups != 0 && st == pd.n_stages - 1 && g >= pd.rem_groups);
                        float sc[R];
#pragma unroll
                        for (int r = 0; r < R; ++r) sc[r] = live ? mxfp4_scale_to_f32((sw_cur[r] >> (8 * i)) & 0xFFu) : 0.0f;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            u32x4 b[NT];
#pragma unroll
                            for (int t = 0; t < NT; ++t) b[t] = b_frag(i, j, t);
#pragma unroll
                            for (int r = 0; r < R; ++r) {
                                uint32_t d[4];
                                mxfp4_dword_to_bf16x8(araw[i][r][j], sc[r], d);
                                const u32x4 av = {d[0], d[1], d[2], d[3]};
#pragma unroll
                                for (int t = 0; t < NT; ++t) acc[r][t] = mfma_16x16x32(av, b[t], acc[r][t]);
                            }
                        }
                    }
                }
                __syncthreads();
            };
            for (;;) {
                const bool d1_first = d1.valid && d1.s0 == 0;
                if (d1_first) set_unit(nxt, d1);
                if constexpr (NT > 0) {
                    if (d0.s0 == 0) {
#pragma unroll
                        for (int r = 0; r < R; ++r)
#pragma unroll
                            for (int t = 0; t < NT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
                        if (cur.active) load_bias<R>(d0.phase ? f.dn : f.gu, d0.e, cur.unit >> 1, (cur.unit & 1) * R, bias_raw);
                    }
                }
                tick(std::integral_constant<int, 0>{}, d1_first);
                tick(std::integral_constant<int, 1>{}, d1_first);
                tick(std::integral_constant<int, 2>{}, d1_first);
                tick(std::integral_constant<int, 3>{}, d1_first);
                if (need_store_wait) {  // everything older than the last tick's loads: the row stores of the quad before
                    wait_vmcnt<R>();
                    need_store_wait = 0;
                }
                bool more = false;
                if constexpr (NT > 0) {
                    if (d0.last) {
                        if (cur.active) {
                            const int group = cur.unit >> 1, r0 = (cur.unit & 1) * R;
                            const int list0 = d0.list0;
                            auto slot_of_row = [&](int i) { return (int)list[list0 + i]; };
                            if (d0.phase) stream_epilogue<R, NT, EPI_ROWS_F32>(f.dn, acc, d0.e, slot_of_row, d0.nrows, group, r0, bias_raw);
                            else stream_epilogue<R, NT, EPI_SWIGLU_BF16>(f.gu, acc, d0.e, slot_of_row, d0.nrows, group, r0, bias_raw);
                            if (d0.drain) {  // all this wave's loads and stores have completed: say so
                                wait_vmcnt<0>();
                                if (lane == 0) __hip_atomic_fetch_add(&drained, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                            } else {
                                need_store_wait = d0.phase == 0;
                            }
                        }
                    } else {
                        more = true;  // the next quad belongs to the same pass
                    }
                }
                if (d1_first) cur = nxt;
#pragma unroll
                for (int r = 0; r < R; ++r) sw_cur[r] = sw_nxt[r];
                ++Q;
                d0 = d1;
                d1 = read_desc(Q + 1);
                if (!more) break;
            }
        };
        load_a(0, cur, false, 0);
        load_a(1, cur, false, 0);
        load_a(2, cur, false, 0);
        __syncthreads();  // the descriptors of quads 0 and 1 are there
        d0 = read_desc(0);
        d1 = read_desc(1);
        while (!d0.stop) {
            const int nt = d0.valid ? (d0.nrows + 15) >> 4 : 0;
            if (nt == 0) run_pass(std::integral_constant<int, 0>{});
            else if (nt == 1) run_pass(std::integral_constant<int, 1>{});
            else if (nt == 2) run_pass(std::integral_constant<int, 2>{});
            else if (nt == 3) run_pass(std::integral_constant<int, 3>{});
            else run_pass(std::integral_constant<int, 4>{});
        }
    } else {
        // bf16: the contraction range is walked in pairs of MFMA steps (64 elements = one 128-byte line of
        // a weight row): in a pair, lane group g takes elements 16g .. 16g+7 in the first step and
        // 16g+8 .. 16g+15 in the second, so a lane's two 16-byte loads are adjacent.  A tick is two
        // pairs; a pair's loads are issued three pairs (one and a half ticks) ahead, into a ring of four.
        const uint32_t lane_off_gu = (uint32_t)((((q >> 2) * 16 + (q & 3)) * dims_gu.K + 16 * g) * 2);
        const uint32_t lane_off_dn = (uint32_t)((((q >> 2) * 16 + (q & 3)) * dims_dn.K + 16 * g) * 2);
        u32x4 ar[4][2][R];  // ring of pairs [2 * (tick parity) + pair][half][row tile]
        auto load_a = [&](int slot, const Unit& u, bool valid, int pair) {
            const PhaseDims pd = dims_of(u.phase);
            const bool real = valid && u.active && pair < pd.n_pairs;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint8_t* base = real ? u.w[r] + (size_t)pair * 128 : dummy;
                const uint32_t vo = real ? (u.phase ? lane_off_dn : lane_off_gu) : (uint32_t)lane * 32;
#pragma unroll
                for (int h = 0; h < 2; ++h) ar[slot][h][r] = *reinterpret_cast<const u32x4*>(base + vo + 16 * h);
            }
        };
        auto run_pass = [&](auto nt_tag) {
            constexpr int NT = decltype(nt_tag)::value;
            constexpr int NA = NT > 0 ? NT : 1;
            f32x4 acc[R][NA];
            auto half_tick = [&](auto i_tag, auto pp_tag, bool d1_first) {
                constexpr int i = decltype(i_tag)::value;
                constexpr int pp = decltype(pp_tag)::value;
                // request the pair three pairs ahead: pair 1 of the next tick (pp = 0) or pair 0 of the tick after
                // that (pp = 1); its ring slot is the one whose pair was consumed in the half tick before this one
                constexpr int ti = i + 1 + pp;  // tick of the quad (or, from 4 on, of the next quad)
                constexpr int tp = 1 - pp;      // pair inside that tick
                constexpr int slot_next = 2 * (ti & 1) + tp;
                if constexpr (ti < 4) load_a(slot_next, cur, d0.valid != 0, 2 * (d0.s0 + ti) + tp);
                else load_a(slot_next, d1_first ? nxt : cur, d1.valid != 0, 2 * (d1.s0 + ti - 4) + tp);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (NT > 0) {
                    constexpr int u = 2 * (i & 1) + pp;
                    const int st = d0.s0 + i;
                    const PhaseDims pd = dims_of(cur.phase);
                    if (d0.valid && cur.active && st < pd.n_stages) {  // wave-uniform
                        const bool live = 2 * st + pp < pd.n_pairs;  // false only in the second half of a ragged stage
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            u32x4 av[R];
#pragma unroll
                            for (int r = 0; r < R; ++r) av[r] = live ? ar[u][h][r] : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
                            for (int t0 = 0; t0 < NT; t0 += 2) {  // two token tiles at a time: eight fragment registers
                                u32x4 b[2];
#pragma unroll
                                for (int t = 0; t < 2; ++t) b[t] = b_frag(i, 2 * pp + h, t0 + t);
#pragma unroll
                                for (int r = 0; r < R; ++r)
#pragma unroll
                                    for (int t = 0; t < 2; ++t) acc[r][t0 + t] = mfma_16x16x32(av[r], b[t], acc[r][t0 + t]);
                            }
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            auto tick = [&](auto i_tag, bool d1_first) {
                half_tick(i_tag, std::integral_constant<int, 0>{}, d1_first);
                half_tick(i_tag, std::integral_constant<int, 1>{}, d1_first);
                __syncthreads();
            };
            for (;;) {
                const bool d1_first = d1.valid && d1.s0 == 0;
                if (d1_first) set_unit(nxt, d1);
                if constexpr (NT > 0) {
                    if (d0.valid && d0.s0 == 0) {
#pragma unroll
                        for (int r = 0; r < R; ++r)
#pragma unroll
                            for (int t = 0; t < NT; ++t) acc[r][t] = f32x4{0.f, 0.f, 0.f, 0.f};
                        if (cur.active) load_bias<R>(d0.phase ? f.dn : f.gu, d0.e, cur.unit >> 1, (cur.unit & 1) * R, bias_raw);
                    }
                }
                tick(std::integral_constant<int, 0>{}, d1_first);
                tick(std::integral_constant<int, 1>{}, d1_first);
                tick(std::integral_constant<int, 2>{}, d1_first);
                tick(std::integral_constant<int, 3>{}, d1_first);
                if (need_store_wait) {  // everything older than the last tick's loads: the row stores of the quad before
                    wait_vmcnt<4 * R>();
                    need_store_wait = 0;
                }
                bool more = false;
                if constexpr (NT > 0) {
                    if (d0.valid && d0.last) {
                        if (cur.active) {
                            const int group = cur.unit >> 1, r0 = (cur.unit & 1) * R;
                            const int list0 = d0.list0;
                            auto slot_of_row = [&](int i) { return (int)list[list0 + i]; };
                            if (d0.phase) stream_epilogue<R, NT, EPI_ROWS_F32>(f.dn, acc, d0.e, slot_of_row, d0.nrows, group, r0, bias_raw);
                            else stream_epilogue<R, NT, EPI_SWIGLU_BF16>(f.gu, acc, d0.e, slot_of_row, d0.nrows, group, r0, bias_raw);
                            if (d0.drain) {  // all this wave's loads and stores have completed: say so
                                wait_vmcnt<0>();
                                if (lane == 0) __hip_atomic_fetch_add(&drained, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                            } else {
                                need_store_wait = d0.phase == 0;
                            }
                        }
                    } else {
                        more = d0.valid != 0;  // the next quad belongs to the same pass
                    }
                }
                if (d1_first) cur = nxt;
                ++Q;
                d0 = d1;
                d1 = read_desc(Q + 1);
                if (!more) break;
            }
        };
        load_a(0, cur, false, 0);
        load_a(1, cur, false, 0);
        load_a(2, cur, false, 0);
        __syncthreads();  // the descriptors of quads 0 and 1 are there
        d0 = read_desc(0);
        d1 = read_desc(1);
        while (!d0.stop) {
            // every token tile is multiplied, also those past the pass's rows (they read stale LDS and are
            // never stored): the matrix work of a bf16 tick is a small part of the time its weights take,
            // and a second variant of the pass costs more registers than are left
            run_pass(std::integral_constant<int, 4>{});
        }
    }
}

}  // namespace

int expert_fused_max_assignments() { return kFusedMaxAssign; }
int expert_fused_max_experts() { return 8 * kFusedMaxLocal; }
int expert_fused_consumers() { return kFusedCons; }

int launch_expert_fused(const ExpertFusedArgs& f, int n_blocks, hipStream_t stream) {
    const ExpertGemmArgs& a = f.gu;
    if (a.rows % 64 != 0 || a.K % 32 != 0 || f.dn.rows % 64 != 0 || f.dn.K % 32 != 0) return MOE_ERR_SHAPE;
    if (!a.topk_i || a.n_assign > kFusedMaxAssign || a.assign_div <= 0 || a.assign_div > 8 || a.n_experts <= 0 ||
        a.n_experts > 8 * kFusedMaxLocal)
        return MOE_ERR_LIMIT;
    if (f.n1 <= 0 || f.n2 <= 0 || !f.ctr || n_blocks <= 0 || a.format != f.dn.format) return MOE_ERR_FORMAT;
    if (ceil_div(a.rows / 32, f.n1) > kFusedCons || ceil_div(f.dn.rows / 32, f.n2) > kFusedCons) return MOE_ERR_FORMAT;
    if (a.format == FMT_BF16) {
        hipLaunchKernelGGL((expert_fused_kernel<FMT_BF16>), dim3(n_blocks), dim3(kFusedWaves * 64), 0, stream, f);
    } else if (a.format == FMT_MXFP4) {
        hipLaunchKernelGGL((expert_fused_kernel<FMT_MXFP4>), dim3(n_blocks), dim3(kFusedWaves * 64), 0, stream, f);
    } else {
        return MOE_ERR_FORMAT;
    }
    return launch_status();
}

}  // namespace moe
