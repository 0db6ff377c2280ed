// row_kernel.h - the row kernel: one launch serves a batch of logits rows.  Row r is scanned
// by `slices` workgroups of 256 threads (grid = slices x rows).  Each workgroup finds the exact
// top-k of its slice; with several slices the last workgroup to arrive (an atomic ticket,
// nobody waits) merges them.  That workgroup then runs the tail.
#pragma once

#include "device_common.h"
#include "select_bitmap.h"
#include "select_exhaustive.h"
#include "select_sparse.h"
#include "select_stream.h"
#include "tail.h"

namespace lily {

// ------------------------------------------------------------------ argmax

// First maximum under float comparison (NaN never wins, -0 == +0), lowest id on
// ties: elementwise.metal:145-150.  Result: the best (value, id) of the slice as a
// composite; id bits all zero when no element qualified.
template <int DT>
__device__ __forceinline__ uint64_t slice_argmax(const RowArgs& a, const Geo<DT>& g, Shared& sh) {
    constexpr int E = Geo<DT>::E;
    const uint32_t tid = threadIdx.x;
    float bv = NEG_INF;
    uint32_t bi = 0xffffffffu;
    for (uint32_t c0 = g.cb; c0 < g.ce; c0 += NT * UNROLL) {
        // Unconditional loads (chunks past the slice's end read its last chunk; `inside`
        // below discards them): a load that may be skipped is waited for as the last one issued.
        u32x4 raw[UNROLL];
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t c = min(c0 + u * NT + tid, g.ce - 1u);
            raw[u] = gload(reinterpret_cast<const u32x4*>(g.base + (size_t)c * 16));
        }
        for (int u = 0; u < UNROLL; ++u) {
            const uint32_t c = c0 + u * NT + tid;
            float v[E];
            unpack<DT>(raw[u], v);
            for (int j = 0; j < E; ++j) {
                const uint32_t id = g.id_of(c, j);
                const bool inside = c >= g.main_lo && c < g.main_hi;
                const float x = v[j];
                if (inside && (x > bv || (x == bv && id < bi))) {
                    bv = x;
                    bi = id;
                }
            }
        }
    }
    for (int side = 0; side < 2; ++side) {
        const uint32_t lo = side == 0 ? g.id_lo : g.edge_hi_begin;
        const uint32_t hi = side == 0 ? g.edge_lo_end : g.id_hi;
        for (uint32_t id = lo + tid; id < hi; id += NT) {
            const float x = load_logit<DT>(a.logits, id);
            if (x > bv || (x == bv && id < bi)) {
                bv = x;
                bi = id;
            }
        }
    }
    uint64_t best = ((uint64_t)lilym_order_key(bv + 0.0f) << 32) | (uint32_t)(~bi);
    best = wave_max_u64(best);
    if ((tid & 63u) == 0) {
        sh.red_u[tid >> 6] = best;
    }
    __syncthreads();
    best = sh.red_u[0];
    for (int i = 1; i < NWAVE; ++i) {
        best = sh.red_u[i] > best ? sh.red_u[i] : best;
    }
    __syncthreads();
    return best;
}

// ------------------------------------------------------------------ the row kernel

// The row's arguments are the same for every thread: read through the constant address
// space they arrive by scalar loads and stay in scalar registers.
__device__ __forceinline__ void load_row_args(RowArgs& a, const LILY_CONST RowArgs* src) {
    static_assert(sizeof(RowArgs) % 16 == 0, "RowArgs is copied in 16-byte pieces");
    const LILY_CONST u32x4* from = (const LILY_CONST u32x4*)src;
    u32x4* to = reinterpret_cast<u32x4*>(&a);
    for (unsigned i = 0; i < sizeof(RowArgs) / 16; ++i) {
        to[i] = from[i];
    }
}

// CHAIN: the kernel of launches whose rows draw in order (compiled apart from the others: what it
// adds behind the selects would cost every other launch registers).
// A workgroup barrier that orders LDS accesses only (outstanding global stores and atomics are
// not waited for).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// The row and the step of a draw that leaves the choice to the device (see RowArgs::sel_row).
__device__ __forceinline__ void apply_selection(RowArgs& a) {
    if (a.sel_row != nullptr) {
        const uint32_t r = min(*(const LILY_CONST uint32_t*)a.sel_row, a.sel_rows - 1u);
        a.logits = static_cast<const char*>(a.logits) + (size_t)r * a.sel_stride;
    }
    if (a.sel_step != nullptr) {
        a.step += *(const LILY_CONST uint32_t*)a.sel_step;
    }
}

template <int DT, int KIND, bool LSE, bool CHAIN = false>
__device__ __forceinline__ void row_body(const LILY_CONST RowArgs* src, const LaunchCfg& cfg, Shared& sh) {
    if (cfg.served != nullptr && *(const LILY_CONST uint32_t*)(cfg.served + blockIdx.y) != 0u) {
        return;
    }
    RowArgs a;
    load_row_args(a, src);
    apply_selection(a);
    // KIND: 0 = rows without masks, penalties or bias lists, 1 = rows with any of them (the
    // bitmap select is compiled for them), 2 = streaming rows only (no bitmap select at all).
    constexpr bool EXCL = KIND == 1;
    const uint32_t tid = threadIdx.x;
    const uint32_t s = blockIdx.x, row = blockIdx.y, S = cfg.slices;
    const uint32_t vocab = cfg.vocab;
    const uint32_t step = a.step + cfg.step_delta;
    const bool want_lse = LSE && a.out_logprob != nullptr;
    uint64_t* cand = dyn_lds;
    uint64_t* found = cand;  // where the select left the slice's candidates
    uint32_t* excl = reinterpret_cast<uint32_t*>(dyn_lds + cfg.cand_cap);

    if ((a.flags & F_FORCED) && !want_lse) {
        if (s == 0 && tid == 0) {
            emit(a, a.forced, vocab);
        }
        return;
    }

    Geo<DT> g;
    g.init(a.logits, vocab, s, S);
    phase(cfg, 0);

    const bool argmax = a.mode == MODE_ARGMAX;
    uint64_t best = 0;
    bool sorted = false;
    if (argmax) {
        best = slice_argmax<DT>(a, g, sh);
    } else {
        // A forced row with a log-probability needs the row sum only: it takes the same
        // selects (their sums are the fast ones) and its candidates are dropped below.
        bool done = false;
        uint32_t took = 2;
        if (cfg.path == 0u && (a.flags & F_STREAM)) {
            done = select_stream<DT, LSE, KIND != 2>(a, g, a.k, sh, cfg, sorted, found);
            if (!done) {
                __syncthreads();
            }
            took = done ? 0u : took;
        }
        if (KIND == 1 && !done && cfg.path == 0u && a.allow != nullptr) {
            done = select_sparse<DT, LSE>(a, g, a.k, cand, min(cfg.dyn_slots, MERGE_CAP), sh, sorted, cfg);
            took = done ? 1u : took;
        }
        if (KIND != 2 && !done && cfg.path != 1u && cfg.bitmap_layout != 0u) {
            const bool special = a.allow != nullptr || (a.flags & F_PEN) || a.n_bias != 0;
            if (EXCL || !special) {
                // A single pass whose running bound let too many candidates in is repeated
                // as two passes (bound first, then collect) before the exhaustive select.
#pragma nounroll
                for (int attempt = 0; attempt < 2 && !done; ++attempt) {
                    const bool two_pass = a.k > 64u || cfg.path == 2u || attempt == 1;
                    if (attempt == 1) {
                        __syncthreads();
                    }
                    done = select_fast<DT, EXCL, LSE>(a, g, a.k, two_pass, cand, cfg.cand_cap, excl, sh,
                                                      cfg, sorted);
                    if (a.k > 64u || cfg.path == 2u) {
                        break;  // it was two passes already
                    }
                }
                took = done ? 1u : took;
            }
        }
        if (cfg.path_stats != nullptr && tid == 0) {
            atomicAdd(&cfg.path_stats[took], 1u);
        }
        if (!done) {
            __syncthreads();
            sorted = false;
            select_exhaustive<DT>(a, g.id_lo, g.id_hi, a.k, want_lse, cand, cfg.cand_cap, sh);
        }
    }

    // What follows reads the row's arguments afresh (scalar loads, served by the scalar cache):
    // kept in registers across the scan, the fields that only the merge and the tail use
    // crowd the scan's own values out of the scalar registers.
    RowArgs t;
    {
        const LILY_CONST RowArgs* again = src;
        asm volatile("" : "+s"(again));
        load_row_args(t, again);
        apply_selection(t);
    }
    const bool forced = (t.flags & F_FORCED) != 0;
    uint32_t n = (argmax || forced) ? 0u : min(sh.n_cand, cfg.cand_cap);
    phase(cfg, 4);
    if (S > 1) {
        const size_t slot = (size_t)row * S + s;
        // Partials go through to memory (no dirty L2 lines to write back), the wave waits
        // for its stores, the workgroup meets, and one thread takes the row's ticket.
        if (argmax) {
            if (tid == 0) {
                handed_store(cfg.ws_cand, slot * cfg.ws_k, best);
            }
        } else {
            // Every slot is written (0 = no candidate), so the merge needs no counts.
            for (uint32_t i = tid; !forced && i < cfg.ws_k; i += NT) {
                handed_store(cfg.ws_cand, slot * cfg.ws_k + i, i < n ? found[i] : (uint64_t)0);
            }
            if (tid == 0) {
                handed_store(cfg.ws_lse, 2 * slot, want_lse ? sh.lse_mc : 0.0);
                handed_store(cfg.ws_lse, 2 * slot + 1, want_lse ? sh.lse_s : 0.0);
            }
        }
        // The hand-over (last_to_arrive(): a release on the ticket and an acquire behind it, or
        // the relaxed form described there).
        const bool last = last_to_arrive(&cfg.ws_ticket[row], S, sh.last, cfg.relaxed_handover != 0u);
        phase(cfg, 5);
        if (!last) {
            return;
        }
        const size_t base = (size_t)row * S;
        if (argmax) {
            best = 0;
            for (uint32_t t = tid; t < S; t += NT) {
                const uint64_t c = handed_load(cfg.ws_cand, (base + t) * cfg.ws_k);
                best = c > best ? c : best;
            }
            best = wave_max_u64(best);
            if ((tid & 63u) == 0) {
                sh.red_u[tid >> 6] = best;
            }
            __syncthreads();
            best = sh.red_u[0];
            for (int i = 1; i < NWAVE; ++i) {
                best = sh.red_u[i] > best ? sh.red_u[i] : best;
            }
        } else {
            // Gather every slice's candidates (0 = no candidate) and the log-sum-exp partials
            // in one round trip.
            constexpr int PER = MERGE_CAP / NT;
            const uint32_t slots = S * cfg.ws_k;
            uint64_t mine[PER];
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                const uint32_t j = tid + (uint32_t)q * NT;
                mine[q] = (!forced && j < slots) ? handed_load(cfg.ws_cand, base * cfg.ws_k + j) : 0ull;
            }
            if (want_lse && tid < 64) {
                double mt = -__builtin_huge_val(), st = 0.0;
                if (tid < S) {
                    mt = handed_load(cfg.ws_lse, 2 * (base + tid));
                    st = handed_load(cfg.ws_lse, 2 * (base + tid) + 1);
                    if (!(st > 0.0)) {
                        mt = -__builtin_huge_val();
                    }
                }
                double m = mt;
                for (int o = 32; o > 0; o >>= 1) {
                    m = fmax(m, __shfl_xor(m, o));
                }
                const double sum = wave_sum_d(st > 0.0 ? st * exp2(mt - m) : 0.0);
                if (tid == 0) {
                    sh.lse_mc = m;
                    sh.lse_s = sum;
                }
            }
            // A bound of the k-th largest from the lanes' best entries (as in the streaming
            // select: each wave's ceil(k / NWAVE)-th largest lane maximum, the minimum over the
            // waves), then only entries at or above it are ranked.
            uint64_t best_mine = 0;
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                best_mine = mine[q] > best_mine ? mine[q] : best_mine;
            }
            const uint32_t kw = (t.k + NWAVE - 1) / NWAVE;
            const uint32_t P = kw <= 64u ? wave_kth_key16((uint32_t)(best_mine >> 48), kw) : 0u;
            if ((tid & 63u) == 0) {
                sh.red_i[tid >> 6] = P;
            }
            if (tid == 0) {
                sh.n_cand = 0;
            }
            __syncthreads();
            uint32_t bound = sh.red_i[0];
            for (int i = 1; i < NWAVE; ++i) {
                bound = min(bound, sh.red_i[i]);
            }
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                if (mine[q] != 0ull && (uint32_t)(mine[q] >> 48) >= bound) {
                    cand[atomicAdd(&sh.n_cand, 1u)] = mine[q];
                }
            }
            __syncthreads();
            n = sh.n_cand;
            sorted = false;
            n = select_topk(cand, n, t.k, sh, sorted);
            found = cand;
        }
    }

    phase(cfg, 6);
    if (argmax) {
        if (tid == 0) {
            const uint32_t id = composite_id(best);
            *t.out_id = id == 0xffffffffu ? 0u : id;
        }
        return;
    }
    if (t.flags & F_FORCED) {
        if (tid == 0) {
            finish_token<DT>(t, sh, t.forced, vocab);
        }
        return;
    }
    if (CHAIN && cfg.chain_rows != 0u) {
        // Rows that draw in order.  This row's candidates - the best t.k under the counts as they
        // stood when the launch began, t.k being the draw's own count plus one for every row
        // before it - are published; the workgroup that publishes last takes the rows one after
        // the other: the ids the earlier rows drew are evaluated again (penalties that can only
        // lower took them down, so the best k_draw of the row as it stands now are still among
        // the candidates), and the tail draws from the best k_draw.
        const uint32_t rows = cfg.chain_rows;
        for (uint32_t i = tid; i < n; i += NT) {
            handed_store(cfg.chain_cand, (size_t)row * CHAIN_CAP + i, found[i]);
        }
        if (tid == 0) {
            handed_store(cfg.chain_n, row, n);
        }
        if (!last_to_arrive(cfg.chain_ticket, rows, sh.last, cfg.relaxed_handover != 0u)) {
            return;
        }
        const LILY_CONST RowArgs* first = src - row;
        if (cfg.accept_ctrl != nullptr && tid < rows) {
            sh.proposal[tid] = gload(cfg.accept_ids + tid);
        }
        // Every row's first 64 candidates, their raw logits and their counts as they stand before
        // any of these rows has drawn are requested together (a wave per row, two rounds for
        // eight rows) and kept in LDS behind the tail's arrays: once the rows draw, nothing waits
        // for memory but the tail's own reads, and the counts the earlier rows left follow from
        // what they drew.  Candidates past the 64th are loaded when their row's turn comes.
        constexpr uint32_t PRE = 64;
        uint64_t* pre_c = dyn_lds + CHAIN_LDS_OFFSET / 8;                           // [rows][PRE]
        float* pre_l = reinterpret_cast<float*>(pre_c + LILY_MAX_VERIFY_ROWS * PRE);  // [rows][PRE]
        uint32_t* pre_cnt = reinterpret_cast<uint32_t*>(pre_l + LILY_MAX_VERIFY_ROWS * PRE);
        // ... and, for the rows that are speculative draws, the proposal and the first 64 entries
        // of the draft's distribution (all of it, as a rule): the tail reads them through the
        // row's pointers, which are turned to these copies.
        uint32_t* pre_qid = pre_cnt + LILY_MAX_VERIFY_ROWS * PRE;                     // [rows][PRE]
        float* pre_qp = reinterpret_cast<float*>(pre_qid + LILY_MAX_VERIFY_ROWS * PRE);
        for (uint32_t j0 = 0; j0 < rows; j0 += NWAVE) {
            const uint32_t j = j0 + (tid >> 6), lane = tid & 63u;
            if (j < rows) {
                const uint32_t nj = min(handed_load(cfg.chain_n, j), CHAIN_CAP);
                if (lane == 0) {
                    sh.chain_n[j] = nj;
                }
                const uint64_t c = handed_load(cfg.chain_cand, (size_t)j * CHAIN_CAP + lane);
                const uint32_t id = min(composite_id(c), vocab - 1u);
                pre_c[j * PRE + lane] = c;
                pre_l[j * PRE + lane] = load_logit<DT>((first + j)->logits, id);
                const LILY_CONST RowArgs* rj = first + j;
                pre_cnt[j * PRE + lane] = (rj->flags & F_PEN) ? load_through(rj->counts + id) : 0u;
                if (rj->mode == MODE_SPEC) {
                    pre_qid[j * PRE + lane] = gload(rj->q_ids + lane);
                    pre_qp[j * PRE + lane] = gload(rj->q_probs + lane);
                    if (lane == 0) {
                        sh.proposal_of[j] = gload(rj->draft);
                        sh.q_n_of[j] = gload(rj->q_n);
                    }
                }
            }
        }
        __syncthreads();
        for (uint32_t j = 0; j < rows; ++j) {
#ifdef LILY_CHAIN_TRACE
            phase(cfg, 8 + j);
#endif
            RowArgs r;
            {
                const LILY_CONST RowArgs* from = first + j;
                asm volatile("" : "+s"(from));
                load_row_args(r, from);
            }
            // What an earlier row drew is evaluated again, with the count it has by now.
            auto times_drawn = [&](uint32_t id) -> uint32_t {
                uint32_t times = 0;
                for (uint32_t q = 0; q < j; ++q) {
                    times += sh.drawn[q] == id ? 1u : 0u;
                }
                return times;
            };
            auto with_count = [&](uint32_t id, float l, uint32_t cnt) -> uint64_t {
                const bool allowed = r.allow == nullptr || bit_of(r.allow, id);
                return composite_of(finish_pre_temperature(r, id, l, cnt, allowed) / r.temperature, id);
            };
            const uint32_t n_now = sh.chain_n[j];
            if (tid < min(n_now, PRE)) {
                const uint64_t c = pre_c[j * PRE + tid];
                const uint32_t id = composite_id(c);
                const uint32_t times = times_drawn(id);
                cand[tid] = times == 0u ? c : with_count(id, pre_l[j * PRE + tid], pre_cnt[j * PRE + tid] + times);
            }
            if (n_now > PRE) {
                // Past what was requested ahead: the earlier rows' increments are waited for
                // (thread 0 issued them) and the counts read as they stand.
                __threadfence();
                __syncthreads();
                for (uint32_t i = tid + PRE; i < n_now; i += NT) {
                    const uint64_t c = handed_load(cfg.chain_cand, (size_t)j * CHAIN_CAP + i);
                    const uint32_t id = composite_id(c);
                    cand[i] = times_drawn(id) == 0u
                                  ? c
                                  : with_count(id, load_logit<DT>(r.logits, id), load_through(r.counts + id));
                }
            }
            __syncthreads();
            // The few candidates that changed are put back in order: up to a workgroup's worth
            // each thread counts the candidates that beat its own (composites are distinct).
            bool ranked = false;
            if (n_now <= NT) {
                // (read eight at a time, the slots up to the next multiple of eight cleared: a
                // loop of one dependent LDS read after the other costs a microsecond a row)
                const uint32_t n_up = (n_now + 7u) & ~7u;
                if (tid >= n_now && tid < n_up) {
                    cand[tid] = 0ull;
                }
                lds_barrier();
                const uint64_t mine = tid < n_now ? cand[tid] : ~0ull;
                uint32_t ahead = 0;
                for (uint32_t q0 = 0; q0 < n_up; q0 += 8u) {
                    uint64_t other[8];
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        other[q] = cand[q0 + (uint32_t)q];
                    }
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        ahead += other[q] > mine ? 1u : 0u;
                    }
                }
                __syncthreads();
                if (tid < n_now) {
                    cand[ahead] = mine;
                }
                __syncthreads();
                ranked = true;
            }
            r.k = r.k_draw;
            if (r.mode == MODE_SPEC && sh.q_n_of[j] <= PRE) {
                r.draft = &sh.proposal_of[j];
                r.q_n = &sh.q_n_of[j];
                r.q_ids = pre_qid + j * PRE;
                r.q_probs = pre_qp + j * PRE;
            }
            tail<DT, KIND != 2, true>(r, vocab, r.step + cfg.step_delta, n_now, ranked, cand, sh, cfg);
            // The workgroup meets over LDS only: a barrier that also waited for thread 0's stores
            // and increments to be acknowledged by memory would cost every row a round trip
            // that nothing here depends on.
            lds_barrier();
            if (tid == 0) {
                sh.drawn[j] = sh.emitted_id;
            }
            lds_barrier();
        }
        // The scratch's largest count (and an id that holds it) follow now, once per draw.  It
        // must never understate a count: thread 0, which issued every increment (device atomics,
        // done where the reads below look), waits for them before anybody reads a count back.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        if (tid < rows && ((first + tid)->flags & F_PEN) && sh.drawn[tid] < vocab) {
            // (row tid's own scratch: the launcher hands every row of such a launch the same one,
            // but nothing here depends on that)
            const LILY_CONST RowArgs* mine = first + tid;
            const uint32_t id = sh.drawn[tid];
            const uint32_t words = (vocab + 31u) / 32u;
            const uint32_t now = load_through(mine->counts + id);
            if (atomicMax(&mine->touched[words], now) <= now) {
                mine->touched[words + 1u] = id;
            }
        }
        if (cfg.accept_ctrl != nullptr && tid == 0) {
            // spec_accept (spec.metal:14-38) on the draws this workgroup just made.
            uint32_t acc = 0;
            while (acc + 1 < rows && sh.drawn[acc] == sh.proposal[acc + 1]) {
                ++acc;
            }
            uint32_t* ctrl = cfg.accept_ctrl;
            ctrl[0] = acc;
            ctrl[LILY_CTRL_STRIDE] = acc + 1;
            for (uint32_t i = 0; i < cfg.accept_chain; ++i) {
                const uint32_t p = cfg.accept_pos0 + acc + 1 + i;
                ctrl[(2 + 3 * i) * LILY_CTRL_STRIDE] = p;
                ctrl[(3 + 3 * i) * LILY_CTRL_STRIDE] = p / cfg.accept_ratio;
                ctrl[(4 + 3 * i) * LILY_CTRL_STRIDE] = ((p + 1) % cfg.accept_ratio == 0) ? 1u : 0u;
            }
        }
        phase(cfg, 7);
        return;
    }
    tail<DT, KIND != 2>(t, vocab, step, n, sorted, found, sh, cfg);
    phase(cfg, 7);
}

// Dynamic LDS: [0, cand_cap) candidates while scanning, then the bitmap.  In the tail the
// first K_CAP slots hold the sorted candidates and the three float arrays follow them
// (the launcher sizes the region for at least K_CAP * 8 + 3 * K_CAP * 4 bytes).
__device__ __forceinline__ void tail_arrays(Shared& sh) {
    float* f = reinterpret_cast<float*>(dyn_lds + K_CAP);
    sh.prob = f;
    sh.cum = f + K_CAP;
    sh.res = f + 2 * K_CAP;
}

template <int DT, int KIND, bool LSE>
__global__ __launch_bounds__(NT, KIND == 1 ? 3 : 4) void k_rows_inline(InlineRows rows, LaunchCfg cfg) {
    __shared__ Shared sh;
    // `rows` is the first kernel argument: index it in the kernel-argument segment itself
    // (indexing the by-value copy would move all of it to scratch memory).
    const LILY_CONST RowArgs* table =
        (const LILY_CONST RowArgs*)__builtin_amdgcn_kernarg_segment_ptr();
    if (threadIdx.x == 0) {
        tail_arrays(sh);
    }
    __syncthreads();
    row_body<DT, KIND, LSE>(table + blockIdx.y, cfg, sh);
}

// Rows that draw in order (the verify pass under penalties): see row_body.
template <int DT, int KIND>
__global__ __launch_bounds__(NT, KIND == 1 ? 3 : 4) void k_rows_chain(InlineRows rows, LaunchCfg cfg) {
    __shared__ Shared sh;
    const LILY_CONST RowArgs* table =
        (const LILY_CONST RowArgs*)__builtin_amdgcn_kernarg_segment_ptr();
    if (threadIdx.x == 0) {
        tail_arrays(sh);
    }
    __syncthreads();
    row_body<DT, KIND, false, true>(table + blockIdx.y, cfg, sh);
}

template <int DT, int KIND, bool LSE>
__global__ __launch_bounds__(NT, KIND == 1 ? 3 : 4) void k_rows_table(LaunchCfg cfg) {
    __shared__ Shared sh;
    const LILY_CONST RowArgs* table = (const LILY_CONST RowArgs*)cfg.table;
    if (threadIdx.x == 0) {
        tail_arrays(sh);
    }
    __syncthreads();
    row_body<DT, KIND, LSE>(table + blockIdx.y, cfg, sh);
}

template <int DT, int KIND, bool LSE>
static hipError_t launch_variant(hipStream_t stream, uint32_t rows, const LaunchCfg& cfg,
                                 const InlineRows* inline_rows, size_t dyn_bytes) {
    const dim3 grid(cfg.slices, rows), block(NT);
    if (cfg.chain_rows != 0u) {
        if constexpr (!LSE) {
            if (inline_rows != nullptr) {
                hipLaunchKernelGGL((k_rows_chain<DT, KIND>), grid, block, dyn_bytes, stream, *inline_rows, cfg);
                return hipGetLastError();
            }
        }
        return hipErrorInvalidValue;   // rows that draw in order travel inline and want no row sum
    }
    if (inline_rows != nullptr) {
        hipLaunchKernelGGL((k_rows_inline<DT, KIND, LSE>), grid, block, dyn_bytes, stream,
                           *inline_rows, cfg);
    } else {
        hipLaunchKernelGGL((k_rows_table<DT, KIND, LSE>), grid, block, dyn_bytes, stream, cfg);
    }
    return hipGetLastError();
}

}  // namespace lily
