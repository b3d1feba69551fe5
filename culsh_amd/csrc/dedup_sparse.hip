// Candidate de-duplication for queries whose candidates are few for the index's row range.
//
// query_from_matched_buckets (core/query.cuh:290-478) hands back, per query, the ascending list of
// distinct rows of the matched buckets.  The bitmap kernel of query.hip marks rows in a bitmap over
// the row range and sweeps it; beyond 2^20 rows that takes several passes per query, each with a
// fixed cost, whatever the query holds.  Here the bitmap has two levels and one pass:
//
//   level 1   one bit per block of 32 rows (n / 1024 words), marked by every candidate row;
//   rank      a prefix sum over level 1 numbers the non-empty blocks in row order;
//   level 2   one entry per non-empty block, at the block's rank: the block's number and a 32-bit
//             word of row bits, both set by one 64-bit OR per candidate row on a second walk over the
//             rows (rank = prefix of the level-1 word + bits below the block's bit);
//   read-out  the level-2 entries in rank order are the ascending duplicate-free list.
//
// The cost follows the number of candidates (two marks per raw candidate, one sweep over the
// non-empty blocks), not the row range: level 1 of 4M rows is 4096 words.  Level 2 holds `cap`
// blocks; a query with more non-empty blocks takes several rank ranges one after the other (counted
// first, then stored).
//
// Lists are packed by the same chained scan over the queries as in the bitmap kernel, so nothing is
// copied afterwards.  A query's count is published as soon as its level 2 is complete, and its rows
// are lined up in level 2's own memory; where its list starts (the sum of all earlier counts) is
// only asked for after the level-1 walk of the workgroup's next query, which needs neither level 2
// nor the answer: by then the earlier queries, which other workgroups work on at the same time,
// have published their counts, and the look-back does not wait.
#include "block_utils.hpp"
#include "common.hpp"
#include "dedup_common.hpp"

namespace culsh_amd {
namespace {

constexpr int SP_STEP = 256;      // level-2 entries a wavefront reads per step (four per lane)
constexpr int SP_MAX_STEPS = 4;   // steps per wavefront and rank range; bounds `cap` to NWAVES * 4 * 256 entries
#ifndef SP_REG
#define SP_REG 40                 // pieces per wavefront of a query whose rows stay in registers (49152 rows per query)
#endif

__global__ __launch_bounds__(DD_THREADS) void dedup_sparse_kernel(SparseDedupArgs a) {
    extern __shared__ uint32_t lds[];
    const int T = a.T, tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int k1 = a.l1_per_thread;
    const uint32_t cap = static_cast<uint32_t>(a.cap);
    const int2* __restrict__ spans = static_cast<const int2*>(a.spans);
    uint2* l1 = reinterpret_cast<uint2*>(lds);  // [DD_THREADS * k1] x: block bits, y: non-empty blocks before this word
    uint2* pb = l1 + DD_THREADS * k1;           // [cap] x: block number, y: the block's row bits
    unsigned long long* sh_base = reinterpret_cast<unsigned long long*>(pb + cap);  // [1]
    int* sh_q = reinterpret_cast<int*>(sh_base + 1);                                // [2]
    int2* tab = reinterpret_cast<int2*>(sh_base + 2);                               // [DD_THREADS]
    int* s_start = reinterpret_cast<int*>(tab + DD_THREADS);                        // [T]
    int* s_len = s_start + T;                                                       // [T]
    uint32_t* s_ppref = reinterpret_cast<uint32_t*>(s_len + T);                     // [T + 1]
    uint32_t* scratch = s_ppref + T + 1;                                            // [17]
    uint32_t* wtot = scratch + 17;                                                  // [NWAVES + 1]

#define SP_TICK(k)                                                             \
    if (a.ticks && tid == 0) {                                                 \
        const unsigned long long now_ = wall_clock64();                        \
        a.ticks[static_cast<size_t>(blockIdx.x) * 8 + (k)] += now_ - tick_;    \
        tick_ = now_;                                                          \
    }
    unsigned long long tick_ = a.ticks ? wall_clock64() : 0ull;

    // Workgroups stay resident and take queries in order from a ticket counter, so every predecessor
    // of a query in the chained scan has been taken by a running workgroup.
    if (tid == 0) *sh_q = static_cast<int>(atomicAdd(a.ticket, 1u));
    {
        uint4* z = reinterpret_cast<uint4*>(lds);
        const int n16 = (DD_THREADS * k1 + static_cast<int>(cap)) / 2;
        for (int i = tid; i < n16; i += DD_THREADS) z[i] = make_uint4(0u, 0u, 0u, 0u);
    }
    __syncthreads();
    // `q` numbers the units of the chained scan: queries, or positions in the list of active queries
    const int n_units = a.active ? static_cast<int>(*a.n_active) : a.n_queries;
    auto query_of = [&](int unit) { return a.active ? a.active[unit] : unit; };
    int q = *sh_q;
    if (q >= n_units) return;
    int2 sp = make_int2(0, 0);
    if (tid < T) sp = spans[static_cast<size_t>(query_of(q)) * T + tid];

    // The query whose rows are lined up in level 2 and wait for the position of their list.
    bool pending = false;
    int pend_q = 0;
    uint32_t pend_pw = 0, pend_total = 0, pend_wave_base = 0;
    uint32_t pend_step[SP_MAX_STEPS] = {0u, 0u, 0u, 0u};  // rows of this wavefront's steps

    auto step_room = [&](uint32_t pw, int j) {  // words of level 2 from the step's first entry on, at most the step's own
        const uint32_t first = static_cast<uint32_t>(wave) * pw + static_cast<uint32_t>(j * SP_STEP);
        return first < cap ? 2u * min(static_cast<uint32_t>(SP_STEP), cap - first) : 0u;
    };
    // First wavefront: the list position of query `qq` with `total` rows, into *sh_base (~0: no room).
    auto place_list = [&](int qq, unsigned long long total) {
        const unsigned long long excl = look_back(a.state, qq, total, a.spin_limit, a.err);
        if (lane == 0) {
            unsigned long long b = excl;
            if (excl + total > a.capacity) {
                atomicOr(a.err, 2u);
                b = ~0ull;
            }
            *sh_base = b;
            const int id = query_of(qq);
            a.counts[id] = total;
            if (!a.active) {  // (with a list of active queries the offsets come from a scan over the counts)
                a.offsets[id] = excl;
                if (qq == n_units - 1) a.offsets[a.n_queries] = excl + total;
            }
        }
    };
    // Stores this wavefront's steps of a rank range whose rows are lined up (or, for a step with more
    // rows than its place held, still sit in their entries) and leaves the entries clean.
    auto copy_out = [&](uint32_t pw, const uint32_t (&st_total)[SP_MAX_STEPS], int32_t* dst, bool store) {
        const int steps = static_cast<int>(pw / SP_STEP);
        __builtin_amdgcn_wave_barrier();  // LDS accesses of one wavefront complete in order
#pragma unroll
        for (int j = 0; j < SP_MAX_STEPS; ++j) {
            if (j >= steps) continue;
            const uint32_t i0 = static_cast<uint32_t>(wave) * pw + static_cast<uint32_t>(j * SP_STEP);
            if (store) {
                if (st_total[j] <= step_room(pw, j)) {
                    const uint32_t* lined = reinterpret_cast<const uint32_t*>(pb + i0);
                    for (uint32_t i = lane; i < st_total[j]; i += 64) dst[i] = static_cast<int32_t>(lined[i]);
                } else {  // dense step: every lane stores the rows of its own four entries
                    uint4 v0 = make_uint4(0u, 0u, 0u, 0u), v1 = make_uint4(0u, 0u, 0u, 0u);
                    if (i0 + static_cast<uint32_t>(lane * 4) < cap) {  // entries behind level 2's end do not exist
                        v0 = *reinterpret_cast<const uint4*>(pb + i0 + lane * 4);
                        v1 = *reinterpret_cast<const uint4*>(pb + i0 + lane * 4 + 2);
                    }
                    const uint32_t blk[4] = {v0.x, v0.z, v1.x, v1.z}, bits[4] = {v0.y, v0.w, v1.y, v1.w};
                    const uint32_t c = __popc(bits[0]) + __popc(bits[1]) + __popc(bits[2]) + __popc(bits[3]);
                    uint32_t pos = wave_inclusive_sum_dpp(c) - c;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        uint32_t left = bits[k];
                        const uint32_t r0 = blk[k] << 5;
                        while (left) {
                            dst[pos++] = static_cast<int32_t>(r0 + static_cast<uint32_t>(__ffs(static_cast<int>(left)) - 1));
                            left &= left - 1u;
                        }
                    }
                }
            }
            dst += st_total[j];
            if (i0 + static_cast<uint32_t>(lane * 4) < cap) {  // row bits must be zero before the next marks
                uint4* z = reinterpret_cast<uint4*>(pb + i0 + lane * 4);
                z[0] = make_uint4(0u, 0u, 0u, 0u);
                z[1] = make_uint4(0u, 0u, 0u, 0u);
            }
        }
    };
    // The pending query leaves: look-back by the first wavefront, then every wavefront stores its part.
    // Contains two barriers.
    auto flush_pending = [&]() {
        if (wave == 0) place_list(pend_q, pend_total);
        __syncthreads();
        const unsigned long long base = *sh_base;
        copy_out(pend_pw, pend_step, a.out + base + pend_wave_base, base != ~0ull);
        __syncthreads();  // level 2 is clean, *sh_base may be rewritten
        pending = false;
    };

    for (;;) {
        int q_next = n_units;
        int2 sp_next = make_int2(0, 0);
        if (tid < T) {
            s_start[tid] = sp.x;
            s_len[tid] = sp.y;
        }
        number_pieces((static_cast<uint32_t>(sp.y) + 63u) >> 6, T, s_ppref, scratch);
        __syncthreads();
        const uint32_t n_pieces = s_ppref[T];
        SP_TICK(0)  // set-up

        // Level 1: every candidate row marks its block.
        // A query of at most SP_REG pieces per wavefront keeps its rows in registers between the two
        // levels, so that they are read from memory once: one piece table, every load in flight at once
        // (in groups of eight that are skipped as a whole beyond the wavefront's last piece), and both
        // levels are marked from the registers.  Lane l holds the table entry of the wavefront's l-th
        // piece; a piece's start and length reach the scalar registers through v_readlane, and a load is
        // a scalar base plus the lane's fixed offset (lanes beyond a piece's end read what follows it in
        // `cand`, which has CAND_PAD readable elements behind its last one, and skip the marks).
        auto mark_block = [&](int row) {
            const uint32_t blk = static_cast<uint32_t>(row) >> 5;
            atomicOr(&l1[blk >> 5].x, 1u << (blk & 31u));
        };
        const bool in_regs = n_pieces <= static_cast<uint32_t>(SP_REG * NWAVES);
        const bool one_round = n_pieces <= static_cast<uint32_t>(DD_THREADS);
        int2 kept = make_int2(0, 0);  // this lane's piece table entry
        int rows[SP_REG];
        const int nk = pieces_of_wave<DD_THREADS>(n_pieces, 0u);
        if (in_regs) {
            kept = piece_table<DD_THREADS>(s_start, s_len, s_ppref, T, n_pieces, 0u, tab);
            // all loads unconditionally (a piece beyond the wavefront's last one reads the start of `cand`):
            // behind branches the compiler could not tell how many younger loads may stay in flight when
            // the first rows are marked, and would wait for nearly all of them
#pragma unroll
            for (int u = 0; u < SP_REG; ++u) rows[u] = stream_fetch(a.cand, kept, u);
#pragma unroll
            for (int u0 = 0; u0 < SP_REG; u0 += 8) {
                if (u0 < nk) {
#pragma unroll
                    for (int u = u0; u < u0 + 8; ++u)
                        if (lane < __builtin_amdgcn_readlane(kept.y, u)) mark_block(rows[u]);
                }
            }
            __syncthreads();
        } else {
            stream_candidates<DD_THREADS>(a.cand, s_start, s_len, s_ppref, T, n_pieces, tab, mark_block, &kept);
        }
        SP_TICK(1)  // level-1 marks

        // Rank: thread `tid` owns the level-1 words [tid * k1, tid * k1 + k1).  Under it the previous
        // query's list leaves: its count was published a level-1 walk ago, so the first wavefront's
        // look-back finds the earlier counts in place; every wavefront then stores its part of the list.
        uint32_t mine = 0;
        for (int j = 0; j < k1; ++j) mine += __popc(l1[tid * k1 + j].x);
        uint32_t n_blocks = 0, before = 0;
        {
            const uint32_t incl = wave_inclusive_sum_dpp(mine);
            if (lane == 63) scratch[wave] = incl;
            if (pending && wave == 0) place_list(pend_q, pend_total);
            __syncthreads();
            SP_TICK(2)  // block count and look-back of the previous query
#pragma unroll
            for (int w = 0; w < NWAVES; ++w) {
                const uint32_t v = scratch[w];
                before += (w < wave) ? v : 0u;
                n_blocks += v;
            }
            before += incl - mine;
            uint32_t run = before;
            for (int j = 0; j < k1; ++j) {
                l1[tid * k1 + j].y = run;
                run += __popc(l1[tid * k1 + j].x);
            }
            if (pending) {
                const unsigned long long base = *sh_base;
                copy_out(pend_pw, pend_step, a.out + base + pend_wave_base, base != ~0ull);
                pending = false;
            }
        }
        __syncthreads();  // the prefix words are in place, level 2 is clean, scratch and *sh_base may be rewritten
        const uint32_t n_pass = n_blocks <= cap ? 1u : (n_blocks + cap - 1u) / cap;
        SP_TICK(3)  // rank, look-back and copy-out of the previous query
        // Level 2, rank range that starts at p0: a row finds its block's rank and sets its bit in the
        // block's entry; the same 64-bit OR leaves the block number there (every row of a block ORs
        // the same number into a word that was zero).
        auto mark_row = [&](int row, uint32_t p0) {
            const uint32_t blk = static_cast<uint32_t>(row) >> 5;
            const uint2 e = l1[blk >> 5];
            const uint32_t r = e.y + __popc(e.x & ((1u << (blk & 31u)) - 1u)) - p0;
            if (r < cap)
                atomicOr(reinterpret_cast<unsigned long long*>(&pb[r]),
                         (static_cast<unsigned long long>(1u << (static_cast<uint32_t>(row) & 31u)) << 32) | blk);
        };
        auto mark_rows = [&](uint32_t p0) {  // a walk over the rows in memory; ends with a barrier
            stream_candidates<DD_THREADS>(a.cand, s_start, s_len, s_ppref, T, n_pieces, tab,
                                          [&](int row) { mark_row(row, p0); }, &kept, one_round);
            if (n_pieces == 0) __syncthreads();
        };
        const bool from_regs = in_regs && n_pass == 1;
        if (from_regs) {  // the rows in registers are used up here, before the read-out needs the registers
#pragma unroll
            for (int u0 = 0; u0 < SP_REG; u0 += 8) {
                if (u0 < nk) {
#pragma unroll
                    for (int u = u0; u < u0 + 8; ++u)
                        if (lane < __builtin_amdgcn_readlane(kept.y, u)) mark_row(rows[u], 0u);
                }
            }
            __syncthreads();
        }

        unsigned long long total = 0;
        if (n_pass > 1) {
            // More non-empty blocks than level 2 holds: count every rank range first (the list's
            // position has to be known before its first row is stored), then take them again below.
            uint32_t cnt = 0;
            for (uint32_t p = 0; p < n_pass; ++p) {
                const uint32_t p0 = p * cap, m = min(cap, n_blocks - p0);
                mark_rows(p0);
                for (uint32_t i = tid; i < m; i += DD_THREADS) {
                    cnt += __popc(pb[i].y);
                    pb[i] = make_uint2(0u, 0u);  // the next rank range puts other blocks here
                }
                __syncthreads();
            }
            cnt = wave_sum(cnt);
            if (lane == 0) wtot[wave] = cnt;
            __syncthreads();
#pragma unroll
            for (int w = 0; w < NWAVES; ++w) total += wtot[w];
            if (wave == 0) {
                if (lane == 0)
                    __hip_atomic_store(&a.state[q], TAG_COUNT | total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                place_list(q, total);
            }
            __syncthreads();  // also: wtot is rewritten below
        }

        unsigned long long running = 0;  // rows of the rank ranges already stored (several ranges only)
        for (uint32_t p = 0; p < n_pass; ++p) {
            const uint32_t p0 = p * cap, m = min(cap, n_blocks - p0);
            const bool last = p == n_pass - 1u;
            if (!from_regs) mark_rows(p0);
            SP_TICK(4)  // level-2 marks
            if (last)  // level 1 is clean for the next query; nobody reads it during the read-out
                for (int j = 0; j < k1; ++j) l1[tid * k1 + j] = make_uint2(0u, 0u);

            // Read-out.  Wavefront w owns the entries [w * pw, (w + 1) * pw) of the rank range; in a step
            // every lane takes four consecutive entries: list order = (wavefront, step, lane, entry, bit).
            const uint32_t pw = ((m + NWAVES - 1u) / NWAVES + (SP_STEP - 1u)) & ~static_cast<uint32_t>(SP_STEP - 1);
            const int steps = static_cast<int>(pw / SP_STEP);  // <= SP_MAX_STEPS
            unsigned int ticket_next = 0;
            if (last && tid == 0) ticket_next = atomicAdd(a.ticket, 1u);  // arrives while the rows are lined up
            // Line-up, step by step: a step's entries go to registers, which frees their place (two words
            // per entry): the rows are written there in list order, ready for full-width stores.  A step
            // with more rows than its place holds stays as it is.
            uint32_t st_total[SP_MAX_STEPS];
#pragma unroll
            for (int j = 0; j < SP_MAX_STEPS; ++j) {
                st_total[j] = 0u;
                if (j >= steps) continue;
                uint4 v0 = make_uint4(0u, 0u, 0u, 0u), v1 = make_uint4(0u, 0u, 0u, 0u);
                const uint32_t i0 = static_cast<uint32_t>(wave) * pw + static_cast<uint32_t>(j * SP_STEP + lane * 4);
                if (i0 < cap) {  // entries behind the range hold no bits
                    v0 = *reinterpret_cast<const uint4*>(pb + i0);
                    v1 = *reinterpret_cast<const uint4*>(pb + i0 + 2);
                }
                const uint32_t blk[4] = {v0.x, v0.z, v1.x, v1.z}, bits[4] = {v0.y, v0.w, v1.y, v1.w};
                const uint32_t c = __popc(bits[0]) + __popc(bits[1]) + __popc(bits[2]) + __popc(bits[3]);
                const uint32_t incl = wave_inclusive_sum_dpp(c);
                st_total[j] = __shfl(incl, 63, 64);
                if (st_total[j] <= step_room(pw, j)) {
                    __builtin_amdgcn_wave_barrier();  // every lane has its entries before the first row lands on them
                    uint32_t* slot = reinterpret_cast<uint32_t*>(pb + static_cast<uint32_t>(wave) * pw + j * SP_STEP) + (incl - c);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        uint32_t left = bits[k];
                        const uint32_t r0 = blk[k] << 5;
                        while (left) {
                            *slot++ = r0 + static_cast<uint32_t>(__ffs(static_cast<int>(left)) - 1);
                            left &= left - 1u;
                        }
                    }
                }
            }
            if (lane == 0) wtot[wave] = st_total[0] + st_total[1] + st_total[2] + st_total[3];
            if (last && wave == 0) {
                const int qn = min(static_cast<int>(__shfl(ticket_next, 0, 64)), n_units);
                if (T <= 64 && qn < n_units && lane < T) sp_next = spans[static_cast<size_t>(query_of(qn)) * T + lane];
                if (lane == 0) *sh_q = qn;
            }
            SP_TICK(5)  // load, line-up
            __syncthreads();  // all rows are lined up; the wavefronts' totals and *sh_q are in place
            uint32_t wave_base = 0, chunk_total = 0;
#pragma unroll
            for (int w = 0; w < NWAVES; ++w) {
                const uint32_t v = wtot[w];
                wave_base += (w < wave) ? v : 0u;
                chunk_total += v;
            }
            wave_base = __builtin_amdgcn_readfirstlane(wave_base);
            chunk_total = __builtin_amdgcn_readfirstlane(chunk_total);
            if (n_pass == 1) {
                // The count is published now; the list leaves after the next query's level-1 walk (or after
                // the last query), when the look-back finds the earlier queries' counts in place.
                if (tid == 0)
                    __hip_atomic_store(&a.state[q], TAG_COUNT | static_cast<unsigned long long>(chunk_total),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                pending = true;
                pend_q = q;
                pend_pw = pw;
                pend_total = chunk_total;
                pend_wave_base = wave_base;
#pragma unroll
                for (int j = 0; j < SP_MAX_STEPS; ++j) pend_step[j] = st_total[j];
            } else {
                const unsigned long long base = *sh_base;
                copy_out(pw, st_total, a.out + base + running + wave_base, base != ~0ull);
                running += chunk_total;
                __syncthreads();  // level 2 and wtot are rewritten by the next rank range / query
            }
            SP_TICK(6)  // totals
            if (last) q_next = *sh_q;
        }
        if (q_next >= n_units) break;
        q = q_next;
        if (T <= 64) {
            sp = sp_next;  // zero outside the first T lanes
        } else {
            sp = make_int2(0, 0);
            if (tid < T) sp = spans[static_cast<size_t>(query_of(q)) * T + tid];
        }
    }
    if (pending) flush_pending();
    SP_TICK(7)
#undef SP_TICK
}

// The queries with at least one non-empty span, in ascending order.  First every query is looked at (one thread
// each, `flags[q]` = it has a candidate; `counts[q]` is zeroed on the way), then a single workgroup writes the
// list: that keeps the order without a scan across workgroups, and reading one flag per query is short work.
__global__ __launch_bounds__(256) void active_flags_kernel(const int2* __restrict__ spans, int n_queries, int T,
                                                          uint32_t* __restrict__ flags, uint64_t* __restrict__ counts) {
    const int q = blockIdx.x * 256 + threadIdx.x;
    if (q >= n_queries) return;
    const int2* s = spans + static_cast<size_t>(q) * T;
    int most = 0;
    for (int t = 0; t < T; ++t) most = max(most, s[t].y);
    flags[q] = most > 0 ? 1u : 0u;
    counts[q] = 0;
}

constexpr int AQ_PER_THREAD = 4;
__global__ __launch_bounds__(DD_THREADS) void active_queries_kernel(const uint32_t* __restrict__ flags, int n_queries,
                                                                   int32_t* __restrict__ active,
                                                                   unsigned int* __restrict__ n_active) {
    __shared__ uint32_t wave_count[NWAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t done = 0;  // active queries before this round's
    for (int base = 0; base < n_queries; base += DD_THREADS * AQ_PER_THREAD) {
        // thread `tid` looks at AQ_PER_THREAD consecutive queries, so that list order = thread order
        const int q0 = base + tid * AQ_PER_THREAD;
        uint32_t mask = 0;
#pragma unroll
        for (int j = 0; j < AQ_PER_THREAD; ++j)
            if (q0 + j < n_queries && flags[q0 + j]) mask |= 1u << j;
        const uint32_t mine = __popc(mask);
        const uint32_t incl = wave_inclusive_sum_dpp(mine);
        if (lane == 63) wave_count[wave] = incl;
        __syncthreads();
        uint32_t before = done, total = 0;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) {
            const uint32_t v = wave_count[w];
            before += (w < wave) ? v : 0u;
            total += v;
        }
        uint32_t pos = before + incl - mine;
#pragma unroll
        for (int j = 0; j < AQ_PER_THREAD; ++j)
            if (mask & (1u << j)) active[pos++] = q0 + j;
        done += total;
        __syncthreads();  // wave_count is rewritten in the next round
    }
    if (tid == 0) *n_active = done;
}

size_t fixed_lds(int T) {
    return (4 + 2 * DD_THREADS + 3 * static_cast<size_t>(T) + 1 + 17 + (NWAVES + 1) + 8) * sizeof(uint32_t);
}

}  // namespace

bool sparse_dedup_geometry(const culsh_ctx* ctx, int n_rows, int T, int cap_limit, SparseDedupGeometry* g) {
    const long long rows_per_l1_thread = 32ll * 32ll * DD_THREADS;  // rows covered by one level-1 word per thread
    const long long k1 = (static_cast<long long>(n_rows) + rows_per_l1_thread - 1) / rows_per_l1_thread;
    const size_t l1_bytes = static_cast<size_t>(k1) * DD_THREADS * sizeof(uint2);
    const size_t fixed = fixed_lds(T);
    if (l1_bytes + fixed + 4096 * sizeof(uint2) > static_cast<size_t>(ctx->lds_max)) return false;
    size_t cap = (static_cast<size_t>(ctx->lds_max) - l1_bytes - fixed) / sizeof(uint2);
    cap = std::min<size_t>(cap, static_cast<size_t>(NWAVES) * SP_MAX_STEPS * SP_STEP);
    if (cap_limit > 0) cap = std::min<size_t>(cap, static_cast<size_t>(cap_limit));
    cap &= ~static_cast<size_t>(3);
    if (cap < 4) return false;
    g->l1_per_thread = static_cast<int>(k1);
    g->cap = static_cast<int>(cap);
    g->lds_bytes = l1_bytes + cap * sizeof(uint2) + fixed;
    return true;
}

culsh_status launch_active_queries(culsh_ctx* ctx, const void* spans, int n_queries, int T, int32_t* active,
                                   unsigned int* n_active, uint64_t* counts) {
    CULSH_REQUIRE(spans && active && n_active && counts && n_queries > 0 && n_queries <= MAX_COMPACT_QUERIES && T > 0,
                  CULSH_ERR_INTERNAL, "active queries: bad argument");
    uint32_t* flags = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n_queries), &flags));
    CULSH_LAUNCH(ctx, active_flags_kernel, dim3(div_up(static_cast<size_t>(n_queries), 256)), dim3(256), 0, ctx->stream,
                 static_cast<const int2*>(spans), n_queries, T, flags, counts);
    CULSH_LAUNCH_CHECK();
    CULSH_LAUNCH(ctx, active_queries_kernel, dim3(1), dim3(DD_THREADS), 0, ctx->stream, flags, n_queries, active, n_active);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status launch_dedup_sparse(culsh_ctx* ctx, const SparseDedupArgs& a, const SparseDedupGeometry& g) {
    static PerDeviceOnce allowed;  // more LDS than a launch may ask for by default: allowed once per device
    if (!allowed.is_set(ctx->device)) {
        CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dedup_sparse_kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, ctx->lds_max));
        allowed.set(ctx->device);
    }
    CULSH_REQUIRE(a.l1_per_thread == g.l1_per_thread && a.cap == g.cap && g.lds_bytes <= static_cast<size_t>(ctx->lds_max),
                  CULSH_ERR_INTERNAL, "sparse de-duplication: geometry mismatch");
    const int per_cu = static_cast<int>(std::max<size_t>(1, std::min<size_t>(2, static_cast<size_t>(ctx->lds_max) / g.lds_bytes)));
    const int resident = std::max(1, ctx->n_cus * per_cu);
    CULSH_LAUNCH(ctx, dedup_sparse_kernel, dim3(std::min(a.n_queries, resident)), dim3(DD_THREADS), g.lds_bytes,
                 ctx->stream, a);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

}  // namespace culsh_amd
