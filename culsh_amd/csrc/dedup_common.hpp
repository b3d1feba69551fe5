// Device helpers shared by the candidate de-duplication kernels: walking the row ids of a query's
// bucket spans, numbering the spans' pieces, and the chained scan over the queries' counts.
#pragma once

#include "block_utils.hpp"
#include "common.hpp"

namespace culsh_amd {

constexpr int DD_THREADS = 1024;
constexpr int NWAVES = DD_THREADS / 64;
constexpr int WALK_U = 16;   // pieces in flight per wavefront (walk_candidates)
constexpr int STREAM_U = 8;  // pieces in flight per wavefront (stream_candidates)

// Visits every row id of the query's spans.  The spans are cut into pieces of up to 64
// consecutive ids (a piece never crosses a span boundary), pieces are dealt round-robin to
// the wavefronts, and a wavefront reads a piece with one load per lane.  Where piece p
// starts is looked up once per piece (one binary search per thread over the spans'
// piece counts, all pieces of a round in parallel) and kept in `tab`, so the per-lane
// work is an add, a compare and the load.  `f` is also called with -1, for the lanes beyond a
// piece's end, and must ignore it.  Contains barriers: all threads must call it.
template <typename F>
__device__ __forceinline__ void walk_candidates(const int32_t* __restrict__ cand, const int* s_start,
                                                const int* s_len, const uint32_t* s_ppref, int T,
                                                uint32_t n_pieces, int2* tab, F&& f) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in every lane: kept in a scalar register
    for (uint32_t r0 = 0; r0 < n_pieces; r0 += DD_THREADS) {
        const uint32_t pc = r0 + static_cast<uint32_t>(tid);
        if (pc < n_pieces) {
            int tl = 0, th = T;  // largest t with s_ppref[t] <= pc; that span owns the piece
            while (th - tl > 1) {
                const int mid = (tl + th) >> 1;
                if (s_ppref[mid] <= pc) tl = mid; else th = mid;
            }
            const int first = static_cast<int>(pc - s_ppref[tl]) * 64;
            tab[tid] = make_int2(s_start[tl] + first, min(64, s_len[tl] - first));
        }
        __syncthreads();
        const uint32_t here = min(static_cast<uint32_t>(DD_THREADS), n_pieces - r0);
        for (uint32_t p0 = wave; p0 < here; p0 += NWAVES * WALK_U) {
            // table entries of all pieces first (one LDS round trip instead of one per piece), then the loads
            int rows[WALK_U];
            int2 ent[WALK_U];
#pragma unroll
            for (int u = 0; u < WALK_U; ++u) ent[u] = tab[min(p0 + u * NWAVES, here - 1u)];
#pragma unroll
            for (int u = 0; u < WALK_U; ++u) {
                const uint32_t pi = p0 + u * NWAVES;
                rows[u] = -1;
                if (pi < here && lane < ent[u].y) rows[u] = cand[static_cast<uint32_t>(ent[u].x + lane)];  // unsigned: no sign extension per load
            }
#pragma unroll
            for (int u = 0; u < WALK_U; ++u) f(rows[u]);  // -1 where the lane has no row: f tells by its range check
        }
        __syncthreads();  // tab is rewritten by the next round
    }
}

// The same visit with loads that never drain: a wavefront keeps STREAM_U pieces in flight and, as soon as
// it has taken a piece's rows out of their register, fetches the piece STREAM_U places further on into
// it, so the walk costs one memory latency plus the work per piece instead of one latency per STREAM_U
// pieces.  Lane l holds the table entry of the wavefront's l-th piece of the round (one LDS read per
// round); a piece's start and length reach the scalar registers through v_readlane, so a load is a
// scalar base plus the lane's fixed offset and costs no vector arithmetic.  Every load is issued
// unconditionally and for all 64 lanes: lanes beyond a piece's end read what follows it in `cand`
// (which therefore has CAND_PAD readable elements behind its last one) and pieces beyond the last one
// read the start of `cand`; their values are dropped.  With loads behind branches the compiler could no
// longer count how many younger loads may stay in flight at a use and would wait for all of them.
// `f` is called for the lanes that hold a row only (never with -1).
// THREADS: size of the workgroup (a multiple of 64); `tab` holds THREADS entries.
// The piece table of the round that starts at piece r0: fills `tab` and hands every lane the entry of the
// wavefront's lane-th piece (length 0: no such piece).  One barrier inside; all threads must call it.
// THREADS: size of the workgroup (a multiple of 64); `tab` holds THREADS entries.
template <int THREADS>
__device__ __forceinline__ int2 piece_table(const int* s_start, const int* s_len, const uint32_t* s_ppref, int T,
                                            uint32_t n_pieces, uint32_t r0, int2* tab) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t pc = r0 + static_cast<uint32_t>(tid);
    if (pc < n_pieces) {
        int tl = 0, th = T;  // largest t with s_ppref[t] <= pc; that span owns the piece
        while (th - tl > 1) {
            const int mid = (tl + th) >> 1;
            if (s_ppref[mid] <= pc) tl = mid; else th = mid;
        }
        const int first = static_cast<int>(pc - s_ppref[tl]) * 64;
        tab[tid] = make_int2(s_start[tl] + first, min(64, s_len[tl] - first));
    }
    __syncthreads();
    const uint32_t here = min(static_cast<uint32_t>(THREADS), n_pieces - r0);
    const uint32_t pi = static_cast<uint32_t>(wave + lane * (THREADS / 64));
    return pi < here ? tab[pi] : make_int2(0, 0);
}

// pieces of this wavefront in the round that starts at piece r0 (at most 64)
template <int THREADS>
__device__ __forceinline__ int pieces_of_wave(uint32_t n_pieces, uint32_t r0) {
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) >> 6);
    const uint32_t here = n_pieces > r0 ? min(static_cast<uint32_t>(THREADS), n_pieces - r0) : 0u;
    return here > static_cast<uint32_t>(wave) ? static_cast<int>((here - wave + THREADS / 64 - 1) / (THREADS / 64)) : 0;
}

// the rows of the wavefront's k-th piece (k < 64, the same in all lanes): one load per lane, unconditional
__device__ __forceinline__ int stream_fetch(const int32_t* __restrict__ cand, const int2& mine, int k) {
    const int32_t* piece = cand + static_cast<uint32_t>(__builtin_amdgcn_readlane(mine.x, k));
    return piece[threadIdx.x & 63];
}

// `kept` (optional): the caller's copy of the wavefront's table entries.  A walk of a single round
// (n_pieces <= THREADS) leaves them there, and a later walk over the same spans that is handed them
// back skips the piece table and its barrier (`reuse` = true; the caller places a barrier between the
// walks if the work of `f` needs one).
template <int THREADS, typename F>
__device__ __forceinline__ void stream_candidates(const int32_t* __restrict__ cand, const int* s_start,
                                                  const int* s_len, const uint32_t* s_ppref, int T,
                                                  uint32_t n_pieces, int2* tab, F&& f, int2* kept = nullptr,
                                                  bool reuse = false) {
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (uint32_t r0 = 0; r0 < n_pieces; r0 += THREADS) {
        const uint32_t here = min(static_cast<uint32_t>(THREADS), n_pieces - r0);
        int2 mine = make_int2(0, 0);  // length 0: no such piece
        if (reuse) {
            mine = *kept;
        } else {
            const uint32_t pc = r0 + static_cast<uint32_t>(tid);
            if (pc < n_pieces) {
                int tl = 0, th = T;  // largest t with s_ppref[t] <= pc; that span owns the piece
                while (th - tl > 1) {
                    const int mid = (tl + th) >> 1;
                    if (s_ppref[mid] <= pc) tl = mid; else th = mid;
                }
                const int first = static_cast<int>(pc - s_ppref[tl]) * 64;
                tab[tid] = make_int2(s_start[tl] + first, min(64, s_len[tl] - first));
            }
            __syncthreads();
            const uint32_t pi = static_cast<uint32_t>(wave + lane * (THREADS / 64));
            if (pi < here) mine = tab[pi];
            if (kept) *kept = mine;
        }
        const int nk = here > static_cast<uint32_t>(wave) ? static_cast<int>((here - wave + THREADS / 64 - 1) / (THREADS / 64)) : 0;  // pieces of this wavefront, <= 64
        auto fetch = [&](int k) {  // k < 64, the same in all lanes
            const int32_t* piece = cand + static_cast<uint32_t>(__builtin_amdgcn_readlane(mine.x, k));
            return piece[lane];
        };
        int rows[STREAM_U];
#pragma unroll
        for (int u = 0; u < STREAM_U; ++u) rows[u] = fetch(u);
        for (int k0 = 0; k0 < nk; k0 += STREAM_U) {
#pragma unroll
            for (int u = 0; u < STREAM_U; ++u) {
                // the rows are used up before their register takes the next load: fetched into another
                // register while these are still needed, they would have to be copied back at the end of
                // every round of the loop, and the copies wait for all loads in flight
                const int len = __builtin_amdgcn_readlane(mine.y, k0 + u);  // 0 beyond the wavefront's last piece
                if (lane < len) f(rows[u]);
                rows[u] = fetch((k0 + STREAM_U + u) & 63);
            }
        }
        __syncthreads();  // tab is rewritten by the next round
    }
}

// Piece numbering of the spans handed to walk_candidates: s_ppref[t] = pieces of the spans before t,
// s_ppref[T] = all pieces.  `pieces` is the piece count of span threadIdx.x (0 beyond the T-th thread).
// Up to 64 spans sit in the first wavefront, which then does it alone, without a barrier; all threads
// must call it, and a barrier has to follow before s_ppref is read.
__device__ __forceinline__ void number_pieces(uint32_t pieces, int T, uint32_t* s_ppref, uint32_t* scratch) {
    const int tid = threadIdx.x;
    if (T <= 64) {
        if (tid < 64) {
            const uint32_t incl = wave_inclusive_sum_dpp(pieces);
            if (tid < T) s_ppref[tid] = incl - pieces;
            if (tid == 63) s_ppref[T] = incl;
        }
    } else {
        uint32_t total;
        const uint32_t ex = block_exclusive_sum(pieces, scratch, &total);
        if (tid < T) s_ppref[tid] = ex;
        if (tid == 0) s_ppref[T] = total;
    }
}

// Chained scan over the queries' counts.  A published word holds a 2-bit tag and a value:
// tag 1 = this query's count, tag 2 = sum of the counts of queries 0..q.  The caller (one
// full wavefront) has published its count; here it sums its predecessors' counts back to
// the nearest running sum, then publishes its own running sum.  Workgroups start in index order, so the
// lowest unfinished query never waits on one that has not started; the poll count is
// bounded all the same and a give-up is reported through `err`.
constexpr unsigned long long TAG_COUNT = 1ull << 62, TAG_SUM = 2ull << 62, TAG_VALUE = TAG_COUNT - 1ull;

__device__ __forceinline__ unsigned long long look_back(unsigned long long* state, int q, unsigned long long total,
                                                        int spin_limit, unsigned int* err) {
    const int lane = threadIdx.x & 63;
    unsigned long long excl = 0;
    int hi = q;  // queries [0, hi) are not accounted for yet
    int polls = 0;
    bool gave_up = false;
    while (hi > 0) {
        const int idx = hi - 1 - lane;  // lane 0 looks at the nearest predecessor
        const unsigned long long v =
            idx >= 0 ? __hip_atomic_load(&state[idx], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : TAG_SUM;
        const unsigned tag = static_cast<unsigned>(v >> 62);
        const unsigned long long has_sum = __ballot(tag == 2u), unpublished = __ballot(tag == 0u);
        const int f = has_sum ? __ffsll(static_cast<long long>(has_sum)) - 1 : 64;  // nearest running sum
        const unsigned long long needed = f >= 63 ? ~0ull : ((2ull << f) - 1ull);  // lanes 0..f
        if (unpublished & needed) {
            if (++polls > spin_limit) { gave_up = true; break; }
            __builtin_amdgcn_s_sleep(2);
            continue;
        }
        excl += wave_sum((lane <= f) ? (v & TAG_VALUE) : 0ull);
        if (f < 64) break;
        hi -= 64;
    }
    if (gave_up) {
        if (lane == 0) atomicOr(err, 1u);
        excl = 0;
    }
    if (lane == 0) __hip_atomic_store(&state[q], TAG_SUM | (excl + total), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return excl;
}

}  // namespace culsh_amd
