// Candidate retrieval on gfx950.
//
// Bucket lookup follows find_matching_buckets_kernel (core/query.cuh:31-101).  The tail
// (core/query.cuh:290-478) produces, per query, the ascending list of distinct row ids
// found in the matched buckets.  The reference gathers all raw candidates, sorts every
// query's segment with a 32-bit segmented radix sort, flags, reduces, scans and compacts.
// Here one workgroup owns a query and marks the row ids of its bucket spans in a bitmap
// held in LDS (up to 2^20 rows per pass of 128 KiB); reading the bitmap in order yields
// the ascending duplicate-free list directly, so raw candidates are never written to
// memory and nothing is sorted.  A first launch counts, a scan places the queries, a
// second launch emits; memory use is O(unique candidates).
#include <algorithm>
#include <cstdlib>

#include "block_utils.hpp"
#include "common.hpp"

namespace culsh_amd {
namespace {

constexpr int DD_THREADS = 1024;

__global__ __launch_bounds__(256) void lookup_kernel(const uint32_t* __restrict__ q_keys,
                                                    const uint32_t* __restrict__ bucket_keys,
                                                    const int32_t* __restrict__ table_bucket_offsets,
                                                    int n_queries, int T, int W, int32_t* __restrict__ matched) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= static_cast<size_t>(n_queries) * T) return;
    const int q = static_cast<int>(idx / T), t = static_cast<int>(idx - static_cast<size_t>(q) * T);
    const uint32_t* key = q_keys + (static_cast<size_t>(t) * n_queries + q) * W;
    int lo = table_bucket_offsets[t], hi = table_bucket_offsets[t + 1] - 1;
    int found = -1;
    while (lo <= hi) {
        const int mid = lo + ((hi - lo) >> 1);
        const uint32_t* m = bucket_keys + static_cast<size_t>(mid) * W;
        int cmp = 0;
        for (int w = 0; w < W && cmp == 0; ++w) cmp = (key[w] > m[w]) - (key[w] < m[w]);
        if (cmp == 0) { found = mid; break; }
        if (cmp < 0) hi = mid - 1; else lo = mid + 1;
    }
    matched[idx] = found;
}

struct DedupArgs {
    const int32_t* matched;                   // [n_queries][T]
    const int32_t* bucket_candidate_offsets;  // [B+1]
    const int32_t* cand;                      // all_candidate_indices
    const uint64_t* offsets;                  // EMIT: per-query output offsets
    uint64_t* counts;                         // COUNT: per-query unique counts
    int32_t* out;                             // EMIT: candidate indices
    int T, n;
    int wpt;       // bitmap words per thread (power of two); a pass covers DD_THREADS*wpt*32 rows
    int n_chunks;  // passes over the row range
    unsigned long long* ticks;  // optional [8] phase timers (wall clock ticks of thread 0), or null
};

constexpr int NWAVES = DD_THREADS / 64;
constexpr int WALK_U = 8;              // 64-row segments in flight per wavefront
constexpr uint32_t ROUND = DD_THREADS * 64u;  // flat candidates per segment-table round

// Visits every row id of the concatenated spans ("flat" order: span 0, span 1, ...), 64
// consecutive ids per wavefront step so that no lane idles on short spans.  The span that
// owns the first id of every 64-id segment is looked up once per segment (one binary
// search per thread, all segments in parallel) and kept in `lut`; lanes then only step
// forward over span boundaries.  Contains barriers: all threads must call it.
template <typename F>
__device__ __forceinline__ void walk_candidates(const int32_t* __restrict__ cand, const int* s_start,
                                                const uint32_t* s_pref, int T, uint32_t total, uint32_t* lut,
                                                F&& f) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (uint32_t r0 = 0; r0 < total; r0 += ROUND) {
        const uint32_t fseg = r0 + static_cast<uint32_t>(tid) * 64u;
        if (fseg < total) {
            int tl = 0, th = T;  // largest t with s_pref[t] <= fseg
            while (th - tl > 1) {
                const int mid = (tl + th) >> 1;
                if (s_pref[mid] <= fseg) tl = mid; else th = mid;
            }
            lut[tid] = static_cast<uint32_t>(tl);
        }
        __syncthreads();
        const uint32_t nseg = min(static_cast<uint32_t>(DD_THREADS), (total - r0 + 63u) >> 6);
        for (uint32_t seg0 = wave; seg0 < nseg; seg0 += NWAVES * WALK_U) {
            int rows[WALK_U];
#pragma unroll
            for (int u = 0; u < WALK_U; ++u) {
                const uint32_t seg = seg0 + u * NWAVES;
                rows[u] = -1;
                if (seg < nseg) {  // uniform across the wavefront
                    const uint32_t fi = r0 + seg * 64u + lane;
                    if (fi < total) {
                        uint32_t t = lut[seg];
                        while (fi >= s_pref[t + 1]) ++t;
                        rows[u] = cand[s_start[t] + (fi - s_pref[t])];
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < WALK_U; ++u)
                if (rows[u] >= 0) f(rows[u]);
        }
        __syncthreads();  // lut is rewritten by the next round
    }
}

// One workgroup per query.  COUNT (EMIT = false) marks the rows of the query's spans in an
// LDS bitmap and counts the bits it set first.  EMIT marks them again, builds a rank table
// (marked rows before every group of 8 bitmap words) and lets every occurrence of a row
// store the row id at its rank: duplicates store the same value to the same place, so the
// output is ascending and duplicate-free without sorting, flagging or compaction.
template <bool EMIT>
__global__ __launch_bounds__(DD_THREADS) void dedup_kernel(DedupArgs a) {
    extern __shared__ uint32_t lds[];
    const int T = a.T, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int chunk_words = DD_THREADS * a.wpt;                  // multiple of 1024
    const int n_groups = chunk_words >> 3;                       // rank groups of 8 words
    uint32_t* bm = lds;                                          // [chunk_words]
    uint32_t* gpref = bm + chunk_words;                          // [n_groups] (EMIT)
    int* s_start = reinterpret_cast<int*>(gpref + (EMIT ? n_groups : 0));  // [T]
    uint32_t* s_pref = reinterpret_cast<uint32_t*>(s_start + T); // [T+1]
    uint32_t* lut = s_pref + T + 1;                              // [DD_THREADS]
    uint32_t* scratch = lut + DD_THREADS;                        // [17]
    uint32_t* wtot = scratch + 17;                               // [NWAVES + 1]

#define DD_TICK(k)                                                                      \
    if (a.ticks && tid == 0) {                                                          \
        const unsigned long long now_ = wall_clock64();                                 \
        atomicAdd(&a.ticks[k], now_ - tick_);                                           \
        tick_ = now_;                                                                   \
    }
    unsigned long long tick_ = a.ticks ? wall_clock64() : 0ull;

    const int q = blockIdx.x;
    uint32_t total;
    {
        int s = 0, len = 0;
        if (tid < T) {
            const int b = a.matched[static_cast<size_t>(q) * T + tid];
            if (b >= 0) {  // span of the matched bucket (count_candidates_kernel, query.cuh:114-132)
                s = a.bucket_candidate_offsets[b];
                len = a.bucket_candidate_offsets[b + 1] - s;
            }
        }
        // the first pass's bitmap is cleared while those loads are in flight
        uint4* bm4 = reinterpret_cast<uint4*>(bm);
        for (int i = tid; i < chunk_words / 4; i += DD_THREADS) bm4[i] = make_uint4(0u, 0u, 0u, 0u);
        if (tid < T) s_start[tid] = s;
        const uint32_t ex = block_exclusive_sum(static_cast<uint32_t>(len), scratch, &total);
        if (tid < T) s_pref[tid] = ex;
        if (tid == 0) s_pref[T] = total;
    }
    uint64_t running = 0;  // unique candidates found in earlier passes
    const uint64_t out_base = EMIT ? a.offsets[q] : 0;
    const uint32_t chunk_rows = static_cast<uint32_t>(chunk_words) * 32u;

    for (int chunk = 0; chunk < a.n_chunks; ++chunk) {
        const uint32_t lo = static_cast<uint32_t>(chunk) * chunk_rows;
        if (chunk > 0) {
            uint4* bm4 = reinterpret_cast<uint4*>(bm);
            for (int i = tid; i < chunk_words / 4; i += DD_THREADS) bm4[i] = make_uint4(0u, 0u, 0u, 0u);
        }
        if (tid <= NWAVES) wtot[tid] = 0;
        __syncthreads();
        DD_TICK(0)  // setup + clear
        // Mark the rows of this pass (collect_candidates_kernel, query.cuh:199-237, but into the
        // bitmap instead of memory).  Rows outside [lo, lo + chunk_rows) belong to another pass.
        uint32_t fresh = 0;  // COUNT: bits this thread set first
        walk_candidates(a.cand, s_start, s_pref, T, total, lut, [&](int row) {
            const uint32_t bit = static_cast<uint32_t>(row) - lo;
            if (bit < chunk_rows) {
                const uint32_t m = 1u << (bit & 31u);
                if (EMIT) {
                    atomicOr(&bm[bit >> 5], m);
                } else {
                    fresh += (atomicOr(&bm[bit >> 5], m) & m) == 0u;
                }
            }
        });
        DD_TICK(1)  // gather
        if (!EMIT) {
            // a row is counted by whichever lane set its bit first
            fresh = wave_sum(fresh);
            if (lane == 0 && fresh) atomicAdd(&wtot[NWAVES], fresh);
            __syncthreads();
            running += wtot[NWAVES];
            __syncthreads();  // wtot and the bitmap are reset by the next pass
            DD_TICK(2)
            continue;
        }
        // Rank table.  Wavefront w owns the consecutive groups [w*gpw, (w+1)*gpw); in step j its
        // lanes take 64 consecutive groups, so group order = (wave, step, lane).
        const int gpw = n_groups / NWAVES;           // >= 8
        const int steps = (gpw + 63) >> 6;           // <= 4
        uint32_t cnt[4], incl[4];
        uint32_t wave_total = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            cnt[j] = 0;
            incl[j] = 0;
            if (j < steps) {
                const int gl = j * 64 + lane;
                if (gl < gpw) {
                    const uint4* p = reinterpret_cast<const uint4*>(&bm[(wave * gpw + gl) << 3]);
                    const uint4 v0 = p[0], v1 = p[1];
                    cnt[j] = __popc(v0.x) + __popc(v0.y) + __popc(v0.z) + __popc(v0.w) + __popc(v1.x) +
                             __popc(v1.y) + __popc(v1.z) + __popc(v1.w);
                }
                incl[j] = wave_inclusive_sum_dpp(cnt[j]) + wave_total;
                wave_total = __shfl(incl[j], 63, 64);
            }
        }
        if (lane == 0) wtot[wave] = wave_total;
        __syncthreads();
        uint32_t wave_base = 0, chunk_total = 0;
#pragma unroll
        for (int w = 0; w < NWAVES; ++w) {
            const uint32_t v = wtot[w];
            wave_base += (w < wave) ? v : 0u;
            chunk_total += v;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gl = j * 64 + lane;
            if (j < steps && gl < gpw) gpref[wave * gpw + gl] = wave_base + incl[j] - cnt[j];
        }
        __syncthreads();
        DD_TICK(2)  // rank table
        int32_t* dst = a.out + out_base + running;
        walk_candidates(a.cand, s_start, s_pref, T, total, lut, [&](int row) {
            const uint32_t bit = static_cast<uint32_t>(row) - lo;
            if (bit < chunk_rows) {
                const uint32_t w = bit >> 5, g = w >> 3, k = w & 7u;
                const uint4* p = reinterpret_cast<const uint4*>(&bm[g << 3]);
                const uint4 v0 = p[0], v1 = p[1];
                const uint32_t words[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
                uint32_t pos = gpref[g];
                uint32_t cur = 0;
#pragma unroll
                for (uint32_t i = 0; i < 8; ++i) {
                    pos += (i < k) ? __popc(words[i]) : 0;
                    cur = (i == k) ? words[i] : cur;
                }
                pos += __popc(cur & ((1u << (bit & 31u)) - 1u));
                dst[pos] = row;
            }
        });
        running += chunk_total;
        DD_TICK(3)  // rank + store
    }
    if (!EMIT && tid == 0) a.counts[q] = running;
#undef DD_TICK
}

}  // namespace

culsh_status launch_find_matching_buckets(culsh_ctx* ctx, const uint32_t* q_keys, int n_queries,
                                          const culsh_index* index, int32_t* matched) {
    const size_t pairs = static_cast<size_t>(n_queries) * index->n_hash_tables;
    CULSH_REQUIRE(pairs / 256 < (1ull << 31), CULSH_ERR_LIMIT, "too many (query, table) pairs");
    CULSH_LAUNCH(ctx, lookup_kernel, dim3(div_up(pairs, 256)), dim3(256), 0, ctx->stream, q_keys,
                       index->bucket_keys, index->table_bucket_offsets, n_queries, index->n_hash_tables,
                       index->key_w, matched);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status query_from_matched(culsh_ctx* ctx, const int32_t* matched, int n_queries,
                                const culsh_index* index, culsh_candidates* out) {
    const int T = index->n_hash_tables;
    CULSH_REQUIRE(T <= DD_THREADS, CULSH_ERR_LIMIT, "query: n_hash_tables > 1024 is not supported");
    CULSH_REQUIRE(n_queries > 0, CULSH_ERR_INVALID, "query: n_queries must be positive");
    // rows addressed by the index: candidates are row ids < n = n_total_candidates / T
    const int n = index->n_total_candidates / T;
    CULSH_REQUIRE(n > 0, CULSH_ERR_INVALID, "query: empty index");

    // Geometry of a pass: DD_THREADS * wpt bitmap words (wpt a power of two); the emit launch
    // adds one rank word per 4 bitmap words.  Smaller bitmaps mean more passes over the row
    // range but let more workgroups share a CU; CULSH_DEDUP_WPT overrides the default cap.
    auto env_int = [](const char* name, int dflt) {
        const char* v = std::getenv(name);
        return (v && *v) ? std::atoi(v) : dflt;
    };
    const size_t fixed = (static_cast<size_t>(2 * T) + 1 + DD_THREADS + 17 + (DD_THREADS / 64 + 1) + 8) * sizeof(uint32_t);
    auto lds_need = [&](int w, bool emit) {
        const size_t cw = static_cast<size_t>(DD_THREADS) * w;
        return (cw + (emit ? cw / 8 : 0)) * 4 + fixed;
    };
    int wpt_max = 1;
    const int wpt_limit = std::max(1, std::min(32, env_int("CULSH_DEDUP_WPT", 32)));
    while (wpt_max * 2 <= wpt_limit && lds_need(wpt_max * 2, true) <= static_cast<size_t>(ctx->lds_max)) wpt_max *= 2;
    int wpt = 1;
    while (wpt < wpt_max && static_cast<long long>(DD_THREADS) * wpt * 32 < n) wpt *= 2;
    DedupArgs a;
    a.matched = matched;
    a.bucket_candidate_offsets = index->bucket_candidate_offsets;
    a.cand = index->all_candidate_indices;
    a.T = T;
    a.n = n;
    a.wpt = wpt;
    a.ticks = nullptr;
    const bool trace = env_int("CULSH_DEDUP_TRACE", 0) != 0;
    unsigned long long* ticks_dev = nullptr;
    if (trace) {
        CULSH_TRY(arena_alloc_t(ctx, 16, &ticks_dev));
        CULSH_HIP(hipMemsetAsync(ticks_dev, 0, 16 * sizeof(unsigned long long), ctx->stream));
    }
    const long long chunk_rows = static_cast<long long>(DD_THREADS) * wpt * 32;
    a.n_chunks = static_cast<int>((n + chunk_rows - 1) / chunk_rows);
    const size_t lds_count = lds_need(wpt, false), lds_emit = lds_need(wpt, true);
    CULSH_REQUIRE(lds_emit <= static_cast<size_t>(ctx->lds_max), CULSH_ERR_INTERNAL, "LDS budget exceeded");
    CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dedup_kernel<false>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_count)));
    CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dedup_kernel<true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_emit)));

    out->n_queries = n_queries;
    CULSH_HIP(hipMalloc(&out->query_candidate_counts, static_cast<size_t>(n_queries) * sizeof(uint64_t)));
    CULSH_HIP(hipMalloc(&out->query_candidate_offsets, (static_cast<size_t>(n_queries) + 1) * sizeof(uint64_t)));

    a.counts = out->query_candidate_counts;
    a.offsets = nullptr;
    a.out = nullptr;
    a.ticks = ticks_dev;
    CULSH_LAUNCH(ctx, dedup_kernel<false>, dim3(n_queries), dim3(DD_THREADS), lds_count, ctx->stream, a);
    CULSH_LAUNCH_CHECK();
    CULSH_TRY(exclusive_scan_u64(ctx, out->query_candidate_counts, out->query_candidate_offsets, n_queries));
    uint64_t U = 0;
    CULSH_TRY(read_back_u64(ctx, out->query_candidate_offsets + n_queries, 1, &U));  // the one host sync
    out->n_total_candidates = U;
    if (U == 0) {  // query.cuh:358-365: counts/offsets stay, indices stay null
        out->query_candidate_indices = nullptr;
        return CULSH_OK;
    }
    CULSH_HIP(hipMalloc(&out->query_candidate_indices, U * sizeof(int32_t)));
    a.offsets = out->query_candidate_offsets;
    a.out = out->query_candidate_indices;
    a.ticks = ticks_dev ? ticks_dev + 8 : nullptr;
    CULSH_LAUNCH(ctx, dedup_kernel<true>, dim3(n_queries), dim3(DD_THREADS), lds_emit, ctx->stream, a);
    CULSH_LAUNCH_CHECK();
    if (trace) {  // 100 MHz wall clock ticks of thread 0, summed over workgroups
        uint64_t tk[16];
        CULSH_TRY(read_back_u64(ctx, reinterpret_cast<const uint64_t*>(ticks_dev), 16, tk));
        fprintf(stderr, "[dedup trace] wpt=%d chunks=%d | count: setup %llu gather %llu reduce %llu | emit: setup %llu gather %llu ranktable %llu rank+store %llu (ticks)\n",
                wpt, a.n_chunks, (unsigned long long)tk[0], (unsigned long long)tk[1], (unsigned long long)tk[2],
                (unsigned long long)tk[8], (unsigned long long)tk[9], (unsigned long long)tk[10],
                (unsigned long long)tk[11]);
    }
    return CULSH_OK;
}

}  // namespace culsh_amd
