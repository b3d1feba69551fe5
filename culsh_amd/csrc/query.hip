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
    int wpt;        // bitmap words per thread (power of two)
    int pad_shift;  // physical word = w + (w >> pad_shift); 31 = no padding
    int n_chunks;   // passes over the row range
};

// first position in cand[s, e) whose value is >= v (spans are ascending row ids)
__device__ __forceinline__ int lower_bound_rows(const int32_t* __restrict__ cand, int s, int e, int v) {
    while (s < e) {
        const int mid = s + ((e - s) >> 1);
        if (cand[mid] < v) s = mid + 1; else e = mid;
    }
    return s;
}

template <bool EMIT>
__global__ __launch_bounds__(DD_THREADS) void dedup_kernel(DedupArgs a) {
    extern __shared__ uint32_t lds[];
    const int T = a.T, tid = threadIdx.x;
    const int chunk_words = DD_THREADS * a.wpt;
    const int phys_words = chunk_words + (chunk_words >> a.pad_shift) + 1;
    uint32_t* bm = lds;
    int* s_start = reinterpret_cast<int*>(lds + phys_words);   // [T] span start of the current pass
    int* s_end = s_start + T;                                  // [T] span end (whole span)
    uint32_t* s_pref = reinterpret_cast<uint32_t*>(s_end + T); // [T+1] exclusive prefix of pass lengths
    uint32_t* scratch = s_pref + T + 1;                        // [17]

    const int q = blockIdx.x;
    if (tid < T) {
        const int b = a.matched[static_cast<size_t>(q) * T + tid];
        int s = 0, e = 0;
        if (b >= 0) {  // span of the matched bucket (count_candidates_kernel, query.cuh:114-132)
            s = a.bucket_candidate_offsets[b];
            e = a.bucket_candidate_offsets[b + 1];
        }
        s_start[tid] = s;
        s_end[tid] = e;
    }
    uint64_t running = 0;  // unique candidates found in earlier passes
    const uint64_t out_base = EMIT ? a.offsets[q] : 0;
    const int chunk_rows = chunk_words * 32;

    for (int chunk = 0; chunk < a.n_chunks; ++chunk) {
        const int lo = chunk * chunk_rows;
        for (int i = tid; i < phys_words; i += DD_THREADS) bm[i] = 0;
        // rows of this pass inside each span: [s_start, cut)
        int len = 0, cut = 0;
        if (tid < T) {
            const int s = s_start[tid], e = s_end[tid];
            cut = (chunk + 1 == a.n_chunks) ? e : lower_bound_rows(a.cand, s, e, lo + chunk_rows);
            len = cut - s;
        }
        uint32_t total;
        const uint32_t ex = block_exclusive_sum(static_cast<uint32_t>(len), scratch, &total);
        if (tid < T) s_pref[tid] = ex;
        if (tid == 0) s_pref[T] = total;
        __syncthreads();
        // flat walk over the concatenated spans (collect_candidates_kernel, query.cuh:199-237,
        // but into the bitmap instead of memory)
        for (uint32_t f = tid; f < total; f += DD_THREADS) {
            int tl = 0, th = T;  // largest t with s_pref[t] <= f
            while (th - tl > 1) {
                const int mid = (tl + th) >> 1;
                if (s_pref[mid] <= f) tl = mid; else th = mid;
            }
            const int row = a.cand[s_start[tl] + (f - s_pref[tl])];
            const uint32_t bit = static_cast<uint32_t>(row - lo);
            const uint32_t w = bit >> 5;
            atomicOr(&bm[w + (w >> a.pad_shift)], 1u << (bit & 31u));
        }
        __syncthreads();
        if (tid < T) s_start[tid] = cut;  // next pass continues where this one stopped
        // thread k owns words [k*wpt, (k+1)*wpt): ascending row order across threads
        uint32_t c = 0;
        const int w0 = tid * a.wpt;
        for (int j = 0; j < a.wpt; ++j) {
            const int w = w0 + j;
            c += __popc(bm[w + (w >> a.pad_shift)]);
        }
        uint32_t chunk_total;
        const uint32_t before = block_exclusive_sum(c, scratch, &chunk_total);
        if (EMIT) {
            int32_t* dst = a.out + out_base + running + before;
            for (int j = 0; j < a.wpt; ++j) {
                const int w = w0 + j;
                uint32_t bits = bm[w + (w >> a.pad_shift)];
                const int row0 = lo + (w << 5);
                while (bits) {
                    *dst++ = row0 + (__ffs(static_cast<int>(bits)) - 1);
                    bits &= bits - 1;
                }
            }
        }
        running += chunk_total;
        __syncthreads();  // bitmap and span arrays are rewritten by the next pass
    }
    if (!EMIT && tid == 0) a.counts[q] = running;
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

    // bitmap geometry: DD_THREADS * wpt words per pass, as large as LDS allows
    const size_t fixed = (static_cast<size_t>(3 * T) + 1 + 17 + 8) * sizeof(uint32_t);
    int wpt_max = 1;
    while (wpt_max < 32) {
        const int nw = wpt_max * 2;
        const size_t need = (static_cast<size_t>(DD_THREADS) * nw + DD_THREADS + 1) * 4 + fixed;
        if (need > static_cast<size_t>(ctx->lds_max)) break;
        wpt_max = nw;
    }
    int wpt = 1;
    while (wpt < wpt_max && static_cast<long long>(DD_THREADS) * wpt * 32 < n) wpt *= 2;
    DedupArgs a;
    a.matched = matched;
    a.bucket_candidate_offsets = index->bucket_candidate_offsets;
    a.cand = index->all_candidate_indices;
    a.T = T;
    a.n = n;
    a.wpt = wpt;
    a.pad_shift = 31;
    if (wpt >= 2) { int s = 0; while ((1 << s) < wpt) ++s; a.pad_shift = s; }
    const long long chunk_rows = static_cast<long long>(DD_THREADS) * wpt * 32;
    a.n_chunks = static_cast<int>((n + chunk_rows - 1) / chunk_rows);
    const int chunk_words = DD_THREADS * wpt;
    const size_t lds_bytes = (static_cast<size_t>(chunk_words) + (chunk_words >> a.pad_shift) + 1) * 4 + fixed;
    CULSH_REQUIRE(lds_bytes <= static_cast<size_t>(ctx->lds_max), CULSH_ERR_INTERNAL, "LDS budget exceeded");
    CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dedup_kernel<false>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dedup_kernel<true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));

    out->n_queries = n_queries;
    CULSH_HIP(hipMalloc(&out->query_candidate_counts, static_cast<size_t>(n_queries) * sizeof(uint64_t)));
    CULSH_HIP(hipMalloc(&out->query_candidate_offsets, (static_cast<size_t>(n_queries) + 1) * sizeof(uint64_t)));

    a.counts = out->query_candidate_counts;
    a.offsets = nullptr;
    a.out = nullptr;
    CULSH_LAUNCH(ctx, dedup_kernel<false>, dim3(n_queries), dim3(DD_THREADS), lds_bytes, ctx->stream, a);
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
    CULSH_LAUNCH(ctx, dedup_kernel<true>, dim3(n_queries), dim3(DD_THREADS), lds_bytes, ctx->stream, a);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

}  // namespace culsh_amd
