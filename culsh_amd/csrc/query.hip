// Candidate retrieval on gfx950.
//
// Bucket lookup follows find_matching_buckets_kernel (core/query.cuh:31-101).  The tail
// (core/query.cuh:290-478) produces, per query, the ascending list of distinct row ids
// found in the matched buckets.  The reference gathers all raw candidates, sorts every
// query's segment with a 32-bit segmented radix sort, flags, reduces, scans and compacts.
// Here one workgroup owns a query and marks the row ids of its bucket spans in a bitmap
// held in LDS (up to 2^20 rows per pass of 128 KiB); reading the bitmap in order yields
// the ascending duplicate-free list directly, so raw candidates are never written to
// memory and nothing is sorted.
//
// Where a query's list starts in the output depends on the counts of all queries before
// it.  When the row range fits one bitmap pass, a single launch does everything: each
// workgroup publishes its count and obtains the sum of its predecessors' counts by
// looking back over their published values (a chained scan), then stores its list.  The
// output is allocated for the number of raw candidates, an upper bound of the result.
// Larger row ranges take several passes per query, in the same launch: rows ascend inside a
// bucket, so a search cuts every span at the passes' row bounds and a pass reads only its own
// part; the query's list is written where its raw candidates would start (no workgroup waits for another), and a copy closes the gaps
// between the lists afterwards.  A path of two launches (count, scan, emit) with no
// cooperation between workgroups stands behind both.
#include <algorithm>
#include <cstdlib>
#include <vector>

#include "block_utils.hpp"
#include "common.hpp"
#include "dedup_common.hpp"

namespace culsh_amd {
namespace {

// Bits to drop from a key's first word to get its directory entry: the entry is made of the
// KEY_DIR_BITS bits from the highest bit that the largest first word has set.
__device__ __forceinline__ int key_dir_shift(uint32_t largest_word) {
    return max(0, 32 - __clz(static_cast<int>(largest_word)) - KEY_DIR_BITS);
}

// Workgroup t sets the entries of table t to ~0 ("no bucket starts here"); workgroup 0 also finds the
// largest first key word over the tables' last buckets (keys ascend inside a table), into dir[0].
__global__ __launch_bounds__(256) void key_dir_init_kernel(const uint32_t* __restrict__ bucket_keys,
                                                          const int32_t* __restrict__ table_bucket_offsets, int T,
                                                          int W, uint32_t* __restrict__ dir,
                                                          const uint32_t* __restrict__ sort_gave_up) {
    __shared__ uint32_t largest[4];
    if (sort_gave_up && *sort_gave_up) return;  // keys and offsets of a failed sort are not to be trusted; the fit is repeated
    const int tid = threadIdx.x;
    uint32_t* entry = dir + 1 + static_cast<size_t>(blockIdx.x) * (KEY_DIR_SIZE + 1);
    for (int x = tid; x <= KEY_DIR_SIZE; x += 256) entry[x] = 0xFFFFFFFFu;
    if (blockIdx.x != 0) return;
    uint32_t m = 0;
    for (int t = tid; t < T; t += 256)
        if (table_bucket_offsets[t + 1] > table_bucket_offsets[t])
            m = max(m, bucket_keys[static_cast<size_t>(table_bucket_offsets[t + 1] - 1) * W]);
#pragma unroll
    for (int step = 32; step > 0; step >>= 1) m = max(m, static_cast<uint32_t>(__shfl_xor(m, step, 64)));
    if ((tid & 63) == 0) largest[tid >> 6] = m;
    __syncthreads();
    if (tid == 0) dir[0] = max(max(largest[0], largest[1]), max(largest[2], largest[3]));
}

// entry[x] of table t = first bucket whose leading bits are >= x; entry[KEY_DIR_SIZE] = the table's
// end.  Two steps.  Mark (table blockIdx.y): the first bucket with leading bits x writes entry[x]; all
// other entries hold ~0 from a fill before.  Close (one workgroup per table): every entry takes the
// smallest value at or behind it, the last one being the table's end.
__global__ __launch_bounds__(256) void key_dir_mark_kernel(const uint32_t* __restrict__ bucket_keys,
                                                          const int32_t* __restrict__ table_bucket_offsets, int W,
                                                          uint32_t* __restrict__ dir,
                                                          const uint32_t* __restrict__ sort_gave_up) {
    if (sort_gave_up && *sort_gave_up) return;
    const int t = blockIdx.y;
    const int shift = key_dir_shift(dir[0]);
    const int begin = table_bucket_offsets[t], end = table_bucket_offsets[t + 1];
    uint32_t* entry = dir + 1 + static_cast<size_t>(t) * (KEY_DIR_SIZE + 1);
    for (int i = begin + blockIdx.x * 256 + threadIdx.x; i < end; i += gridDim.x * 256) {
        const uint32_t lead = bucket_keys[static_cast<size_t>(i) * W] >> shift;  // < KEY_DIR_SIZE
        if (i == begin || (bucket_keys[static_cast<size_t>(i - 1) * W] >> shift) != lead) entry[lead] = static_cast<uint32_t>(i);
    }
}

__global__ __launch_bounds__(256) void key_dir_close_kernel(const int32_t* __restrict__ table_bucket_offsets,
                                                           uint32_t* __restrict__ dir,
                                                           const uint32_t* __restrict__ sort_gave_up) {
    constexpr int PER = KEY_DIR_SIZE / 256;  // entries per thread
    __shared__ uint32_t tail[256];
    if (sort_gave_up && *sort_gave_up) return;
    const int t = blockIdx.x, tid = threadIdx.x;
    uint32_t* entry = dir + 1 + static_cast<size_t>(t) * (KEY_DIR_SIZE + 1);
    const uint32_t end = static_cast<uint32_t>(table_bucket_offsets[t + 1]);
    uint32_t v[PER];
    uint32_t low = end;  // smallest value at or behind this thread's entries, inside its own part
#pragma unroll
    for (int k = PER - 1; k >= 0; --k) {
        low = min(low, entry[tid * PER + k]);
        v[k] = low;
    }
    // smallest value of the threads behind this one: inside the wavefront by shuffles, then over the
    // wavefronts behind
    const int lane = tid & 63, wave = tid >> 6;
    uint32_t incl = low;  // minimum over lanes >= this one
#pragma unroll
    for (int step = 1; step < 64; step <<= 1) {
        const uint32_t other = __shfl_down(incl, step, 64);
        if (lane + step < 64) incl = min(incl, other);
    }
    uint32_t behind = __shfl_down(incl, 1, 64);
    if (lane == 63) behind = end;
    if (lane == 0) tail[wave] = incl;
    __syncthreads();
    for (int w = wave + 1; w < 4; ++w) behind = min(behind, tail[w]);
#pragma unroll
    for (int k = 0; k < PER; ++k) entry[tid * PER + k] = min(v[k], behind);
    if (tid == 0) entry[KEY_DIR_SIZE] = end;
}

// Binary search of every (query, table) key among the table's sorted bucket keys, inside the range
// the directory gives for the key's leading bits (the whole table without a directory); writes
// the matched bucket id (-1 = none) and / or its span (start, length) of candidate rows.
__global__ __launch_bounds__(256) void lookup_kernel(const uint32_t* __restrict__ q_keys,
                                                    const uint32_t* __restrict__ bucket_keys,
                                                    const uint32_t* __restrict__ dir,
                                                    const int32_t* __restrict__ table_bucket_offsets,
                                                    const int32_t* __restrict__ bucket_candidate_offsets,
                                                    int n_queries, int T, int W, int32_t* __restrict__ matched,
                                                    int2* __restrict__ spans,
                                                    unsigned long long* __restrict__ raw_total, int key_rows,
                                                    int key_first) {
    __shared__ unsigned long long block_raw;
    if (threadIdx.x == 0) block_raw = 0ull;
    __syncthreads();
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    const bool live = idx < static_cast<size_t>(n_queries) * T;
    // neighbouring threads: neighbouring queries of one table (their keys are neighbours in memory and
    // they walk the same table's directory and buckets); results are stored per query
    const int t = live ? static_cast<int>(idx / n_queries) : 0, q = live ? static_cast<int>(idx - static_cast<size_t>(t) * n_queries) : 0;
    const size_t slot = static_cast<size_t>(q) * T + t;
    // the keys are [T][key_rows][W]; the queries of this call are the rows key_first .. key_first + n_queries of every table
    const uint32_t* key = q_keys + (static_cast<size_t>(t) * key_rows + key_first + q) * W;
    int lo = live ? table_bucket_offsets[t] : 0, hi = live ? table_bucket_offsets[t + 1] - 1 : -1;
    if (live && dir) {
        const uint32_t lead = key[0] >> key_dir_shift(dir[0]);
        if (lead >= static_cast<uint32_t>(KEY_DIR_SIZE)) {
            hi = lo - 1;  // beyond every bucket key
        } else {
            const uint32_t* entry = dir + 1 + static_cast<size_t>(t) * (KEY_DIR_SIZE + 1) + lead;
            lo = static_cast<int>(entry[0]);
            hi = static_cast<int>(entry[1]) - 1;
        }
    }
    int found = -1;
    while (lo <= hi) {
        const int mid = lo + ((hi - lo) >> 1);
        const uint32_t* m = bucket_keys + static_cast<size_t>(mid) * W;
        int cmp = 0;
        for (int w = 0; w < W && cmp == 0; ++w) cmp = (key[w] > m[w]) - (key[w] < m[w]);
        if (cmp == 0) { found = mid; break; }
        if (cmp < 0) hi = mid - 1; else lo = mid + 1;
    }
    if (live && matched) matched[slot] = found;
    if (spans) {
        int2 sp = make_int2(0, 0);
        if (found >= 0) {
            sp.x = bucket_candidate_offsets[found];
            sp.y = bucket_candidate_offsets[found + 1] - sp.x;
        }
        if (live) spans[slot] = sp;
        // number of raw candidates: one atomic per wavefront in LDS, one per workgroup in memory
        const unsigned long long wsum = wave_sum(static_cast<unsigned long long>(sp.y));
        if ((threadIdx.x & 63) == 0 && wsum) atomicAdd(&block_raw, wsum);
        __syncthreads();
        if (threadIdx.x == 0 && block_raw) atomicAdd(raw_total, block_raw);
    }
}

// Span of every matched bucket (count_candidates_kernel, core/query.cuh:114-132).
__global__ __launch_bounds__(256) void span_kernel(const int32_t* __restrict__ matched,
                                                  const int32_t* __restrict__ bucket_candidate_offsets,
                                                  size_t pairs, int n_buckets, int2* __restrict__ spans,
                                                  unsigned long long* __restrict__ raw_total) {
    __shared__ unsigned long long block_raw;
    if (threadIdx.x == 0) block_raw = 0ull;
    __syncthreads();
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    int2 sp = make_int2(0, 0);
    if (idx < pairs) {
        const int b = matched[idx];
        if (b >= 0 && b < n_buckets) {  // -1 = no bucket; an id beyond the buckets is taken the same way
            sp.x = bucket_candidate_offsets[b];
            sp.y = bucket_candidate_offsets[b + 1] - sp.x;
        }
        spans[idx] = sp;
    }
    const unsigned long long wsum = wave_sum(static_cast<unsigned long long>(sp.y));
    if ((threadIdx.x & 63) == 0 && wsum) atomicAdd(&block_raw, wsum);
    __syncthreads();
    if (threadIdx.x == 0 && block_raw) atomicAdd(raw_total, block_raw);
}

// Raw candidates per query: the sum of its span lengths.
__global__ __launch_bounds__(256) void raw_counts_kernel(const int2* __restrict__ spans, int n_queries, int T,
                                                        uint64_t* __restrict__ raw_counts) {
    const int q = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (q >= n_queries) return;
    unsigned long long sum = 0;
    for (int t = lane; t < T; t += 64) sum += static_cast<unsigned long long>(spans[static_cast<size_t>(q) * T + t].y);
    sum = wave_sum(sum);
    if (lane == 0) raw_counts[q] = sum;
}

// Closes the gaps between the queries' lists: list q moves from src_offsets[q] to dst_offsets[q].
__global__ __launch_bounds__(256) void close_gaps_kernel(const int32_t* __restrict__ src,
                                                        const uint64_t* __restrict__ src_offsets,
                                                        const uint64_t* __restrict__ dst_offsets,
                                                        const uint64_t* __restrict__ counts,
                                                        int32_t* __restrict__ dst) {
    const int q = blockIdx.x;
    const int32_t* from = src + src_offsets[q];
    int32_t* to = dst + dst_offsets[q];
    const uint64_t count = counts[q];
    for (uint64_t i = threadIdx.x; i < count; i += 256) to[i] = from[i];
}


constexpr int SPARSE_WORDS = 2;  // a pass is read out through the summary when its range has this many bitmap words per row, or more
constexpr int REG_U = 32;  // several passes: pieces per wavefront of a query whose rows stay in registers (at most 32768 rows per query)
constexpr int SPLIT_BATCH = 3;  // row bounds located per search round of split_spans

// The rows of a span ascend.  For every span t < T and each of the K row bounds bound0 + k * chunk_rows
// this counts the span's rows below the bound, into s_split[k * T + t].  Four neighbouring lanes share
// one search and cut its range into five parts per round: a span of 500 rows takes four dependent
// loads, and 256 searches run side by side.  All threads must call it; the caller places the barriers.
__device__ __forceinline__ void split_spans(const int32_t* __restrict__ cand, const int* s_org_start,
                                            const int* s_org_len, int T, int K, uint32_t bound0,
                                            uint32_t chunk_rows, int* s_split) {
    const int sub = threadIdx.x & 3, group_shift = threadIdx.x & 60;
    for (int task = threadIdx.x >> 2; task < T * K; task += DD_THREADS / 4) {
        const int k = task / T, t = task - k * T;
        const uint32_t bound = bound0 + static_cast<uint32_t>(k) * chunk_rows;
        const int32_t* rows = cand + s_org_start[t];
        int first = 0, len = s_org_len[t];  // rows before `first` are below the bound, rows from first + len on are not
        while (len > 0) {
            const int step = (len + 4) / 5, end = first + len;
            const int pos = first + (sub + 1) * step - 1;  // last row of part `sub`
            const bool below = pos < end && static_cast<uint32_t>(rows[pos]) < bound;
            const int nb = __popc(static_cast<uint32_t>(__ballot(below) >> group_shift) & 15u);  // parts wholly below
            first += nb * step;
            len = nb == 4 ? end - first : min(step - 1, end - first);  // what is left of part `nb`, minus its probed last row
        }
        if (sub == 0) s_split[task] = first;
    }
}

enum DedupMode { DD_COUNT = 0, DD_EMIT = 1, DD_FUSED = 2, DD_FUSED_PASSES = 3 };  // FUSED: one bitmap pass per query

struct DedupArgs {
    const int2* spans;            // [n_queries][T] (start, length) in `cand`
    const int32_t* cand;          // all_candidate_indices
    int32_t* out;                 // EMIT, FUSED: candidate indices
    uint64_t* counts;             // COUNT, FUSED: per-query unique counts (written)
    uint64_t* offsets;            // EMIT: per-query output offsets (read); FUSED: [n_queries+1] (written)
    unsigned long long* state;    // FUSED, one pass: [n_queries] published counts / running sums, zero before the launch
    const uint64_t* raw_offsets;  // FUSED, several passes: [n_queries] where a query's list starts in `out` (spaced by raw counts)
    unsigned int* err;            // FUSED: set when the look-back gave up or the output would overflow
    unsigned int* ticket;         // FUSED: next query to hand out (workgroups stay and take queries in order)
    unsigned long long capacity;  // FUSED: elements available in `out`
    int T, n_queries;
    int wpt;       // bitmap words per thread (power of two); a pass covers DD_THREADS*wpt*32 rows
    int n_chunks;  // passes over the row range
    int spin_limit;  // FUSED: polls of an unpublished predecessor before giving up
    unsigned long long* ticks;  // optional [n_queries][8] phase timers (wall clock ticks of thread 0), or null
};


// Where bitmap word `w` sits in LDS.  With eight words per lane and step a lane reads two 16-byte
// halves at a lane stride of 32 bytes, and sixteen neighbouring lanes would hit every bank twice per
// read.  Lanes 8-15 of every sixteen keep their two halves in swapped places (index bit 2 = the half,
// bit 6 = lane bit 3), so that the sixteen reads cover sixteen different 16-byte columns.
__device__ __forceinline__ uint32_t bitmap_slot(uint32_t w, uint32_t swap_mask) {  // swap_mask: 4 for eight words per lane, else 0
    return w ^ ((w >> 4) & swap_mask);
}

// The `ew` (8, 4 or 1) consecutive bitmap words a lane owns in one read-out step, whose region starts
// at `region`.  The words are merged from the three cases as two vector values and only then spread
// into the array: filling the array inside the branches makes the compiler keep it in scratch memory.
__device__ __forceinline__ void load_step_words(const uint32_t* region, int lane, int ew, uint32_t (&words)[8]) {
    uint4 v0 = make_uint4(0u, 0u, 0u, 0u), v1 = make_uint4(0u, 0u, 0u, 0u);
    if (ew == 8) {
        const int swap = (lane >> 1) & 4;  // bitmap_slot of this lane's words
        v0 = *reinterpret_cast<const uint4*>(region + ((lane * 8) ^ swap));
        v1 = *reinterpret_cast<const uint4*>(region + ((lane * 8 + 4) ^ swap));
    } else if (ew == 4) {
        v0 = *reinterpret_cast<const uint4*>(region + lane * 4);
    } else {
        v0.x = region[lane];
    }
    words[0] = v0.x; words[1] = v0.y; words[2] = v0.z; words[3] = v0.w;
    words[4] = v1.x; words[5] = v1.y; words[6] = v1.z; words[7] = v1.w;
}

// One workgroup per query.  COUNT marks the rows of the query's spans in the LDS bitmap and
// counts the bits it set first.  EMIT and FUSED mark them and read the bitmap out in row
// order: the list is ascending and duplicate-free without sorting, and raw candidates
// never reach memory.
template <int MODE>
__global__ __launch_bounds__(DD_THREADS) void dedup_kernel(DedupArgs a) {
    constexpr bool FUSED = MODE == DD_FUSED || MODE == DD_FUSED_PASSES;
    extern __shared__ uint32_t lds[];
    const int T = a.T, tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int chunk_words = DD_THREADS * a.wpt;                  // multiple of 1024
    uint32_t* bm = lds;                                          // [chunk_words]
    uint32_t* sm = bm + chunk_words;                             // [chunk_words / 32] one bit per non-zero bitmap word (sparse passes)
    unsigned long long* sh_base = reinterpret_cast<unsigned long long*>(sm + chunk_words / 32);  // [1]
    int* sh_q = reinterpret_cast<int*>(sh_base + 1);             // [2] query handed to the workgroup
    int2* tab = reinterpret_cast<int2*>(sh_base + 2);            // [DD_THREADS]
    int* s_start = reinterpret_cast<int*>(tab + DD_THREADS);     // [T]
    int* s_len = s_start + T;                                    // [T]
    uint32_t* s_ppref = reinterpret_cast<uint32_t*>(s_len + T);  // [T+1]
    uint32_t* scratch = s_ppref + T + 1;                         // [17]
    uint32_t* wtot = scratch + 17;                               // [NWAVES + 1]
    // several passes per query: the query's spans as given, and where the next row bounds cut them
    int* s_org_start = reinterpret_cast<int*>(wtot + NWAVES + 1);  // [T]
    int* s_org_len = s_org_start + T;                              // [T]
    int* s_split = s_org_len + T;                                  // [SPLIT_BATCH][T]

#define DD_TICK(k)                                                                      \
    if (a.ticks && tid == 0) {                                                          \
        const unsigned long long now_ = wall_clock64();                                 \
        a.ticks[static_cast<size_t>(blockIdx.x) * 8 + (k)] += now_ - tick_;             \
        tick_ = now_;                                                                   \
    }
    unsigned long long tick_ = a.ticks ? wall_clock64() : 0ull;

    // COUNT, EMIT: one workgroup per query.  FUSED: workgroups stay resident and take queries in
    // order from a ticket counter, so a query's predecessors in the chained scan have always been
    // taken by a running workgroup; the next ticket and its spans are fetched under the current
    // query's read-out.
    int q = blockIdx.x;
    if (FUSED && tid == 0) *sh_q = static_cast<int>(atomicAdd(a.ticket, 1u));
    {   // the bitmap is cleared while the first loads are in flight; FUSED keeps it clean afterwards
        uint4* bm4 = reinterpret_cast<uint4*>(bm);
        for (int i = tid; i < (chunk_words + chunk_words / 32) / 4; i += DD_THREADS) bm4[i] = make_uint4(0u, 0u, 0u, 0u);
    }
    if (FUSED) {
        __syncthreads();
        q = *sh_q;
        if (q >= a.n_queries) return;
    }
    int2 sp = make_int2(0, 0);
    if (tid < T) sp = a.spans[static_cast<size_t>(q) * T + tid];
  for (;;) {  // the queries of this workgroup (a single one unless FUSED)
    int q_next = a.n_queries;
    int2 sp_next = make_int2(0, 0);
    // FUSED with several passes: a query's list starts where its raw candidates would (no dependence
    // on other queries, the host closes the gaps afterwards), and every pass walks the part of each
    // span whose rows fall into its range; split_spans finds those parts, a few passes ahead.
    constexpr bool several = MODE == DD_FUSED_PASSES;
    const bool cut = MODE != DD_FUSED && a.n_chunks > 1;  // several passes, in one launch or two
    uint32_t n_pieces;
    int covered = 0;  // several passes: rows of span `tid` that earlier passes walked
    if (cut) {
        if (tid < T) {
            s_org_start[tid] = sp.x;
            s_org_len[tid] = sp.y;
        }
    } else {
        if (tid < T) {
            s_start[tid] = sp.x;
            s_len[tid] = sp.y;
        }
        number_pieces((static_cast<uint32_t>(sp.y) + 63u) >> 6, T, s_ppref, scratch);
    }
    uint64_t running = 0;  // unique candidates found in earlier passes
    const uint64_t out_base = MODE == DD_EMIT ? a.offsets[q] : 0;
    const uint32_t chunk_rows = static_cast<uint32_t>(chunk_words) * 32u;
    const int wpw = chunk_words / NWAVES;                  // bitmap words per wavefront in the read-out, >= 64
    const int ew = wpw >= 512 ? 8 : (wpw >= 256 ? 4 : 1);  // words per lane and read-out step
    const uint32_t swap_mask = ew == 8 ? 4u : 0u;

    const unsigned long long raw_base = several ? a.raw_offsets[q] : 0ull;
    if (several && cut) {
        // A query with few candidates (at most REG_U pieces per wavefront) keeps its rows in registers: one
        // piece table and one fetch for the whole query, and every pass marks the rows of its range from the
        // registers and is read out through the summary of non-zero words.  No span is cut at the passes'
        // row bounds and nothing is fetched twice.
        number_pieces((static_cast<uint32_t>(sp.y) + 63u) >> 6, T, s_ppref, scratch);
        if (tid < T) {
            s_start[tid] = sp.x;
            s_len[tid] = sp.y;
        }
        __syncthreads();
        const uint32_t whole = s_ppref[T];
        if (whole <= static_cast<uint32_t>(REG_U * NWAVES)) {
            if (static_cast<uint32_t>(tid) < whole) {
                int tl = 0, th = T;  // largest t with s_ppref[t] <= tid; that span owns the piece
                while (th - tl > 1) {
                    const int mid = (tl + th) >> 1;
                    if (s_ppref[mid] <= static_cast<uint32_t>(tid)) tl = mid; else th = mid;
                }
                const int first = static_cast<int>(static_cast<uint32_t>(tid) - s_ppref[tl]) * 64;
                tab[tid] = make_int2(s_start[tl] + first, min(64, s_len[tl] - first));
            }
            __syncthreads();
            int rows[REG_U];
            {
#pragma unroll
                for (int u0 = 0; u0 < REG_U; u0 += 16) {  // table entries of sixteen pieces, then their loads
                    int2 ent[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u)
                        ent[u] = tab[min(static_cast<uint32_t>(wave + (u0 + u) * NWAVES), max(whole, 1u) - 1u)];
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        rows[u0 + u] = -1;
                        if (static_cast<uint32_t>(wave + (u0 + u) * NWAVES) < whole && lane < ent[u].y)
                            rows[u0 + u] = a.cand[static_cast<uint32_t>(ent[u].x + lane)];
                    }
                }
            }
            uint32_t* wbm = bm + wave * wpw;
            unsigned int ticket_next = 0;
            for (int chunk = 0; chunk < a.n_chunks; ++chunk) {
                const uint32_t lo = static_cast<uint32_t>(chunk) * chunk_rows;
                const bool last = chunk == a.n_chunks - 1;
                if (last && tid == 0) ticket_next = atomicAdd(a.ticket, 1u);  // arrives while the rows are marked and counted
#pragma unroll
                for (int u = 0; u < REG_U; ++u) {
                    const uint32_t bit = static_cast<uint32_t>(rows[u]) - lo;
                    if (bit < chunk_rows) {  // also false for -1 (no row)
                        const uint32_t w = bit >> 5;
                        atomicOr(&bm[bitmap_slot(w, swap_mask)], 1u << (bit & 31u));
                        atomicOr(&sm[w >> 5], 1u << (w & 31u));
                    }
                }
                __syncthreads();
                uint32_t sp_words = 0;
                if (lane < wpw / 32) sp_words = sm[wave * (wpw / 32) + lane];
                uint32_t c = 0;
                for (uint32_t left = sp_words; left; left &= left - 1u)
                    c += __popc(wbm[bitmap_slot(static_cast<uint32_t>(lane * 32 + __ffs(static_cast<int>(left)) - 1), swap_mask)]);
                const uint32_t incl = wave_inclusive_sum_dpp(c);
                if (lane == 63) wtot[wave] = incl;
                if (last && wave == 0) {
                    const int qn = min(static_cast<int>(__shfl(ticket_next, 0, 64)), a.n_queries);
                    if (T <= 64 && qn < a.n_queries && lane < T) sp_next = a.spans[static_cast<size_t>(qn) * T + lane];
                    if (lane == 0) *sh_q = qn;
                }
                __syncthreads();
                uint32_t wave_base = 0, chunk_total = 0;
#pragma unroll
                for (int w = 0; w < NWAVES; ++w) {
                    const uint32_t v = wtot[w];
                    wave_base += (w < wave) ? v : 0u;
                    chunk_total += v;
                }
                const uint64_t base = raw_base + running;
                const bool store = base + chunk_total <= a.capacity;  // cannot fail with capacity = raw candidates
                if (tid == 0) {
                    if (!store) atomicOr(a.err, 2u);
                    if (last) a.counts[q] = running + chunk_total;
                }
                if (last) q_next = *sh_q;
                int32_t* dst = a.out + base + wave_base + (incl - c);
                const uint32_t row_base = lo + (static_cast<uint32_t>(wave * wpw + lane * 32) << 5);
                for (uint32_t left = sp_words; left; left &= left - 1u) {
                    const uint32_t k = static_cast<uint32_t>(__ffs(static_cast<int>(left)) - 1);
                    uint32_t* word = &wbm[bitmap_slot(static_cast<uint32_t>(lane * 32) + k, swap_mask)];
                    uint32_t bits = *word;
                    *word = 0u;
                    const uint32_t r0 = row_base + (k << 5);
                    while (bits && store) {
                        *dst++ = static_cast<int32_t>(r0 + (__ffs(static_cast<int>(bits)) - 1));
                        bits &= bits - 1u;
                    }
                }
                if (sp_words) sm[wave * (wpw / 32) + lane] = 0u;
                running += chunk_total;
                __syncthreads();  // bitmap, summary and wtot are rewritten by the next pass
            }
            if (q_next >= a.n_queries) break;
            q = q_next;
            if (T <= 64) {
                sp = sp_next;  // zero outside the first T lanes
            } else {
                sp = make_int2(0, 0);
                if (tid < T) sp = a.spans[static_cast<size_t>(q) * T + tid];
            }
            continue;
        }
        __syncthreads();  // the general path below rewrites the piece numbering
    }
    for (int chunk = 0; chunk < a.n_chunks; ++chunk) {
        const uint32_t lo = static_cast<uint32_t>(chunk) * chunk_rows;
        const bool last = MODE == DD_FUSED || chunk == a.n_chunks - 1;  // DD_FUSED is launched for one pass only
        if (chunk > 0 && !FUSED) {  // FUSED leaves the bitmap clean after every read-out
            uint4* bm4 = reinterpret_cast<uint4*>(bm);
            for (int i = tid; i < chunk_words / 4; i += DD_THREADS) bm4[i] = make_uint4(0u, 0u, 0u, 0u);
        }
        if (cut) {
            const int ahead = chunk % SPLIT_BATCH;
            if (ahead == 0 && !last) {
                __syncthreads();  // the spans are in place, the previous bounds are used up
                split_spans(a.cand, s_org_start, s_org_len, T, min(SPLIT_BATCH, a.n_chunks - 1 - chunk),
                            lo + chunk_rows, chunk_rows, s_split);
                __syncthreads();
            }
            uint32_t pieces = 0;
            if (tid < T) {
                const int end = last ? sp.y : s_split[ahead * T + tid];
                s_start[tid] = sp.x + covered;
                s_len[tid] = end - covered;
                pieces = (static_cast<uint32_t>(end - covered) + 63u) >> 6;
                covered = end;
            }
            number_pieces(pieces, T, s_ppref, scratch);
        }
        if (tid <= NWAVES) wtot[tid] = 0;
        __syncthreads();
        n_pieces = s_ppref[T];
        if (several && n_pieces == 0 && !last) {  // no row in this range; the bitmap is clean
            __syncthreads();                      // s_ppref is rewritten by the next pass
            continue;
        }
        DD_TICK(0)  // setup + clear
        // Mark the rows of this pass (collect_candidates_kernel, core/query.cuh:199-237, but into
        // the bitmap instead of memory).  Rows outside [lo, lo + chunk_rows) belong to another pass.
        // Several passes per query: a pass with few rows for its range (its pieces hold at most one row per
        // SPARSE_WORDS bitmap words) is read out through a summary: every mark also sets its bitmap word's
        // bit in `sm`, and the read-out visits the words that have one instead of sweeping the whole
        // range.  (Not with one pass per query: there the chained scan's look-back runs under the sweep,
        // and without the sweep the waits for predecessors pile up and cost more than the sweep did.)
        const bool sparse = several && static_cast<size_t>(n_pieces) * 64u * SPARSE_WORDS <= static_cast<size_t>(chunk_words);
        auto mark_sparse = [&](int row) {
            const uint32_t bit = static_cast<uint32_t>(row) - lo;
            if (bit < chunk_rows) {
                const uint32_t m = 1u << (bit & 31u), w = bit >> 5;
                // both without a returned value: waiting for the first one's answer to decide on the
                // second costs more than the second
                atomicOr(&bm[bitmap_slot(w, swap_mask)], m);
                atomicOr(&sm[w >> 5], 1u << (w & 31u));
            }
        };
        uint32_t fresh = 0;  // COUNT: bits this thread set first
        auto mark = [&](int row) {
            const uint32_t bit = static_cast<uint32_t>(row) - lo;
            if (bit < chunk_rows) {  // also false for -1 (no row): lo + chunk_rows stays below 2^32
                const uint32_t m = 1u << (bit & 31u), slot = bitmap_slot(bit >> 5, swap_mask);
                if (MODE == DD_COUNT) {
                    fresh += (atomicOr(&bm[slot], m) & m) == 0u;
                } else {
                    atomicOr(&bm[slot], m);
                }
            }
        };
        if (sparse) walk_candidates(a.cand, s_start, s_len, s_ppref, T, n_pieces, tab, mark_sparse);
        else walk_candidates(a.cand, s_start, s_len, s_ppref, T, n_pieces, tab, mark);
        DD_TICK(1)  // gather
        if (MODE == DD_COUNT) {
            // a row is counted by whichever lane set its bit first
            fresh = wave_sum(fresh);
            if (lane == 0 && fresh) atomicAdd(&wtot[NWAVES], fresh);
            __syncthreads();
            running += wtot[NWAVES];
            __syncthreads();  // wtot and the bitmap are reset by the next pass
            DD_TICK(2)
            continue;
        }
        // Ordered read-out.  Wavefront w owns the consecutive words [w*wpw, (w+1)*wpw); in a step
        // every lane takes EW consecutive words, so row order = (wave, step, lane, word, bit).
        const int steps = wpw / (64 * ew);
        uint32_t* wbm = bm + wave * wpw;
        // How many rows each wavefront holds.  One pass per query: counted first, so that the query's
        // count is published before the line-up.  Several passes: nobody waits for the count, and the
        // line-up's own totals serve.
        uint32_t wave_total = 0;
        // Sparse pass: lane l owns the 32 consecutive words [32 l, 32 l + 32) of the wavefront's part and
        // the summary word that stands for them; row order = (wave, lane, word, bit).
        uint32_t sp_words = 0, sp_before = 0;  // this lane's summary word; rows of the lower lanes
        if (sparse) {
            if (lane < wpw / 32) sp_words = sm[wave * (wpw / 32) + lane];
            uint32_t c = 0;
            for (uint32_t left = sp_words; left; left &= left - 1u)
                c += __popc(wbm[bitmap_slot(static_cast<uint32_t>(lane * 32 + __ffs(static_cast<int>(left)) - 1), swap_mask)]);
            sp_before = wave_inclusive_sum_dpp(c) - c;
            wave_total = c;
        }
        for (int i = lane; !sparse && !several && i < wpw / 4; i += 64) {  // in any order: contiguous reads
            const uint4 v = reinterpret_cast<const uint4*>(wbm)[i];
            wave_total += __popc(v.x) + __popc(v.y) + __popc(v.z) + __popc(v.w);
        }
        uint32_t wave_base = 0, chunk_total = 0;
        if (!several) {
            wave_total = wave_sum(wave_total);
            if (lane == 0) wtot[wave] = wave_total;
            __syncthreads();
#pragma unroll
            for (int w = 0; w < NWAVES; ++w) {
                const uint32_t v = wtot[w];
                wave_base += (w < wave) ? v : 0u;
                chunk_total += v;
            }
            // the same in every lane: summed here and kept in scalar registers, not as 16 values until their use
            wave_base = __builtin_amdgcn_readfirstlane(wave_base);
            chunk_total = __builtin_amdgcn_readfirstlane(chunk_total);
        }
        // FUSED: the first wavefront publishes the count before anything else, so that later
        // queries can go on, and looks back only after lining up its own rows.
        DD_TICK(4)
        unsigned int ticket_next = 0;
        if (FUSED && wave == 0 && lane == 0) {
            if (!several)
                __hip_atomic_store(&a.state[q], TAG_COUNT | static_cast<unsigned long long>(chunk_total),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (last) ticket_next = atomicAdd(a.ticket, 1u);  // arrives while the rows are lined up
        }
        // Line-up.  A step's words go to registers, which frees its part of the bitmap: the rows are
        // written there in list order, ready for full-width wavefront stores.  No step needs the
        // position of the query's list for this.  A dense step (more rows than slots) is left alone.
        const uint32_t region = 64u * ew;  // words (= list slots) a step covers
        uint32_t st_total[4] = {0u, 0u, 0u, 0u};  // steps <= 4 for every geometry
        if (sparse && several) st_total[0] = wave_sum(wave_total);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (sparse || j >= steps) break;
            const int w0 = (j * 64 + lane) * ew;
            uint32_t* sreg = wbm + j * region;
            uint32_t words[8];
            load_step_words(sreg, lane, ew, words);
            uint32_t c = 0;
#pragma unroll
            for (int k = 0; k < 8; ++k) c += __popc(words[k]);
            const uint32_t incl = wave_inclusive_sum_dpp(c);
            st_total[j] = __shfl(incl, 63, 64);
            if (st_total[j] <= region) {
                uint32_t* slot = sreg + (incl - c);  // runs on from word to word
                const uint32_t row_base = lo + (static_cast<uint32_t>(wave * wpw + w0) << 5);
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    uint32_t bits = words[k];
                    const uint32_t r0 = row_base + (k << 5);
                    while (bits) {
                        *slot++ = r0 + (__ffs(static_cast<int>(bits)) - 1);
                        bits &= bits - 1u;
                    }
                }
            }
        }
        DD_TICK(5)
        uint64_t base = out_base + running;
        bool store = true;
        if (several) {
            if (lane == 0) wtot[wave] = st_total[0] + st_total[1] + st_total[2] + st_total[3];
            if (last && wave == 0) {
                const int qn = min(static_cast<int>(__shfl(ticket_next, 0, 64)), a.n_queries);
                if (T <= 64 && qn < a.n_queries && lane < T) sp_next = a.spans[static_cast<size_t>(qn) * T + lane];
                if (lane == 0) *sh_q = qn;
            }
            DD_TICK(6)
            __syncthreads();
#pragma unroll
            for (int w = 0; w < NWAVES; ++w) {
                const uint32_t v = wtot[w];
                wave_base += (w < wave) ? v : 0u;
                chunk_total += v;
            }
            // the same in every lane: summed here and kept in scalar registers, not as 16 values until their use
            wave_base = __builtin_amdgcn_readfirstlane(wave_base);
            chunk_total = __builtin_amdgcn_readfirstlane(chunk_total);
            base = raw_base + running;
            store = base + chunk_total <= a.capacity;  // cannot fail with capacity = raw candidates
            if (tid == 0) {
                if (!store) atomicOr(a.err, 2u);
                if (last) a.counts[q] = running + chunk_total;
            }
            if (last) q_next = *sh_q;
        } else if (FUSED) {
            if (wave == 0) {
                const int qn = min(static_cast<int>(__shfl(ticket_next, 0, 64)), a.n_queries);
                // spans of the next query (they all sit in this wavefront when T <= 64)
                if (T <= 64 && qn < a.n_queries && lane < T) sp_next = a.spans[static_cast<size_t>(qn) * T + lane];
                const unsigned long long excl = look_back(a.state, q, chunk_total, a.spin_limit, a.err);
                if (lane == 0) {
                    *sh_q = qn;
                    unsigned long long b = excl;
                    if (excl + chunk_total > a.capacity) {  // cannot happen with capacity = raw candidates
                        atomicOr(a.err, 2u);
                        b = ~0ull;
                    }
                    *sh_base = b;
                    a.counts[q] = running + chunk_total;
                    a.offsets[q] = excl;
                    if (q == a.n_queries - 1) a.offsets[a.n_queries] = excl + chunk_total;
                }
            }
            DD_TICK(6)
            __syncthreads();
            base = *sh_base;
            store = base != ~0ull;
            if (last) q_next = *sh_q;
        }
        DD_TICK(2)  // count, line-up (+ look-back)
        if (sparse) {
            // every lane writes the rows of its own words where the lower lanes' rows end, and leaves the
            // words and its summary word clean (also when nothing may be stored)
            int32_t* dst = a.out + base + wave_base + sp_before;
            const uint32_t row_base = lo + (static_cast<uint32_t>(wave * wpw + lane * 32) << 5);
            for (uint32_t left = sp_words; left; left &= left - 1u) {
                const uint32_t k = static_cast<uint32_t>(__ffs(static_cast<int>(left)) - 1);
                uint32_t* word = &wbm[bitmap_slot(static_cast<uint32_t>(lane * 32) + k, swap_mask)];
                uint32_t bits = *word;
                *word = 0u;
                const uint32_t r0 = row_base + (k << 5);
                while (bits && store) {
                    *dst++ = static_cast<int32_t>(r0 + (__ffs(static_cast<int>(bits)) - 1));
                    bits &= bits - 1u;
                }
            }
            if (sp_words) sm[wave * (wpw / 32) + lane] = 0u;
        } else if (store) {
            int32_t* dst = a.out + base + wave_base;
            __builtin_amdgcn_wave_barrier();  // LDS accesses of one wavefront complete in order
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (j >= steps) break;
                const uint32_t* sreg = wbm + j * region;
                if (st_total[j] <= region) {
                    for (uint32_t i = lane; i < st_total[j]; i += 64) dst[i] = static_cast<int32_t>(sreg[i]);
                } else {  // dense step: every lane stores the rows of its own words
                    const int w0 = (j * 64 + lane) * ew;
                    uint32_t words[8];
                    load_step_words(sreg, lane, ew, words);
                    uint32_t c = 0;
#pragma unroll
                    for (int k = 0; k < 8; ++k) c += __popc(words[k]);
                    uint32_t pos = wave_inclusive_sum_dpp(c) - c;
                    const uint32_t row_base = lo + (static_cast<uint32_t>(wave * wpw + w0) << 5);
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        uint32_t bits = words[k];
                        const uint32_t r0 = row_base + (k << 5);
                        while (bits) {
                            dst[pos++] = static_cast<int32_t>(r0 + (__ffs(static_cast<int>(bits)) - 1));
                            bits &= bits - 1u;
                        }
                    }
                }
                dst += st_total[j];
            }
        }
        if (FUSED && !sparse) {  // leave this wavefront's part of the bitmap clean for the next query
            uint4* z = reinterpret_cast<uint4*>(wbm);
            for (int i = lane; i < wpw / 4; i += 64) z[i] = make_uint4(0u, 0u, 0u, 0u);
        }
        running += chunk_total;
        __syncthreads();  // bitmap and wtot are rewritten by the next pass
        DD_TICK(3)  // ordered store
    }
    if (MODE == DD_COUNT && tid == 0) a.counts[q] = running;
    if (!FUSED || q_next >= a.n_queries) break;
    q = q_next;
    if (T <= 64) {
        sp = sp_next;  // zero outside the first T lanes
    } else {
        sp = make_int2(0, 0);
        if (tid < T) sp = a.spans[static_cast<size_t>(q) * T + tid];
    }
  }
#undef DD_TICK
}

}  // namespace

culsh_status build_key_directory(culsh_ctx* ctx, culsh_index* index, size_t bucket_bound) {
    const int T = index->n_hash_tables;
    dev_free(index->key_dir);
    index->key_dir = nullptr;
    if (T > KEY_DIR_MAX_TABLES || index->key_w < 1) return CULSH_OK;
    const size_t words = 1 + static_cast<size_t>(T) * (KEY_DIR_SIZE + 1);
    CULSH_HIP(dev_malloc(&index->key_dir, words * sizeof(uint32_t)));
    const uint32_t* gave_up = ctx->sort_err_dev;  // null outside a fit (loaded indices)
    CULSH_LAUNCH(ctx, key_dir_init_kernel, dim3(static_cast<unsigned>(T)), dim3(256), 0, ctx->stream,
                 index->bucket_keys, index->table_bucket_offsets, T, index->key_w, index->key_dir, gave_up);
    CULSH_LAUNCH_CHECK();
    // about two buckets per thread for tables of even size; larger tables take more rounds
    const unsigned per_table = static_cast<unsigned>(std::max<size_t>(1, std::min<size_t>(4096, div_up(bucket_bound / T + 1, 512))));
    CULSH_LAUNCH(ctx, key_dir_mark_kernel, dim3(per_table, static_cast<unsigned>(T)), dim3(256), 0, ctx->stream,
                 index->bucket_keys, index->table_bucket_offsets, index->key_w, index->key_dir, gave_up);
    CULSH_LAUNCH_CHECK();
    CULSH_LAUNCH(ctx, key_dir_close_kernel, dim3(static_cast<unsigned>(T)), dim3(256), 0, ctx->stream,
                 index->table_bucket_offsets, index->key_dir, gave_up);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status launch_find_matching_buckets(culsh_ctx* ctx, const uint32_t* q_keys, int n_queries,
                                          const culsh_index* index, int32_t* matched, void* spans,
                                          unsigned long long* raw_total, int key_rows, int key_first) {
    if (key_rows <= 0) { key_rows = n_queries; key_first = 0; }
    CULSH_REQUIRE(key_first >= 0 && key_first + n_queries <= key_rows, CULSH_ERR_INTERNAL, "lookup: queries outside the key array");
    const size_t pairs = static_cast<size_t>(n_queries) * index->n_hash_tables;
    CULSH_REQUIRE(pairs / 256 < (1ull << 31), CULSH_ERR_LIMIT, "too many (query, table) pairs");
    CULSH_REQUIRE(!spans || raw_total, CULSH_ERR_INTERNAL, "spans need a raw candidate counter");
    CULSH_LAUNCH(ctx, lookup_kernel, dim3(div_up(pairs, 256)), dim3(256), 0, ctx->stream, q_keys,
                 index->bucket_keys, index->key_dir, index->table_bucket_offsets, index->bucket_candidate_offsets, n_queries,
                 index->n_hash_tables, index->key_w, matched, static_cast<int2*>(spans), raw_total, key_rows, key_first);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

namespace {

int env_int(const char* name, int dflt) {
    const char* v = std::getenv(name);
    return (v && *v) ? std::atoi(v) : dflt;
}

// Geometry of a de-duplication pass: DD_THREADS * wpt bitmap words, wpt a power of two; row ranges
// beyond one bitmap take n_chunks passes.  Debug knob: CULSH_DEDUP_WPT lowers the cap on wpt (more passes).
struct DedupGeometry {
    int wpt = 1, n_chunks = 1;
    size_t lds_bytes = 0;
};

culsh_status dedup_geometry(const culsh_ctx* ctx, const culsh_index* index, DedupGeometry* g) {
    const int T = index->n_hash_tables;
    const int n = index->n_total_candidates / T;  // candidates are row ids < n
    const int wpt_limit = std::max(1, std::min(32, env_int("CULSH_DEDUP_WPT", 32)));
    // beside the bitmap: 3T + 1 words of spans for one pass, 2T + SPLIT_BATCH * T more when a query takes several
    for (int several = 0; several < 2; ++several) {
        const size_t per_table = several ? 5 + SPLIT_BATCH : 3;
        const size_t fixed = (4 + per_table * T + 1 + 2 * DD_THREADS + 17 + (NWAVES + 1) + 8) * sizeof(uint32_t);
        // bitmap, its summary (one bit per bitmap word), the rest
        auto lds_need = [&](int w) { return static_cast<size_t>(DD_THREADS) * w * 4 + static_cast<size_t>(DD_THREADS) * w / 8 + fixed; };
        int wpt_max = 1;
        while (wpt_max * 2 <= wpt_limit && lds_need(wpt_max * 2) <= static_cast<size_t>(ctx->lds_max)) wpt_max *= 2;
        int wpt = 1;
        while (wpt < wpt_max && static_cast<long long>(DD_THREADS) * wpt * 32 < n) wpt *= 2;
        const long long chunk_rows = static_cast<long long>(DD_THREADS) * wpt * 32;
        g->wpt = wpt;
        g->n_chunks = static_cast<int>((n + chunk_rows - 1) / chunk_rows);
        g->lds_bytes = lds_need(wpt);
        if (g->n_chunks == 1) break;
    }
    CULSH_REQUIRE(g->lds_bytes <= static_cast<size_t>(ctx->lds_max), CULSH_ERR_INTERNAL, "LDS budget exceeded");
    return CULSH_OK;
}

// The zero-initialised words a query needs, in one block cleared by one memset:
// [0] raw candidate total, [1] error flags (low half) and ticket counter (high half),
// [2 .. 2 + n_queries) the published words of the chained scan (kernels that pack the lists themselves).
culsh_status alloc_query_words(culsh_ctx* ctx, int n_queries, const DedupGeometry& g, unsigned long long** words) {
    (void)g;
    const size_t count = 2 + static_cast<size_t>(n_queries);
    CULSH_TRY(arena_alloc_t(ctx, count, words));
    CULSH_HIP(hipMemsetAsync(*words, 0, count * sizeof(unsigned long long), ctx->stream));
    return CULSH_OK;
}

// `raw_total` points at the block of alloc_query_words; its first word holds the number of raw
// candidates = sum of all span lengths.  Debug knobs: CULSH_DEDUP_TWO_PASS=1 forces the
// count / scan / emit path, CULSH_DEDUP_TRACE=1 prints phase timers.
culsh_status query_from_spans(culsh_ctx* ctx, const int2* spans, const unsigned long long* raw_total, int n_queries,
                              const culsh_index* index, const DedupGeometry& g, culsh_candidates* out,
                              int32_t* lists_dst = nullptr, uint64_t lists_cap = 0) {
    const int T = index->n_hash_tables;
    const int n = index->n_total_candidates / T;
    const int wpt = g.wpt, n_chunks = g.n_chunks;
    const size_t lds_bytes = g.lds_bytes;
    const bool trace = env_int("CULSH_DEDUP_TRACE", 0) != 0;
    unsigned long long* ticks_dev = nullptr;
    if (trace) {
        CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n_queries) * 8, &ticks_dev));
        CULSH_HIP(hipMemsetAsync(ticks_dev, 0, static_cast<size_t>(n_queries) * 8 * sizeof(unsigned long long), ctx->stream));
    }

    out->n_queries = n_queries;
    CULSH_HIP(dev_malloc(&out->query_candidate_counts, static_cast<size_t>(n_queries) * sizeof(uint64_t)));
    CULSH_HIP(dev_malloc(&out->query_candidate_offsets, (static_cast<size_t>(n_queries) + 1) * sizeof(uint64_t)));

    DedupArgs a;
    a.spans = spans;
    a.cand = index->all_candidate_indices;
    a.out = nullptr;
    a.counts = out->query_candidate_counts;
    a.offsets = out->query_candidate_offsets;
    a.state = nullptr;
    a.raw_offsets = nullptr;
    a.err = nullptr;
    a.ticket = nullptr;
    a.capacity = 0;
    a.T = T;
    a.n_queries = n_queries;
    a.wpt = wpt;
    a.n_chunks = n_chunks;
    a.spin_limit = env_int("CULSH_DEDUP_SPIN_LIMIT", 1 << 16);  // tests set 0 to reach the give-up path
    a.ticks = ticks_dev;

    bool fused = env_int("CULSH_DEDUP_TWO_PASS", 0) == 0;
    const bool several = n_chunks > 1;
    uint64_t U = 0;
    // Which kernel.  Row ranges of one bitmap pass: the bitmap kernel, unless the queries hold next to
    // nothing (fewer than one raw candidate per 2048 rows: the sweep over the bitmap is then most of a
    // query's time, and the two-level kernel sweeps a 32nd of it).  Larger ranges: the two-level
    // kernel (dedup_sparse.hip) when its level 1 fits and a query's distinct rows are expected to fit
    // its level 2, else the bitmap kernel with several passes per query.
    // CULSH_DEDUP_SPARSE (tests, tuning): 0 = never, 1 = whenever the geometry allows; CULSH_DEDUP_SPARSE_CAP
    // lowers the number of level-2 entries.
    enum Path { P_FUSED, P_PASSES, P_SPARSE };
    SparseDedupGeometry sg;
    const int sparse_knob = env_int("CULSH_DEDUP_SPARSE", -1);
    const bool sparse_ok = sparse_knob != 0 && sparse_dedup_geometry(ctx, n, T, env_int("CULSH_DEDUP_SPARSE_CAP", 0), &sg);
    auto choose_path = [&](double raw_per_query, double uniq_per_query) {  // uniq_per_query < 0: not known
        if (sparse_ok && sparse_knob == 1) return P_SPARSE;
        if (!several) return sparse_ok && sparse_knob != 0 && raw_per_query * 2048.0 <= static_cast<double>(n) ? P_SPARSE : P_FUSED;
        if (!sparse_ok) return P_PASSES;
        const bool fits = uniq_per_query >= 0.0 ? uniq_per_query <= 0.9 * sg.cap : raw_per_query <= 4.0 * sg.cap;
        return fits ? P_SPARSE : P_PASSES;
    };
    // The output is sized by the number of raw candidates R, an upper bound of the result.  When an
    // earlier call went to an index of the same shape (the same index, or one fitted again), its
    // distinct candidates per query (plus a quarter) size this call's output and R is read back together
    // with the result, one host round trip instead of two; the kernels do not write beyond the
    // capacity, and a call that would have is redone with R known.
    // CULSH_QUERY_RAW_GUESS (tests): candidates per query to assume, 0 = never guess.
    const int forced_guess = env_int("CULSH_QUERY_RAW_GUESS", -1);
    const uint64_t shape = ((static_cast<uint64_t>(index->n_total_candidates) << 32 ^ static_cast<uint64_t>(index->n_total_buckets)) *
                                0x9E3779B97F4A7C15ull +
                            (static_cast<uint64_t>(T) << 20 ^ static_cast<uint64_t>(index->n_hashes))) | 1ull;
    culsh_ctx::QueryGuess* slot = nullptr;
    for (auto& s : ctx->query_guess)
        if (s.key == shape) slot = &s;
    double guess_raw = forced_guess >= 0 ? static_cast<double>(forced_guess) : (slot ? slot->raw_per_query : 0.0);
    double guess_uniq = forced_guess >= 0 ? static_cast<double>(forced_guess) : (slot ? slot->uniq_per_query : 0.0);
    if (!slot) {
        slot = &ctx->query_guess[ctx->query_guess_next];
        ctx->query_guess_next = (ctx->query_guess_next + 1) % static_cast<int>(sizeof(ctx->query_guess) / sizeof(ctx->query_guess[0]));
        *slot = culsh_ctx::QueryGuess();
    }
    for (int attempt = 0; fused && attempt < 2; ++attempt) {
        const uint64_t bound = static_cast<uint64_t>(n_queries) * static_cast<uint64_t>(n);
        bool guessed = attempt == 0 && guess_raw > 0.0;
        Path path = guessed ? choose_path(guess_raw, guess_uniq) : P_FUSED;
        if (path == P_PASSES) guessed = false;  // lists at raw-count spacing: R sizes the output
        // The caller's array takes the lists when the kernel packs them itself and the size need not be
        // known first (the guessed mode: a batch behind the first one); a batch that does not fit is
        // redone with an array of its own.
        const bool in_place = guessed && lists_dst != nullptr && lists_cap > 0;
        unsigned long long* words = const_cast<unsigned long long*>(raw_total);
        uint64_t R = 0;
        if (attempt == 1) {  // the guess was too small: R is known by now, the kernel's words start from zero again
            R = ctx->pinned[2];
            CULSH_HIP(hipMemsetAsync(words + 1, 0, (1 + static_cast<size_t>(n_queries)) * sizeof(unsigned long long), ctx->stream));
        } else if (!guessed) {
            CULSH_TRY(read_back_u64(ctx, reinterpret_cast<const uint64_t*>(raw_total), 1, &R));  // host sync 1 of 2
        }
        if (!guessed) {
            path = choose_path(static_cast<double>(R) / n_queries, -1.0);
            slot->key = shape;
            slot->raw_per_query = static_cast<double>(R) / n_queries;
        }
        if (!guessed && R == 0) {  // no query matched any bucket (query.cuh:358-365: counts/offsets stay, indices stay null)
            CULSH_HIP(hipMemsetAsync(out->query_candidate_counts, 0, static_cast<size_t>(n_queries) * sizeof(uint64_t), ctx->stream));
            CULSH_HIP(hipMemsetAsync(out->query_candidate_offsets, 0, (static_cast<size_t>(n_queries) + 1) * sizeof(uint64_t), ctx->stream));
            out->n_total_candidates = 0;
            out->query_candidate_indices = nullptr;
            slot->uniq_per_query = 0.0;
            return CULSH_OK;
        }
        // Packed lists (bitmap kernel with one pass, two-level kernel): a chained scan over the queries
        // places them; a query holds at most n distinct rows, which bounds the output when buckets
        // overlap heavily.  Several bitmap passes: list q starts at the sum of the raw counts of the
        // queries before it, and the gaps are closed below.
        const uint64_t cap = path == P_PASSES ? R
                             : in_place ? lists_cap
                             : guessed ? std::min<uint64_t>(bound, static_cast<uint64_t>(guess_uniq * n_queries * 1.25) + 1024)
                                       : std::min<uint64_t>(R, bound);
        unsigned int* err = reinterpret_cast<unsigned int*>(words + 1);  // [0] error flags, [1] ticket counter
        a.state = words + 2;
        a.ticket = err + 1;
        uint64_t* raw_offsets = nullptr;
        if (path == P_PASSES) {
            uint64_t* raw_counts = nullptr;
            CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n_queries), &raw_counts));
            CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n_queries) + 1, &raw_offsets));
            CULSH_LAUNCH(ctx, raw_counts_kernel, dim3(div_up(static_cast<size_t>(n_queries), 4)), dim3(256), 0, ctx->stream,
                         spans, n_queries, T, raw_counts);
            CULSH_LAUNCH_CHECK();
            CULSH_TRY(exclusive_scan_u64(ctx, raw_counts, raw_offsets, n_queries));
            a.raw_offsets = raw_offsets;
            a.state = nullptr;
        }
        bool compacted = false;  // the two-level kernel works on the queries that matched a bucket only
        int32_t* lists = lists_dst;
        if (!in_place) {
            lists = nullptr;
            CULSH_HIP(dev_malloc(&lists, cap * sizeof(int32_t)));
            out->query_candidate_indices = lists;  // owned by `out` from here on, also if a later step fails
        }
        a.out = lists;
        a.err = err;
        a.capacity = cap;
        if (path == P_SPARSE) {
            SparseDedupArgs s;
            s.spans = spans;
            s.cand = a.cand;
            s.out = lists;
            s.counts = a.counts;
            s.offsets = a.offsets;
            s.state = a.state;
            s.err = err;
            s.ticket = a.ticket;
            s.capacity = cap;
            s.T = T;
            s.n_queries = n_queries;
            s.l1_per_thread = sg.l1_per_thread;
            s.cap = sg.cap;
            s.spin_limit = a.spin_limit;
            s.ticks = ticks_dev;
            // Inside one bitmap pass this kernel is only taken for queries with next to no candidates, and
            // most of those match no bucket at all: they are left out (their counts are zero, a query
            // costs the kernel several barriers whatever it holds) and the offsets come from a scan.
            compacted = !several && n_queries <= MAX_COMPACT_QUERIES && env_int("CULSH_DEDUP_COMPACT", 1) != 0;
            if (compacted) {
                int32_t* active = nullptr;
                unsigned int* n_active = nullptr;
                CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n_queries), &active));
                CULSH_TRY(arena_alloc_t(ctx, 1, &n_active));
                CULSH_TRY(launch_active_queries(ctx, spans, n_queries, T, active, n_active, out->query_candidate_counts));
                s.active = active;
                s.n_active = n_active;
            }
            CULSH_TRY(launch_dedup_sparse(ctx, s, sg));
        } else {
            {   // more LDS than a launch may ask for by default: allowed once per kernel and device, not per call
                static PerDeviceOnce allowed[2];
                PerDeviceOnce& done = allowed[path == P_PASSES ? 1 : 0];
                if (!done.is_set(ctx->device)) {
                    const void* kernel = path == P_PASSES ? reinterpret_cast<const void*>(dedup_kernel<DD_FUSED_PASSES>)
                                                          : reinterpret_cast<const void*>(dedup_kernel<DD_FUSED>);
                    CULSH_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, ctx->lds_max));
                    done.set(ctx->device);
                }
            }
            // as many workgroups as fit on the device at once (LDS and 2048 threads per CU bound it)
            const int per_cu = static_cast<int>(std::max<size_t>(1, std::min<size_t>(2, static_cast<size_t>(ctx->lds_max) / lds_bytes)));
            const int resident = std::max(1, ctx->n_cus * per_cu);
            if (path == P_PASSES)
                CULSH_LAUNCH(ctx, dedup_kernel<DD_FUSED_PASSES>, dim3(std::min(n_queries, resident)), dim3(DD_THREADS),
                             lds_bytes, ctx->stream, a);
            else
                CULSH_LAUNCH(ctx, dedup_kernel<DD_FUSED>, dim3(std::min(n_queries, resident)), dim3(DD_THREADS), lds_bytes,
                             ctx->stream, a);
            CULSH_LAUNCH_CHECK();
        }
        if (path == P_PASSES || compacted)
            CULSH_TRY(exclusive_scan_u64(ctx, out->query_candidate_counts, out->query_candidate_offsets, n_queries));
        CULSH_HIP(hipMemcpyAsync(&ctx->pinned[0], out->query_candidate_offsets + n_queries, sizeof(uint64_t),
                                 hipMemcpyDeviceToHost, ctx->stream));
        CULSH_HIP(hipMemcpyAsync(&ctx->pinned[1], err, sizeof(unsigned int), hipMemcpyDeviceToHost, ctx->stream));
        if (guessed)
            CULSH_HIP(hipMemcpyAsync(&ctx->pinned[2], raw_total, sizeof(uint64_t), hipMemcpyDeviceToHost, ctx->stream));
        CULSH_HIP(hipStreamSynchronize(ctx->stream));  // host sync 2 of 2 (the only one after a guess)
        U = ctx->pinned[0];
        const unsigned int e = static_cast<unsigned int>(ctx->pinned[1] & 0xffffffffu);
        if (guessed) {
            slot->key = shape;
            slot->raw_per_query = static_cast<double>(ctx->pinned[2]) / n_queries;
        }
        if (in_place) lists = nullptr;  // not this function's to free
        if (guessed && e == 2u) {  // the guess (or the caller's array) was too small and nothing else went wrong: once more with R
            dev_free(lists);
            out->query_candidate_indices = nullptr;
            guess_raw = 0.0;
            continue;
        }
        if (e != 0) {  // never seen; the two-launch path below needs no cooperation between workgroups
            dev_free(lists);
            out->query_candidate_indices = nullptr;
            fused = false;
        } else if (U == 0) {
            dev_free(lists);
            out->query_candidate_indices = nullptr;
            slot->uniq_per_query = 0.0;
        } else if (in_place) {
            slot->uniq_per_query = static_cast<double>(U) / n_queries;
            out->lists_in_place = true;
        } else if (path == P_PASSES) {
            slot->uniq_per_query = static_cast<double>(U) / n_queries;
            int32_t* packed = nullptr;
            CULSH_HIP(dev_malloc(&packed, U * sizeof(int32_t)));
            out->query_candidate_indices = packed;
            hipError_t err_copy = hipSuccess;
            {
                StageTimer st(ctx, "close_gaps_kernel");
                hipLaunchKernelGGL(close_gaps_kernel, dim3(n_queries), dim3(256), 0, ctx->stream, lists, raw_offsets,
                                   out->query_candidate_offsets, out->query_candidate_counts, packed);
                err_copy = hipGetLastError();
            }
            if (err_copy == hipSuccess) err_copy = hipStreamSynchronize(ctx->stream);
            dev_free(lists);
            CULSH_HIP(err_copy);
        } else {
            slot->uniq_per_query = static_cast<double>(U) / n_queries;
            if (U < cap - cap / 4 && (cap - U) * sizeof(int32_t) > (size_t(1) << 20)) {
                // more than a quarter of the block would stay unused (tables that overlap, a first call
                // sized by the raw candidates): hand out an exact-size array instead
                int32_t* exact = nullptr;
                CULSH_HIP(dev_malloc(&exact, U * sizeof(int32_t)));
                out->query_candidate_indices = exact;
                hipError_t err_copy = hipMemcpyAsync(exact, lists, U * sizeof(int32_t), hipMemcpyDeviceToDevice, ctx->stream);
                if (err_copy == hipSuccess) err_copy = hipStreamSynchronize(ctx->stream);
                dev_free(lists);
                CULSH_HIP(err_copy);
            }
        }
        break;
    }
    if (!fused) {
        static PerDeviceOnce allowed_two_launch;
        if (!allowed_two_launch.is_set(ctx->device)) {
            CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dedup_kernel<DD_COUNT>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, ctx->lds_max));
            CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(dedup_kernel<DD_EMIT>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, ctx->lds_max));
            allowed_two_launch.set(ctx->device);
        }
        CULSH_LAUNCH(ctx, dedup_kernel<DD_COUNT>, dim3(n_queries), dim3(DD_THREADS), lds_bytes, ctx->stream, a);
        CULSH_LAUNCH_CHECK();
        CULSH_TRY(exclusive_scan_u64(ctx, out->query_candidate_counts, out->query_candidate_offsets, n_queries));
        CULSH_TRY(read_back_u64(ctx, out->query_candidate_offsets + n_queries, 1, &U));
        if (U != 0) {
            CULSH_HIP(dev_malloc(&out->query_candidate_indices, U * sizeof(int32_t)));
            a.out = out->query_candidate_indices;
            a.ticks = nullptr;
            CULSH_LAUNCH(ctx, dedup_kernel<DD_EMIT>, dim3(n_queries), dim3(DD_THREADS), lds_bytes, ctx->stream, a);
            CULSH_LAUNCH_CHECK();
        } else {
            out->query_candidate_indices = nullptr;
        }
    }
    out->n_total_candidates = U;
    if (trace) {  // 100 MHz wall clock ticks of thread 0, summed over workgroups
        std::vector<uint64_t> all(static_cast<size_t>(n_queries) * 8);
        CULSH_HIP(hipStreamSynchronize(ctx->stream));
        CULSH_HIP(hipMemcpy(all.data(), ticks_dev, all.size() * sizeof(uint64_t), hipMemcpyDeviceToHost));
        uint64_t tk[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (size_t i = 0; i < all.size(); ++i) tk[i & 7] += all[i];
        if (sparse_ok)
            fprintf(stderr, "[two-level trace, if taken] set-up %llu level-1 %llu look-back %llu rank+copy-out %llu level-2 %llu line-up %llu totals %llu tail %llu\n",
                    (unsigned long long)tk[0], (unsigned long long)tk[1], (unsigned long long)tk[2], (unsigned long long)tk[3],
                    (unsigned long long)tk[4], (unsigned long long)tk[5], (unsigned long long)tk[6], (unsigned long long)tk[7]);
        fprintf(stderr, "[dedup trace] wpt=%d chunks=%d fused=%d | setup %llu gather %llu count %llu store %llu (ticks) | popc %llu line-up %llu look-back %llu barrier %llu\n",
                wpt, n_chunks, int(fused), (unsigned long long)tk[0], (unsigned long long)tk[1],
                (unsigned long long)tk[2], (unsigned long long)tk[3], (unsigned long long)tk[4],
                (unsigned long long)tk[5], (unsigned long long)tk[6], (unsigned long long)tk[2]);
    }
    return CULSH_OK;
}

culsh_status check_query_args(int n_queries, const culsh_index* index) {
    static_assert(CULSH_MAX_TABLES <= DD_THREADS, "one thread per table");
    CULSH_REQUIRE(index->n_hash_tables <= CULSH_MAX_TABLES, CULSH_ERR_LIMIT, "query: n_hash_tables > 1024 is not supported");
    CULSH_REQUIRE(n_queries > 0, CULSH_ERR_INVALID, "query: n_queries must be positive");
    CULSH_REQUIRE(index->n_total_candidates / index->n_hash_tables > 0, CULSH_ERR_INVALID, "query: empty index");
    return CULSH_OK;
}

}  // namespace

culsh_status query_from_matched(culsh_ctx* ctx, const int32_t* matched, int n_queries,
                                const culsh_index* index, culsh_candidates* out) {
    CULSH_TRY(check_query_args(n_queries, index));
    const size_t pairs = static_cast<size_t>(n_queries) * index->n_hash_tables;
    CULSH_REQUIRE(pairs / 256 < (1ull << 31), CULSH_ERR_LIMIT, "too many (query, table) pairs");
    int2* spans = nullptr;
    unsigned long long* raw_total = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, pairs, &spans));
    DedupGeometry g;
    CULSH_TRY(dedup_geometry(ctx, index, &g));
    CULSH_TRY(alloc_query_words(ctx, n_queries, g, &raw_total));
    CULSH_LAUNCH(ctx, span_kernel, dim3(div_up(pairs, 256)), dim3(256), 0, ctx->stream, matched,
                 index->bucket_candidate_offsets, pairs, index->n_total_buckets, spans, raw_total);
    CULSH_LAUNCH_CHECK();
    return query_from_spans(ctx, spans, raw_total, n_queries, index, g, out);
}

culsh_status query_from_keys(culsh_ctx* ctx, const uint32_t* q_keys, int n_queries, const culsh_index* index,
                             culsh_candidates* out, int32_t* lists_dst, uint64_t lists_cap, int key_rows, int key_first) {
    CULSH_TRY(check_query_args(n_queries, index));
    int2* spans = nullptr;
    unsigned long long* raw_total = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n_queries) * index->n_hash_tables, &spans));
    DedupGeometry g;
    CULSH_TRY(dedup_geometry(ctx, index, &g));
    CULSH_TRY(alloc_query_words(ctx, n_queries, g, &raw_total));
    CULSH_TRY(launch_find_matching_buckets(ctx, q_keys, n_queries, index, nullptr, spans, raw_total, key_rows, key_first));
    return query_from_spans(ctx, spans, raw_total, n_queries, index, g, out, lists_dst, lists_cap);
}

}  // namespace culsh_amd
