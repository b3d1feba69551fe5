// Internal definitions shared by the HIP translation units of libculsh_amd.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "../../include/culsh_amd.h"

namespace culsh_amd {

// ---------------------------------------------------------------- errors
void set_error(const char* fmt, ...);

struct Status {
    culsh_status code = CULSH_OK;
    bool ok() const { return code == CULSH_OK; }
};

#define CULSH_HIP(call)                                                                   \
    do {                                                                                  \
        hipError_t e_ = (call);                                                           \
        if (e_ != hipSuccess) {                                                           \
            ::culsh_amd::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                                   __FILE__, __LINE__);                                   \
            return (e_ == hipErrorOutOfMemory) ? CULSH_ERR_NOMEM : CULSH_ERR_HIP;         \
        }                                                                                 \
    } while (0)

// "Done once per device" flags.  Contexts are used by one host thread each, but two threads with a
// context each may reach the same flag together: doing the step twice is harmless, a torn flag is not.
struct PerDeviceOnce {
    std::atomic<bool> done[64] = {};
    bool is_set(int device) const { return done[device & 63].load(std::memory_order_acquire); }
    void set(int device) { done[device & 63].store(true, std::memory_order_release); }
};

#define CULSH_TRY(expr)                    \
    do {                                   \
        culsh_status s_ = (expr);          \
        if (s_ != CULSH_OK) return s_;     \
    } while (0)

#define CULSH_REQUIRE(cond, code, ...)         \
    do {                                       \
        if (!(cond)) {                         \
            ::culsh_amd::set_error(__VA_ARGS__); \
            return (code);                     \
        }                                      \
    } while (0)

// Checks the launch itself (bad configuration); execution errors surface at the next sync.
#define CULSH_LAUNCH_CHECK() CULSH_HIP(hipGetLastError())

// ---------------------------------------------------------------- key encodings
// Signatures are opaque byte strings ordered lexicographically (unsigned bytes, byte 0
// most significant).  Internally every signature is held as `W` 32-bit key words whose
// unsigned word-lexicographic order is that byte order:
//   ENC_BE   word w = big-endian load of signature bytes [4w, 4w+4), zero padded
//   ENC_BITS (signatures made of 0/1 bytes) hash h -> bit (31 - h%32) of word h/32
//   ENC_PSC  (p-stable int32 hashes) per-hash ranks in byte order, `bits` each, MSB first;
//            the width comes from the index's codec (pscodec.hip)
//   ENC_MHR  (MinHash uint32 hashes) per-hash rank of the minimising column among all columns,
//            in byte order of the hash values, `bits` each, MSB first (mhcodec.hip)
enum KeyEnc : int { ENC_BE = 0, ENC_BITS = 1, ENC_PSC = 2, ENC_MHR = 3 };

inline int key_words(KeyEnc enc, int sig_nbytes) {
    return enc == ENC_BITS ? (sig_nbytes + 31) / 32 : (sig_nbytes + 3) / 4;
}

// Rank tables of the p-stable key compression (device arrays, owned by the index).
struct PsCodec {
    int bits = 0;             // bits per hash in a compressed key
    int rmax = 0;             // row pitch of fwd / inv
    int32_t* vmin = nullptr;  // [T*H] smallest hash value seen at fit time
    int32_t* range = nullptr; // [T*H] number of values in [vmin, vmax]
    uint32_t* fwd = nullptr;  // [T*H][rmax] value - vmin -> rank in byte order (0-based)
    int32_t* inv = nullptr;   // [T*H][rmax] rank -> value
};

// Rank tables of the MinHash key compression (device arrays, owned by the index).
struct MhCodec {
    int bits = 0;              // bits per hash in a compressed key
    int d = 0;                 // n_features; codes: 0..d-1 ranks, d = empty row, d+1 = matches nothing
    uint32_t* rank = nullptr;  // [T*H][d] column -> rank of its hash value (signature byte order)
    uint32_t* inv = nullptr;   // [T*H][d] rank -> hash value
    uint32_t* ainv = nullptr;  // [T*H] inverse of the multiplier modulo the prime (0: multiplier is a multiple of it)
};

}  // namespace culsh_amd

// ---------------------------------------------------------------- opaque objects
struct culsh_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    // scratch arena (bump allocated per call, grown between calls)
    char* arena = nullptr;
    size_t arena_cap = 0;
    size_t arena_off = 0;
    size_t arena_live = 0;               // bytes handed out and not rewound in this call (arena + overflow)
    size_t arena_want = 0;               // high-water mark of arena_live
    std::vector<void*> overflow;         // freed at the end of the call
    uint64_t arena_overflow_blocks = 0;  // blocks that did not fit the arena, over the context's life
    uint64_t arena_grow_failures = 0;    // grows of the arena that found no memory (the calls went on with overflow blocks)
    uint64_t* pinned = nullptr;          // 64 x u64 pinned host words for D2H scalars
    // pinned staging for hash parameters on their way to the device (grown on demand); calls end
    // with the stream idle, so a call may reuse it from the start
    char* param_stage = nullptr;
    size_t param_stage_cap = 0, param_stage_off = 0;
    // the hash parameters last generated from a seed (a model that is fitted again with the same
    // settings draws the same parameters; generating them on the host costs more than a fit)
    struct GenCache {
        int family = -1, window = 0, elem = 0;
        uint64_t seed = 0;
        size_t rows = 0, d = 0;
        std::vector<char> p, b;  // P and b, or A and B
    } gen_cache;
    // chained scan of the radix sort: give-up flag of the last sort (device, arena) and the
    // switch to the unchained passes after a give-up
    uint32_t* sort_err_dev = nullptr;
    uint32_t* aux_flag_dev = nullptr;  // a family's own flag that travels with the end-of-build read-back, or null
    uint32_t aux_flag_host = 0;        // its value after that read-back
    bool sort_unchained = false;
    int mh_prime_kind = 0;  // the prime MinHash fits of this context hash with (culsh_ctx_set_minhash_prime)
    // raw and distinct candidates per query of the last query calls, by the shape of the index they
    // went to (rows, buckets, tables, hashes): sizes the next call's output on an index of that shape
    // without a host round trip (query.hip).  A few shapes are kept, so that a caller who alternates
    // between indices keeps the short path on each.
    struct QueryGuess { uint64_t key = 0; double raw_per_query = 0.0, uniq_per_query = 0.0; };
    QueryGuess query_guess[8];
    int query_guess_next = 0;  // slot the next unknown shape replaces
    int lds_max = 0;                     // max LDS bytes per workgroup
    int n_cus = 0;
    // per-kernel timing with HIP events on `stream` (off unless enabled)
    bool profiling = false;
    std::string prof_filter;             // when not empty: only kernels whose name contains it are timed
    struct ProfPending { int stage; hipEvent_t start, stop; };
    struct ProfStage { std::string name; double total_ms = 0.0; long launches = 0; };
    std::vector<ProfPending> prof_pending;
    std::vector<hipEvent_t> prof_pool;
    std::vector<ProfStage> prof_stages;
};

struct culsh_index {
    // core::Index (core/index.cuh:12-40)
    int32_t* all_candidate_indices = nullptr;
    uint8_t* all_bucket_signatures = nullptr;
    int32_t* bucket_candidate_offsets = nullptr;
    int32_t* table_bucket_offsets = nullptr;
    int n_total_candidates = 0, n_total_buckets = 0, n_hash_tables = 0, n_hashes = 0;
    int sig_nbytes = 0, n_features = 0;
    uint64_t seed = 0;
    // sort-order form of the bucket signatures: uint32 [n_total_buckets][key_w]
    uint32_t* bucket_keys = nullptr;
    uint32_t* key_dir = nullptr;  // directory over the keys' leading bits (build_key_directory), or null
    culsh_amd::KeyEnc enc = culsh_amd::ENC_BE;
    int key_w = 0;
    culsh_amd::PsCodec psc;  // enc == ENC_PSC only
    culsh_amd::MhCodec mhc;  // enc == ENC_MHR only
    int mh_prime_kind = 0;   // MinHash: the prime the index was hashed with (mh_prime.hpp)
    // family parameters (device): rplsh/index.cuh, pslsh/index.cuh, minhash/index.cuh
    culsh_kind kind = CULSH_KIND_CORE;
    bool is_double = false;
    int window_size = 0;
    void* P = nullptr;    // [T*H][d] f32/f64
    void* b = nullptr;    // [T*H] f32/f64
    uint32_t* A = nullptr;
    uint32_t* B = nullptr;
    int device = 0;
};

struct culsh_candidates {
    // core::Candidates (core/candidates.cuh:14-40)
    int32_t* query_candidate_indices = nullptr;
    uint64_t* query_candidate_counts = nullptr;
    uint64_t* query_candidate_offsets = nullptr;
    int n_queries = 0;
    uint64_t n_total_candidates = 0;
    int device = 0;
    // Batched queries only (a batch's result before the batches are put together): the lists were
    // written straight into the caller's array, or have been copied there already.
    bool lists_in_place = false;
};

namespace culsh_amd {

// Calls into the HIP allocator made by this library in this process (hipMalloc, hipHostMalloc, hipFree,
// hipEventCreate): what culsh_debug_allocation_calls reports, so that a test can tell that a call
// allocated nothing.
extern std::atomic<uint64_t> g_allocation_calls;
inline void count_allocation_call() { g_allocation_calls.fetch_add(1, std::memory_order_relaxed); }

// ---------------------------------------------------------------- object memory (pool.hip)
// Device blocks owned by index / candidate objects; freed blocks are cached for reuse.
hipError_t dev_malloc(void** out, size_t bytes);
template <typename T>
inline hipError_t dev_malloc(T** out, size_t bytes) {
    void* p = nullptr;
    const hipError_t e = dev_malloc(&p, bytes);
    *out = static_cast<T*>(p);
    return e;
}
void dev_free(void* ptr);
void dev_trim();

// ---------------------------------------------------------------- scratch arena
culsh_status arena_begin(culsh_ctx* ctx);                 // start of an API call
culsh_status arena_alloc(culsh_ctx* ctx, size_t bytes, void** out);
culsh_status arena_end(culsh_ctx* ctx);                   // syncs the stream, frees overflow
struct ArenaMark { size_t off, live; };
ArenaMark arena_mark(const culsh_ctx* ctx);
void arena_rewind(culsh_ctx* ctx, const ArenaMark& mark);  // stream idle; frees what came after the mark
template <typename T>
inline culsh_status arena_alloc_t(culsh_ctx* ctx, size_t count, T** out) {
    void* p = nullptr;
    culsh_status s = arena_alloc(ctx, count * sizeof(T), &p);
    *out = static_cast<T*>(p);
    return s;
}
// RAII: arena_begin at construction, arena_end at scope exit.
struct ArenaScope {
    culsh_ctx* ctx;
    culsh_status begin_status;
    explicit ArenaScope(culsh_ctx* c) : ctx(c), begin_status(arena_begin(c)) {}
    ~ArenaScope() { arena_end(ctx); }
};

// Brackets the launches issued during its lifetime with two events on the context's stream
// when profiling is enabled; elapsed times are folded into per-name totals at the next
// end-of-call synchronisation.
struct StageTimer {
    culsh_ctx* ctx;
    int pending = -1;
    StageTimer(culsh_ctx* c, const char* name);
    ~StageTimer();
};
void profile_collect(culsh_ctx* ctx);  // call with the stream idle

// Kernel launch on the context's stream, timed under the kernel's name when profiling is on.
#define CULSH_LAUNCH(ctx, kernel, ...)                    \
    do {                                                  \
        ::culsh_amd::StageTimer st_(ctx, #kernel);        \
        hipLaunchKernelGGL(kernel, __VA_ARGS__);          \
    } while (0)

// Copies a small host array to device memory through pinned staging, asynchronously on the context's
// stream (api.hip); only valid inside a fit, which resets the staging area at its start.
culsh_status upload_async(culsh_ctx* ctx, const void* host, size_t bytes, void* dev);
// Reads `count` (<= 64) device u64/u32 words into host memory; synchronises the stream.
culsh_status read_back_u64(culsh_ctx* ctx, const uint64_t* dev, int count, uint64_t* host);
culsh_status read_back_u32(culsh_ctx* ctx, const uint32_t* dev, int count, uint32_t* host);
// one u64 and (optionally) one u32 from different places with a single synchronisation
culsh_status read_back_pair(culsh_ctx* ctx, const uint64_t* dev_a, const uint32_t* dev_b_or_null, uint64_t* a,
                            uint32_t* b);
// Internal status: the radix sort's chained scan gave up; the caller switches the context to
// unchained passes and repeats the fit.  Never returned through the C ABI.
constexpr culsh_status CULSH_RETRY_UNCHAINED = static_cast<culsh_status>(7);
// Internal: a MinHash fit with rank keys met a column id at or beyond n_features; the fit is
// repeated with plain keys, which hash any id.
constexpr culsh_status CULSH_RETRY_PLAIN_KEYS = static_cast<culsh_status>(6);

// ---------------------------------------------------------------- projection (project.hip)
// Output modes of the projection kernels.
enum ProjEpilogue : int {
    EPI_SIGN_KEYS = 0,   // RPLSH, fused: packed sign bits -> key words [T][n][W] (ENC_BITS)
    EPI_SIGN_BYTES = 1,  // RPLSH, reference layout: uint8 [T][n][H]
    EPI_FLOOR_I32 = 3    // p-stable, reference layout: int32 [T][n][H]
};
// `minmax` (EPI_FLOOR_I32 only, may be null): [T*H][2] words preset to INT_MAX / INT_MIN.  Where the
// kernel can (H a multiple of 4, `out` and `b` 16-byte aligned) it folds the smallest and largest
// hash of every column into them while it stores the hashes, and says so in *minmax_folded; else
// the caller sweeps `out` itself.
culsh_status launch_project_f32(culsh_ctx* ctx, const float* X, const float* P, const float* b,
                                int n, int d, int T, int H, ProjEpilogue epi, void* out,
                                int32_t* minmax = nullptr, bool* minmax_folded = nullptr);
culsh_status launch_project_f64(culsh_ctx* ctx, const double* X, const double* P, const double* b,
                                int n, int d, int T, int H, ProjEpilogue epi, void* out);

// ---------------------------------------------------------------- minhash (minhash.hip)
// as_keys: write byte-swapped values (ENC_BE key words) instead of the raw uint32.
// prime_kind: which prime the family is taken modulo (mh_prime.hpp; 0 = the reference's 2^32 - 5).
culsh_status launch_minhash(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr,
                            const uint32_t* A, const uint32_t* B, int n, int T, int H,
                            bool as_keys, uint32_t* out, int prime_kind);

// ---------------------------------------------------------------- key codec (index.hip)
// signature bytes [T][n][S] -> key words [T][n][W]
culsh_status launch_sig_to_keys(culsh_ctx* ctx, const uint8_t* sig, size_t n_items, int S,
                                KeyEnc enc, int W, uint32_t* keys);
// key words [count][W] -> signature bytes [count][S]; count_dev (may be null) caps count by a
// value that only the device knows yet
culsh_status launch_keys_to_sig(culsh_ctx* ctx, const uint32_t* keys, size_t count, const uint64_t* count_dev,
                                int S, KeyEnc enc, int W, uint8_t* sig);

// ---------------------------------------------------------------- p-stable key compression (pscodec.hip)
// Measures the value range of every (table, hash) of sig [T][n][H]; when the ranges are
// narrow, fills ix->psc, sets ix->enc = ENC_PSC and ix->key_w, and reports compressed = true.
// `mm_folded`: the ranges when the projection has folded them already ([T*H][2] from ps_minmax_prepare),
// else null and sig is swept here.
culsh_status ps_build_codec(culsh_ctx* ctx, const int32_t* sig, int n, int T, int H, culsh_index* ix,
                            bool* compressed, int32_t* mm_folded = nullptr);
// [T*H][2] range words in the arena, preset to INT_MAX / INT_MIN
culsh_status ps_minmax_prepare(culsh_ctx* ctx, int T, int H, int32_t** mm_dev);
// The same from value ranges on the host: mm[2c] / mm[2c + 1] = smallest / largest hash of column c = t * H + h.
culsh_status ps_build_codec_from_ranges(culsh_ctx* ctx, const int32_t* mm, int T, int H, culsh_index* ix, bool* compressed);
// int32 hashes [T][rows][H] -> compressed key words [T][rows][ix->key_w]; the T tables of `sig` are the
// index's tables t0 .. t0 + T - 1
culsh_status launch_ps_compress(culsh_ctx* ctx, const int32_t* sig, size_t rows, int T, int H, const culsh_index* ix,
                                uint32_t* keys, int t0 = 0);
// ix->bucket_keys -> little-endian int32 signatures of the buckets (needs table_bucket_offsets)
culsh_status launch_ps_keys_to_sig(culsh_ctx* ctx, const culsh_index* ix, size_t count, const uint64_t* count_dev,
                                   uint8_t* sig);
void free_ps_codec(culsh_index* ix);

// ---------------------------------------------------------------- MinHash key compression (mhcodec.hip)
// Builds the rank tables from ix->A / ix->B when that shortens the keys; then fills ix->mhc, sets
// ix->enc = ENC_MHR and ix->key_w, and reports used = true.  Rank codes stand for column ids below
// n_features `d` only: the fit's rank kernel flags any other id (see launch_minhash_rank).
// May return CULSH_RETRY_UNCHAINED (its column sort is a chained radix sort).
culsh_status mh_build_codec(culsh_ctx* ctx, int T, int H, int d, culsh_index* ix, bool* used);
// CSR rows -> packed rank codes [T][n][ix->key_w].  `fit_flag` non-null (the fit): ids are taken to
// be below the codec's n_features, for which a cheaper hash applies, and the word is set to 1 when
// one is not — the keys are then wrong (never out of bounds) and the caller fits again with plain
// keys.  Null (queries): any id is hashed as it is; ids the fit never saw match nothing.
culsh_status launch_minhash_rank(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr, int n, int T, int H,
                                 const culsh_index* ix, uint32_t* fit_flag, uint32_t* keys);
// uint32 signatures [T][rows][H] -> packed rank codes; T < 0: all tables of the index, else the T tables
// t0 .. t0 + T - 1.  unknown_flag (device, may be null) is set to 1 when a value is no column's hash
// (its code then matches nothing).
culsh_status launch_mh_sig_to_keys(culsh_ctx* ctx, const uint32_t* sig, size_t rows, const culsh_index* ix,
                                   uint32_t* keys, int T = -1, int t0 = 0, uint32_t* unknown_flag = nullptr);
// ix->bucket_keys -> little-endian uint32 signatures of the buckets (needs table_bucket_offsets)
culsh_status launch_mh_keys_to_sig(culsh_ctx* ctx, const culsh_index* ix, size_t count, const uint64_t* count_dev,
                                   uint8_t* sig);
void free_mh_codec(culsh_index* ix);

// ---------------------------------------------------------------- sort (sort.hip)
// Stable sort of each table's n items by key words (word 0 most significant), starting
// from the identity permutation.  keys_in [T][n][W] is clobbered.  On return
// *sorted_keys points at whichever of keys_in / keys_tmp holds the sorted keys and
// rows_out [T][n] holds the row ids in sorted order.  known_vary (host, [W], may be null):
// bits that may differ between keys; when null they are measured (one host sync).
culsh_status sort_tables(culsh_ctx* ctx, uint32_t* keys_in, uint32_t* keys_tmp, int32_t* rows_tmp,
                         int32_t* rows_out, int n, int T, int W, const uint32_t* known_vary,
                         uint32_t** sorted_keys);
size_t sort_scratch_bytes(int n, int T, int W);

// ---------------------------------------------------------------- index build (index.hip)
// From sorted keys + rows to the core::Index arrays (allocates them; one host sync).
culsh_status build_index_from_sorted(culsh_ctx* ctx, const uint32_t* sorted_keys, int32_t* rows_sorted_owned,
                                     int n, int T, int H, int S, KeyEnc enc, int W,
                                     int32_t* item_to_bucket_opt, culsh_index* index);
// Full pipeline from unsorted key words (arena-owned, clobbered).
culsh_status fit_index_from_keys(culsh_ctx* ctx, uint32_t* keys, int n, int T, int H, int S,
                                 KeyEnc enc, int W, int32_t* item_to_bucket_opt, culsh_index* index);

// ---------------------------------------------------------------- query (query.hip)
// `matched` ([n_queries][T] bucket ids, -1 = none) and `spans` ([n_queries][T] int2 (start,
// length) into all_candidate_indices) are both optional outputs; with `spans` the sum of
// the span lengths is added to *raw_total (device).
// Directory in front of the bucket lookup's binary search: for every table and every value of the
// KEY_DIR_BITS leading bits of a key's first word (counted from the highest bit any bucket key has
// set), where the buckets with that value start.  Layout: [0] = largest first word of any bucket key,
// then per table KEY_DIR_SIZE + 1 bucket numbers.  Not built for more than KEY_DIR_MAX_TABLES tables.
constexpr int KEY_DIR_BITS = 12, KEY_DIR_SIZE = 1 << KEY_DIR_BITS, KEY_DIR_MAX_TABLES = 1024;
// `bucket_bound`: the number of buckets or an upper bound of it (sizes the launch only).
culsh_status build_key_directory(culsh_ctx* ctx, culsh_index* index, size_t bucket_bound);

culsh_status launch_find_matching_buckets(culsh_ctx* ctx, const uint32_t* q_keys, int n_queries,
                                          const culsh_index* index, int32_t* matched, void* spans = nullptr,
                                          unsigned long long* raw_total = nullptr, int key_rows = 0, int key_first = 0);
culsh_status query_from_matched(culsh_ctx* ctx, const int32_t* matched, int n_queries,
                                const culsh_index* index, culsh_candidates* out);
// lookup + candidate retrieval from key words [T][n_queries][key_w]
// `lists_dst` (may be null): `lists_cap` elements of the caller's own, into which the lists are written when
// that can be done without a copy and they fit (out->lists_in_place says so; out->query_candidate_indices stays
// null then); else the result gets an array of its own as always.
// `key_rows` > 0: the key array holds `key_rows` rows per table and this call's queries are the rows
// key_first .. key_first + n_queries of every table (a batch out of keys that were hashed in one go).
culsh_status query_from_keys(culsh_ctx* ctx, const uint32_t* q_keys, int n_queries, const culsh_index* index,
                             culsh_candidates* out, int32_t* lists_dst = nullptr, uint64_t lists_cap = 0,
                             int key_rows = 0, int key_first = 0);

// Most hash tables an index may have (every fit, load and query checks it): the query kernels give each
// table of a query one thread of a workgroup.
constexpr int CULSH_MAX_TABLES = 1024;

// Elements that can be read (not used) behind the last one of an index's all_candidate_indices: the
// query kernels fetch whole 64-row pieces.
constexpr size_t CAND_PAD = 64;

// ---------------------------------------------------------------- sparse de-duplication (dedup_sparse.hip)
// One launch that turns the queries' bucket spans into packed ascending duplicate-free lists through a
// two-level bitmap whose cost follows the candidates, not the row range.
struct SparseDedupArgs {
    const void* spans;            // int2 [n_queries][T] (start, length) in `cand`
    const int32_t* cand;          // all_candidate_indices
    int32_t* out;                 // candidate indices, `capacity` elements
    uint64_t* counts;             // [n_queries] (written)
    uint64_t* offsets;            // [n_queries + 1] (written)
    unsigned long long* state;    // [n_queries] words of the chained scan, zero before the launch
    unsigned int* err;            // bit 0: the chained scan gave up, bit 1: `out` too small
    unsigned int* ticket;         // next query to hand out, zero before the launch
    unsigned long long capacity;
    int T, n_queries;
    int l1_per_thread;            // level-1 words per thread (SparseDedupGeometry)
    int cap;                      // level-2 entries (SparseDedupGeometry)
    int spin_limit;               // polls of an unpublished predecessor before giving up
    unsigned long long* ticks;    // optional [workgroups][8] phase timers (wall clock ticks of thread 0), or null
    // Optional: only the queries that matched a bucket at all are worked on.  `active` lists them in ascending
    // order, `*n_active` says how many; the chained scan then runs over positions in that list, `counts` of
    // the other queries are zero already, and `offsets` are left to a scan over `counts` afterwards.
    const int32_t* active = nullptr;
    const unsigned int* n_active = nullptr;
};
// Fills `active` / `*n_active` for SparseDedupArgs from the spans of `n_queries` (<= MAX_COMPACT_QUERIES)
// queries and zeroes `counts`.
constexpr int MAX_COMPACT_QUERIES = 1 << 18;
culsh_status launch_active_queries(culsh_ctx* ctx, const void* spans, int n_queries, int T, int32_t* active,
                                   unsigned int* n_active, uint64_t* counts);
struct SparseDedupGeometry {
    int l1_per_thread = 0, cap = 0;
    size_t lds_bytes = 0;
};
// false when level 1 of `n_rows` rows leaves no room for level 2 in LDS; cap_limit > 0 lowers `cap` (tests)
bool sparse_dedup_geometry(const culsh_ctx* ctx, int n_rows, int T, int cap_limit, SparseDedupGeometry* g);
culsh_status launch_dedup_sparse(culsh_ctx* ctx, const SparseDedupArgs& a, const SparseDedupGeometry& g);

// ---------------------------------------------------------------- scans (scan.hip)
// Exclusive prefix sum of `n` u64 values; out[n] receives the total (out has n+1 slots).
culsh_status exclusive_scan_u64(culsh_ctx* ctx, const uint64_t* in, uint64_t* out, size_t n);

// ---------------------------------------------------------------- host-side generator (rng.cpp part of api)
void gen_normals_f64(uint64_t seed, int stream, size_t n, double* out);
void gen_raw_u64(uint64_t seed, int stream, size_t n, uint64_t* out);

void free_index_arrays(culsh_index* ix);
void free_candidates_arrays(culsh_candidates* c);

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline unsigned div_up(size_t a, size_t b) { return static_cast<unsigned>((a + b - 1) / b); }

}  // namespace culsh_amd
