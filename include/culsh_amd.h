/*
 * culsh_amd - C ABI of the MI355X (gfx950) implementation of cuLSH's fit/query path.
 *
 * This is the drop-in boundary: the entry points below are what a binding for this
 * path binds (the reference binds the same operations from C++ through pybind11 in
 * python/csrc/bindings.cu).  Every function returns a culsh_status; on failure
 * culsh_last_error() holds a message for the calling thread.  No exceptions, no C++
 * types and no framework types cross this boundary.
 *
 * Conventions
 *   - `*_dev` pointers are device (HBM) addresses, `*_host` pointers are host addresses.
 *   - Dense inputs are C-contiguous row-major [rows][n_features]; CSR inputs are int32.
 *   - Signature matrices are table-major opaque bytes X_sig[n_hash_tables][rows][sig_nbytes]
 *     exactly as in the reference (cuda/README.md:14-36): RPLSH one uint8 (0/1) per hash,
 *     p-stable one little-endian int32 per hash, MinHash one little-endian uint32 per hash.
 *   - Every call runs on the context's stream and returns after that stream is idle
 *     (the reference binding synchronises the same way, bindings.cu:41,68,97).
 *   - Objects are not thread-safe; one context per host thread.
 *   - Limits: n_samples * n_hash_tables < 2^31 (int32 candidate positions, as
 *     core/index.cuh:32); n_hash_tables <= 1024 for every fit, load and query (refused with
 *     CULSH_ERR_LIMIT before any device work: a query gives each table one thread of a workgroup).
 *
 * Citations are file:line in the reference checkout (cuda/culsh/src/... unless noted).
 */
#ifndef CULSH_AMD_H
#define CULSH_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    CULSH_OK = 0,
    CULSH_ERR_INVALID = 1, /* bad argument (null pointer, non-positive size, dtype mismatch) */
    CULSH_ERR_HIP = 2,     /* a HIP runtime call failed */
    CULSH_ERR_NOMEM = 3,   /* device or host allocation failed */
    CULSH_ERR_LIMIT = 4,   /* a documented size limit was exceeded */
    CULSH_ERR_INTERNAL = 5
} culsh_status;

/* Which hashing family produced an index (selects the extra parameter arrays). */
typedef enum { CULSH_KIND_CORE = 0, CULSH_KIND_RPLSH = 1, CULSH_KIND_PSLSH = 2, CULSH_KIND_MINHASH = 3 } culsh_kind;

/* Names of the arrays held by an index / a candidates object (for the copy calls). */
typedef enum {
    CULSH_ARR_CANDIDATE_INDICES = 0,        /* int32  [n_total_candidates]           core/index.cuh:16 */
    CULSH_ARR_BUCKET_SIGNATURES = 1,        /* uint8  [n_total_buckets * sig_nbytes] core/index.cuh:20 */
    CULSH_ARR_BUCKET_CANDIDATE_OFFSETS = 2, /* int32  [n_total_buckets + 1]          core/index.cuh:24 */
    CULSH_ARR_TABLE_BUCKET_OFFSETS = 3,     /* int32  [n_hash_tables + 1]            core/index.cuh:28 */
    CULSH_ARR_PROJECTION = 4,               /* f32/f64 [T*H*n_features]  rplsh/index.cuh:15, pslsh/index.cuh:15 */
    CULSH_ARR_BIAS = 5,                     /* f32/f64 [T*H]             pslsh/index.cuh:16 */
    CULSH_ARR_HASH_A = 6,                   /* uint32 [T*H]              minhash/index.cuh:16 */
    CULSH_ARR_HASH_B = 7,                   /* uint32 [T*H]              minhash/index.cuh:17 */
    CULSH_ARR_QUERY_INDICES = 16,           /* int32  [n_total_candidates] core/candidates.cuh:18 */
    CULSH_ARR_QUERY_COUNTS = 17,            /* uint64 [n_queries]          core/candidates.cuh:22 */
    CULSH_ARR_QUERY_OFFSETS = 18            /* uint64 [n_queries + 1]      core/candidates.cuh:27 */
} culsh_array;

typedef struct culsh_ctx culsh_ctx;               /* stream + scratch arena (role of CUDAResourceManager, python/csrc/common/cuda_utils.cuh:30-62) */
typedef struct culsh_index culsh_index;           /* core::Index + per-family parameters */
typedef struct culsh_candidates culsh_candidates; /* core::Candidates */

/* Metadata of an index (core/index.cuh:30-40 plus the family fields). */
typedef struct {
    int32_t kind;              /* culsh_kind */
    int32_t n_total_candidates;
    int32_t n_total_buckets;
    int32_t n_hash_tables;
    int32_t n_hashes;
    int32_t sig_nbytes;
    int32_t n_features;
    int32_t is_double;         /* RPLSH / p-stable only */
    int32_t window_size;       /* p-stable only (0 when loaded without it) */
    uint64_t seed;
    uint64_t size_bytes;       /* as Index::size_bytes(), core/index.cuh:148-165 + family arrays */
} culsh_index_meta;

typedef struct {
    int32_t n_queries;
    uint64_t n_total_candidates;
    int32_t is_empty; /* Candidates::empty(), core/candidates.cuh:102-105 */
} culsh_candidates_meta;

/* ---- library / context ------------------------------------------------------------- */
const char* culsh_last_error(void);
const char* culsh_version(void);

/* Creates a context on `device` with its own stream (python/csrc/common/cuda_utils.cuh:36-39). */
culsh_status culsh_ctx_create(int device, culsh_ctx** out);
void culsh_ctx_destroy(culsh_ctx* ctx);
culsh_status culsh_ctx_synchronize(culsh_ctx* ctx);
/* The context's hipStream_t, for callers that want to order their own work after it. */
void* culsh_ctx_stream(culsh_ctx* ctx);

/* ---- per-kernel timing ------------------------------------------------------------------
 * No counterpart in the reference (it has wall-clock timing only, cuda/benchmark/bench.cu:144-163).
 * When enabled, every kernel launch is bracketed by two HIP events on the context's stream;
 * totals per kernel name are available after the call that launched them has returned.
 * The events keep consecutive kernels about 10 us apart, so a caller that times whole calls
 * restricts the timing to the kernel it needs with culsh_profile_filter (a substring of the
 * kernel name; NULL or "" = every kernel). */
culsh_status culsh_profile_enable(culsh_ctx* ctx, int on);
culsh_status culsh_profile_filter(culsh_ctx* ctx, const char* substring);
culsh_status culsh_profile_reset(culsh_ctx* ctx);
int culsh_profile_count(const culsh_ctx* ctx);
culsh_status culsh_profile_get(const culsh_ctx* ctx, int i, const char** name, double* total_ms, int64_t* launches);

/* ---- object memory ------------------------------------------------------------------
 * No counterpart in the reference (it allocates with cudaMalloc per array,
 * core/index.cuh:42-77, core/candidates.cuh:42-70).  Index and candidate arrays come from
 * a per-device cache of freed blocks (bounded by CULSH_POOL_MAX_MB, default 8192, 0 = off);
 * this call hands every cached block back to the driver. */
void culsh_memory_trim(void);

/* ---- seeded hash parameters (host side) -------------------------------------------------
 * Role of generate_random_projections (rplsh/hash.cuh:58-78),
 * generate_random_projections_biases (pslsh/hash.cuh:59-89) and generate_hash_integers
 * (minhash/hash.cuh:42-54).  The reference draws from cuRAND XORWOW, whose stream no
 * reference test pins and which is not reproduced; this generator is splitmix64 counter
 * based with Box-Muller normals.  `n_rows` = n_hash_tables * n_hashes. */
culsh_status culsh_generate_projection_f32(uint64_t seed, int n_rows, int n_features, float* P_host);
culsh_status culsh_generate_projection_f64(uint64_t seed, int n_rows, int n_features, double* P_host);
culsh_status culsh_generate_pslsh_params_f32(uint64_t seed, int n_rows, int n_features, int window_size, float* P_host, float* b_host);
culsh_status culsh_generate_pslsh_params_f64(uint64_t seed, int n_rows, int n_features, int window_size, double* P_host, double* b_host);
culsh_status culsh_generate_minhash_params(uint64_t seed, int n_rows, uint32_t* A_host, uint32_t* B_host);
/* The same normalised for another prime of the family (see culsh_ctx_set_minhash_prime). */
culsh_status culsh_generate_minhash_params_mod(uint64_t seed, int n_rows, uint32_t prime, uint32_t* A_host, uint32_t* B_host);

/* ---- RPLSH (rplsh/rplsh.cu) --------------------------------------------------------------
 * `P_host_opt`: NULL draws P from `seed`; otherwise a host array [T*H][n_features] of
 * the input's precision is used as the projection matrix (the only way the reference
 * offers to do this is RPLSHIndex.load_*, bindings.cu:428-442). */
culsh_status culsh_rplsh_fit_f32(culsh_ctx*, const float* X_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, uint64_t seed, const float* P_host_opt, culsh_index** out);   /* rplsh.cu:18-51 */
culsh_status culsh_rplsh_fit_f64(culsh_ctx*, const double* X_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, uint64_t seed, const double* P_host_opt, culsh_index** out); /* rplsh.cu:53-86 */
/* batch_size <= 0 or >= n_queries: unbatched (rplsh.cu:190-192). Fails with CULSH_ERR_INVALID
 * when the index precision differs from the query's (bindings.cu:58-60, 75-77). */
culsh_status culsh_rplsh_query_f32(culsh_ctx*, const float* Q_dev, int n_queries, const culsh_index*, int batch_size, culsh_candidates** out);   /* rplsh.cu:88-108,188-206 */
culsh_status culsh_rplsh_query_f64(culsh_ctx*, const double* Q_dev, int n_queries, const culsh_index*, int batch_size, culsh_candidates** out); /* rplsh.cu:110-128,208-226 */
culsh_status culsh_rplsh_fit_query_f32(culsh_ctx*, const float* X_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, uint64_t seed, const float* P_host_opt, culsh_candidates** out);   /* rplsh.cu:130-157 */
culsh_status culsh_rplsh_fit_query_f64(culsh_ctx*, const double* X_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, uint64_t seed, const double* P_host_opt, culsh_candidates** out); /* rplsh.cu:159-186 */

/* ---- p-stable LSH (pslsh/pslsh.cu) --------------------------------------------------------
 * `P_host_opt` / `b_host_opt` (both or neither): P already divided by the window and
 * b in (0,1], as stored by the reference (pslsh/hash.cuh:71-86). */
culsh_status culsh_pslsh_fit_f32(culsh_ctx*, const float* X_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, int window_size, uint64_t seed, const float* P_host_opt, const float* b_host_opt, culsh_index** out);    /* pslsh.cu:18-53 */
culsh_status culsh_pslsh_fit_f64(culsh_ctx*, const double* X_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, int window_size, uint64_t seed, const double* P_host_opt, const double* b_host_opt, culsh_index** out); /* pslsh.cu:55-91 */
culsh_status culsh_pslsh_query_f32(culsh_ctx*, const float* Q_dev, int n_queries, const culsh_index*, int batch_size, culsh_candidates** out);   /* pslsh.cu:93-114,202-220 */
culsh_status culsh_pslsh_query_f64(culsh_ctx*, const double* Q_dev, int n_queries, const culsh_index*, int batch_size, culsh_candidates** out); /* pslsh.cu:116-137,222-242 */
culsh_status culsh_pslsh_fit_query_f32(culsh_ctx*, const float* X_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, int window_size, uint64_t seed, const float* P_host_opt, const float* b_host_opt, culsh_candidates** out);    /* pslsh.cu:139-169 */
culsh_status culsh_pslsh_fit_query_f64(culsh_ctx*, const double* X_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, int window_size, uint64_t seed, const double* P_host_opt, const double* b_host_opt, culsh_candidates** out); /* pslsh.cu:171-200 */

/* ---- MinHash LSH (minhash/minhash.cu) -----------------------------------------------------
 * CSR column ids / row pointers are int32 device arrays; values are not read
 * (minhash_lsh.py:99-100).  `A_host_opt` / `B_host_opt` (both or neither) are already
 * normalised: A in [1,p-1], B in [0,p-1], p = 4294967291 (minhash/hash.cuh:17,26-32).
 *
 * The prime is a parameter of the hashing kernels.  The reference fixes it at 4294967291 = 2^32 - 5
 * (`MINHASH_PRIME`, minhash/hash.cuh:17), which is the default and what every parity statement refers to;
 * culsh_ctx_set_minhash_prime switches the fits, `culsh_minhash_compute` calls and loads of a context to
 * 2147483647 = 2^31 - 1, the other usual choice (no counterpart in the reference; any other value is
 * refused).  An index keeps the prime it was fitted with and its queries hash with it; the saved arrays of
 * the reference's format do not name it, so a load takes the context's. */
culsh_status culsh_ctx_set_minhash_prime(culsh_ctx*, uint32_t prime);
culsh_status culsh_ctx_get_minhash_prime(const culsh_ctx*, uint32_t* prime);
culsh_status culsh_index_minhash_prime(const culsh_index*, uint32_t* prime);
culsh_status culsh_minhash_fit(culsh_ctx*, const int32_t* indices_dev, const int32_t* indptr_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, uint64_t seed, const uint32_t* A_host_opt, const uint32_t* B_host_opt, culsh_index** out); /* minhash.cu:19-50 */
culsh_status culsh_minhash_query(culsh_ctx*, const int32_t* indices_dev, const int32_t* indptr_dev, int n_queries, const culsh_index*, culsh_candidates** out); /* minhash.cu:52-74 */
culsh_status culsh_minhash_fit_query(culsh_ctx*, const int32_t* indices_dev, const int32_t* indptr_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, uint64_t seed, const uint32_t* A_host_opt, const uint32_t* B_host_opt, culsh_candidates** out); /* minhash.cu:76-102 */

/* ---- stage-level entry points (signatures in, so bucket tables and candidate lists can be
 *      compared bit for bit given identical signatures) --------------------------------- */
/* hash<T> of rplsh/hash.cuh:92-129: uint8 sig_dev[T][n][H]; P_dev is a device array. */
culsh_status culsh_rplsh_hash_f32(culsh_ctx*, const float* X_dev, const float* P_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, uint8_t* sig_dev);
culsh_status culsh_rplsh_hash_f64(culsh_ctx*, const double* X_dev, const double* P_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, uint8_t* sig_dev);
/* hash<T> of pslsh/hash.cuh:104-142: int32 sig_dev[T][n][H]. */
culsh_status culsh_pslsh_hash_f32(culsh_ctx*, const float* X_dev, const float* P_dev, const float* b_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, int32_t* sig_dev);
culsh_status culsh_pslsh_hash_f64(culsh_ctx*, const double* X_dev, const double* P_dev, const double* b_dev, int n_samples, int n_features, int n_hash_tables, int n_hashes, int32_t* sig_dev);
/* compute_minhash of minhash/hash.cuh:142-155: uint32 sig_dev[T][n][H]. */
culsh_status culsh_minhash_compute(culsh_ctx*, const int32_t* indices_dev, const int32_t* indptr_dev, const uint32_t* A_dev, const uint32_t* B_dev, int n_samples, int n_hash_tables, int n_hashes, uint32_t* sig_dev);
/* core::detail::fit_index, core/fit.cuh:222-374.  `item_to_bucket_dev_opt`: NULL or int32 [n*T]
 * receiving bucket ids at [row * T + table] (fit.cuh:180-185). */
culsh_status culsh_core_fit_index(culsh_ctx*, const void* X_sig_dev, int n_samples, int n_hash_tables, int n_hashes, int sig_nbytes, int32_t* item_to_bucket_dev_opt, culsh_index** out);
/* core::detail::query_index, core/query.cuh:490-522. */
culsh_status culsh_core_query_index(culsh_ctx*, const void* Q_sig_dev, int n_queries, int sig_nbytes, const culsh_index*, culsh_candidates** out);
/* find_matching_buckets_kernel, core/query.cuh:72-101: int32 matched_dev[n_queries * T]. */
culsh_status culsh_core_find_matching_buckets(culsh_ctx*, const void* Q_sig_dev, int n_queries, int sig_nbytes, const culsh_index*, int32_t* matched_dev);
/* The same lookup for callers that cannot allocate (tight serving loops, harnesses that forbid hipMalloc,
 * code that must not allocate because a HIP graph is being captured elsewhere in the process; the call
 * itself still sets the current device and checks the launch status, and has not been run on a capturing
 * stream).  No counterpart in the reference.  The key words of the queries,
 * which culsh_core_find_matching_buckets keeps in the context's scratch arena, live in a workspace that
 * is part of the library's device image (CULSH_STATIC_SCRATCH_WORDS 32-bit words per GPU, held until the
 * process ends); the call makes no hipMalloc / hipFree, creates no events and does not wait for the
 * stream: it enqueues its kernels on the context's stream and returns, and `matched_dev` is complete
 * after culsh_ctx_synchronize (or any other call on the context, all of which end with the stream
 * idle).  n_queries * n_hash_tables * key words per signature beyond the workspace is refused with
 * CULSH_ERR_LIMIT (key words: ceil(n_hashes / 32) for RPLSH indices, at most ceil(sig_nbytes / 4)
 * otherwise).  All calls on one GPU share that GPU's workspace, which keeps the last call's contents
 * (every call overwrites the part it reads): calls on one context follow each other on its stream, but
 * calls of two contexts that overlap in time on one GPU race. */
#define CULSH_STATIC_SCRATCH_WORDS (1u << 20) /* 4 MiB */
culsh_status culsh_core_find_matching_buckets_static(culsh_ctx*, const void* Q_sig_dev, int n_queries, int sig_nbytes, const culsh_index*, int32_t* matched_dev);
/* core::detail::query_from_matched_buckets, core/query.cuh:290-478. */
culsh_status culsh_core_query_from_matched_buckets(culsh_ctx*, const int32_t* matched_dev, int n_queries, const culsh_index*, culsh_candidates** out);
/* core::detail::fit_query, core/fit_query.cuh:30-55. */
culsh_status culsh_core_fit_query(culsh_ctx*, const void* X_sig_dev, int n_samples, int n_hash_tables, int n_hashes, int sig_nbytes, culsh_candidates** out);

/* ---- index object ------------------------------------------------------------------------ */
culsh_status culsh_index_get_meta(const culsh_index*, culsh_index_meta* out);
/* Debugging aids (no counterpart in the reference).  culsh_debug_allocation_calls: how often this
 * library has called the HIP allocator in this process (hipMalloc, hipHostMalloc, hipFree,
 * hipEventCreate): unchanged across a call means the call allocated nothing.  culsh_debug_arena_state:
 * out[0] = bytes of the context's scratch arena, out[1] = bytes of it in use, out[2] = scratch blocks
 * that did not fit the arena so far, out[3] = grows of the arena that found no memory (such calls go on
 * with separate blocks and the next call tries again). */
uint64_t culsh_debug_allocation_calls(void);
culsh_status culsh_debug_arena_state(const culsh_ctx*, uint64_t out[4]);
/* Internal form of the lookup keys (no counterpart in the reference; for tests and tuning): 32-bit words
 * per bucket key, and how a signature becomes a key: 0 = its bytes, big-endian word by word, 1 = one bit per
 * RPLSH hash, 2 = p-stable hashes as ranks among the values seen at fit time, 3 = MinHash values as ranks
 * of their columns.  A loaded index gets the form a fit of the same data would have chosen. */
culsh_status culsh_index_key_form(const culsh_index*, int32_t* key_words, int32_t* encoding);
/* Number of elements / element size of one of the index's arrays (0 elements when absent). */
culsh_status culsh_index_array_info(const culsh_index*, culsh_array which, uint64_t* n_elems, uint32_t* elem_size);
/* Copies an array to the host (getters of bindings.cu:341-378) or to a device buffer. */
culsh_status culsh_index_copy_array(culsh_ctx*, const culsh_index*, culsh_array which, void* dst, uint64_t dst_bytes, int dst_is_device);
/* Rebuilds an index from host arrays: load_rplsh_index / load_pslsh_index / load_minhash_index
 * (bindings.cu:407-476).  `param0_host`: projection (RPLSH, p-stable) or hash_a (MinHash);
 * `param1_host`: bias (p-stable) or hash_b (MinHash), NULL for RPLSH.  Unlike the reference, arrays that
 * do not add up (offsets that decrease or do not span the arrays, candidate indices outside
 * [0, n_total_candidates / n_hash_tables)) are refused with CULSH_ERR_INVALID: the query kernels trust them. */
culsh_status culsh_index_load(culsh_ctx*, culsh_kind kind, int is_double,
                              const int32_t* candidate_indices_host, const uint8_t* bucket_signatures_host,
                              const int32_t* bucket_candidate_offsets_host, const int32_t* table_bucket_offsets_host,
                              const void* param0_host, const void* param1_host,
                              int n_total_candidates, int n_total_buckets, int n_hash_tables, int n_hashes,
                              int sig_nbytes, int n_features, uint64_t seed, culsh_index** out);
void culsh_index_free(culsh_index*);

/* ---- candidates object --------------------------------------------------------------------- */
culsh_status culsh_candidates_get_meta(const culsh_candidates*, culsh_candidates_meta* out);
/* get_indices / get_counts / get_offsets (bindings.cu:268-338). */
culsh_status culsh_candidates_copy_array(culsh_ctx*, const culsh_candidates*, culsh_array which, void* dst, uint64_t dst_bytes, int dst_is_device);
/* Device address of one of the arrays (NULL when empty); valid until the object is freed. */
const void* culsh_candidates_device_ptr(const culsh_candidates*, culsh_array which);
/* Candidates::merge, core/candidates.cuh:139-197: appends `other` to `*acc` (consuming `other`);
 * `*acc` may be NULL, in which case it becomes `other`. */
culsh_status culsh_candidates_merge(culsh_ctx*, culsh_candidates** acc, culsh_candidates* other);
void culsh_candidates_free(culsh_candidates*);

#ifdef __cplusplus
}
#endif
#endif /* CULSH_AMD_H */
