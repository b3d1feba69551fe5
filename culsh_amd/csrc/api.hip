// C ABI of libculsh_amd: context, scratch arena, seeded parameter generator, and the
// orchestration of fit / query / fit_query for the three hashing families
// (role of rplsh/rplsh.cu, pslsh/pslsh.cu, minhash/minhash.cu and of the *Core classes in
// python/csrc/bindings.cu of the reference).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <memory>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "common.hpp"
#include "mh_prime.hpp"

namespace culsh_amd {

std::atomic<uint64_t> g_allocation_calls{0};


// ---------------------------------------------------------------- errors
static thread_local std::string g_last_error;

void set_error(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
}

// ---------------------------------------------------------------- arena
static constexpr size_t ARENA_ALIGN = 256;

culsh_status arena_begin(culsh_ctx* ctx) {
    CULSH_HIP(hipSetDevice(ctx->device));
    ctx->arena_off = 0;
    ctx->arena_live = 0;
    ctx->sort_err_dev = nullptr;  // pointed into the arena of an earlier call
    ctx->aux_flag_dev = nullptr;  // likewise
    ctx->aux_flag_host = 0;
    if (ctx->arena_want > ctx->arena_cap) {  // stream is idle here: every call ends with a sync
        // the new block first: a grow that fails keeps the arena there is
        const size_t want = align_up(ctx->arena_want + ctx->arena_want / 8, 1 << 20);
        void* p = nullptr;
        count_allocation_call();
        hipError_t grown = hipMalloc(&p, want);
        if (grown != hipSuccess && ctx->arena) {
            // both blocks do not fit side by side: the stream is idle and nothing in the old one is
            // live, so it goes first and the new one is tried once more
            (void)hipGetLastError();
            count_allocation_call();
            (void)hipFree(ctx->arena);
            const size_t old_cap = ctx->arena_cap;
            ctx->arena = nullptr;
            ctx->arena_cap = 0;
            count_allocation_call();
            grown = hipMalloc(&p, want);
            if (grown != hipSuccess) {  // not even alone: back to the size that did fit
                (void)hipGetLastError();
                void* old = nullptr;
                count_allocation_call();
                if (hipMalloc(&old, old_cap) == hipSuccess) {
                    ctx->arena = static_cast<char*>(old);
                    ctx->arena_cap = old_cap;
                } else {
                    (void)hipGetLastError();
                }
            }
        }
        if (grown == hipSuccess) {
            if (ctx->arena) {  // (the grow fitted beside it)
                count_allocation_call();
                (void)hipFree(ctx->arena);
            }
            ctx->arena = static_cast<char*>(p);
            ctx->arena_cap = want;
        } else {
            ++ctx->arena_grow_failures;  // visible through culsh_debug_arena_state
            (void)hipGetLastError();  // what does not fit falls back to per-allocation blocks
        }
    }
    ctx->arena_want = 0;
    return CULSH_OK;
}

// `arena_want` is the high-water mark of the bytes live at once (arena + overflow blocks), which is
// what the next call's arena is sized by; a caller that rewinds with arena_rewind (batched queries)
// therefore asks for one batch's scratch, not the sum over the batches.
culsh_status arena_alloc(culsh_ctx* ctx, size_t bytes, void** out) {
    bytes = align_up(std::max<size_t>(bytes, 1), ARENA_ALIGN);
    ctx->arena_live += bytes;
    ctx->arena_want = std::max(ctx->arena_want, ctx->arena_live);
    if (ctx->arena && ctx->arena_off + bytes <= ctx->arena_cap) {
        *out = ctx->arena + ctx->arena_off;
        ctx->arena_off += bytes;
        return CULSH_OK;
    }
    void* p = nullptr;
    count_allocation_call();
    CULSH_HIP(hipMalloc(&p, bytes));
    ctx->overflow.push_back(p);
    ++ctx->arena_overflow_blocks;
    *out = p;
    return CULSH_OK;
}

ArenaMark arena_mark(const culsh_ctx* ctx) { return ArenaMark{ctx->arena_off, ctx->arena_live}; }

// Gives back what was allocated since `mark`.  The stream must be idle (the memory may be handed out
// again at once); overflow blocks stay until the end of the call.
void arena_rewind(culsh_ctx* ctx, const ArenaMark& mark) {
    ctx->arena_off = mark.off;
    ctx->arena_live = mark.live;
}

StageTimer::StageTimer(culsh_ctx* c, const char* name) : ctx(c) {
    if (!c->profiling) return;
    if (!c->prof_filter.empty() && std::strstr(name, c->prof_filter.c_str()) == nullptr) return;
    int stage = -1;
    for (size_t i = 0; i < c->prof_stages.size(); ++i)
        if (c->prof_stages[i].name == name) { stage = static_cast<int>(i); break; }
    if (stage < 0) {
        c->prof_stages.push_back({name, 0.0, 0});
        stage = static_cast<int>(c->prof_stages.size()) - 1;
    }
    hipEvent_t ev[2];
    for (auto& e : ev) {
        if (!c->prof_pool.empty()) {
            e = c->prof_pool.back();
            c->prof_pool.pop_back();
        } else if (count_allocation_call(), hipEventCreate(&e) != hipSuccess) {
            (void)hipGetLastError();
            return;
        }
    }
    (void)hipEventRecord(ev[0], c->stream);
    c->prof_pending.push_back({stage, ev[0], ev[1]});
    pending = static_cast<int>(c->prof_pending.size()) - 1;
}

StageTimer::~StageTimer() {
    if (pending >= 0) (void)hipEventRecord(ctx->prof_pending[pending].stop, ctx->stream);
}

void profile_collect(culsh_ctx* ctx) {
    for (auto& p : ctx->prof_pending) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, p.start, p.stop) == hipSuccess) {
            ctx->prof_stages[p.stage].total_ms += ms;
            ctx->prof_stages[p.stage].launches += 1;
        } else {
            (void)hipGetLastError();
        }
        ctx->prof_pool.push_back(p.start);
        ctx->prof_pool.push_back(p.stop);
    }
    ctx->prof_pending.clear();
}

culsh_status arena_end(culsh_ctx* ctx) {
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e == hipSuccess) profile_collect(ctx);
    for (void* p : ctx->overflow) {
        count_allocation_call();
        (void)hipFree(p);
    }
    ctx->overflow.clear();
    if (e != hipSuccess) {
        set_error("stream synchronize failed: %s", hipGetErrorString(e));
        return CULSH_ERR_HIP;
    }
    return CULSH_OK;
}

culsh_status read_back_u64(culsh_ctx* ctx, const uint64_t* dev, int count, uint64_t* host) {
    CULSH_REQUIRE(count <= 64, CULSH_ERR_INTERNAL, "read_back: too many words");
    CULSH_HIP(hipMemcpyAsync(ctx->pinned, dev, count * sizeof(uint64_t), hipMemcpyDeviceToHost, ctx->stream));
    CULSH_HIP(hipStreamSynchronize(ctx->stream));
    std::memcpy(host, ctx->pinned, count * sizeof(uint64_t));
    return CULSH_OK;
}

culsh_status read_back_pair(culsh_ctx* ctx, const uint64_t* dev_a, const uint32_t* dev_b_or_null, uint64_t* a,
                            uint32_t* b) {
    ctx->pinned[1] = 0;
    CULSH_HIP(hipMemcpyAsync(&ctx->pinned[0], dev_a, sizeof(uint64_t), hipMemcpyDeviceToHost, ctx->stream));
    if (dev_b_or_null)
        CULSH_HIP(hipMemcpyAsync(&ctx->pinned[1], dev_b_or_null, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    ctx->pinned[2] = 0;
    if (ctx->aux_flag_dev)  // a family's own flag rides along
        CULSH_HIP(hipMemcpyAsync(&ctx->pinned[2], ctx->aux_flag_dev, sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    CULSH_HIP(hipStreamSynchronize(ctx->stream));
    ctx->aux_flag_host = static_cast<uint32_t>(ctx->pinned[2] & 0xffffffffu);
    *a = ctx->pinned[0];
    *b = static_cast<uint32_t>(ctx->pinned[1] & 0xffffffffu);
    return CULSH_OK;
}

culsh_status read_back_u32(culsh_ctx* ctx, const uint32_t* dev, int count, uint32_t* host) {
    CULSH_REQUIRE(count <= 128, CULSH_ERR_INTERNAL, "read_back: too many words");
    CULSH_HIP(hipMemcpyAsync(ctx->pinned, dev, count * sizeof(uint32_t), hipMemcpyDeviceToHost, ctx->stream));
    CULSH_HIP(hipStreamSynchronize(ctx->stream));
    std::memcpy(host, ctx->pinned, count * sizeof(uint32_t));
    return CULSH_OK;
}

// ---------------------------------------------------------------- seeded generator
// splitmix64 counter streams: r[i] = sm64(key + i), key = sm64(sm64(seed) ^ sm64(stream)).
static inline uint64_t sm64(uint64_t x) {
    uint64_t z = x + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
enum { STREAM_PROJECTION = 1, STREAM_BIAS = 2, STREAM_HASH_A = 3, STREAM_HASH_B = 4 };

void gen_raw_u64(uint64_t seed, int stream, size_t n, uint64_t* out) {
    const uint64_t key = sm64(sm64(seed) ^ sm64(static_cast<uint64_t>(stream)));
    for (size_t i = 0; i < n; ++i) out[i] = sm64(key + i);
}

// Box-Muller: z = sqrt(-2 ln u1) cos(2 pi u2), u1 in (0,1], u2 in [0,1), 53-bit uniforms.
// Element i depends on (key, i) alone, so large requests are cut into ranges for a few host threads.
void gen_normals_f64(uint64_t seed, int stream, size_t n, double* out) {
    const uint64_t key = sm64(sm64(seed) ^ sm64(static_cast<uint64_t>(stream)));
    auto range = [key, out](size_t lo, size_t hi) {
        const double inv = 1.0 / 9007199254740992.0;
        const double two_pi = 6.283185307179586476925286766559;
        for (size_t i = lo; i < hi; ++i) {
            const double u1 = static_cast<double>((sm64(key + 2 * i) >> 11) + 1) * inv;
            const double u2 = static_cast<double>(sm64(key + 2 * i + 1) >> 11) * inv;
            out[i] = std::sqrt(-2.0 * std::log(u1)) * std::cos(two_pi * u2);
        }
    };
    const size_t per_thread = 8192;
    const unsigned hw = std::max(1u, std::thread::hardware_concurrency());
    const size_t want = std::min<size_t>({static_cast<size_t>(16), static_cast<size_t>(hw), n / per_thread});
    if (want < 2) {
        range(0, n);
        return;
    }
    std::vector<std::thread> workers;
    const size_t chunk = (n + want - 1) / want;
    for (size_t w = 1; w < want; ++w) {
        const size_t lo = std::min(n, w * chunk), hi = std::min(n, lo + chunk);
        try {
            workers.emplace_back(range, lo, hi);
        } catch (...) {  // no thread to be had: this one does the range itself
            range(lo, hi);
        }
    }
    range(0, std::min(n, chunk));
    for (std::thread& t : workers) t.join();
}

template <typename T>
static void gen_projection(uint64_t seed, size_t count, int window, T* P) {
    std::vector<double> z(count);
    gen_normals_f64(seed, STREAM_PROJECTION, count, z.data());
    for (size_t i = 0; i < count; ++i) {
        T v = static_cast<T>(z[i]);
        if (window > 0) v = v / static_cast<T>(window);  // pslsh/hash.cuh:85-86
        P[i] = v;
    }
}

template <typename T>
static void gen_bias(uint64_t seed, size_t count, T* b) {  // uniform in (0,1], pslsh/hash.cuh:71-73
    std::vector<uint64_t> r(count);
    gen_raw_u64(seed, STREAM_BIAS, count, r.data());
    for (size_t i = 0; i < count; ++i)
        b[i] = static_cast<T>(static_cast<double>((r[i] >> 11) + 1) * (1.0 / 9007199254740992.0));
}

static void gen_minhash(uint64_t seed, size_t count, uint32_t* A, uint32_t* B, int prime_kind = MH_PRIME_2_32_M5) {
    const uint64_t p = mh_prime_value(prime_kind);  // the reference's: minhash/hash.cuh:17
    std::vector<uint64_t> r(count);
    gen_raw_u64(seed, STREAM_HASH_A, count, r.data());
    for (size_t i = 0; i < count; ++i) A[i] = static_cast<uint32_t>(((r[i] >> 32) % (p - 1)) + 1);  // :27-28
    gen_raw_u64(seed, STREAM_HASH_B, count, r.data());
    for (size_t i = 0; i < count; ++i) B[i] = static_cast<uint32_t>((r[i] >> 32) % p);              // :30-31
}

// ---------------------------------------------------------------- object helpers
void free_index_arrays(culsh_index* ix) {
    if (!ix) return;
    dev_free(ix->all_candidate_indices);
    dev_free(ix->all_bucket_signatures);
    dev_free(ix->bucket_candidate_offsets);
    dev_free(ix->table_bucket_offsets);
    dev_free(ix->bucket_keys);
    dev_free(ix->key_dir);
    dev_free(ix->P);
    dev_free(ix->b);
    dev_free(ix->A);
    dev_free(ix->B);
    free_ps_codec(ix);
    free_mh_codec(ix);
    ix->all_candidate_indices = nullptr;
    ix->all_bucket_signatures = nullptr;
    ix->bucket_candidate_offsets = nullptr;
    ix->table_bucket_offsets = nullptr;
    ix->bucket_keys = nullptr;
    ix->key_dir = nullptr;
    ix->P = ix->b = nullptr;
    ix->A = ix->B = nullptr;
}

void free_candidates_arrays(culsh_candidates* c) {
    if (!c) return;
    dev_free(c->query_candidate_indices);
    dev_free(c->query_candidate_counts);
    dev_free(c->query_candidate_offsets);
    c->query_candidate_indices = nullptr;
    c->query_candidate_counts = nullptr;
    c->query_candidate_offsets = nullptr;
}

struct IndexDeleter {
    void operator()(culsh_index* p) const { free_index_arrays(p); delete p; }
};
struct CandDeleter {
    void operator()(culsh_candidates* p) const { free_candidates_arrays(p); delete p; }
};
using IndexPtr = std::unique_ptr<culsh_index, IndexDeleter>;
using CandPtr = std::unique_ptr<culsh_candidates, CandDeleter>;

template <typename T>
static culsh_status upload(const T* host, size_t count, T** dev) {
    *dev = nullptr;
    if (count == 0) return CULSH_OK;  // empty array -> nullptr (array_utils.cuh:34-36)
    CULSH_HIP(dev_malloc(dev, count * sizeof(T)));
    CULSH_HIP(hipMemcpy(*dev, host, count * sizeof(T), hipMemcpyHostToDevice));
    return CULSH_OK;
}

// Small host arrays (hash parameters, rank tables) go through pinned staging and an asynchronous copy
// on the context's stream: the kernels queued behind it see the data, and the host does not wait for
// the copy.  The staging area is filled from param_stage_off on, which every fit resets at its start
// (the stream is idle then, so nothing reads the area any more).
culsh_status upload_async(culsh_ctx* ctx, const void* host, size_t bytes, void* dev) {
    if (bytes == 0) return CULSH_OK;
    const size_t need = ctx->param_stage_off + align_up(bytes, 256);
    if (need > ctx->param_stage_cap) {
        if (ctx->param_stage_off != 0 || bytes > (size_t(64) << 20)) {  // staging in use or not worth pinning
            CULSH_HIP(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice));
            return CULSH_OK;
        }
        if (ctx->param_stage) (void)hipHostFree(ctx->param_stage);
        ctx->param_stage = nullptr;
        ctx->param_stage_cap = 0;
        const size_t cap = std::max<size_t>(size_t(1) << 20, 2 * align_up(bytes, 256));
        count_allocation_call();
        if (hipHostMalloc(reinterpret_cast<void**>(&ctx->param_stage), cap, hipHostMallocDefault) != hipSuccess) {
            (void)hipGetLastError();
            ctx->param_stage = nullptr;
            CULSH_HIP(hipMemcpy(dev, host, bytes, hipMemcpyHostToDevice));
            return CULSH_OK;
        }
        ctx->param_stage_cap = cap;
    }
    char* slot = ctx->param_stage + ctx->param_stage_off;
    std::memcpy(slot, host, bytes);
    ctx->param_stage_off += align_up(bytes, 256);
    CULSH_HIP(hipMemcpyAsync(dev, slot, bytes, hipMemcpyHostToDevice, ctx->stream));
    return CULSH_OK;
}

template <typename T>
static culsh_status upload_params(culsh_ctx* ctx, const T* host, size_t count, T** dev) {
    *dev = nullptr;
    if (count == 0) return CULSH_OK;
    CULSH_HIP(dev_malloc(dev, count * sizeof(T)));
    return upload_async(ctx, host, count * sizeof(T), *dev);
}

// More than CULSH_MAX_TABLES tables are refused by every fit (and by culsh_index_load), before any device
// work: the query kernels give every table of a query a thread of one workgroup, so such an index could be
// built and saved but never queried.  (The reference has no stated bound; its kernels are written for tens
// of tables, core/fit.cuh:59-68.)
static culsh_status check_fit_args(culsh_ctx* ctx, const void* X, int n, int d, int T, int H, void* out) {
    CULSH_REQUIRE(ctx && X && out, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(n > 0 && d > 0, CULSH_ERR_INVALID, "n_samples and n_features must be positive");
    CULSH_REQUIRE(T > 0 && H > 0, CULSH_ERR_INVALID, "n_hash_tables and n_hashes must be positive");
    CULSH_REQUIRE(T <= CULSH_MAX_TABLES, CULSH_ERR_LIMIT, "n_hash_tables > 1024 is not supported");
    CULSH_REQUIRE(static_cast<long long>(n) * T < (1ll << 31), CULSH_ERR_LIMIT,
                  "n_samples * n_hash_tables must be below 2^31 (int32 candidate positions)");
    return CULSH_OK;
}

// ---------------------------------------------------------------- hashing to key words
enum Family { FAM_RPLSH, FAM_PSLSH };

// Dense rows -> key words [T][rows][W] in the arena.  For p-stable hashing at fit time
// (`fit_ix` given) the key encoding is chosen here and recorded in the index; at query time
// (`ix` given) the index's encoding is used.
template <typename T>
static culsh_status hash_dense_to_keys(culsh_ctx* ctx, Family fam, const T* X, int rows, int d, int nT, int H,
                                       const void* P, const void* b, culsh_index* fit_ix, const culsh_index* ix,
                                       uint32_t** keys_out, int* W_out) {
    const size_t N = static_cast<size_t>(rows) * nT;
    uint32_t* keys = nullptr;
    if (fam == FAM_RPLSH) {
        const int W = key_words(ENC_BITS, H);
        CULSH_TRY(arena_alloc_t(ctx, N * W, &keys));
        if constexpr (std::is_same_v<T, float>) {
            CULSH_TRY(launch_project_f32(ctx, X, static_cast<const float*>(P), nullptr, rows, d, nT, H, EPI_SIGN_KEYS, keys));
        } else {
            CULSH_TRY(launch_project_f64(ctx, X, static_cast<const double*>(P), nullptr, rows, d, nT, H, EPI_SIGN_KEYS, keys));
        }
        *keys_out = keys;
        *W_out = W;
        return CULSH_OK;
    }
    // p-stable: int32 hashes in the reference layout first (pslsh/hash.cuh:25-47)
    int32_t* sig = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, N * H, &sig));
    int32_t* mm = nullptr;     // fit: value range of every hash function, folded by the projection where it can
    bool mm_folded = false;
    if constexpr (std::is_same_v<T, float>) {
        if (fit_ix && H <= 1024) CULSH_TRY(ps_minmax_prepare(ctx, nT, H, &mm));
        CULSH_TRY(launch_project_f32(ctx, X, static_cast<const float*>(P), static_cast<const float*>(b), rows, d, nT, H,
                                     EPI_FLOOR_I32, sig, mm, &mm_folded));
    } else {
        CULSH_TRY(launch_project_f64(ctx, X, static_cast<const double*>(P), static_cast<const double*>(b), rows, d, nT,
                                     H, EPI_FLOOR_I32, sig));
    }
    if (fit_ix) {
        bool compressed = false;
        CULSH_TRY(ps_build_codec(ctx, sig, rows, nT, H, fit_ix, &compressed, mm_folded ? mm : nullptr));
        if (!compressed) { fit_ix->enc = ENC_BE; fit_ix->key_w = H; }
        ix = fit_ix;
    }
    const int W = ix->key_w;
    CULSH_TRY(arena_alloc_t(ctx, N * W, &keys));
    if (ix->enc == ENC_PSC)
        CULSH_TRY(launch_ps_compress(ctx, sig, rows, nT, H, ix, keys));
    else
        CULSH_TRY(launch_sig_to_keys(ctx, reinterpret_cast<const uint8_t*>(sig), N, 4 * H, ENC_BE, W, keys));
    *keys_out = keys;
    *W_out = W;
    return CULSH_OK;
}

// ---------------------------------------------------------------- candidates concatenation
__global__ void shift_offsets_kernel(const uint64_t* __restrict__ src, uint64_t* __restrict__ dst, size_t count,
                                     uint64_t base) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < count) dst[i] = src[i] + base;
}

// One pre-sized result instead of the reference's re-allocation per batch
// (Candidates::merge, core/candidates.cuh:139-197); same contents.
// `lists` (may be null): an array of `lists_cap` elements that already holds, at its final place, the lists of
// the parts marked lists_in_place.  It becomes the result's array when everything fits; `*lists` is taken over
// or freed here either way.
static culsh_status concat_candidates(culsh_ctx* ctx, const std::vector<culsh_candidates*>& parts,
                                      culsh_candidates* out, int32_t** lists = nullptr, uint64_t lists_cap = 0) {
    size_t nq = 0;
    uint64_t total = 0;
    for (auto* p : parts) { nq += p->n_queries; total += p->n_total_candidates; }
    int32_t* placed = lists ? *lists : nullptr;  // owned here from now on
    if (lists) *lists = nullptr;
    struct Guard { int32_t* p; ~Guard() { dev_free(p); } } guard{placed};
    CULSH_REQUIRE(nq < (1ull << 31), CULSH_ERR_LIMIT, "too many queries");
    out->n_queries = static_cast<int>(nq);
    out->n_total_candidates = total;
    CULSH_HIP(dev_malloc(&out->query_candidate_counts, std::max<size_t>(1, nq) * sizeof(uint64_t)));
    CULSH_HIP(dev_malloc(&out->query_candidate_offsets, (nq + 1) * sizeof(uint64_t)));
    const bool keep = placed && total > 0 && total <= lists_cap;  // the pre-filled array is the result's
    if (keep) {
        out->query_candidate_indices = placed;
        guard.p = nullptr;
    } else if (total) {
        CULSH_HIP(dev_malloc(&out->query_candidate_indices, total * sizeof(int32_t)));
    }
    size_t q0 = 0;
    uint64_t c0 = 0;
    CULSH_HIP(hipMemsetAsync(out->query_candidate_offsets, 0, sizeof(uint64_t), ctx->stream));
    for (auto* p : parts) {
        if (p->n_total_candidates) {
            const int32_t* src = p->lists_in_place ? (placed ? placed + c0 : nullptr) : p->query_candidate_indices;
            CULSH_REQUIRE(src, CULSH_ERR_INTERNAL, "a batch's candidate lists are missing");
            if (!(keep && p->lists_in_place))
                CULSH_HIP(hipMemcpyAsync(out->query_candidate_indices + c0, src, p->n_total_candidates * sizeof(int32_t),
                                         hipMemcpyDeviceToDevice, ctx->stream));
        }
        if (p->n_queries) {
            CULSH_HIP(hipMemcpyAsync(out->query_candidate_counts + q0, p->query_candidate_counts,
                                     p->n_queries * sizeof(uint64_t), hipMemcpyDeviceToDevice, ctx->stream));
            // offsets[1..] of the part, shifted by the running total (candidates.cuh:178-183)
            CULSH_LAUNCH(ctx, shift_offsets_kernel, dim3(div_up(p->n_queries, 256)), dim3(256), 0, ctx->stream,
                               p->query_candidate_offsets + 1, out->query_candidate_offsets + q0 + 1,
                               static_cast<size_t>(p->n_queries), c0);
            CULSH_LAUNCH_CHECK();
        }
        q0 += p->n_queries;
        c0 += p->n_total_candidates;
    }
    if (guard.p) CULSH_HIP(hipStreamSynchronize(ctx->stream));  // copies out of the array that the guard frees
    return CULSH_OK;
}

// query over key words that are already in the arena
static culsh_status query_keys(culsh_ctx* ctx, const uint32_t* q_keys, int nq, const culsh_index* ix,
                               culsh_candidates* out, int32_t* lists_dst = nullptr, uint64_t lists_cap = 0,
                               int key_rows = 0, int key_first = 0) {
    return query_from_keys(ctx, q_keys, nq, ix, out, lists_dst, lists_cap, key_rows, key_first);
}

template <typename T>
static culsh_status dense_query(culsh_ctx* ctx, Family fam, const T* Q, int nq, const culsh_index* ix,
                                int batch_size, culsh_candidates** out) {
    CULSH_REQUIRE(ctx && Q && ix && out, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(nq > 0, CULSH_ERR_INVALID, "n_queries must be positive");
    CULSH_REQUIRE(ix->kind == (fam == FAM_RPLSH ? CULSH_KIND_RPLSH : CULSH_KIND_PSLSH), CULSH_ERR_INVALID,
                  "index was built by a different hashing family");
    const bool want_double = std::is_same_v<T, double>;
    if (ix->is_double && !want_double) {
        set_error("Index was fitted with float64, but query is float32");  // bindings.cu:58-60
        return CULSH_ERR_INVALID;
    }
    if (!ix->is_double && want_double) {
        set_error("Index was fitted with float32, but query is float64");  // bindings.cu:75-77
        return CULSH_ERR_INVALID;
    }
    CULSH_REQUIRE(ix->P && (fam == FAM_RPLSH || ix->b), CULSH_ERR_INVALID, "index holds no hash parameters");
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    const int d = ix->n_features, nT = ix->n_hash_tables, H = ix->n_hashes;
    if (batch_size <= 0 || batch_size >= nq) batch_size = nq;  // rplsh.cu:190-192
    std::vector<CandPtr> parts;
    // The batches' lists go straight into one array, sized after the first batch by what it found per
    // query (plus 15 %): the first batch's lists are copied there once, later batches write theirs behind
    // what is there already; a batch that does not fit gets an array of its own and everything is put
    // together at the end, as for the reference's merge.
    struct Lists { int32_t* p = nullptr; ~Lists() { dev_free(p); } } lists;
    uint64_t lists_cap = 0, lists_used = 0;
    bool contiguous = true;  // all lists so far are (or can be put) in `lists` one behind the other
    // The queries of all batches are hashed in one launch when their key words are a modest amount of memory
    // (the batches bound the candidates, which are what is large): a batch of some thousand rows fills a
    // fraction of the device, 10,000 rows x 768 x 1024 run at 0.62 of the fp32 MFMA peak against 0.87 for
    // 100,000.  Every batch then looks its rows up in the key array of all queries.
    uint32_t* all_keys = nullptr;
    int W_all = 0;
    // (p-stable hashing also holds the int32 hashes of all rows until the keys are made)
    const size_t key_bytes = static_cast<size_t>(nq) * nT * (static_cast<size_t>(std::max(1, ix->key_w)) + (fam == FAM_RPLSH ? 0 : H)) *
                             sizeof(uint32_t);
    if (batch_size < nq && key_bytes <= (size_t(1) << 30))
        CULSH_TRY(hash_dense_to_keys<T>(ctx, fam, Q, nq, d, nT, H, ix->P, ix->b, nullptr, ix, &all_keys, &W_all));
    for (int start = 0; start < nq; start += batch_size) {
        const int bn = std::min(batch_size, nq - start);
        const ArenaMark mark = arena_mark(ctx);
        uint32_t* keys = all_keys;
        int W = W_all;
        if (!all_keys)
            CULSH_TRY(hash_dense_to_keys<T>(ctx, fam, Q + static_cast<size_t>(start) * d, bn, d, nT, H, ix->P, ix->b,
                                            nullptr, ix, &keys, &W));
        CandPtr part(new (std::nothrow) culsh_candidates());
        CULSH_REQUIRE(part, CULSH_ERR_NOMEM, "host allocation failed");
        part->device = ctx->device;
        const bool room = lists.p && contiguous && lists_used < lists_cap;
        CULSH_TRY(query_keys(ctx, keys, bn, ix, part.get(), room ? lists.p + lists_used : nullptr,
                             room ? lists_cap - lists_used : 0, all_keys ? nq : 0, all_keys ? start : 0));
        const uint64_t found = part->n_total_candidates;
        if (start == 0 && bn < nq && found > 0) {
            const double per_query = static_cast<double>(found) / bn;
            lists_cap = static_cast<uint64_t>(per_query * nq * 1.15) + 4096;
            if (dev_malloc(&lists.p, lists_cap * sizeof(int32_t)) == hipSuccess) {
                CULSH_HIP(hipMemcpyAsync(lists.p, part->query_candidate_indices, found * sizeof(int32_t),
                                         hipMemcpyDeviceToDevice, ctx->stream));
                part->lists_in_place = true;  // (it keeps its own array until the parts are freed)
            } else {
                (void)hipGetLastError();
                lists.p = nullptr;
                lists_cap = 0;
            }
        }
        if (lists.p && contiguous) {
            if (part->lists_in_place || found == 0) lists_used += found;
            else contiguous = false;  // this batch's lists sit elsewhere: the ones behind it cannot be placed yet
        }
        parts.push_back(std::move(part));
        arena_rewind(ctx, mark);  // the batch's query has ended with the stream idle
    }
    if (parts.size() == 1) {
        CULSH_TRY(arena_end(ctx));
        *out = parts[0].release();
        return CULSH_OK;
    }
    CandPtr result(new (std::nothrow) culsh_candidates());
    CULSH_REQUIRE(result, CULSH_ERR_NOMEM, "host allocation failed");
    result->device = ctx->device;
    std::vector<culsh_candidates*> raw;
    for (auto& p : parts) raw.push_back(p.get());
    CULSH_TRY(concat_candidates(ctx, raw, result.get(), &lists.p, lists_cap));
    CULSH_TRY(arena_end(ctx));  // parts are freed after the copies have run
    *out = result.release();
    return CULSH_OK;
}

// Shared tail of every fit: keys -> index (+ optional fit_query).
static culsh_status finish_fit(culsh_ctx* ctx, uint32_t* keys, int n, int T, int H, int S, KeyEnc enc, int W,
                               culsh_index* ix, culsh_candidates* cands_or_null) {
    int32_t* item_to_bucket = nullptr;
    if (cands_or_null) CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n) * T, &item_to_bucket));
    CULSH_TRY(fit_index_from_keys(ctx, keys, n, T, H, S, enc, W, item_to_bucket, ix));
    // A family's own flag has come back with the end-of-build read-back (MinHash rank keys: a column id
    // at or beyond n_features).  The keys are void then; the caller fits again with plain keys, and the
    // query of the fitted rows is not run on an index that is about to be dropped.
    if (ctx->aux_flag_host) return CULSH_RETRY_PLAIN_KEYS;
    if (cands_or_null)  // core/fit_query.cuh:46-50
        CULSH_TRY(query_from_matched(ctx, item_to_bucket, n, ix, cands_or_null));
    return CULSH_OK;
}

template <typename T>
static culsh_status dense_fit_once(culsh_ctx* ctx, Family fam, const T* X, int n, int d, int nT, int H, int window,
                              uint64_t seed, const T* P_host, const T* b_host, culsh_index** index_out,
                              culsh_candidates** cands_out) {
    CULSH_TRY(check_fit_args(ctx, X, n, d, nT, H, index_out ? static_cast<void*>(index_out) : static_cast<void*>(cands_out)));
    if (fam == FAM_PSLSH) {
        CULSH_REQUIRE(window > 0, CULSH_ERR_INVALID, "window_size must be positive");
        CULSH_REQUIRE((P_host == nullptr) == (b_host == nullptr), CULSH_ERR_INVALID,
                      "projection and bias must be given together");
    }
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    IndexPtr ix(new (std::nothrow) culsh_index());
    CULSH_REQUIRE(ix, CULSH_ERR_NOMEM, "host allocation failed");
    ix->device = ctx->device;
    ix->kind = (fam == FAM_RPLSH) ? CULSH_KIND_RPLSH : CULSH_KIND_PSLSH;
    ix->is_double = std::is_same_v<T, double>;
    ix->window_size = (fam == FAM_PSLSH) ? window : 0;
    const size_t TH = static_cast<size_t>(nT) * H;
    {
        ctx->param_stage_off = 0;
        if (!P_host) {
            culsh_ctx::GenCache& gc = ctx->gen_cache;
            const int win = fam == FAM_PSLSH ? window : 0;
            if (!(gc.family == static_cast<int>(fam) && gc.seed == seed && gc.rows == TH && gc.d == static_cast<size_t>(d) &&
                  gc.window == win && gc.elem == static_cast<int>(sizeof(T)))) {
                gc.family = -1;
                gc.p.resize(TH * d * sizeof(T));
                gen_projection<T>(seed, TH * d, win, reinterpret_cast<T*>(gc.p.data()));
                gc.b.clear();
                if (fam == FAM_PSLSH) {
                    gc.b.resize(TH * sizeof(T));
                    gen_bias<T>(seed, TH, reinterpret_cast<T*>(gc.b.data()));
                }
                gc.family = static_cast<int>(fam);
                gc.seed = seed;
                gc.rows = TH;
                gc.d = static_cast<size_t>(d);
                gc.window = win;
                gc.elem = static_cast<int>(sizeof(T));
            }
            P_host = reinterpret_cast<const T*>(gc.p.data());
            if (fam == FAM_PSLSH) b_host = reinterpret_cast<const T*>(gc.b.data());
        }
        T* dP = nullptr;
        CULSH_TRY(upload_params(ctx, P_host, TH * d, &dP));
        ix->P = dP;
        if (fam == FAM_PSLSH) {
            T* db = nullptr;
            CULSH_TRY(upload_params(ctx, b_host, TH, &db));
            ix->b = db;
        }
    }
    uint32_t* keys = nullptr;
    int W = 0;
    CULSH_TRY(hash_dense_to_keys<T>(ctx, fam, X, n, d, nT, H, ix->P, ix->b, ix.get(), nullptr, &keys, &W));
    const KeyEnc enc = (fam == FAM_RPLSH) ? ENC_BITS : ix->enc;
    const int S = (fam == FAM_RPLSH) ? H : 4 * H;  // rplsh.cu:37, pslsh.cu:39
    CandPtr cands;
    if (cands_out) {
        cands.reset(new (std::nothrow) culsh_candidates());
        CULSH_REQUIRE(cands, CULSH_ERR_NOMEM, "host allocation failed");
        cands->device = ctx->device;
    }
    CULSH_TRY(finish_fit(ctx, keys, n, nT, H, S, enc, W, ix.get(), cands.get()));
    ix->n_features = d;
    ix->seed = seed;
    CULSH_TRY(arena_end(ctx));
    if (index_out) *index_out = ix.release();
    if (cands_out) *cands_out = cands.release();  // the index (and P) is dropped, rplsh.cu:152-155
    return CULSH_OK;
}

static culsh_status minhash_fit_once(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr, int n, int d,
                                     int nT, int H, uint64_t seed, const uint32_t* A_host, const uint32_t* B_host,
                                     bool plain_keys, culsh_index** index_out, culsh_candidates** cands_out) {
    CULSH_TRY(check_fit_args(ctx, indptr, n, d, nT, H, index_out ? static_cast<void*>(index_out) : static_cast<void*>(cands_out)));
    CULSH_REQUIRE((A_host == nullptr) == (B_host == nullptr), CULSH_ERR_INVALID, "hash_a and hash_b must be given together");
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    IndexPtr ix(new (std::nothrow) culsh_index());
    CULSH_REQUIRE(ix, CULSH_ERR_NOMEM, "host allocation failed");
    ix->device = ctx->device;
    ix->kind = CULSH_KIND_MINHASH;
    ix->mh_prime_kind = ctx->mh_prime_kind;
    const size_t TH = static_cast<size_t>(nT) * H;
    {
        ctx->param_stage_off = 0;
        if (!A_host) {
            culsh_ctx::GenCache& gc = ctx->gen_cache;
            const int FAM_MINHASH_TAG = 100 + ctx->mh_prime_kind;
            if (!(gc.family == FAM_MINHASH_TAG && gc.seed == seed && gc.rows == TH)) {
                gc.family = -1;
                gc.p.resize(TH * sizeof(uint32_t));
                gc.b.resize(TH * sizeof(uint32_t));
                gen_minhash(seed, TH, reinterpret_cast<uint32_t*>(gc.p.data()), reinterpret_cast<uint32_t*>(gc.b.data()),
                            ctx->mh_prime_kind);
                gc.family = FAM_MINHASH_TAG;
                gc.seed = seed;
                gc.rows = TH;
            }
            A_host = reinterpret_cast<const uint32_t*>(gc.p.data());
            B_host = reinterpret_cast<const uint32_t*>(gc.b.data());
        }
        CULSH_TRY(upload_params(ctx, A_host, TH, &ix->A));
        CULSH_TRY(upload_params(ctx, B_host, TH, &ix->B));
    }
    const size_t N = static_cast<size_t>(n) * nT;
    // rank codes instead of raw hash values where that shortens the keys
    bool ranked = false;
    if (!plain_keys) CULSH_TRY(mh_build_codec(ctx, nT, H, d, ix.get(), &ranked));
    uint32_t* keys = nullptr;
    KeyEnc enc = ENC_BE;
    int W = H;
    if (ranked) {
        enc = ENC_MHR;
        W = ix->key_w;
        CULSH_TRY(arena_alloc_t(ctx, N * W, &keys));
        // rank codes cover column ids below n_features; the kernel flags any other id in a word that
        // comes back with the end-of-build read-back
        CULSH_TRY(arena_alloc_t(ctx, 1, &ctx->aux_flag_dev));
        CULSH_HIP(hipMemsetAsync(ctx->aux_flag_dev, 0, sizeof(uint32_t), ctx->stream));
        CULSH_TRY(launch_minhash_rank(ctx, indices, indptr, n, nT, H, ix.get(), ctx->aux_flag_dev, keys));
    } else {
        CULSH_TRY(arena_alloc_t(ctx, N * H, &keys));
        CULSH_TRY(launch_minhash(ctx, indices, indptr, ix->A, ix->B, n, nT, H, true, keys, ix->mh_prime_kind));
    }
    CandPtr cands;
    if (cands_out) {
        cands.reset(new (std::nothrow) culsh_candidates());
        CULSH_REQUIRE(cands, CULSH_ERR_NOMEM, "host allocation failed");
        cands->device = ctx->device;
    }
    {
        const culsh_status st = finish_fit(ctx, keys, n, nT, H, 4 * H, enc, W, ix.get(), cands.get());  // minhash.cu:37
        if (st == CULSH_RETRY_PLAIN_KEYS) {  // a column id at or beyond n_features: these keys are void
            CULSH_TRY(arena_end(ctx));
            return CULSH_RETRY_PLAIN_KEYS;
        }
        CULSH_TRY(st);
    }
    ix->n_features = d;
    ix->seed = seed;
    CULSH_TRY(arena_end(ctx));
    if (index_out) *index_out = ix.release();
    if (cands_out) *cands_out = cands.release();
    return CULSH_OK;
}

static size_t elem_size_of(const culsh_index* ix, culsh_array which) {
    switch (which) {
        case CULSH_ARR_BUCKET_SIGNATURES: return 1;
        case CULSH_ARR_PROJECTION:
        case CULSH_ARR_BIAS: return ix->is_double ? 8 : 4;
        default: return 4;
    }
}

static culsh_status index_array(const culsh_index* ix, culsh_array which, const void** ptr, uint64_t* count) {
    const uint64_t TH = static_cast<uint64_t>(ix->n_hash_tables) * ix->n_hashes;
    switch (which) {
        case CULSH_ARR_CANDIDATE_INDICES: *ptr = ix->all_candidate_indices; *count = ix->n_total_candidates; break;
        case CULSH_ARR_BUCKET_SIGNATURES:
            *ptr = ix->all_bucket_signatures;
            *count = static_cast<uint64_t>(ix->n_total_buckets) * ix->sig_nbytes;
            break;
        case CULSH_ARR_BUCKET_CANDIDATE_OFFSETS:
            *ptr = ix->bucket_candidate_offsets; *count = static_cast<uint64_t>(ix->n_total_buckets) + 1; break;
        case CULSH_ARR_TABLE_BUCKET_OFFSETS:
            *ptr = ix->table_bucket_offsets; *count = static_cast<uint64_t>(ix->n_hash_tables) + 1; break;
        case CULSH_ARR_PROJECTION: *ptr = ix->P; *count = ix->P ? TH * ix->n_features : 0; break;
        case CULSH_ARR_BIAS: *ptr = ix->b; *count = ix->b ? TH : 0; break;
        case CULSH_ARR_HASH_A: *ptr = ix->A; *count = ix->A ? TH : 0; break;
        case CULSH_ARR_HASH_B: *ptr = ix->B; *count = ix->B ? TH : 0; break;
        default: set_error("not an index array: %d", static_cast<int>(which)); return CULSH_ERR_INVALID;
    }
    if (*ptr == nullptr) *count = 0;
    return CULSH_OK;
}

}  // namespace culsh_amd

using namespace culsh_amd;

// ======================================================================================
// The radix sort's chained scan cannot stall as long as workgroups start in index order;
// should it ever give up, the context switches to unchained passes and the fit is repeated
// from the hashing step (the sort has overwritten its input by then).
template <typename F>
static culsh_status with_sort_retry(culsh_ctx* ctx, F&& fit) {
    culsh_status s = fit();
    if (s == CULSH_RETRY_UNCHAINED && ctx) {
        ctx->sort_unchained = true;
        s = fit();
    }
    if (s == CULSH_RETRY_UNCHAINED) {
        set_error("radix sort: chained scan gave up and no unchained retry was possible");
        s = CULSH_ERR_INTERNAL;
    }
    return s;
}

template <typename T>
static culsh_status dense_fit(culsh_ctx* ctx, Family fam, const T* X, int n, int d, int nT, int H, int window,
                              uint64_t seed, const T* P_host, const T* b_host, culsh_index** index_out,
                              culsh_candidates** cands_out) {
    return with_sort_retry(ctx, [&] {
        return dense_fit_once<T>(ctx, fam, X, n, d, nT, H, window, seed, P_host, b_host, index_out, cands_out);
    });
}

static culsh_status minhash_fit_impl(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr, int n, int d,
                                     int nT, int H, uint64_t seed, const uint32_t* A_host, const uint32_t* B_host,
                                     culsh_index** index_out, culsh_candidates** cands_out) {
    culsh_status s = with_sort_retry(ctx, [&] {
        return minhash_fit_once(ctx, indices, indptr, n, d, nT, H, seed, A_host, B_host, false, index_out, cands_out);
    });
    if (s == CULSH_RETRY_PLAIN_KEYS)
        s = with_sort_retry(ctx, [&] {
            return minhash_fit_once(ctx, indices, indptr, n, d, nT, H, seed, A_host, B_host, true, index_out, cands_out);
        });
    return s;
}

extern "C" {

const char* culsh_last_error(void) { return g_last_error.c_str(); }
const char* culsh_version(void) { return "culsh_amd 0.1.0 (gfx950)"; }

// ---- the entry point that allocates nothing
// Key words of the queries on their way to the lookup kernel live in this array instead of the
// context's arena.  Every device the library runs on holds its own copy at its own address; the
// array's name is only a host-side handle of the symbol, so the address is asked for once per device
// (culsh_ctx_create, with that device current) and kept.
static __device__ __align__(256) uint32_t g_static_scratch[CULSH_STATIC_SCRATCH_WORDS];
static std::mutex g_static_scratch_mutex;
static uint32_t* g_static_scratch_ptr[64] = {};

static culsh_status static_scratch_init(int device) {  // `device` is current
    if (device < 0 || device >= 64) return CULSH_OK;   // such a device has no static entry point
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (g_static_scratch_ptr[device]) return CULSH_OK;
    void* p = nullptr;
    CULSH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_scratch)));
    CULSH_REQUIRE(p != nullptr, CULSH_ERR_HIP, "hipGetSymbolAddress returned a null address");
    g_static_scratch_ptr[device] = static_cast<uint32_t*>(p);
    return CULSH_OK;
}

culsh_status culsh_ctx_create(int device, culsh_ctx** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    *out = nullptr;
    int count = 0;
    CULSH_HIP(hipGetDeviceCount(&count));
    CULSH_REQUIRE(device >= 0 && device < count, CULSH_ERR_INVALID, "device %d out of range (%d visible)", device, count);
    CULSH_HIP(hipSetDevice(device));
    std::unique_ptr<culsh_ctx> ctx(new (std::nothrow) culsh_ctx());
    CULSH_REQUIRE(ctx, CULSH_ERR_NOMEM, "host allocation failed");
    ctx->device = device;
    hipDeviceProp_t prop;
    CULSH_HIP(hipGetDeviceProperties(&prop, device));
    CULSH_REQUIRE(std::strncmp(prop.gcnArchName, "gfx950", 6) == 0, CULSH_ERR_INVALID,
                  "device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
    ctx->n_cus = prop.multiProcessorCount;
    int lds_optin = 0;
    if (hipDeviceGetAttribute(&lds_optin, hipDeviceAttributeMaxSharedMemoryPerBlock, device) != hipSuccess) {
        (void)hipGetLastError();
        lds_optin = 0;
    }
    ctx->lds_max = std::max<int>(static_cast<int>(prop.sharedMemPerBlock), lds_optin);
    if (ctx->lds_max <= 0) ctx->lds_max = 65536;
    CULSH_HIP(hipStreamCreate(&ctx->stream));  // default priority
    void* pinned = nullptr;
    if (hipHostMalloc(&pinned, 64 * sizeof(uint64_t), hipHostMallocDefault) != hipSuccess) {
        (void)hipStreamDestroy(ctx->stream);
        set_error("hipHostMalloc failed");
        return CULSH_ERR_NOMEM;
    }
    ctx->pinned = static_cast<uint64_t*>(pinned);
    // The workspace of the entry point that allocates nothing.  If its address cannot be had, only that
    // entry point is affected (it reports the missing workspace); everything else works without it.
    if (static_scratch_init(device) != CULSH_OK) (void)hipGetLastError();
    *out = ctx.release();
    return CULSH_OK;
}

void culsh_ctx_destroy(culsh_ctx* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipStreamDestroy(ctx->stream);
    }
    profile_collect(ctx);
    for (hipEvent_t e : ctx->prof_pool) (void)hipEventDestroy(e);
    for (void* p : ctx->overflow) {
        count_allocation_call();
        (void)hipFree(p);
    }
    if (ctx->arena) (void)hipFree(ctx->arena);
    if (ctx->pinned) (void)hipHostFree(ctx->pinned);
    if (ctx->param_stage) (void)hipHostFree(ctx->param_stage);
    delete ctx;
}

culsh_status culsh_ctx_synchronize(culsh_ctx* ctx) {
    CULSH_REQUIRE(ctx, CULSH_ERR_INVALID, "null argument");
    CULSH_HIP(hipStreamSynchronize(ctx->stream));
    return CULSH_OK;
}

void* culsh_ctx_stream(culsh_ctx* ctx) { return ctx ? static_cast<void*>(ctx->stream) : nullptr; }

void culsh_memory_trim(void) { culsh_amd::dev_trim(); }

culsh_status culsh_profile_enable(culsh_ctx* ctx, int on) {
    CULSH_REQUIRE(ctx, CULSH_ERR_INVALID, "null argument");
    CULSH_HIP(hipStreamSynchronize(ctx->stream));
    profile_collect(ctx);
    ctx->profiling = on != 0;
    return CULSH_OK;
}
culsh_status culsh_profile_filter(culsh_ctx* ctx, const char* substring) {
    CULSH_REQUIRE(ctx, CULSH_ERR_INVALID, "null argument");
    ctx->prof_filter = substring ? substring : "";
    return CULSH_OK;
}
culsh_status culsh_profile_reset(culsh_ctx* ctx) {
    CULSH_REQUIRE(ctx, CULSH_ERR_INVALID, "null argument");
    CULSH_HIP(hipStreamSynchronize(ctx->stream));
    profile_collect(ctx);
    ctx->prof_stages.clear();
    return CULSH_OK;
}
int culsh_profile_count(const culsh_ctx* ctx) { return ctx ? static_cast<int>(ctx->prof_stages.size()) : 0; }
culsh_status culsh_profile_get(const culsh_ctx* ctx, int i, const char** name, double* total_ms, int64_t* launches) {
    CULSH_REQUIRE(ctx && name && total_ms && launches, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(i >= 0 && i < static_cast<int>(ctx->prof_stages.size()), CULSH_ERR_INVALID, "stage index out of range");
    *name = ctx->prof_stages[i].name.c_str();
    *total_ms = ctx->prof_stages[i].total_ms;
    *launches = ctx->prof_stages[i].launches;
    return CULSH_OK;
}

// ---- generators
culsh_status culsh_generate_projection_f32(uint64_t seed, int n_rows, int d, float* P) {
    CULSH_REQUIRE(P && n_rows > 0 && d > 0, CULSH_ERR_INVALID, "bad argument");
    gen_projection<float>(seed, static_cast<size_t>(n_rows) * d, 0, P);
    return CULSH_OK;
}
culsh_status culsh_generate_projection_f64(uint64_t seed, int n_rows, int d, double* P) {
    CULSH_REQUIRE(P && n_rows > 0 && d > 0, CULSH_ERR_INVALID, "bad argument");
    gen_projection<double>(seed, static_cast<size_t>(n_rows) * d, 0, P);
    return CULSH_OK;
}
culsh_status culsh_generate_pslsh_params_f32(uint64_t seed, int n_rows, int d, int w, float* P, float* b) {
    CULSH_REQUIRE(P && b && n_rows > 0 && d > 0 && w > 0, CULSH_ERR_INVALID, "bad argument");
    gen_projection<float>(seed, static_cast<size_t>(n_rows) * d, w, P);
    gen_bias<float>(seed, n_rows, b);
    return CULSH_OK;
}
culsh_status culsh_generate_pslsh_params_f64(uint64_t seed, int n_rows, int d, int w, double* P, double* b) {
    CULSH_REQUIRE(P && b && n_rows > 0 && d > 0 && w > 0, CULSH_ERR_INVALID, "bad argument");
    gen_projection<double>(seed, static_cast<size_t>(n_rows) * d, w, P);
    gen_bias<double>(seed, n_rows, b);
    return CULSH_OK;
}
culsh_status culsh_generate_minhash_params(uint64_t seed, int n_rows, uint32_t* A, uint32_t* B) {
    CULSH_REQUIRE(A && B && n_rows > 0, CULSH_ERR_INVALID, "bad argument");
    gen_minhash(seed, n_rows, A, B);
    return CULSH_OK;
}
static bool prime_kind_of(uint32_t prime, int* kind) {
    if (prime == mh_prime_value(MH_PRIME_2_32_M5)) { *kind = MH_PRIME_2_32_M5; return true; }
    if (prime == mh_prime_value(MH_PRIME_2_31_M1)) { *kind = MH_PRIME_2_31_M1; return true; }
    return false;
}
culsh_status culsh_generate_minhash_params_mod(uint64_t seed, int n_rows, uint32_t prime, uint32_t* A, uint32_t* B) {
    int kind = 0;
    CULSH_REQUIRE(A && B && n_rows > 0, CULSH_ERR_INVALID, "bad argument");
    CULSH_REQUIRE(prime_kind_of(prime, &kind), CULSH_ERR_INVALID, "MinHash prime must be 4294967291 or 2147483647");
    gen_minhash(seed, n_rows, A, B, kind);
    return CULSH_OK;
}
culsh_status culsh_ctx_set_minhash_prime(culsh_ctx* ctx, uint32_t prime) {
    int kind = 0;
    CULSH_REQUIRE(ctx, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(prime_kind_of(prime, &kind), CULSH_ERR_INVALID, "MinHash prime must be 4294967291 or 2147483647");
    ctx->mh_prime_kind = kind;
    return CULSH_OK;
}
culsh_status culsh_ctx_get_minhash_prime(const culsh_ctx* ctx, uint32_t* prime) {
    CULSH_REQUIRE(ctx && prime, CULSH_ERR_INVALID, "null argument");
    *prime = mh_prime_value(ctx->mh_prime_kind);
    return CULSH_OK;
}
culsh_status culsh_index_minhash_prime(const culsh_index* ix, uint32_t* prime) {
    CULSH_REQUIRE(ix && prime, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(ix->kind == CULSH_KIND_MINHASH, CULSH_ERR_INVALID, "not a MinHash index");
    *prime = mh_prime_value(ix->mh_prime_kind);
    return CULSH_OK;
}

// ---- RPLSH
culsh_status culsh_rplsh_fit_f32(culsh_ctx* ctx, const float* X, int n, int d, int T, int H, uint64_t seed,
                                 const float* P, culsh_index** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return dense_fit<float>(ctx, FAM_RPLSH, X, n, d, T, H, 0, seed, P, nullptr, out, nullptr);
}
culsh_status culsh_rplsh_fit_f64(culsh_ctx* ctx, const double* X, int n, int d, int T, int H, uint64_t seed,
                                 const double* P, culsh_index** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return dense_fit<double>(ctx, FAM_RPLSH, X, n, d, T, H, 0, seed, P, nullptr, out, nullptr);
}
culsh_status culsh_rplsh_query_f32(culsh_ctx* ctx, const float* Q, int nq, const culsh_index* ix, int batch,
                                   culsh_candidates** out) {
    return dense_query<float>(ctx, FAM_RPLSH, Q, nq, ix, batch, out);
}
culsh_status culsh_rplsh_query_f64(culsh_ctx* ctx, const double* Q, int nq, const culsh_index* ix, int batch,
                                   culsh_candidates** out) {
    return dense_query<double>(ctx, FAM_RPLSH, Q, nq, ix, batch, out);
}
culsh_status culsh_rplsh_fit_query_f32(culsh_ctx* ctx, const float* X, int n, int d, int T, int H, uint64_t seed,
                                       const float* P, culsh_candidates** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return dense_fit<float>(ctx, FAM_RPLSH, X, n, d, T, H, 0, seed, P, nullptr, nullptr, out);
}
culsh_status culsh_rplsh_fit_query_f64(culsh_ctx* ctx, const double* X, int n, int d, int T, int H, uint64_t seed,
                                       const double* P, culsh_candidates** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return dense_fit<double>(ctx, FAM_RPLSH, X, n, d, T, H, 0, seed, P, nullptr, nullptr, out);
}

// ---- p-stable
culsh_status culsh_pslsh_fit_f32(culsh_ctx* ctx, const float* X, int n, int d, int T, int H, int w, uint64_t seed,
                                 const float* P, const float* b, culsh_index** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return dense_fit<float>(ctx, FAM_PSLSH, X, n, d, T, H, w, seed, P, b, out, nullptr);
}
culsh_status culsh_pslsh_fit_f64(culsh_ctx* ctx, const double* X, int n, int d, int T, int H, int w, uint64_t seed,
                                 const double* P, const double* b, culsh_index** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return dense_fit<double>(ctx, FAM_PSLSH, X, n, d, T, H, w, seed, P, b, out, nullptr);
}
culsh_status culsh_pslsh_query_f32(culsh_ctx* ctx, const float* Q, int nq, const culsh_index* ix, int batch,
                                   culsh_candidates** out) {
    return dense_query<float>(ctx, FAM_PSLSH, Q, nq, ix, batch, out);
}
culsh_status culsh_pslsh_query_f64(culsh_ctx* ctx, const double* Q, int nq, const culsh_index* ix, int batch,
                                   culsh_candidates** out) {
    return dense_query<double>(ctx, FAM_PSLSH, Q, nq, ix, batch, out);
}
culsh_status culsh_pslsh_fit_query_f32(culsh_ctx* ctx, const float* X, int n, int d, int T, int H, int w,
                                       uint64_t seed, const float* P, const float* b, culsh_candidates** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return dense_fit<float>(ctx, FAM_PSLSH, X, n, d, T, H, w, seed, P, b, nullptr, out);
}
culsh_status culsh_pslsh_fit_query_f64(culsh_ctx* ctx, const double* X, int n, int d, int T, int H, int w,
                                       uint64_t seed, const double* P, const double* b, culsh_candidates** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return dense_fit<double>(ctx, FAM_PSLSH, X, n, d, T, H, w, seed, P, b, nullptr, out);
}

// ---- MinHash
culsh_status culsh_minhash_fit(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr, int n, int d, int T,
                               int H, uint64_t seed, const uint32_t* A, const uint32_t* B, culsh_index** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return minhash_fit_impl(ctx, indices, indptr, n, d, T, H, seed, A, B, out, nullptr);
}
culsh_status culsh_minhash_fit_query(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr, int n, int d,
                                     int T, int H, uint64_t seed, const uint32_t* A, const uint32_t* B,
                                     culsh_candidates** out) {
    CULSH_REQUIRE(out, CULSH_ERR_INVALID, "null argument");
    return minhash_fit_impl(ctx, indices, indptr, n, d, T, H, seed, A, B, nullptr, out);
}
culsh_status culsh_minhash_query(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr, int nq,
                                 const culsh_index* ix, culsh_candidates** out) {
    CULSH_REQUIRE(ctx && indptr && ix && out, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(nq > 0, CULSH_ERR_INVALID, "n_queries must be positive");
    CULSH_REQUIRE(ix->kind == CULSH_KIND_MINHASH && ix->A && ix->B, CULSH_ERR_INVALID, "not a MinHash index");
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    const int T = ix->n_hash_tables, H = ix->n_hashes;
    uint32_t* keys = nullptr;
    if (ix->enc == ENC_MHR) {
        CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(nq) * T * ix->key_w, &keys));
        CULSH_TRY(launch_minhash_rank(ctx, indices, indptr, nq, T, H, ix, nullptr, keys));
    } else {
        CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(nq) * T * H, &keys));
        CULSH_TRY(launch_minhash(ctx, indices, indptr, ix->A, ix->B, nq, T, H, true, keys, ix->mh_prime_kind));
    }
    CandPtr c(new (std::nothrow) culsh_candidates());
    CULSH_REQUIRE(c, CULSH_ERR_NOMEM, "host allocation failed");
    c->device = ctx->device;
    CULSH_TRY(query_keys(ctx, keys, nq, ix, c.get()));
    CULSH_TRY(arena_end(ctx));
    *out = c.release();
    return CULSH_OK;
}

// ---- stage level
#define STAGE_PROLOGUE()                                   \
    CULSH_REQUIRE(ctx, CULSH_ERR_INVALID, "null argument"); \
    ArenaScope scope(ctx);                                  \
    CULSH_TRY(scope.begin_status)

culsh_status culsh_rplsh_hash_f32(culsh_ctx* ctx, const float* X, const float* P, int n, int d, int T, int H,
                                  uint8_t* sig) {
    STAGE_PROLOGUE();
    CULSH_TRY(launch_project_f32(ctx, X, P, nullptr, n, d, T, H, EPI_SIGN_BYTES, sig));
    return arena_end(ctx);
}
culsh_status culsh_rplsh_hash_f64(culsh_ctx* ctx, const double* X, const double* P, int n, int d, int T, int H,
                                  uint8_t* sig) {
    STAGE_PROLOGUE();
    CULSH_TRY(launch_project_f64(ctx, X, P, nullptr, n, d, T, H, EPI_SIGN_BYTES, sig));
    return arena_end(ctx);
}
culsh_status culsh_pslsh_hash_f32(culsh_ctx* ctx, const float* X, const float* P, const float* b, int n, int d,
                                  int T, int H, int32_t* sig) {
    STAGE_PROLOGUE();
    CULSH_TRY(launch_project_f32(ctx, X, P, b, n, d, T, H, EPI_FLOOR_I32, sig));
    return arena_end(ctx);
}
culsh_status culsh_pslsh_hash_f64(culsh_ctx* ctx, const double* X, const double* P, const double* b, int n, int d,
                                  int T, int H, int32_t* sig) {
    STAGE_PROLOGUE();
    CULSH_TRY(launch_project_f64(ctx, X, P, b, n, d, T, H, EPI_FLOOR_I32, sig));
    return arena_end(ctx);
}
culsh_status culsh_minhash_compute(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr, const uint32_t* A,
                                   const uint32_t* B, int n, int T, int H, uint32_t* sig) {
    STAGE_PROLOGUE();
    CULSH_TRY(launch_minhash(ctx, indices, indptr, A, B, n, T, H, false, sig, ctx->mh_prime_kind));
    return arena_end(ctx);
}

static culsh_status core_fit_index_once(culsh_ctx* ctx, const void* X_sig, int n, int T, int H, int S,
                                  int32_t* item_to_bucket, culsh_index** out) {
    CULSH_TRY(check_fit_args(ctx, X_sig, n, 1, T, H, out));
    CULSH_REQUIRE(S > 0, CULSH_ERR_INVALID, "sig_nbytes must be > 0");  // core/fit.cuh:224
    CULSH_REQUIRE(S <= 256, CULSH_ERR_LIMIT, "sig_nbytes > 256 is not supported");
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    IndexPtr ix(new (std::nothrow) culsh_index());
    CULSH_REQUIRE(ix, CULSH_ERR_NOMEM, "host allocation failed");
    ix->device = ctx->device;
    const int W = key_words(ENC_BE, S);
    uint32_t* keys = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n) * T * W, &keys));
    CULSH_TRY(launch_sig_to_keys(ctx, static_cast<const uint8_t*>(X_sig), static_cast<size_t>(n) * T, S, ENC_BE, W, keys));
    CULSH_TRY(fit_index_from_keys(ctx, keys, n, T, H, S, ENC_BE, W, item_to_bucket, ix.get()));
    CULSH_TRY(arena_end(ctx));
    *out = ix.release();
    return CULSH_OK;
}

culsh_status culsh_core_fit_index(culsh_ctx* ctx, const void* X_sig, int n, int T, int H, int S,
                                  int32_t* item_to_bucket, culsh_index** out) {
    return with_sort_retry(ctx, [&] { return core_fit_index_once(ctx, X_sig, n, T, H, S, item_to_bucket, out); });
}

// Query signatures in the reference layout -> key words of the index's encoding, into `keys`
// ([T][nq][key_w] words that the caller provides).
static culsh_status sig_query_keys_into(culsh_ctx* ctx, const void* Q_sig, int nq, int S, const culsh_index* ix,
                                        uint32_t* keys) {
    CULSH_REQUIRE(ctx && Q_sig && ix, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(nq > 0, CULSH_ERR_INVALID, "n_queries must be positive");
    CULSH_REQUIRE(S == ix->sig_nbytes, CULSH_ERR_INVALID, "sig_nbytes (%d) != index sig_nbytes (%d)", S,
                  ix->sig_nbytes);  // core/query.cuh:494
    if (ix->enc == ENC_PSC) {
        CULSH_REQUIRE(reinterpret_cast<uintptr_t>(Q_sig) % 4 == 0, CULSH_ERR_INVALID, "signatures must be 4-byte aligned");
        return launch_ps_compress(ctx, static_cast<const int32_t*>(Q_sig), nq, ix->n_hash_tables, ix->n_hashes, ix, keys);
    }
    if (ix->enc == ENC_MHR) {
        CULSH_REQUIRE(reinterpret_cast<uintptr_t>(Q_sig) % 4 == 0, CULSH_ERR_INVALID, "signatures must be 4-byte aligned");
        return launch_mh_sig_to_keys(ctx, static_cast<const uint32_t*>(Q_sig), nq, ix, keys);
    }
    return launch_sig_to_keys(ctx, static_cast<const uint8_t*>(Q_sig), static_cast<size_t>(nq) * ix->n_hash_tables,
                              S, ix->enc, ix->key_w, keys);
}

static culsh_status sig_query_keys(culsh_ctx* ctx, const void* Q_sig, int nq, int S, const culsh_index* ix,
                                   uint32_t** keys) {
    CULSH_REQUIRE(ctx && Q_sig && ix, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(nq > 0, CULSH_ERR_INVALID, "n_queries must be positive");
    CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(nq) * ix->n_hash_tables * ix->key_w, keys));
    return sig_query_keys_into(ctx, Q_sig, nq, S, ix, *keys);
}

culsh_status culsh_core_find_matching_buckets(culsh_ctx* ctx, const void* Q_sig, int nq, int S,
                                              const culsh_index* ix, int32_t* matched) {
    CULSH_REQUIRE(ctx && matched, CULSH_ERR_INVALID, "null argument");
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    uint32_t* keys = nullptr;
    CULSH_TRY(sig_query_keys(ctx, Q_sig, nq, S, ix, &keys));
    CULSH_TRY(launch_find_matching_buckets(ctx, keys, nq, ix, matched));
    return arena_end(ctx);
}

// ---- the entry point that allocates nothing (workspace: g_static_scratch, set up in culsh_ctx_create)
culsh_status culsh_core_find_matching_buckets_static(culsh_ctx* ctx, const void* Q_sig, int nq, int S,
                                                     const culsh_index* ix, int32_t* matched) {
    CULSH_REQUIRE(ctx && Q_sig && ix && matched, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(nq > 0, CULSH_ERR_INVALID, "n_queries must be positive");
    CULSH_REQUIRE(ix->device == ctx->device, CULSH_ERR_INVALID, "index and context are on different devices");
    const size_t words = static_cast<size_t>(nq) * ix->n_hash_tables * ix->key_w;
    CULSH_REQUIRE(words <= CULSH_STATIC_SCRATCH_WORDS, CULSH_ERR_LIMIT,
                  "find_matching_buckets_static: n_queries * n_hash_tables * key words = %zu exceeds the static "
                  "workspace of %zu words; use culsh_core_find_matching_buckets",
                  words, static_cast<size_t>(CULSH_STATIC_SCRATCH_WORDS));
    uint32_t* keys = (ctx->device >= 0 && ctx->device < 64) ? g_static_scratch_ptr[ctx->device] : nullptr;
    CULSH_REQUIRE(keys != nullptr, CULSH_ERR_INTERNAL, "static workspace of device %d was not set up", ctx->device);
    CULSH_HIP(hipSetDevice(ctx->device));
    // no event objects either: launches of this call are not timed
    const bool profiling = ctx->profiling;
    ctx->profiling = false;
    culsh_status st = sig_query_keys_into(ctx, Q_sig, nq, S, ix, keys);
    if (st == CULSH_OK) st = launch_find_matching_buckets(ctx, keys, nq, ix, matched);
    ctx->profiling = profiling;
    return st;
}

culsh_status culsh_core_query_index(culsh_ctx* ctx, const void* Q_sig, int nq, int S, const culsh_index* ix,
                                    culsh_candidates** out) {
    CULSH_REQUIRE(ctx && out, CULSH_ERR_INVALID, "null argument");
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    uint32_t* keys = nullptr;
    CULSH_TRY(sig_query_keys(ctx, Q_sig, nq, S, ix, &keys));
    CandPtr c(new (std::nothrow) culsh_candidates());
    CULSH_REQUIRE(c, CULSH_ERR_NOMEM, "host allocation failed");
    c->device = ctx->device;
    CULSH_TRY(query_keys(ctx, keys, nq, ix, c.get()));
    CULSH_TRY(arena_end(ctx));
    *out = c.release();
    return CULSH_OK;
}

culsh_status culsh_core_query_from_matched_buckets(culsh_ctx* ctx, const int32_t* matched, int nq,
                                                   const culsh_index* ix, culsh_candidates** out) {
    CULSH_REQUIRE(ctx && matched && ix && out, CULSH_ERR_INVALID, "null argument");
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    CandPtr c(new (std::nothrow) culsh_candidates());
    CULSH_REQUIRE(c, CULSH_ERR_NOMEM, "host allocation failed");
    c->device = ctx->device;
    CULSH_TRY(query_from_matched(ctx, matched, nq, ix, c.get()));
    CULSH_TRY(arena_end(ctx));
    *out = c.release();
    return CULSH_OK;
}

static culsh_status core_fit_query_once(culsh_ctx* ctx, const void* X_sig, int n, int T, int H, int S,
                                  culsh_candidates** out) {
    CULSH_TRY(check_fit_args(ctx, X_sig, n, 1, T, H, out));
    CULSH_REQUIRE(S > 0 && S <= 256, CULSH_ERR_INVALID, "sig_nbytes must be in [1, 256]");
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    IndexPtr ix(new (std::nothrow) culsh_index());
    CandPtr c(new (std::nothrow) culsh_candidates());
    CULSH_REQUIRE(ix && c, CULSH_ERR_NOMEM, "host allocation failed");
    ix->device = c->device = ctx->device;
    const int W = key_words(ENC_BE, S);
    uint32_t* keys = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(n) * T * W, &keys));
    CULSH_TRY(launch_sig_to_keys(ctx, static_cast<const uint8_t*>(X_sig), static_cast<size_t>(n) * T, S, ENC_BE, W, keys));
    CULSH_TRY(finish_fit(ctx, keys, n, T, H, S, ENC_BE, W, ix.get(), c.get()));
    CULSH_TRY(arena_end(ctx));
    *out = c.release();
    return CULSH_OK;
}

culsh_status culsh_core_fit_query(culsh_ctx* ctx, const void* X_sig, int n, int T, int H, int S,
                                  culsh_candidates** out) {
    return with_sort_retry(ctx, [&] { return core_fit_query_once(ctx, X_sig, n, T, H, S, out); });
}

// ---- index object
culsh_status culsh_index_get_meta(const culsh_index* ix, culsh_index_meta* m) {
    CULSH_REQUIRE(ix && m, CULSH_ERR_INVALID, "null argument");
    m->kind = ix->kind;
    m->n_total_candidates = ix->n_total_candidates;
    m->n_total_buckets = ix->n_total_buckets;
    m->n_hash_tables = ix->n_hash_tables;
    m->n_hashes = ix->n_hashes;
    m->sig_nbytes = ix->sig_nbytes;
    m->n_features = ix->n_features;
    m->is_double = ix->is_double ? 1 : 0;
    m->window_size = ix->window_size;
    m->seed = ix->seed;
    // Index::size_bytes (core/index.cuh:148-165) + family arrays (rplsh/index.cuh:45-53 etc.)
    uint64_t sz = 0;
    const bool core_empty = !ix->all_candidate_indices && !ix->all_bucket_signatures &&
                            !ix->bucket_candidate_offsets && !ix->table_bucket_offsets;
    if (!core_empty) {
        sz += (static_cast<uint64_t>(ix->n_total_buckets) + 1) * 4 + (static_cast<uint64_t>(ix->n_hash_tables) + 1) * 4;
        sz += static_cast<uint64_t>(ix->n_total_buckets) * ix->sig_nbytes;
        sz += static_cast<uint64_t>(ix->n_total_candidates) * 4;
    }
    const uint64_t TH = static_cast<uint64_t>(ix->n_hash_tables) * ix->n_hashes;
    const uint64_t fsz = ix->is_double ? 8 : 4;
    if (ix->P && ix->n_features > 0) sz += TH * ix->n_features * fsz;
    if (ix->b) sz += TH * fsz;
    if (ix->A) sz += TH * 4;
    if (ix->B) sz += TH * 4;
    m->size_bytes = sz;
    return CULSH_OK;
}

culsh_status culsh_index_array_info(const culsh_index* ix, culsh_array which, uint64_t* n_elems, uint32_t* elem_size) {
    CULSH_REQUIRE(ix && n_elems && elem_size, CULSH_ERR_INVALID, "null argument");
    const void* p = nullptr;
    CULSH_TRY(index_array(ix, which, &p, n_elems));
    *elem_size = static_cast<uint32_t>(elem_size_of(ix, which));
    return CULSH_OK;
}

culsh_status culsh_index_copy_array(culsh_ctx* ctx, const culsh_index* ix, culsh_array which, void* dst,
                                    uint64_t dst_bytes, int dst_is_device) {
    CULSH_REQUIRE(ctx && ix, CULSH_ERR_INVALID, "null argument");
    const void* p = nullptr;
    uint64_t count = 0;
    CULSH_TRY(index_array(ix, which, &p, &count));
    const uint64_t bytes = count * elem_size_of(ix, which);
    CULSH_REQUIRE(dst_bytes >= bytes, CULSH_ERR_INVALID, "destination too small (%llu < %llu bytes)",
                  static_cast<unsigned long long>(dst_bytes), static_cast<unsigned long long>(bytes));
    if (bytes == 0) return CULSH_OK;
    CULSH_REQUIRE(dst, CULSH_ERR_INVALID, "null destination");
    CULSH_HIP(hipSetDevice(ctx->device));
    CULSH_HIP(hipMemcpy(dst, p, bytes, dst_is_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost));
    return CULSH_OK;
}

culsh_status culsh_index_load(culsh_ctx* ctx, culsh_kind kind, int is_double, const int32_t* cand,
                              const uint8_t* bsig, const int32_t* bco, const int32_t* tbo, const void* param0,
                              const void* param1, int n_total_candidates, int n_total_buckets, int T, int H, int S,
                              int d, uint64_t seed, culsh_index** out) {
    CULSH_REQUIRE(ctx && out, CULSH_ERR_INVALID, "null argument");
    CULSH_REQUIRE(kind == CULSH_KIND_RPLSH || kind == CULSH_KIND_PSLSH || kind == CULSH_KIND_MINHASH ||
                      kind == CULSH_KIND_CORE, CULSH_ERR_INVALID, "unknown index kind");
    CULSH_REQUIRE(n_total_candidates >= 0 && n_total_buckets >= 0 && T > 0 && H > 0 && S > 0 && d >= 0,
                  CULSH_ERR_INVALID, "bad index metadata");
    CULSH_REQUIRE(T <= CULSH_MAX_TABLES, CULSH_ERR_LIMIT, "n_hash_tables > 1024 is not supported");
    CULSH_REQUIRE(S <= 256, CULSH_ERR_LIMIT, "sig_nbytes > 256 is not supported");
    CULSH_REQUIRE((n_total_candidates == 0 || cand) && (n_total_buckets == 0 || bsig) && bco && tbo,
                  CULSH_ERR_INVALID, "missing index array");
    KeyEnc enc = ENC_BE;
    if (kind == CULSH_KIND_RPLSH) {
        CULSH_REQUIRE(S == H, CULSH_ERR_INVALID, "RPLSH signatures hold one byte per hash (sig_nbytes == n_hashes)");
        const size_t nb = static_cast<size_t>(n_total_buckets) * S;
        for (size_t i = 0; i < nb; ++i)
            CULSH_REQUIRE(bsig[i] <= 1, CULSH_ERR_INVALID, "RPLSH bucket signatures must hold 0/1 bytes");
        enc = ENC_BITS;
    } else if (kind != CULSH_KIND_CORE) {
        CULSH_REQUIRE(S == 4 * H, CULSH_ERR_INVALID, "sig_nbytes must be 4 * n_hashes for this family");
    }
    // The kernels trust these arrays (a span outside all_candidate_indices or a row id outside the
    // bitmap's range would be a stray access on the device), so a file that does not add up is refused here.
    CULSH_REQUIRE(n_total_candidates % T == 0, CULSH_ERR_INVALID, "n_total_candidates is not a multiple of n_hash_tables");
    CULSH_REQUIRE(tbo[0] == 0 && tbo[T] == n_total_buckets, CULSH_ERR_INVALID, "table_bucket_offsets do not span the buckets");
    for (int t = 0; t < T; ++t)
        CULSH_REQUIRE(tbo[t] <= tbo[t + 1], CULSH_ERR_INVALID, "table_bucket_offsets must not decrease");
    CULSH_REQUIRE(bco[0] == 0 && bco[n_total_buckets] == n_total_candidates, CULSH_ERR_INVALID,
                  "bucket_candidate_offsets do not span the candidates");
    for (int i = 0; i < n_total_buckets; ++i)
        CULSH_REQUIRE(bco[i] <= bco[i + 1], CULSH_ERR_INVALID, "bucket_candidate_offsets must not decrease");
    {
        const uint32_t n_rows = static_cast<uint32_t>(n_total_candidates / T);
        uint32_t beyond = 0;
        for (int i = 0; i < n_total_candidates; ++i) beyond |= static_cast<uint32_t>(static_cast<uint32_t>(cand[i]) >= n_rows);
        CULSH_REQUIRE(beyond == 0, CULSH_ERR_INVALID, "candidate index outside [0, n_total_candidates / n_hash_tables)");
    }
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    IndexPtr ix(new (std::nothrow) culsh_index());
    CULSH_REQUIRE(ix, CULSH_ERR_NOMEM, "host allocation failed");
    ix->device = ctx->device;
    ix->kind = kind;
    ix->is_double = is_double != 0;
    ix->n_total_candidates = n_total_candidates;
    ix->n_total_buckets = n_total_buckets;
    ix->n_hash_tables = T;
    ix->n_hashes = H;
    ix->sig_nbytes = S;
    ix->n_features = d;
    ix->seed = seed;
    ix->enc = enc;
    ix->key_w = key_words(enc, S);
    {   // readable behind its end, see CAND_PAD
        const size_t count = static_cast<size_t>(n_total_candidates);
        if (count) {  // empty array -> nullptr (array_utils.cuh:34-36)
            CULSH_HIP(dev_malloc(&ix->all_candidate_indices, (count + CAND_PAD) * sizeof(int32_t)));
            CULSH_HIP(hipMemcpy(ix->all_candidate_indices, cand, count * sizeof(int32_t), hipMemcpyHostToDevice));
        }
    }
    CULSH_TRY(upload(bsig, static_cast<size_t>(n_total_buckets) * S, &ix->all_bucket_signatures));
    CULSH_TRY(upload(bco, static_cast<size_t>(n_total_buckets) + 1, &ix->bucket_candidate_offsets));
    CULSH_TRY(upload(tbo, static_cast<size_t>(T) + 1, &ix->table_bucket_offsets));
    const size_t TH = static_cast<size_t>(T) * H;
    if (kind == CULSH_KIND_RPLSH || kind == CULSH_KIND_PSLSH) {
        CULSH_REQUIRE(param0, CULSH_ERR_INVALID, "projection is required");
        if (ix->is_double) {
            double* p = nullptr;
            CULSH_TRY(upload(static_cast<const double*>(param0), TH * d, &p));
            ix->P = p;
        } else {
            float* p = nullptr;
            CULSH_TRY(upload(static_cast<const float*>(param0), TH * d, &p));
            ix->P = p;
        }
        if (kind == CULSH_KIND_PSLSH) {
            CULSH_REQUIRE(param1, CULSH_ERR_INVALID, "bias is required");
            if (ix->is_double) {
                double* p = nullptr;
                CULSH_TRY(upload(static_cast<const double*>(param1), TH, &p));
                ix->b = p;
            } else {
                float* p = nullptr;
                CULSH_TRY(upload(static_cast<const float*>(param1), TH, &p));
                ix->b = p;
            }
        }
    } else if (kind == CULSH_KIND_MINHASH) {
        CULSH_REQUIRE(param0 && param1, CULSH_ERR_INVALID, "hash_a and hash_b are required");
        ix->mh_prime_kind = ctx->mh_prime_kind;  // the saved arrays do not name the prime: the context's is taken
        CULSH_TRY(upload(static_cast<const uint32_t*>(param0), TH, &ix->A));
        CULSH_TRY(upload(static_cast<const uint32_t*>(param1), TH, &ix->B));
    }
    // The key form a fit would have chosen, so that a loaded model runs the same lookup as a fitted one
    // (bindings.cu:407-476 loads into the same Index type that fit returns).  p-stable: the value ranges
    // come from the bucket signatures themselves (every fitted row sits in a bucket, so they are the
    // fit's ranges).  MinHash: the rank tables depend on hash_a / hash_b / n_features only; a bucket
    // value that is no column's hash (the fit met column ids beyond n_features and kept plain keys) sends
    // the index back to plain keys.
    bool compact = false;
    if (kind == CULSH_KIND_PSLSH && n_total_buckets > 0 && H <= 1024) {
        std::vector<int32_t> mm(2 * TH);
        const int32_t* values = reinterpret_cast<const int32_t*>(bsig);
        for (int t = 0; t < T; ++t) {
            int32_t* m = mm.data() + 2 * static_cast<size_t>(t) * H;
            for (int h = 0; h < H; ++h) { m[2 * h] = INT32_MAX; m[2 * h + 1] = INT32_MIN; }
            for (int b = tbo[t]; b < tbo[t + 1]; ++b) {
                const int32_t* v = values + static_cast<size_t>(b) * H;
                for (int h = 0; h < H; ++h) {
                    m[2 * h] = std::min(m[2 * h], v[h]);
                    m[2 * h + 1] = std::max(m[2 * h + 1], v[h]);
                }
            }
            for (int h = 0; h < H; ++h)
                if (m[2 * h] > m[2 * h + 1]) m[2 * h] = m[2 * h + 1] = 0;  // a table without buckets
        }
        ctx->param_stage_off = 0;  // the rank tables go up through the pinned staging area (stream idle here)
        CULSH_TRY(ps_build_codec_from_ranges(ctx, mm.data(), T, H, ix.get(), &compact));
    } else if (kind == CULSH_KIND_MINHASH && n_total_buckets > 0) {
        culsh_status st = mh_build_codec(ctx, T, H, d, ix.get(), &compact);
        if (st == CULSH_RETRY_UNCHAINED) {  // its column sort gave up on the chained scan: once more without
            free_mh_codec(ix.get());
            ctx->sort_unchained = true;
            st = mh_build_codec(ctx, T, H, d, ix.get(), &compact);
        }
        CULSH_REQUIRE(st != CULSH_RETRY_UNCHAINED, CULSH_ERR_INTERNAL, "radix sort: chained scan gave up twice");
        CULSH_TRY(st);
    }
    CULSH_HIP(dev_malloc(&ix->bucket_keys, std::max<size_t>(1, static_cast<size_t>(n_total_buckets) * ix->key_w) * 4));
    if (compact) {
        uint32_t* unknown = nullptr;
        CULSH_TRY(arena_alloc_t(ctx, 1, &unknown));
        CULSH_HIP(hipMemsetAsync(unknown, 0, sizeof(uint32_t), ctx->stream));
        for (int t = 0; t < T; ++t) {  // the tables hold different numbers of buckets: one launch each
            const size_t first = static_cast<size_t>(tbo[t]), count = static_cast<size_t>(tbo[t + 1] - tbo[t]);
            uint32_t* keys = ix->bucket_keys + first * ix->key_w;
            if (kind == CULSH_KIND_PSLSH)
                CULSH_TRY(launch_ps_compress(ctx, reinterpret_cast<const int32_t*>(ix->all_bucket_signatures) + first * H, count,
                                             1, H, ix.get(), keys, t));
            else
                CULSH_TRY(launch_mh_sig_to_keys(ctx, reinterpret_cast<const uint32_t*>(ix->all_bucket_signatures) + first * H,
                                                count, ix.get(), keys, 1, t, unknown));
        }
        uint32_t any_unknown = 0;
        CULSH_TRY(read_back_u32(ctx, unknown, 1, &any_unknown));
        if (any_unknown) {
            free_mh_codec(ix.get());
            ix->enc = ENC_BE;
            ix->key_w = key_words(ENC_BE, S);
            dev_free(ix->bucket_keys);
            ix->bucket_keys = nullptr;
            CULSH_HIP(dev_malloc(&ix->bucket_keys, std::max<size_t>(1, static_cast<size_t>(n_total_buckets) * ix->key_w) * 4));
            compact = false;
        }
    }
    if (!compact)
        CULSH_TRY(launch_sig_to_keys(ctx, ix->all_bucket_signatures, n_total_buckets, S, ix->enc, ix->key_w, ix->bucket_keys));
    CULSH_TRY(build_key_directory(ctx, ix.get(), static_cast<size_t>(n_total_buckets)));
    CULSH_TRY(arena_end(ctx));
    *out = ix.release();
    return CULSH_OK;
}

uint64_t culsh_debug_allocation_calls(void) { return g_allocation_calls.load(std::memory_order_relaxed); }

culsh_status culsh_debug_arena_state(const culsh_ctx* ctx, uint64_t out[4]) {
    CULSH_REQUIRE(ctx && out, CULSH_ERR_INVALID, "null argument");
    out[0] = ctx->arena_cap;
    out[1] = ctx->arena_off;
    out[2] = ctx->arena_overflow_blocks;
    out[3] = ctx->arena_grow_failures;
    return CULSH_OK;
}

culsh_status culsh_index_key_form(const culsh_index* ix, int32_t* key_words_out, int32_t* encoding) {
    CULSH_REQUIRE(ix && key_words_out && encoding, CULSH_ERR_INVALID, "null argument");
    *key_words_out = ix->key_w;
    *encoding = static_cast<int32_t>(ix->enc);
    return CULSH_OK;
}

void culsh_index_free(culsh_index* ix) {
    if (!ix) return;
    (void)hipSetDevice(ix->device);
    free_index_arrays(ix);
    delete ix;
}

// ---- candidates object
culsh_status culsh_candidates_get_meta(const culsh_candidates* c, culsh_candidates_meta* m) {
    CULSH_REQUIRE(c && m, CULSH_ERR_INVALID, "null argument");
    m->n_queries = c->n_queries;
    m->n_total_candidates = c->n_total_candidates;
    m->is_empty = (!c->query_candidate_indices && !c->query_candidate_counts && !c->query_candidate_offsets) ? 1 : 0;
    return CULSH_OK;
}

static culsh_status cand_array(const culsh_candidates* c, culsh_array which, const void** p, uint64_t* bytes) {
    switch (which) {
        case CULSH_ARR_QUERY_INDICES: *p = c->query_candidate_indices; *bytes = c->n_total_candidates * 4; break;
        case CULSH_ARR_QUERY_COUNTS: *p = c->query_candidate_counts; *bytes = static_cast<uint64_t>(c->n_queries) * 8; break;
        case CULSH_ARR_QUERY_OFFSETS:
            *p = c->query_candidate_offsets; *bytes = (static_cast<uint64_t>(c->n_queries) + 1) * 8; break;
        default: set_error("not a candidates array: %d", static_cast<int>(which)); return CULSH_ERR_INVALID;
    }
    if (*p == nullptr) *bytes = 0;
    return CULSH_OK;
}

culsh_status culsh_candidates_copy_array(culsh_ctx* ctx, const culsh_candidates* c, culsh_array which, void* dst,
                                         uint64_t dst_bytes, int dst_is_device) {
    CULSH_REQUIRE(ctx && c, CULSH_ERR_INVALID, "null argument");
    const void* p = nullptr;
    uint64_t bytes = 0;
    CULSH_TRY(cand_array(c, which, &p, &bytes));
    CULSH_REQUIRE(dst_bytes >= bytes, CULSH_ERR_INVALID, "destination too small");
    if (bytes == 0) return CULSH_OK;
    CULSH_REQUIRE(dst, CULSH_ERR_INVALID, "null destination");
    CULSH_HIP(hipSetDevice(ctx->device));
    CULSH_HIP(hipMemcpy(dst, p, bytes, dst_is_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost));
    return CULSH_OK;
}

const void* culsh_candidates_device_ptr(const culsh_candidates* c, culsh_array which) {
    if (!c) return nullptr;
    const void* p = nullptr;
    uint64_t bytes = 0;
    if (cand_array(c, which, &p, &bytes) != CULSH_OK) return nullptr;
    return p;
}

culsh_status culsh_candidates_merge(culsh_ctx* ctx, culsh_candidates** acc, culsh_candidates* other) {
    CULSH_REQUIRE(ctx && acc, CULSH_ERR_INVALID, "null argument");
    if (!other) return CULSH_OK;
    const bool other_empty = !other->query_candidate_indices && !other->query_candidate_counts &&
                             !other->query_candidate_offsets;
    if (other_empty) {  // candidates.cuh:140-142
        culsh_candidates_free(other);
        return CULSH_OK;
    }
    culsh_candidates* a = *acc;
    const bool acc_empty = !a || (!a->query_candidate_indices && !a->query_candidate_counts &&
                                  !a->query_candidate_offsets);
    if (acc_empty) {  // candidates.cuh:144-148
        if (a) culsh_candidates_free(a);
        *acc = other;
        return CULSH_OK;
    }
    ArenaScope scope(ctx);
    CULSH_TRY(scope.begin_status);
    CandPtr result(new (std::nothrow) culsh_candidates());
    CULSH_REQUIRE(result, CULSH_ERR_NOMEM, "host allocation failed");
    result->device = ctx->device;
    CULSH_TRY(concat_candidates(ctx, {a, other}, result.get()));
    CULSH_TRY(arena_end(ctx));
    culsh_candidates_free(a);
    culsh_candidates_free(other);
    *acc = result.release();
    return CULSH_OK;
}

void culsh_candidates_free(culsh_candidates* c) {
    if (!c) return;
    (void)hipSetDevice(c->device);
    free_candidates_arrays(c);
    delete c;
}

}  // extern "C"
