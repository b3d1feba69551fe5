// Index build from sorted keys, and the signature <-> key-word codec.
//
// Role of mark_boundaries_kernel, the bucket-flag scan, the table-offset selection and
// build_final_index_kernel of the reference (core/fit.cuh:97-208, 305-362), fused into
// two passes over the sorted items: count bucket heads per tile, then (after a scan of
// the tile counts) write bucket offsets, bucket keys, table offsets and, optionally, the
// (row, table) -> bucket map.
#include <algorithm>

#include "block_utils.hpp"
#include "common.hpp"

namespace culsh_amd {
namespace {

constexpr int IB_THREADS = 256;
constexpr int IB_ITEMS = 8;
constexpr int IB_TILE = IB_THREADS * IB_ITEMS;

// head(i): first item of its table, or key differs from the previous item
// (mark_boundaries_kernel, core/fit.cuh:97-143)
__device__ __forceinline__ uint32_t is_head(const uint32_t* __restrict__ keys, size_t i, int n, int W) {
    if (i % n == 0) return 1u;
    const uint32_t* a = keys + i * W;
    const uint32_t* b = a - W;
    uint32_t diff = 0;
    for (int w = 0; w < W; ++w) diff |= a[w] ^ b[w];
    return diff != 0u;
}

// Flags of the IB_ITEMS consecutive items owned by one thread.  Keys of 1, 2 or 4 words of a
// full run are fetched with 16-byte loads plus the predecessor's key.
template <int KW>
__device__ __forceinline__ uint64_t thread_flags_vec(const uint32_t* __restrict__ keys, size_t base, int n,
                                                     uint32_t (&flag)[IB_ITEMS]) {
    constexpr int NV = IB_ITEMS * KW / 4;  // uint4 loads per thread
    uint32_t k[(IB_ITEMS + 1) * KW];
#pragma unroll
    for (int w = 0; w < KW; ++w) k[w] = base ? keys[(base - 1) * KW + w] : 0u;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const uint4 q = *reinterpret_cast<const uint4*>(keys + base * KW + 4 * v);
        k[KW + 4 * v + 0] = q.x;
        k[KW + 4 * v + 1] = q.y;
        k[KW + 4 * v + 2] = q.z;
        k[KW + 4 * v + 3] = q.w;
    }
    uint64_t c = 0;
    uint32_t r = static_cast<uint32_t>(base % n);  // position inside the table
#pragma unroll
    for (int i = 0; i < IB_ITEMS; ++i) {
        uint32_t diff = 0;
#pragma unroll
        for (int w = 0; w < KW; ++w) diff |= k[(i + 1) * KW + w] ^ k[i * KW + w];
        flag[i] = (r == 0u) || (diff != 0u);
        c += flag[i];
        if (++r == static_cast<uint32_t>(n)) r = 0u;
    }
    return c;
}

__device__ __forceinline__ uint64_t thread_flags(const uint32_t* __restrict__ keys, size_t base, size_t N, int n,
                                                 int W, uint32_t (&flag)[IB_ITEMS]) {
    static_assert(IB_ITEMS == 8, "vector paths assume 8 items per thread");
    if (base + IB_ITEMS <= N) {
        if (W == 1) return thread_flags_vec<1>(keys, base, n, flag);
        if (W == 2) return thread_flags_vec<2>(keys, base, n, flag);
        if (W == 4) return thread_flags_vec<4>(keys, base, n, flag);
    }
    uint64_t c = 0;
#pragma unroll
    for (int i = 0; i < IB_ITEMS; ++i) {
        flag[i] = (base + i < N) ? is_head(keys, base + i, n, W) : 0u;
        c += flag[i];
    }
    return c;
}

__global__ __launch_bounds__(IB_THREADS) void count_heads_kernel(const uint32_t* __restrict__ keys, size_t N,
                                                                int n, int W, uint64_t* __restrict__ tile_counts) {
    __shared__ uint64_t scratch[17];
    const size_t base = static_cast<size_t>(blockIdx.x) * IB_TILE + threadIdx.x * IB_ITEMS;
    uint32_t flag[IB_ITEMS];
    const uint64_t c = thread_flags(keys, base, N, n, W, flag);
    uint64_t total;
    block_exclusive_sum(c, scratch, &total);
    if (threadIdx.x == 0) tile_counts[blockIdx.x] = total;
}

// Bucket heads of a tile are first gathered in LDS in order, then their offsets and keys are
// written by consecutive threads to consecutive addresses (a head-per-thread write would touch
// one cache line per lane when most items open a bucket of their own).
__global__ __launch_bounds__(IB_THREADS) void build_index_kernel(
    const uint32_t* __restrict__ keys, const int32_t* __restrict__ rows, size_t N, int n, int T, int W,
    const uint64_t* __restrict__ tile_base, const uint64_t* __restrict__ n_buckets_dev,
    int32_t* __restrict__ bucket_candidate_offsets,
    uint32_t* __restrict__ bucket_keys, int32_t* __restrict__ table_bucket_offsets,
    int32_t* __restrict__ item_to_bucket, const uint32_t* __restrict__ sort_gave_up) {
    __shared__ uint64_t scratch[17];
    __shared__ uint16_t head_slot[IB_TILE];  // tile-local item numbers of the heads, ascending
    // A sort that gave up leaves slots of keys and rows unwritten: the bucket count may then exceed
    // the arrays sized for it and the rows are no valid addresses.  The flag is final by now (same
    // stream); the host repeats the fit.
    if (sort_gave_up && *sort_gave_up) return;
    const size_t tile_start = static_cast<size_t>(blockIdx.x) * IB_TILE;
    const size_t base = tile_start + threadIdx.x * IB_ITEMS;
    uint32_t flag[IB_ITEMS];
    const uint64_t c = thread_flags(keys, base, N, n, W, flag);
    uint64_t total;
    const uint64_t first_bucket = tile_base[blockIdx.x];
    const uint64_t ex = block_exclusive_sum(c, scratch, &total);
    uint64_t run = first_bucket + ex;
    uint32_t local = static_cast<uint32_t>(ex);
#pragma unroll
    for (int i = 0; i < IB_ITEMS; ++i) {
        const size_t pos = base + i;
        if (pos >= N) break;
        run += flag[i];
        const int32_t bucket = static_cast<int32_t>(run) - 1;  // scan + flag - 1 (fit.cuh:183)
        if (flag[i]) {
            head_slot[local++] = static_cast<uint16_t>(threadIdx.x * IB_ITEMS + i);
            if (pos % n == 0) table_bucket_offsets[pos / n] = bucket;      // fit.cuh:317-326
        }
        if (item_to_bucket) {
            const size_t t = pos / n;
            const uint32_t row = static_cast<uint32_t>(rows[pos]);
            if (row < static_cast<uint32_t>(n)) item_to_bucket[static_cast<size_t>(row) * T + t] = bucket;  // fit.cuh:180-185
        }
    }
    __syncthreads();
    const uint32_t heads = static_cast<uint32_t>(total);
    for (uint32_t j = threadIdx.x; j < heads; j += IB_THREADS)
        bucket_candidate_offsets[first_bucket + j] = static_cast<int32_t>(tile_start + head_slot[j]);  // fit.cuh:190-191
    uint32_t* kout = bucket_keys + first_bucket * W;
    if (W == 1) {
        for (uint32_t j = threadIdx.x; j < heads; j += IB_THREADS) kout[j] = keys[tile_start + head_slot[j]];
    } else {
        const uint32_t words = heads * static_cast<uint32_t>(W);
        for (uint32_t idx = threadIdx.x; idx < words; idx += IB_THREADS) {
            const uint32_t j = idx / static_cast<uint32_t>(W), w = idx - j * static_cast<uint32_t>(W);
            kout[idx] = keys[(tile_start + head_slot[j]) * W + w];
        }
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {  // terminators, fit.cuh:351-357
        const int32_t n_buckets = static_cast<int32_t>(*n_buckets_dev);
        table_bucket_offsets[T] = n_buckets;
        bucket_candidate_offsets[n_buckets] = static_cast<int32_t>(N);
    }
}

__global__ __launch_bounds__(256) void sig_to_keys_kernel(const uint8_t* __restrict__ sig, size_t n_items,
                                                         int S, int enc, int W, uint32_t* __restrict__ keys) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= n_items * W) return;
    const size_t item = idx / W;
    const int w = static_cast<int>(idx - item * W);
    const uint8_t* s = sig + item * S;
    uint32_t k = 0;
    if (enc == ENC_BE) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int byte = 4 * w + j;
            if (byte < S) k |= static_cast<uint32_t>(s[byte]) << (24 - 8 * j);
        }
    } else {
        for (int j = 0; j < 32; ++j) {
            const int h = 32 * w + j;
            if (h < S && s[h] != 0) k |= 1u << (31 - j);
        }
    }
    keys[idx] = k;
}

// Four consecutive signature bytes per thread (one 32-bit store where all four exist).
__global__ __launch_bounds__(256) void keys_to_sig_kernel(const uint32_t* __restrict__ keys, size_t count,
                                                         const uint64_t* __restrict__ count_dev, int S, int enc,
                                                         int W, uint8_t* __restrict__ sig) {
    if (count_dev) count = min(count, static_cast<size_t>(*count_dev));  // exact count known on the device only
    const size_t total = count * S;
    const size_t b0 = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
    if (b0 >= total) return;
    size_t item = b0 / S;
    int byte = static_cast<int>(b0 - item * S);
    uint32_t packed = 0;
    const int nb = static_cast<int>(min(static_cast<size_t>(4), total - b0));
    for (int j = 0; j < nb; ++j) {
        const uint32_t* k = keys + item * W;
        const uint32_t v = (enc == ENC_BE) ? ((k[byte >> 2] >> (24 - 8 * (byte & 3))) & 0xFFu)
                                           : ((k[byte >> 5] >> (31 - (byte & 31))) & 1u);
        packed |= v << (8 * j);
        if (++byte == S) { byte = 0; ++item; }
    }
    if (nb == 4) {
        *reinterpret_cast<uint32_t*>(sig + b0) = packed;  // sig comes from the allocator: 4-byte aligned
    } else {
        for (int j = 0; j < nb; ++j) sig[b0 + j] = static_cast<uint8_t>(packed >> (8 * j));
    }
}

// Sign-bit keys, signature width a multiple of four bytes: a thread expands VEC (1 or 4) groups of four
// key bits into four 0/1 bytes each and stores them at once.  The four bits, highest first, go to
// bytes 0..3 of a word: ((nibble * 0x08040201) >> 3) & 0x01010101.
template <int VEC>
__global__ __launch_bounds__(256) void bit_keys_to_sig_kernel(const uint32_t* __restrict__ keys, size_t count,
                                                             const uint64_t* __restrict__ count_dev, int S, int W,
                                                             uint32_t* __restrict__ sig) {
    if (count_dev) count = min(count, static_cast<size_t>(*count_dev));  // exact count known on the device only
    const uint32_t per_item = static_cast<uint32_t>(S) / (4u * VEC);     // stores per bucket
    const size_t g = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (g >= count * per_item) return;
    const size_t item = g / per_item;
    const uint32_t first = static_cast<uint32_t>(g - item * per_item) * VEC;  // first group of four bits
    const uint32_t word = keys[item * W + (first >> 3)];
    uint32_t out[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
        const uint32_t nibble = (word >> (28u - 4u * ((first + v) & 7u))) & 15u;
        out[v] = ((nibble * 0x08040201u) >> 3) & 0x01010101u;
    }
    if (VEC == 4)
        reinterpret_cast<uint4*>(sig)[g] = make_uint4(out[0], out[VEC > 1 ? 1 : 0], out[VEC > 2 ? 2 : 0], out[VEC > 3 ? 3 : 0]);
    else
        sig[g] = out[0];
}

}  // namespace

culsh_status launch_sig_to_keys(culsh_ctx* ctx, const uint8_t* sig, size_t n_items, int S, KeyEnc enc, int W,
                                uint32_t* keys) {
    if (n_items == 0) return CULSH_OK;
    const size_t total = n_items * W;
    CULSH_REQUIRE(div_up(total, 256) < (1u << 31) && total / 256 < (1ull << 31), CULSH_ERR_LIMIT, "too many items");
    CULSH_LAUNCH(ctx, sig_to_keys_kernel, dim3(div_up(total, 256)), dim3(256), 0, ctx->stream, sig, n_items, S,
                       static_cast<int>(enc), W, keys);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status launch_keys_to_sig(culsh_ctx* ctx, const uint32_t* keys, size_t count, const uint64_t* count_dev,
                                int S, KeyEnc enc, int W, uint8_t* sig) {
    if (count == 0) return CULSH_OK;
    const size_t total = count * S;
    CULSH_REQUIRE(total / 1024 < (1ull << 31), CULSH_ERR_LIMIT, "too many buckets");
    CULSH_REQUIRE(reinterpret_cast<uintptr_t>(sig) % 4 == 0, CULSH_ERR_INTERNAL, "signature array is not 4-byte aligned");
    if (enc == ENC_BITS && S % 16 == 0 && reinterpret_cast<uintptr_t>(sig) % 16 == 0) {
        CULSH_LAUNCH(ctx, bit_keys_to_sig_kernel<4>, dim3(div_up(total / 16, 256)), dim3(256), 0, ctx->stream, keys, count,
                     count_dev, S, W, reinterpret_cast<uint32_t*>(sig));
    } else if (enc == ENC_BITS && S % 4 == 0) {
        CULSH_LAUNCH(ctx, bit_keys_to_sig_kernel<1>, dim3(div_up(total / 4, 256)), dim3(256), 0, ctx->stream, keys, count,
                     count_dev, S, W, reinterpret_cast<uint32_t*>(sig));
    } else {
        CULSH_LAUNCH(ctx, keys_to_sig_kernel, dim3(div_up(div_up(total, 4), 256)), dim3(256), 0, ctx->stream, keys, count,
                     count_dev, S, static_cast<int>(enc), W, sig);
    }
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status build_index_from_sorted(culsh_ctx* ctx, const uint32_t* sorted_keys, int32_t* rows_sorted_owned,
                                     int n, int T, int H, int S, KeyEnc enc, int W,
                                     int32_t* item_to_bucket_opt, culsh_index* index) {
    const size_t N = static_cast<size_t>(n) * T;
    const size_t tiles = (N + IB_TILE - 1) / IB_TILE;
    uint64_t* tile_counts = nullptr;
    uint64_t* tile_base = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, tiles, &tile_counts));
    CULSH_TRY(arena_alloc_t(ctx, tiles + 1, &tile_base));
    CULSH_LAUNCH(ctx, count_heads_kernel, dim3(static_cast<unsigned>(tiles)), dim3(IB_THREADS), 0, ctx->stream,
                       sorted_keys, N, n, W, tile_counts);
    CULSH_LAUNCH_CHECK();
    CULSH_TRY(exclusive_scan_u64(ctx, tile_counts, tile_base, tiles));
    const uint64_t* total_dev = tile_base + tiles;

    // Sign-bit keys admit at most 2^S buckets per table.  When that bound is small the bucket
    // arrays are sized by it and the exact count is fetched at the end of the call, so the
    // device never waits for the host in the middle of the build.
    size_t B_bound = N;
    if (enc == ENC_BITS && S < 31) B_bound = std::min<size_t>(N, static_cast<size_t>(T) << S);
    const bool deferred = B_bound * (8 + static_cast<size_t>(4) * W + S) <= (static_cast<size_t>(256) << 20);
    uint64_t n_buckets64 = 0;
    uint32_t sort_gave_up = 0;
    if (!deferred) {
        // host sync (fit.cuh:332-337); the sort's give-up flag comes along, before anything is sized
        // by a count taken from keys that a failed sort left incomplete
        CULSH_TRY(read_back_pair(ctx, total_dev, ctx->sort_err_dev, &n_buckets64, &sort_gave_up));
        if (sort_gave_up) {
            ctx->sort_err_dev = nullptr;
            return CULSH_RETRY_UNCHAINED;
        }
        B_bound = static_cast<size_t>(n_buckets64);
    }
    index->all_candidate_indices = rows_sorted_owned;
    index->n_total_candidates = static_cast<int>(N);
    index->n_hash_tables = T;
    index->n_hashes = H;
    index->sig_nbytes = S;
    index->enc = enc;
    index->key_w = W;
    CULSH_HIP(dev_malloc(&index->bucket_candidate_offsets, (B_bound + 1) * sizeof(int32_t)));
    CULSH_HIP(dev_malloc(&index->table_bucket_offsets, (static_cast<size_t>(T) + 1) * sizeof(int32_t)));
    CULSH_HIP(dev_malloc(&index->bucket_keys, std::max<size_t>(1, B_bound * W) * sizeof(uint32_t)));
    CULSH_HIP(dev_malloc(&index->all_bucket_signatures, std::max<size_t>(1, B_bound * S)));
    CULSH_LAUNCH(ctx, build_index_kernel, dim3(static_cast<unsigned>(tiles)), dim3(IB_THREADS), 0, ctx->stream,
                       sorted_keys, rows_sorted_owned, N, n, T, W, tile_base, total_dev, index->bucket_candidate_offsets,
                       index->bucket_keys, index->table_bucket_offsets, item_to_bucket_opt,
                       static_cast<const uint32_t*>(ctx->sort_err_dev));
    CULSH_LAUNCH_CHECK();
    CULSH_TRY(build_key_directory(ctx, index, B_bound));
    if (enc == ENC_PSC)
        CULSH_TRY(launch_ps_keys_to_sig(ctx, index, B_bound, total_dev, index->all_bucket_signatures));
    else if (enc == ENC_MHR)
        CULSH_TRY(launch_mh_keys_to_sig(ctx, index, B_bound, total_dev, index->all_bucket_signatures));
    else
        CULSH_TRY(launch_keys_to_sig(ctx, index->bucket_keys, B_bound, total_dev, S, enc, W, index->all_bucket_signatures));
    // end-of-build read-back: the bucket count and the sort's give-up flag (unless fetched above); the
    // kernels launched since then have skipped their work if the flag was set
    if (deferred) CULSH_TRY(read_back_pair(ctx, total_dev, ctx->sort_err_dev, &n_buckets64, &sort_gave_up));
    ctx->sort_err_dev = nullptr;
    if (sort_gave_up) return CULSH_RETRY_UNCHAINED;
    index->n_total_buckets = static_cast<int>(n_buckets64);
    return CULSH_OK;
}

culsh_status fit_index_from_keys(culsh_ctx* ctx, uint32_t* keys, int n, int T, int H, int S, KeyEnc enc, int W,
                                 int32_t* item_to_bucket_opt, culsh_index* index) {
    const size_t N = static_cast<size_t>(n) * T;
    CULSH_REQUIRE(N < (1ull << 31), CULSH_ERR_LIMIT,
                  "n_samples * n_hash_tables must be below 2^31 (int32 candidate positions)");
    uint32_t* keys_tmp = nullptr;
    int32_t* rows_tmp = nullptr;
    int32_t* rows_out = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, N * W, &keys_tmp));
    CULSH_TRY(arena_alloc_t(ctx, N, &rows_tmp));
    CULSH_HIP(dev_malloc(&rows_out, (N + CAND_PAD) * sizeof(int32_t)));  // readable behind its end, see CAND_PAD
    index->all_candidate_indices = rows_out;  // owned by the index from here on (freed with it)
    uint32_t* sorted = nullptr;
    uint32_t bits_vary[64];
    const uint32_t* known_vary = nullptr;
    if ((enc == ENC_PSC || enc == ENC_MHR) && W <= 64) {
        const int nb = H * (enc == ENC_PSC ? index->psc.bits : index->mhc.bits);  // compressed keys occupy the top H*bits bits
        for (int w = 0; w < W; ++w) {
            const int nbits = std::min(32, nb - 32 * w);
            bits_vary[w] = nbits >= 32 ? 0xFFFFFFFFu : (0xFFFFFFFFu << (32 - nbits));
        }
        known_vary = bits_vary;
    } else if (enc == ENC_BITS && W <= 64) {
        // sign-bit keys: exactly the top S bits of the key string can differ, so the radix
        // passes are known without looking at the data (and without a host round trip)
        for (int w = 0; w < W; ++w) {
            const int nbits = std::min(32, S - 32 * w);
            bits_vary[w] = nbits >= 32 ? 0xFFFFFFFFu : (0xFFFFFFFFu << (32 - nbits));
        }
        known_vary = bits_vary;
    }
    CULSH_TRY(sort_tables(ctx, keys, keys_tmp, rows_tmp, rows_out, n, T, W, known_vary, &sorted));
    return build_index_from_sorted(ctx, sorted, rows_out, n, T, H, S, enc, W, item_to_bucket_opt, index);
}

}  // namespace culsh_amd
