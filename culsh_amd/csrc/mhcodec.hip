// Order-preserving key compression for MinHash signatures.
//
// A MinHash signature is H little-endian uint32 hashes, ordered by the raw bytes
// (core/fit.cuh:265-272); as key words that is 4*H bytes in which every byte varies, i.e.
// 4*H radix passes over 4*H-byte keys.  Every hash value is (a*f + b) mod p of one column id
// f < n_features, and for a fixed hash function that map is one-to-one (0 < a < p), so a hash
// value can be replaced by the rank of its column among all n_features columns under that hash
// function, taken in the byte order of the hash values.  Ranks need ceil(log2(n_features + 2))
// bits (two more codes stand for "empty row" = 0xFFFFFFFF, which sorts last, and for "the minimum
// came from a column >= n_features", which no fitted row can produce and therefore matches
// nothing); packed MSB first they keep the bucket order bit for bit.  For 50,000 columns and 4
// hashes a key shrinks from 128 to 64 bits and the sort from 16 passes to 8.
//
// The rank tables are built on the device: hash all columns, sort every hash function's column
// list with the table sort of sort.hip, invert the permutation.
#include <algorithm>

#include "common.hpp"
#include "mh_prime.hpp"

namespace culsh_amd {
namespace {

// ainv[c] = A[c]^(p-2) mod p: the inverse of the multiplier, with which the column that produced a
// hash value is recovered from the value (the hash is a bijection of [0, p) unless A[c] = 0 mod p)
template <int PK>
__global__ __launch_bounds__(256) void mh_inverse_kernel(const uint32_t* __restrict__ A, int count,
                                                        uint32_t* __restrict__ ainv) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= count) return;
    uint32_t base = MhPrime<PK>::hash(A[c], 1u, 0u), acc = 1u;
    for (uint32_t e = MhPrime<PK>::P - 2u; e; e >>= 1) {
        if (e & 1u) acc = MhPrime<PK>::hash(acc, base, 0u);
        base = MhPrime<PK>::hash(base, base, 0u);
    }
    ainv[c] = acc;  // 0 for a multiplier that is 0 mod p (p - 2 is odd, so the first step already gives 0)
}

// keys[c][f] = byte-order form of hash_c(f): the sort then ranks columns in signature byte order
template <int PK>
__global__ __launch_bounds__(256) void mh_hash_columns_kernel(const uint32_t* __restrict__ A,
                                                             const uint32_t* __restrict__ B, int d,
                                                             uint32_t* __restrict__ keys) {
    const int c = blockIdx.y;
    const int f = blockIdx.x * 256 + threadIdx.x;
    if (f < d) keys[static_cast<size_t>(c) * d + f] = __builtin_bswap32(MhPrime<PK>::hash(A[c], static_cast<uint32_t>(f), B[c]));
}

// sorted_cols[c][r] = column of rank r; sorted_keys[c][r] = its byte-swapped hash
__global__ __launch_bounds__(256) void mh_invert_kernel(const int32_t* __restrict__ sorted_cols,
                                                       const uint32_t* __restrict__ sorted_keys, size_t total, int d,
                                                       uint32_t* __restrict__ rank, uint32_t* __restrict__ inv,
                                                       const uint32_t* __restrict__ sort_gave_up) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    // a column sort that gave up leaves slots unwritten: their columns are no valid addresses (the
    // host reads the flag next and repeats the fit)
    if (sort_gave_up && *sort_gave_up) return;
    const size_t c = i / d;
    const uint32_t r = static_cast<uint32_t>(i - c * d);
    // A multiplier that is 0 mod p gives every column the same value, hence the same rank (0); any
    // other multiplier gives d different values.
    const uint32_t col = static_cast<uint32_t>(sorted_cols[i]);
    if (col < static_cast<uint32_t>(d)) rank[c * d + col] = sorted_keys[i] == sorted_keys[c * d] ? 0u : r;
    inv[i] = __builtin_bswap32(sorted_keys[i]);
}

constexpr int RB = 32;  // rows per workgroup (RB_SMALL for launches that would otherwise leave compute units idle)
constexpr int RB_SMALL = 8;
constexpr int NTHREADS = 256;

// MinHash of CSR rows written as packed rank codes (role of compute_minhash_kernel,
// minhash/hash.cuh:69-128, plus the key packing).  Same work split as minhash_kernel: items are
// (row, hash) pairs with hashes fastest; besides the running minimum a thread keeps the column
// that produced it.  SMALL: every column id is below 2^25; then only the minimum is kept and
// its column is computed from it at the end, ainv * (min - b) mod p.
template <bool SMALL, int PK>
__global__ __launch_bounds__(NTHREADS) void minhash_rank_kernel(const int32_t* __restrict__ indices,
                                                               const int32_t* __restrict__ indptr,
                                                               const uint32_t* __restrict__ A,
                                                               const uint32_t* __restrict__ B,
                                                               const uint32_t* __restrict__ ainv,
                                                               const uint32_t* __restrict__ rank, int n, int T, int H,
                                                               int d, int bits, int W, int th_chunk, int rb,
                                                               uint32_t* __restrict__ out,
                                                               uint32_t* __restrict__ id_beyond_d) {
    extern __shared__ uint32_t stage[];  // [th_chunk][rb] codes
    const int TH = T * H;
    const int row0 = blockIdx.x * rb;
    const int rows = min(rb, n - row0);
    if (SMALL && id_beyond_d) {
        // The cheaper hash and the rank codes hold for ids below d only: the workgroup looks once at
        // the ids of its rows (one contiguous stretch; negative ids read as huge) and tells the host.
        // Every lane that sees such an id stores the same word.
        uint32_t fmax = 0;
        for (int j = indptr[row0] + static_cast<int>(threadIdx.x), e = indptr[row0 + rows]; j < e; j += NTHREADS)
            fmax = max(fmax, static_cast<uint32_t>(indices[j]));
        if (fmax >= static_cast<uint32_t>(d)) *id_beyond_d = 1u;
    }
    for (int c0 = 0; c0 < TH; c0 += th_chunk) {
        const int nc = min(th_chunk, TH - c0);
        // (row r, hash c0 + c) -> stage[c][r]
        auto one = [&](int r, int c) {
            const int s = indptr[row0 + r], e = indptr[row0 + r + 1];
            const uint32_t a = A[c0 + c], b = B[c0 + c];
            uint32_t m = 0xFFFFFFFFu, col = 0xFFFFFFFFu;
            auto take = [&](uint32_t f) {
                if (SMALL) {
                    m = min(m, MhPrime<PK>::hash_small(a, f, b));
                } else {
                    const uint32_t h = MhPrime<PK>::hash(a, f, b);
                    const bool less = h < m;
                    m = less ? h : m;
                    col = less ? f : col;
                }
            };
            int j = s;
            for (; j + 4 <= e; j += 4) {  // four loads in flight, then four hash chains
                const uint32_t f0 = static_cast<uint32_t>(indices[j]), f1 = static_cast<uint32_t>(indices[j + 1]);
                const uint32_t f2 = static_cast<uint32_t>(indices[j + 2]), f3 = static_cast<uint32_t>(indices[j + 3]);
                take(f0);
                take(f1);
                take(f2);
                take(f3);
            }
            for (; j < e; ++j) take(static_cast<uint32_t>(indices[j]));
            if (SMALL && s < e) {
                const uint32_t ai = ainv[c0 + c];
                constexpr uint32_t P = MhPrime<PK>::P;
                const uint32_t bp = MhPrime<PK>::hash(1u, b, 0u);   // b mod p (an injected b may be any 32-bit value)
                const uint32_t x = m - bp + (m < bp ? P : 0u);      // (m - b) mod p; wraps to the exact value
                col = ai ? MhPrime<PK>::hash(ai, x, 0u) : static_cast<uint32_t>(indices[s]);  // all hashes equal: the first stays
            }
            uint32_t code = static_cast<uint32_t>(d);                      // empty row: sorts last
            if (s < e) code = col < static_cast<uint32_t>(d) ? rank[static_cast<size_t>(c0 + c) * d + col]
                                                              : static_cast<uint32_t>(d) + 1u;  // matches nothing
            stage[c * rb + r] = code;
        };
        if ((nc & 63) == 0) {
            // every wavefront works on one row at a time: saying so lets the row's column ids be fetched
            // once per wavefront, through the scalar unit
            for (int item = threadIdx.x; item < rows * nc; item += NTHREADS) {
                const int r = item / nc;
                one(__builtin_amdgcn_readfirstlane(r), item - r * nc);
            }
        } else {
            for (int item = threadIdx.x; item < rows * nc; item += NTHREADS) {
                const int r = item / nc;
                one(r, item - r * nc);
            }
        }
        __syncthreads();
        // one thread per (table, row): pack the H codes of the table MSB first
        const int tables = nc / H;  // th_chunk is a whole number of tables
        for (int item = threadIdx.x; item < tables * rows; item += NTHREADS) {
            const int tl = item / rows, r = item - tl * rows;
            const int t = c0 / H + tl;
            uint32_t* k = out + (static_cast<size_t>(t) * n + row0 + r) * W;
            unsigned long long acc = 0;
            int nbits = 0, w = 0;
            for (int h = 0; h < H; ++h) {
                acc = (acc << bits) | stage[(tl * H + h) * rb + r];
                nbits += bits;
                if (nbits >= 32) {
                    k[w++] = static_cast<uint32_t>(acc >> (nbits - 32));
                    nbits -= 32;
                    acc &= (1ull << nbits) - 1ull;
                }
            }
            if (nbits > 0) k[w++] = static_cast<uint32_t>(acc << (32 - nbits));
        }
        __syncthreads();
    }
}

// uint32 signatures [T][rows][H] (reference layout) -> packed rank codes.  A value is looked
// up among the sorted hash values of its hash function (rank = position).
__global__ __launch_bounds__(256) void mh_sig_to_keys_kernel(const uint32_t* __restrict__ sig, size_t rows, int T,
                                                            int H, int d, int bits, int W, int t0,
                                                            const uint32_t* __restrict__ inv,
                                                            uint32_t* __restrict__ keys,
                                                            uint32_t* __restrict__ unknown_flag) {
    const size_t item = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (item >= rows * T) return;
    const int t = t0 + static_cast<int>(item / rows);  // t0: number of the first table of `sig`
    bool unknown = false;  // a value that is no column's hash (unknown_flag, may be null, is set to 1 then)
    const uint32_t* s = sig + item * H;
    uint32_t* k = keys + item * W;
    unsigned long long acc = 0;
    int nbits = 0, w = 0;
    for (int h = 0; h < H; ++h) {
        const uint32_t v = s[h];
        uint32_t code = static_cast<uint32_t>(d) + 1u;
        if (v == 0xFFFFFFFFu) {
            code = static_cast<uint32_t>(d);
        } else {
            // inv holds hash values in the byte order of their little-endian form
            const uint32_t* tab = inv + static_cast<size_t>(t * H + h) * d;
            const uint32_t key = __builtin_bswap32(v);
            int lo = 0, hi = d - 1;
            if (__builtin_bswap32(tab[0]) == key) { code = 0u; hi = -1; }  // also the rank of a constant hash
            while (lo <= hi) {
                const int mid = lo + ((hi - lo) >> 1);
                const uint32_t mk = __builtin_bswap32(tab[mid]);
                if (mk == key) { code = static_cast<uint32_t>(mid); break; }
                if (mk < key) lo = mid + 1; else hi = mid - 1;
            }
            unknown |= code == static_cast<uint32_t>(d) + 1u;
        }
        acc = (acc << bits) | code;
        nbits += bits;
        if (nbits >= 32) {
            k[w++] = static_cast<uint32_t>(acc >> (nbits - 32));
            nbits -= 32;
            acc &= (1ull << nbits) - 1ull;
        }
    }
    if (nbits > 0) k[w++] = static_cast<uint32_t>(acc << (32 - nbits));
    if (unknown && unknown_flag) *unknown_flag = 1u;
}

// Signatures of the buckets from their rank keys.  A workgroup takes `bpb` consecutive buckets (a
// multiple of 256 chosen by the host so that the key words fit in 16 KiB of LDS) and searches the
// tables of its first and last bucket once; nearly every workgroup lies inside one table or across one
// boundary, and then a bucket's table follows from one comparison.
constexpr int MH_BPB_MIN = 256;

// largest t in [lo, hi) with table_bucket_offsets[t] <= bucket
__device__ __forceinline__ int mh_table_of(const int32_t* __restrict__ table_bucket_offsets, int lo, int hi, size_t bucket) {
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (static_cast<size_t>(table_bucket_offsets[mid]) <= bucket) lo = mid; else hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(256) void mh_keys_to_sig_kernel(const uint32_t* __restrict__ keys, size_t count,
                                                            const uint64_t* __restrict__ count_dev,
                                                            const int32_t* __restrict__ table_bucket_offsets, int T,
                                                            int H, int d, int bits, int W, int bpb,
                                                            const uint32_t* __restrict__ inv,
                                                            uint32_t* __restrict__ sig) {
    extern __shared__ uint32_t mh_lds[];  // [2] first and last table, then [bpb][W] key words
    uint32_t* trange = mh_lds;
    uint32_t* kw = mh_lds + 2;
    if (count_dev) count = min(count, static_cast<size_t>(*count_dev));
    const size_t b0 = static_cast<size_t>(blockIdx.x) * bpb;
    if (b0 >= count) return;
    const int nb = static_cast<int>(min(static_cast<size_t>(bpb), count - b0));
    if (threadIdx.x < 2)
        trange[threadIdx.x] = static_cast<uint32_t>(
            mh_table_of(table_bucket_offsets, 0, T, threadIdx.x == 0 ? b0 : b0 + static_cast<size_t>(nb) - 1));
    for (int i = threadIdx.x; i < nb * W; i += 256) kw[i] = keys[b0 * W + i];
    __syncthreads();
    const int t_first = static_cast<int>(trange[0]), t_last = static_cast<int>(trange[1]);
    const bool near = t_last - t_first <= 1;  // uniform over the workgroup
    const size_t second = t_last > t_first ? static_cast<size_t>(table_bucket_offsets[t_first + 1]) : ~size_t(0);
    const uint32_t mask = (1u << bits) - 1u;
    auto value = [&](int bl, int t, int h) -> uint32_t {
        const uint32_t* k = kw + bl * W;
        const int o = h * bits, w0 = o >> 5, sh = o & 31;
        const unsigned long long two = (static_cast<unsigned long long>(k[w0]) << 32) | (w0 + 1 < W ? k[w0 + 1] : 0u);
        const uint32_t code = static_cast<uint32_t>(two >> (64 - sh - bits)) & mask;
        return code < static_cast<uint32_t>(d) ? inv[static_cast<size_t>(t * H + h) * d + code] : 0xFFFFFFFFu;
    };
    auto table = [&](int bl) -> int {
        const size_t bucket = b0 + bl;
        return near ? t_first + (bucket >= second ? 1 : 0) : mh_table_of(table_bucket_offsets, t_first, t_last + 1, bucket);
    };
    uint32_t* out = sig + b0 * H;
    if (H % 4 == 0 && reinterpret_cast<uintptr_t>(sig) % 16 == 0) {  // four hashes of a bucket per thread and store
        const int qpb = H >> 2;
        for (int q = threadIdx.x; q < nb * qpb; q += 256) {
            const int bl = q / qpb, h = (q - bl * qpb) << 2;
            const int t = table(bl);
            *reinterpret_cast<uint4*>(out + 4 * static_cast<size_t>(q)) =
                make_uint4(value(bl, t, h), value(bl, t, h + 1), value(bl, t, h + 2), value(bl, t, h + 3));
        }
    } else {
        for (int i = threadIdx.x; i < nb * H; i += 256) {
            const int bl = i / H;
            out[i] = value(bl, table(bl), i - bl * H);
        }
    }
}

}  // namespace

void free_mh_codec(culsh_index* ix) {
    dev_free(ix->mhc.rank);
    dev_free(ix->mhc.inv);
    dev_free(ix->mhc.ainv);
    ix->mhc = MhCodec();
}

culsh_status mh_build_codec(culsh_ctx* ctx, int T, int H, int d, culsh_index* ix, bool* used) {
    *used = false;
    const size_t TH = static_cast<size_t>(T) * H;
    if (d < 1 || TH * static_cast<size_t>(d) > (size_t(1) << 25) || TH > 65535) return CULSH_OK;
    int bits = 1;
    while ((1ll << bits) < static_cast<long long>(d) + 2) ++bits;
    const int W = (H * bits + 31) / 32;
    if (W >= H || W > 56) return CULSH_OK;  // nothing to gain, or more than the restore kernel keeps in LDS (256 keys of W words)
    const size_t total = TH * d;
    uint32_t *keys = nullptr, *keys_tmp = nullptr, *sorted = nullptr;
    int32_t *cols_tmp = nullptr, *cols = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, total, &keys));
    CULSH_TRY(arena_alloc_t(ctx, total, &keys_tmp));
    CULSH_TRY(arena_alloc_t(ctx, total, &cols_tmp));
    CULSH_TRY(arena_alloc_t(ctx, total, &cols));
    const bool mersenne = ix->mh_prime_kind == MH_PRIME_2_31_M1;
    if (mersenne)
        CULSH_LAUNCH(ctx, mh_hash_columns_kernel<MH_PRIME_2_31_M1>, dim3(div_up(d, 256), static_cast<unsigned>(TH)), dim3(256), 0,
                     ctx->stream, ix->A, ix->B, d, keys);
    else
        CULSH_LAUNCH(ctx, mh_hash_columns_kernel<MH_PRIME_2_32_M5>, dim3(div_up(d, 256), static_cast<unsigned>(TH)), dim3(256), 0,
                     ctx->stream, ix->A, ix->B, d, keys);
    CULSH_LAUNCH_CHECK();
    const uint32_t all_bits = 0xFFFFFFFFu;
    CULSH_TRY(sort_tables(ctx, keys, keys_tmp, cols_tmp, cols, d, static_cast<int>(TH), 1, &all_bits, &sorted));
    MhCodec& mc = ix->mhc;
    CULSH_HIP(dev_malloc(&mc.rank, total * sizeof(uint32_t)));
    CULSH_HIP(dev_malloc(&mc.inv, total * sizeof(uint32_t)));
    CULSH_HIP(dev_malloc(&mc.ainv, TH * sizeof(uint32_t)));
    CULSH_LAUNCH(ctx, mh_invert_kernel, dim3(div_up(total, 256)), dim3(256), 0, ctx->stream, cols, sorted, total, d,
                 mc.rank, mc.inv, static_cast<const uint32_t*>(ctx->sort_err_dev));
    CULSH_LAUNCH_CHECK();
    if (mersenne)
        CULSH_LAUNCH(ctx, mh_inverse_kernel<MH_PRIME_2_31_M1>, dim3(div_up(TH, 256)), dim3(256), 0, ctx->stream, ix->A,
                     static_cast<int>(TH), mc.ainv);
    else
        CULSH_LAUNCH(ctx, mh_inverse_kernel<MH_PRIME_2_32_M5>, dim3(div_up(TH, 256)), dim3(256), 0, ctx->stream, ix->A,
                     static_cast<int>(TH), mc.ainv);
    CULSH_LAUNCH_CHECK();
    if (ctx->sort_err_dev) {  // the column sort used the chained scan: its flag is settled here
        uint32_t gave_up = 0;
        CULSH_TRY(read_back_u32(ctx, ctx->sort_err_dev, 1, &gave_up));
        ctx->sort_err_dev = nullptr;
        if (gave_up) return CULSH_RETRY_UNCHAINED;
    }
    mc.bits = bits;
    mc.d = d;
    ix->enc = ENC_MHR;
    ix->key_w = W;
    *used = true;
    return CULSH_OK;
}

culsh_status launch_minhash_rank(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr, int n, int T, int H,
                                 const culsh_index* ix, uint32_t* fit_flag, uint32_t* keys) {
    CULSH_REQUIRE(indptr && keys && ix->mhc.rank, CULSH_ERR_INVALID, "minhash: null pointer");
    CULSH_REQUIRE(n > 0, CULSH_ERR_INVALID, "minhash: sizes must be positive");
    CULSH_REQUIRE(H <= 384, CULSH_ERR_LIMIT, "minhash: n_hashes > 384 is not supported");
    // fewer rows per workgroup when 32 would give the compute units less than four workgroups each
    const int rb = (n + RB - 1) / RB >= 4 * ctx->n_cus ? RB : RB_SMALL;
    int tables_per_chunk = static_cast<int>(std::min<long long>(T, std::max(1, (12288 / rb) / H)));
    const int th_chunk = tables_per_chunk * H;
    const size_t lds = static_cast<size_t>(th_chunk) * rb * sizeof(uint32_t);
    const dim3 grid((n + rb - 1) / rb);
    const bool small = fit_flag && ix->mhc.d <= (1 << 25);
    uint32_t* flag = small ? fit_flag : nullptr;
#define MH_RANK_CASE(S, PK)                                                                                              \
    CULSH_LAUNCH(ctx, (minhash_rank_kernel<S, PK>), grid, dim3(NTHREADS), lds, ctx->stream, indices, indptr, ix->A, ix->B, \
                 ix->mhc.ainv, ix->mhc.rank, n, T, H, ix->mhc.d, ix->mhc.bits, ix->key_w, th_chunk, rb, keys, flag)
    if (ix->mh_prime_kind == MH_PRIME_2_31_M1) {
        if (small) MH_RANK_CASE(true, MH_PRIME_2_31_M1); else MH_RANK_CASE(false, MH_PRIME_2_31_M1);
    } else {
        if (small) MH_RANK_CASE(true, MH_PRIME_2_32_M5); else MH_RANK_CASE(false, MH_PRIME_2_32_M5);
    }
#undef MH_RANK_CASE
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status launch_mh_sig_to_keys(culsh_ctx* ctx, const uint32_t* sig, size_t rows, const culsh_index* ix,
                                   uint32_t* keys, int T, int t0, uint32_t* unknown_flag) {
    if (T < 0) T = ix->n_hash_tables;
    const size_t items = rows * T;
    if (items == 0) return CULSH_OK;
    CULSH_REQUIRE(items / 256 < (1ull << 31), CULSH_ERR_LIMIT, "too many items");
    CULSH_LAUNCH(ctx, mh_sig_to_keys_kernel, dim3(div_up(items, 256)), dim3(256), 0, ctx->stream, sig, rows, T,
                 ix->n_hashes, ix->mhc.d, ix->mhc.bits, ix->key_w, t0, ix->mhc.inv, keys, unknown_flag);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status launch_mh_keys_to_sig(culsh_ctx* ctx, const culsh_index* ix, size_t count, const uint64_t* count_dev,
                                   uint8_t* sig) {
    if (count == 0) return CULSH_OK;
    // buckets per workgroup: as many as 16 KiB of key words hold, 256 to 2048
    const int bpb = std::max(MH_BPB_MIN, std::min(2048, (4096 / ix->key_w) / 256 * 256));
    CULSH_REQUIRE(count / bpb < (1ull << 31), CULSH_ERR_LIMIT, "too many buckets");
    const size_t lds = (2 + static_cast<size_t>(bpb) * ix->key_w) * sizeof(uint32_t);
    CULSH_LAUNCH(ctx, mh_keys_to_sig_kernel, dim3(div_up(count, bpb)), dim3(256), lds, ctx->stream, ix->bucket_keys,
                 count, count_dev, ix->table_bucket_offsets, ix->n_hash_tables, ix->n_hashes, ix->mhc.d, ix->mhc.bits,
                 ix->key_w, bpb, ix->mhc.inv, reinterpret_cast<uint32_t*>(sig));
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

}  // namespace culsh_amd
