// MinHash signatures over CSR rows on gfx950 (role of compute_minhash_kernel,
// minhash/hash.cuh:69-128).
//
// A workgroup owns RB consecutive rows and all T*H hash functions.  Work items are
// (row, hash) pairs: a thread walks its row's column ids (the lanes that share a row read
// the same addresses, which the vector cache serves as one broadcast) and keeps the
// running minimum in a register, so there is no cross-lane reduction at all.  Results are
// staged in LDS and written table-major so that each table receives RB*H consecutive
// words.
#include "common.hpp"
#include "mh_prime.hpp"

namespace culsh_amd {
namespace {

constexpr int RB = 32;  // rows per workgroup
constexpr int NTHREADS = 256;

// PK: the prime of the hash family (mh_prime.hpp; the reference's is minhash/hash.cuh:17)
template <bool AS_KEYS, int PK>
__global__ __launch_bounds__(NTHREADS) void minhash_kernel(const int32_t* __restrict__ indices,
                                                          const int32_t* __restrict__ indptr,
                                                          const uint32_t* __restrict__ A,
                                                          const uint32_t* __restrict__ B, int n, int T,
                                                          int H, int th_chunk, uint32_t* __restrict__ out) {
    extern __shared__ uint32_t stage[];  // [th_chunk][RB]
    const int TH = T * H;
    const int row0 = blockIdx.x * RB;
    const int rows = min(RB, n - row0);
    for (int c0 = 0; c0 < TH; c0 += th_chunk) {
        const int nc = min(th_chunk, TH - c0);
        // item -> (row, hash): hashes vary fastest so the lanes of a wavefront share a row
        for (int item = threadIdx.x; item < rows * nc; item += NTHREADS) {
            const int r = item / nc, c = item - r * nc;
            const int s = indptr[row0 + r], e = indptr[row0 + r + 1];
            const uint32_t a = A[c0 + c], b = B[c0 + c];
            uint32_t m = 0xFFFFFFFFu;  // empty row (minhash/hash.cuh:86-89)
            int j = s;
            for (; j + 4 <= e; j += 4) {  // four loads in flight, then four hash chains
                const uint32_t f0 = static_cast<uint32_t>(indices[j]), f1 = static_cast<uint32_t>(indices[j + 1]);
                const uint32_t f2 = static_cast<uint32_t>(indices[j + 2]), f3 = static_cast<uint32_t>(indices[j + 3]);
                m = min(min(m, MhPrime<PK>::hash(a, f0, b)), MhPrime<PK>::hash(a, f1, b));
                m = min(min(m, MhPrime<PK>::hash(a, f2, b)), MhPrime<PK>::hash(a, f3, b));
            }
            for (; j < e; ++j) m = min(m, MhPrime<PK>::hash(a, static_cast<uint32_t>(indices[j]), b));
            stage[c * RB + r] = m;
        }
        __syncthreads();
        // table-major write: out[(t*n + row)*H + h]; for one table the block's rows are
        // consecutive, so (row, h) pairs of a table form one contiguous run of rows*H words
        for (int item = threadIdx.x; item < rows * nc; item += NTHREADS) {
            // enumerate in output order within each table: (t, r, h)
            const int per_table = rows * H;
            const int c_first = c0;  // chunk starts on a table boundary (th_chunk % H == 0)
            const int tl = item / per_table, rem = item - tl * per_table;
            const int r = rem / H, h = rem - r * H;
            const int t = c_first / H + tl;
            const uint32_t v = stage[(tl * H + h) * RB + r];
            out[(static_cast<size_t>(t) * n + row0 + r) * H + h] = AS_KEYS ? __builtin_bswap32(v) : v;
        }
        __syncthreads();
    }
}

}  // namespace

culsh_status launch_minhash(culsh_ctx* ctx, const int32_t* indices, const int32_t* indptr,
                            const uint32_t* A, const uint32_t* B, int n, int T, int H, bool as_keys,
                            uint32_t* out, int prime_kind) {
    CULSH_REQUIRE(indptr && A && B && out, CULSH_ERR_INVALID, "minhash: null pointer");
    CULSH_REQUIRE(n > 0 && T > 0 && H > 0, CULSH_ERR_INVALID, "minhash: sizes must be positive");
    CULSH_REQUIRE(H <= 384, CULSH_ERR_LIMIT, "minhash: n_hashes > 384 is not supported");
    const long long TH = static_cast<long long>(T) * H;
    CULSH_REQUIRE(TH < (1ll << 30), CULSH_ERR_LIMIT, "T*H too large");
    // hashes per LDS stage: whole tables, at most 12288 words (48 KiB) of staging
    int tables_per_chunk = static_cast<int>(std::min<long long>(T, std::max(1, (12288 / RB) / H)));
    const int th_chunk = tables_per_chunk * H;
    const size_t lds = static_cast<size_t>(th_chunk) * RB * sizeof(uint32_t);
    dim3 grid((n + RB - 1) / RB), block(NTHREADS);
#define MINHASH_CASE(K, PK)                                                                                          \
    CULSH_LAUNCH(ctx, (minhash_kernel<K, PK>), grid, block, lds, ctx->stream, indices, indptr, A, B, n, T, H, th_chunk, out)
    if (prime_kind == MH_PRIME_2_31_M1) {
        if (as_keys) MINHASH_CASE(true, MH_PRIME_2_31_M1); else MINHASH_CASE(false, MH_PRIME_2_31_M1);
    } else {
        if (as_keys) MINHASH_CASE(true, MH_PRIME_2_32_M5); else MINHASH_CASE(false, MH_PRIME_2_32_M5);
    }
#undef MINHASH_CASE
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

}  // namespace culsh_amd
