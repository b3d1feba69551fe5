// Stable per-table radix sort of (key words, row id) on gfx950.
//
// Replaces the reference's loop of {gather one signature byte through the permutation,
// 8-bit CUB SortPairs over all items} run sig_nbytes + 1 times (core/fit.cuh:254-282).
// Here every table is its own sort segment (so no table-id pass), keys travel with the
// row ids (no random gathers), and byte positions in which no key differs from the first
// key of its table are skipped - for sign-bit keys of H hashes that leaves ceil(H/8)
// passes instead of H + 1.
//
// One pass = three launches with no inter-workgroup waiting: per-tile digit histograms,
// an exclusive scan of [table][digit][tile], and a scatter that ranks items inside the
// tile with wavefront ballots (stable: tile order, then wave order, then lane order).
#include "block_utils.hpp"
#include "common.hpp"

namespace culsh_amd {
namespace {

constexpr int SORT_THREADS = 256;
constexpr int SORT_ITEMS = 16;
constexpr int SORT_TILE = SORT_THREADS * SORT_ITEMS;  // 4096 items per workgroup

// vary[w] |= key[t][i][w] ^ key[t][0][w]
__global__ __launch_bounds__(256) void varying_bits_kernel(const uint32_t* __restrict__ keys, int n,
                                                          int W, uint32_t* __restrict__ vary) {
    const int t = blockIdx.y;
    const uint32_t* tk = keys + static_cast<size_t>(t) * n * W;
    const size_t total = static_cast<size_t>(n) * W;
    // thread strides by a multiple of W so that it always sees the same word position
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x * W;
    for (int w = 0; w < W; ++w) {
        const uint32_t first = tk[w];
        uint32_t acc = 0;
        for (size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * W + w; i < total;
             i += stride)
            acc |= tk[i] ^ first;
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) acc |= __shfl_xor(acc, d, 64);
        if ((threadIdx.x & 63) == 0 && acc) atomicOr(&vary[w], acc);
    }
}

__global__ __launch_bounds__(256) void iota_rows_kernel(int32_t* __restrict__ rows, int n, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < total) rows[i] = static_cast<int32_t>(i % n);
}

__global__ __launch_bounds__(SORT_THREADS) void radix_hist_kernel(const uint32_t* __restrict__ keys, int n,
                                                                 int W, int word, int shift, int tiles,
                                                                 uint32_t* __restrict__ hist) {
    __shared__ uint32_t h[256];
    const int tile = blockIdx.x, t = blockIdx.y;
    h[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t* tk = keys + static_cast<size_t>(t) * n * W;
#pragma unroll 4
    for (int j = 0; j < SORT_ITEMS; ++j) {
        const int idx = tile * SORT_TILE + j * SORT_THREADS + threadIdx.x;
        if (idx < n) atomicAdd(&h[(tk[static_cast<size_t>(idx) * W + word] >> shift) & 255u], 1u);
    }
    __syncthreads();
    hist[(static_cast<size_t>(t) * 256 + threadIdx.x) * tiles + tile] = h[threadIdx.x];
}

// In-place exclusive scan of one table's [256][tiles] histogram (digit major).
__global__ __launch_bounds__(1024) void radix_scan_kernel(uint32_t* __restrict__ hist, int tiles) {
    __shared__ uint32_t scratch[17];
    uint32_t* base = hist + static_cast<size_t>(blockIdx.x) * 256 * tiles;
    const int len = 256 * tiles;
    uint32_t carry = 0;
    for (int start = 0; start < len; start += 1024) {
        const int i = start + threadIdx.x;
        const uint32_t v = (i < len) ? base[i] : 0;
        uint32_t total;
        const uint32_t ex = block_exclusive_sum(v, scratch, &total);
        if (i < len) base[i] = carry + ex;
        carry += total;
    }
}

template <bool ONE_WORD>
__global__ __launch_bounds__(SORT_THREADS) void radix_scatter_kernel(
    const uint32_t* __restrict__ keys_in, const int32_t* __restrict__ rows_in,
    uint32_t* __restrict__ keys_out, int32_t* __restrict__ rows_out,
    const uint32_t* __restrict__ hist_scanned, int n, int W, int word, int shift, int tiles) {
    __shared__ uint32_t whist[SORT_THREADS / 64][256];
    const int tile = blockIdx.x, t = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int i = tid; i < (SORT_THREADS / 64) * 256; i += SORT_THREADS) (&whist[0][0])[i] = 0;
    __syncthreads();

    const size_t tbase = static_cast<size_t>(t) * n;
    const int base_idx = tile * SORT_TILE + wave * (SORT_ITEMS * 64);
    uint32_t kw[SORT_ITEMS], rank[SORT_ITEMS];
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
#pragma unroll
    for (int j = 0; j < SORT_ITEMS; ++j) {
        const int idx = base_idx + j * 64 + lane;
        const bool valid = idx < n;
        const uint32_t k = valid ? keys_in[(tbase + idx) * W + word] : 0u;
        kw[j] = k;
        const uint32_t d = (k >> shift) & 255u;
        // lanes holding the same digit
        unsigned long long peers = __builtin_amdgcn_ballot_w64(valid);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const bool bit = (d >> b) & 1u;
            const unsigned long long m = __builtin_amdgcn_ballot_w64(bit);
            peers &= bit ? m : ~m;
        }
        uint32_t old = 0;
        int leader = lane;
        if (valid) {
            leader = __ffsll(static_cast<long long>(peers)) - 1;
            if (lane == leader) {
                old = whist[wave][d];
                whist[wave][d] = old + static_cast<uint32_t>(__popcll(peers));
            }
        }
        old = __shfl(old, leader, 64);
        rank[j] = old + static_cast<uint32_t>(__popcll(peers & lt_mask));
    }
    __syncthreads();
    {   // digit `tid`: global base of this tile, then exclusive over the waves
        uint32_t b = hist_scanned[(static_cast<size_t>(t) * 256 + tid) * tiles + tile];
#pragma unroll
        for (int w = 0; w < SORT_THREADS / 64; ++w) {
            const uint32_t c = whist[w][tid];
            whist[w][tid] = b;
            b += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < SORT_ITEMS; ++j) {
        const int idx = base_idx + j * 64 + lane;
        if (idx < n) {
            const uint32_t d = (kw[j] >> shift) & 255u;
            const size_t dst = tbase + whist[wave][d] + rank[j];
            if (ONE_WORD) {
                keys_out[dst] = kw[j];
            } else {
                for (int w = 0; w < W; ++w) keys_out[dst * W + w] = keys_in[(tbase + idx) * W + w];
            }
            rows_out[dst] = rows_in ? rows_in[tbase + idx] : idx;
        }
    }
}

}  // namespace

size_t sort_scratch_bytes(int n, int T, int W) {
    const size_t tiles = (static_cast<size_t>(n) + SORT_TILE - 1) / SORT_TILE;
    return align_up(static_cast<size_t>(T) * 256 * tiles * sizeof(uint32_t), 256) +
           align_up(static_cast<size_t>(W) * sizeof(uint32_t), 256) + 512;
}

culsh_status sort_tables(culsh_ctx* ctx, uint32_t* keys_in, uint32_t* keys_tmp, int32_t* rows_tmp,
                         int32_t* rows_out, int n, int T, int W, uint32_t** sorted_keys) {
    CULSH_REQUIRE(n > 0 && T > 0 && W > 0 && W <= 64, CULSH_ERR_INVALID, "sort: bad sizes (W must be <= 64 words)");
    CULSH_REQUIRE(T <= 65535, CULSH_ERR_LIMIT, "n_hash_tables > 65535 is not supported");
    const int tiles = (n + SORT_TILE - 1) / SORT_TILE;
    const size_t N = static_cast<size_t>(n) * T;

    // which byte positions differ anywhere
    uint32_t* vary_dev = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(W), &vary_dev));
    CULSH_HIP(hipMemsetAsync(vary_dev, 0, W * sizeof(uint32_t), ctx->stream));
    {
        const unsigned bx = std::max(1u, std::min(64u, div_up(n, 256 * 8)));
        CULSH_LAUNCH(ctx, varying_bits_kernel, dim3(bx, T), dim3(256), 0, ctx->stream, keys_in, n, W, vary_dev);
        CULSH_LAUNCH_CHECK();
    }
    uint32_t vary[64];
    CULSH_TRY(read_back_u32(ctx, vary_dev, W, vary));

    // least significant digit first: last word, low byte
    struct Pass { int word, shift; };
    std::vector<Pass> passes;
    for (int w = W - 1; w >= 0; --w)
        for (int byte = 0; byte < 4; ++byte)
            if ((vary[w] >> (8 * byte)) & 0xFFu) passes.push_back({w, 8 * byte});

    if (passes.empty()) {  // every table holds one distinct key: identity order
        CULSH_LAUNCH(ctx, iota_rows_kernel, dim3(div_up(N, 256)), dim3(256), 0, ctx->stream, rows_out, n, N);
        CULSH_LAUNCH_CHECK();
        *sorted_keys = keys_in;
        return CULSH_OK;
    }

    uint32_t* hist = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(T) * 256 * tiles, &hist));
    uint32_t* kin = keys_in;
    uint32_t* kout = keys_tmp;
    const int np = static_cast<int>(passes.size());
    const int32_t* rin = nullptr;
    for (int p = 0; p < np; ++p) {
        // the last pass must land in rows_out
        int32_t* rout = ((np - 1 - p) % 2 == 0) ? rows_out : rows_tmp;
        const dim3 grid(tiles, T);
        CULSH_LAUNCH(ctx, radix_hist_kernel, grid, dim3(SORT_THREADS), 0, ctx->stream, kin, n, W,
                           passes[p].word, passes[p].shift, tiles, hist);
        CULSH_LAUNCH_CHECK();
        CULSH_LAUNCH(ctx, radix_scan_kernel, dim3(T), dim3(1024), 0, ctx->stream, hist, tiles);
        CULSH_LAUNCH_CHECK();
        if (W == 1)
            CULSH_LAUNCH(ctx, radix_scatter_kernel<true>, grid, dim3(SORT_THREADS), 0, ctx->stream, kin, rin,
                               kout, rout, hist, n, W, passes[p].word, passes[p].shift, tiles);
        else
            CULSH_LAUNCH(ctx, radix_scatter_kernel<false>, grid, dim3(SORT_THREADS), 0, ctx->stream, kin, rin,
                               kout, rout, hist, n, W, passes[p].word, passes[p].shift, tiles);
        CULSH_LAUNCH_CHECK();
        std::swap(kin, kout);
        rin = rout;
    }
    *sorted_keys = kin;
    return CULSH_OK;
}

}  // namespace culsh_amd
