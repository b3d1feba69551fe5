// Device-wide exclusive prefix sums (role of cub::DeviceScan::ExclusiveSum at
// core/fit.cuh:305-310 and core/query.cuh:330-336, 425-431).
//
// Three launches: per-tile sums, one workgroup that scans the tile sums, per-tile scan
// with the tile's base added.  No inter-workgroup waiting, so every wave reaches its exit.
#include "block_utils.hpp"
#include "common.hpp"

namespace culsh_amd {
namespace {

constexpr int SCAN_THREADS = 256;
constexpr int SCAN_ITEMS = 8;
constexpr int SCAN_TILE = SCAN_THREADS * SCAN_ITEMS;

__global__ __launch_bounds__(SCAN_THREADS) void tile_sums_kernel(const uint64_t* __restrict__ in,
                                                                size_t n, uint64_t* __restrict__ sums) {
    __shared__ uint64_t scratch[17];
    const size_t base = static_cast<size_t>(blockIdx.x) * SCAN_TILE + threadIdx.x * SCAN_ITEMS;
    uint64_t s = 0;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i)
        if (base + i < n) s += in[base + i];
    uint64_t total;
    block_exclusive_sum(s, scratch, &total);
    if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// In-place exclusive scan of `m` values by one workgroup; writes the grand total to *total_out.
__global__ __launch_bounds__(1024) void spine_scan_kernel(uint64_t* __restrict__ sums, size_t m,
                                                         uint64_t* __restrict__ total_out) {
    __shared__ uint64_t scratch[17];
    uint64_t carry = 0;
    for (size_t start = 0; start < m; start += 1024) {
        const size_t i = start + threadIdx.x;
        const uint64_t v = (i < m) ? sums[i] : 0;
        uint64_t total;
        const uint64_t ex = block_exclusive_sum(v, scratch, &total);
        if (i < m) sums[i] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) *total_out = carry;
}

__global__ __launch_bounds__(SCAN_THREADS) void tile_scan_kernel(const uint64_t* __restrict__ in,
                                                                size_t n,
                                                                const uint64_t* __restrict__ tile_base,
                                                                uint64_t* __restrict__ out) {
    __shared__ uint64_t scratch[17];
    const size_t base = static_cast<size_t>(blockIdx.x) * SCAN_TILE + threadIdx.x * SCAN_ITEMS;
    uint64_t v[SCAN_ITEMS];
    uint64_t s = 0;
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) {
        v[i] = (base + i < n) ? in[base + i] : 0;
        s += v[i];
    }
    uint64_t total;
    uint64_t run = tile_base[blockIdx.x] + block_exclusive_sum(s, scratch, &total);
#pragma unroll
    for (int i = 0; i < SCAN_ITEMS; ++i) {
        if (base + i < n) out[base + i] = run;
        run += v[i];
    }
}

}  // namespace

culsh_status exclusive_scan_u64(culsh_ctx* ctx, const uint64_t* in, uint64_t* out, size_t n) {
    CULSH_REQUIRE(in && out, CULSH_ERR_INVALID, "scan: null pointer");
    if (n == 0) {
        CULSH_HIP(hipMemsetAsync(out, 0, sizeof(uint64_t), ctx->stream));
        return CULSH_OK;
    }
    const size_t tiles = (n + SCAN_TILE - 1) / SCAN_TILE;
    CULSH_REQUIRE(tiles < (1ull << 31), CULSH_ERR_LIMIT, "scan: input too large");
    uint64_t* sums = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, tiles, &sums));
    CULSH_LAUNCH(ctx, tile_sums_kernel, dim3(static_cast<unsigned>(tiles)), dim3(SCAN_THREADS), 0,
                       ctx->stream, in, n, sums);
    CULSH_LAUNCH_CHECK();
    CULSH_LAUNCH(ctx, spine_scan_kernel, dim3(1), dim3(1024), 0, ctx->stream, sums, tiles, out + n);
    CULSH_LAUNCH_CHECK();
    CULSH_LAUNCH(ctx, tile_scan_kernel, dim3(static_cast<unsigned>(tiles)), dim3(SCAN_THREADS), 0,
                       ctx->stream, in, n, sums, out);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

}  // namespace culsh_amd
