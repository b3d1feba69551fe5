// Stable per-table radix sort of (key words, row id) on gfx950.
//
// Replaces the reference's loop of {gather one signature byte through the permutation,
// 8-bit CUB SortPairs over all items} run sig_nbytes + 1 times (core/fit.cuh:254-282).
// Here every table is its own sort segment (so no table-id pass), keys travel with the
// row ids (no random gathers), and byte positions in which no key differs from the first
// key of its table are skipped - for sign-bit keys of H hashes that leaves ceil(H/8)
// passes instead of H + 1.
//
// A pass is one scatter launch that ranks items inside a tile with wavefront ballots
// (stable: tile order, then wave order, then lane order).  Where a tile's digit runs start
// is found by a chained scan: one launch before the first pass counts every digit of every
// pass per table (the counts do not depend on the order of the items), and in a pass the
// workgroup of tile k publishes its digit counts and sums those of tiles < k by looking
// back over the published words.  Workgroups are numbered tile-major, so the tiles of one
// table that run at the same time are few and the look-back is short.  The poll count is
// bounded; a give-up is reported and the caller repeats the fit with the unchained form of
// a pass: per-tile digit histograms, an exclusive scan of [table][digit][tile], scatter.
#include <cstdlib>
#include <vector>

#include "block_utils.hpp"
#include "common.hpp"

namespace culsh_amd {
namespace {

constexpr int SORT_THREADS = 256;  // histogram kernels; also the number of digits

// Tile of a scatter pass: THREADS * ITEMS items per workgroup.  A tile leaves in 256 digit runs, so
// bigger tiles mean longer runs of consecutive addresses per store (what the pass is bound by) and
// fewer, larger workgroups per CU (LDS holds the whole tile).
struct TileShape {
    int threads, items;
    constexpr int tile() const { return threads * items; }
};
constexpr TileShape SHAPE_W1{512, 16}, SHAPE_W2{512, 8}, SHAPE_ANY{256, 16};
inline TileShape tile_shape(int W) { return W == 1 ? SHAPE_W1 : (W == 2 ? SHAPE_W2 : SHAPE_ANY); }

// vary[w] |= key[t][i][w] ^ key[t][0][w]
__device__ __forceinline__ void publish_vary(uint32_t acc, uint32_t* __restrict__ slot) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) acc |= __shfl_xor(acc, d, 64);
    // most wavefronts add nothing new once a few have reported: skip their atomics
    if ((threadIdx.x & 63) == 0 && (acc & ~__atomic_load_n(slot, __ATOMIC_RELAXED))) atomicOr(slot, acc);
}

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
#pragma unroll 4
        for (size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * W + w; i < total;
             i += stride)
            acc |= tk[i] ^ first;
        publish_vary(acc, &vary[w]);
    }
}

// Same for W in {1, 2, 4} with 16-byte loads (component c of a uint4 is word position c % W).
__global__ __launch_bounds__(256) void varying_bits_vec_kernel(const uint32_t* __restrict__ keys, int n,
                                                              int W, uint32_t* __restrict__ vary) {
    const int t = blockIdx.y;
    const uint32_t* tk = keys + static_cast<size_t>(t) * n * W;
    const size_t nvec = static_cast<size_t>(n) * W / 4;  // caller guarantees n*W % 4 == 0
    const uint4* tv = reinterpret_cast<const uint4*>(tk);
    const uint32_t f0 = tk[0], f1 = tk[1 % W], f2 = tk[2 % W], f3 = tk[3 % W];
    uint32_t a0 = 0, a1 = 0, a2 = 0, a3 = 0;
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
#pragma unroll 4
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        const uint4 v = tv[i];
        a0 |= v.x ^ f0;
        a1 |= v.y ^ f1;
        a2 |= v.z ^ f2;
        a3 |= v.w ^ f3;
    }
    if (W == 1) {
        publish_vary(a0 | a1 | a2 | a3, &vary[0]);
    } else if (W == 2) {
        publish_vary(a0 | a2, &vary[0]);
        publish_vary(a1 | a3, &vary[1]);
    } else {
        publish_vary(a0, &vary[0]);
        publish_vary(a1, &vary[1]);
        publish_vary(a2, &vary[2]);
        publish_vary(a3, &vary[3]);
    }
}

__global__ __launch_bounds__(256) void iota_rows_kernel(int32_t* __restrict__ rows, int n, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < total) rows[i] = static_cast<int32_t>(i % n);
}

constexpr int MAX_PASSES_PER_LAUNCH = 16;
struct PassList {
    int count;
    int word[MAX_PASSES_PER_LAUNCH];
    int shift[MAX_PASSES_PER_LAUNCH];
};

// Digit totals per (pass, table, digit) for up to 16 passes in one read of the keys (tiles of its
// own size: the totals do not depend on how the scatter cuts a table).
constexpr int TOT_ITEMS = 32;
constexpr int TOT_TILE = SORT_THREADS * TOT_ITEMS;
constexpr int TOT_ROW = 257;  // words per histogram row
__global__ __launch_bounds__(SORT_THREADS) void radix_totals_kernel(const uint32_t* __restrict__ keys, int n, int W,
                                                                   PassList pl, int T, int copies,
                                                                   uint32_t* __restrict__ dtot /*[pass][T][256]*/) {
    // Several copies of every pass's histogram, one per lane residue: lanes of one wavefront that hold
    // the same digit (frequent with skewed keys) then add to different words, and a row of 257 words
    // puts those words into different banks as well.
    extern __shared__ uint32_t h[];  // [copies][pl.count][TOT_ROW]
    const int t = blockIdx.y;
    const int mine = static_cast<int>(threadIdx.x & 63) % copies;
    for (int i = threadIdx.x; i < copies * pl.count * TOT_ROW; i += SORT_THREADS) h[i] = 0;
    __syncthreads();
    const uint32_t* tk = keys + static_cast<size_t>(t) * n * W;
    const int last_idx = n - 1;
    // A workgroup takes every gridDim.x-th tile of its table: the atomics on the totals in memory at
    // the end are what bounds this kernel, so there are few workgroups with many tiles each.
    const int tiles = (n + TOT_TILE - 1) / TOT_TILE;
    for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        uint32_t kw[TOT_ITEMS];
        int last_word = -1;
        for (int p = 0; p < pl.count; ++p) {  // passes are ordered by word, so a word is fetched once
            if (pl.word[p] != last_word) {
                last_word = pl.word[p];
#pragma unroll
                for (int j = 0; j < TOT_ITEMS; ++j) {  // clamped, not predicated: nothing stands between the loads
                    const int idx = min(tile * TOT_TILE + j * SORT_THREADS + static_cast<int>(threadIdx.x), last_idx);
                    kw[j] = tk[static_cast<size_t>(idx) * W + last_word];
                }
            }
            uint32_t* hp = h + (mine * pl.count + p) * TOT_ROW;
            const int shift = pl.shift[p];
#pragma unroll
            for (int j = 0; j < TOT_ITEMS; ++j) {
                const int idx = tile * TOT_TILE + j * SORT_THREADS + threadIdx.x;
                if (idx < n) atomicAdd(&hp[(kw[j] >> shift) & 255u], 1u);
            }
        }
    }
    __syncthreads();
    for (int p = 0; p < pl.count; ++p) {
        uint32_t c = 0;
        for (int r = 0; r < copies; ++r) c += h[(r * pl.count + p) * TOT_ROW + threadIdx.x];
        if (c) atomicAdd(&dtot[(static_cast<size_t>(p) * T + t) * 256 + threadIdx.x], c);
    }
}

// Published word of the chained scan: 2-bit tag, 30-bit value.
constexpr uint32_t ST_COUNT = 1u << 30, ST_SUM = 2u << 30, ST_VALUE = ST_COUNT - 1u;

__global__ __launch_bounds__(SORT_THREADS) void radix_hist_kernel(const uint32_t* __restrict__ keys, int n,
                                                                 int W, int word, int shift, int tiles,
                                                                 int tile_items, uint32_t* __restrict__ hist,
                                                                 uint32_t* __restrict__ dtot) {
    __shared__ uint32_t h[SORT_THREADS / 64][256];  // one copy per wavefront: fewer same-bank atomics
    const int tile = blockIdx.x, t = blockIdx.y, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < (SORT_THREADS / 64) * 256; i += SORT_THREADS) (&h[0][0])[i] = 0;
    __syncthreads();
    const uint32_t* tk = keys + static_cast<size_t>(t) * n * W;
    const int end = static_cast<int>(min(static_cast<long long>(n), static_cast<long long>(tile + 1) * tile_items));
#pragma unroll 4
    for (int idx = tile * tile_items + threadIdx.x; idx < end; idx += SORT_THREADS)
        atomicAdd(&h[wave][(tk[static_cast<size_t>(idx) * W + word] >> shift) & 255u], 1u);
    __syncthreads();
    uint32_t c = 0;
#pragma unroll
    for (int w = 0; w < SORT_THREADS / 64; ++w) c += h[w][threadIdx.x];
    hist[(static_cast<size_t>(t) * 256 + threadIdx.x) * tiles + tile] = c;
    if (c) atomicAdd(&dtot[t * 256 + threadIdx.x], c);  // digit totals of the table (zeroed by the host)
}

// In-place exclusive scan of one table's [256][tiles] histogram (digit major).  The digit
// totals give every digit row its base; each wavefront then scans whole rows with wave
// scans only.  Grid (T, SCAN_PARTS): a workgroup handles 256 / SCAN_PARTS digit rows.
constexpr int SCAN_PARTS = 8;
__global__ __launch_bounds__(256) void radix_scan_kernel(uint32_t* __restrict__ hist,
                                                        const uint32_t* __restrict__ dtot, int tiles) {
    __shared__ uint32_t scratch[17];
    __shared__ uint32_t dbase[256];
    const int t = blockIdx.x, part = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t total;
    dbase[threadIdx.x] = block_exclusive_sum(dtot[t * 256 + threadIdx.x], scratch, &total);
    __syncthreads();
    constexpr int ROWS_PER_WAVE = 256 / SCAN_PARTS / 4;
    for (int k = 0; k < ROWS_PER_WAVE; ++k) {
        const int d = part * (256 / SCAN_PARTS) + wave * ROWS_PER_WAVE + k;
        uint32_t* row = hist + (static_cast<size_t>(t) * 256 + d) * tiles;
        uint32_t carry = dbase[d];
        for (int c0 = 0; c0 < tiles; c0 += 64) {
            const int i = c0 + lane;
            const uint32_t v = (i < tiles) ? row[i] : 0u;
            const uint32_t incl = wave_inclusive_sum(v);
            if (i < tiles) row[i] = carry + incl - v;
            carry += __shfl(incl, 63, 64);
        }
    }
}

// KW: key words known at compile time (1, 2 or 4: keys move as one vector), 0 = any W.
// CHAINED: `hist_scanned` is null; `dtot` holds this pass's digit totals [T][256], `state`
// the published words [T][tiles][256] (zero at launch), `err` the give-up flag; the grid is
// one-dimensional and tile-major.
// LDS bytes of a scatter workgroup (the kernel carves the same layout).
constexpr size_t scatter_lds_bytes(int KW, TileShape sh) {
    const size_t tile = static_cast<size_t>(sh.tile());
    const size_t staged = (KW == 1 || KW == 2) ? tile * KW + tile : tile;  // keys + rows, else source slots
    return ((sh.threads / 64) * 256 + 256 + 256 + 32 + staged) * sizeof(uint32_t);
}

template <int KW, bool CHAINED, int THREADS, int ITEMS>
__global__ __launch_bounds__(THREADS) void radix_scatter_kernel(
    const uint32_t* __restrict__ keys_in, const int32_t* __restrict__ rows_in,
    uint32_t* __restrict__ keys_out, int32_t* __restrict__ rows_out,
    const uint32_t* __restrict__ hist_scanned, int n, int W, int word, int shift, int tiles, int T,
    const uint32_t* __restrict__ dtot, uint32_t* __restrict__ state, uint32_t* __restrict__ err,
    int spin_limit) {
    constexpr bool ONE_WORD = (KW == 1);
    constexpr int NW = THREADS / 64;
    constexpr int TILE = THREADS * ITEMS;
    constexpr bool TWO_WORDS = (KW == 2);                  // staged in full as well (8-byte keys)
    constexpr bool STAGED = ONE_WORD || TWO_WORDS;
    extern __shared__ __attribute__((aligned(16))) uint32_t scatter_lds[];
    uint32_t (*whist)[256] = reinterpret_cast<uint32_t (*)[256]>(scatter_lds);  // [NW] per-wave digit counts, then per-wave offsets inside a digit run
    uint32_t* dstart = scatter_lds + NW * 256;   // [256] start of each digit's run inside the sorted tile
    uint32_t* gbase = dstart + 256;              // [256] global position of the run minus dstart (wraps, used additively)
    uint32_t* scratch = gbase + 256;             // [32]
    uint32_t* st_key = scratch + 32;             // [TILE * (1 or 2)] staged keys (8-byte aligned), else [TILE] source slots
    int32_t* st_row = reinterpret_cast<int32_t*>(st_key + TILE * (TWO_WORDS ? 2 : 1));  // [TILE] when staged
    const int tile = CHAINED ? static_cast<int>(blockIdx.x / T) : static_cast<int>(blockIdx.x);
    const int t = CHAINED ? static_cast<int>(blockIdx.x - static_cast<unsigned>(tile) * T) : static_cast<int>(blockIdx.y);
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in every lane: scalar
    for (int i = tid; i < NW * 256; i += THREADS) (&whist[0][0])[i] = 0;
    __syncthreads();

    // table bases are wavefront-uniform; inside a table 32-bit element offsets suffice for the
    // fixed key widths (n < 2^30 there)
    const size_t tbase = static_cast<size_t>(t) * n;
    const int Wc = KW > 0 ? KW : W;
    const uint32_t* tkeys_in = keys_in + tbase * Wc;
    const int32_t* trows_in = rows_in ? rows_in + tbase : nullptr;
    uint32_t* tkeys_out = keys_out + tbase * Wc;
    int32_t* trows_out = rows_out + tbase;
    const int tile0 = tile * TILE;
    const int base_idx = tile0 + wave * (ITEMS * 64);
    uint32_t kw[ITEMS], rank[ITEMS];
    int32_t rw[STAGED ? ITEMS : 1];
    uint32_t kw_other[TWO_WORDS ? ITEMS : 1];  // the word of a two-word key that is not the digit word
    // All loads of the tile are issued before the first is used: indices past the end are clamped
    // instead of predicated, so nothing stands between the loads (a branch per load would make every
    // item wait for its own round trip to memory).
    const int last_idx = n - 1;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const uint32_t idc = static_cast<uint32_t>(min(base_idx + j * 64 + lane, last_idx));
        if (TWO_WORDS) {
            const uint2 kv = *reinterpret_cast<const uint2*>(tkeys_in + idc * 2u);
            kw[j] = word == 0 ? kv.x : kv.y;
            kw_other[j] = word == 0 ? kv.y : kv.x;
        } else {
            kw[j] = KW > 0 ? tkeys_in[idc * static_cast<uint32_t>(KW) + static_cast<uint32_t>(word)]
                           : tkeys_in[static_cast<size_t>(idc) * W + word];
        }
    }
    if (STAGED) {
        if (trows_in) {
#pragma unroll
            for (int j = 0; j < ITEMS; ++j)
                rw[j] = trows_in[static_cast<uint32_t>(min(base_idx + j * 64 + lane, last_idx))];
        } else {
#pragma unroll
            for (int j = 0; j < ITEMS; ++j) rw[j] = base_idx + j * 64 + lane;
        }
    }
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int idx = base_idx + j * 64 + lane;
        const bool valid = idx < n;
        const uint32_t k = kw[j];
        const uint32_t d = (k >> shift) & 255u;
        // lanes holding the same digit
        const unsigned long long live = __builtin_amdgcn_ballot_w64(valid);
        uint32_t peers_lo = static_cast<uint32_t>(live), peers_hi = static_cast<uint32_t>(live >> 32);
        // Per digit bit b: x = all ones if the bit is set in this lane, else zero, and m = the lanes where
        // it is set.  Lanes agreeing with this one on the bit are m where x is ones and ~m where x is
        // zero, i.e. ~(m ^ x); peers &= ~(m ^ x) is one three-input bit operation per half.  Written out
        // by hand: eight compares first, then the sixteen bit operations, which keeps every vector read
        // of a compare's scalar result at least two instructions behind the compare (gfx950 needs that
        // distance and nothing pads inline assembly).
        uint32_t x[8];
        unsigned long long m[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) x[b] = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(d), b, 1));
#pragma unroll
        for (int b = 0; b < 8; ++b) asm volatile("v_cmp_ne_u32_e64 %0, 0, %1" : "=s"(m[b]) : "v"(x[b]));
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            asm volatile("v_bitop3_b32 %0, %0, %1, %2 bitop3:0x90"
                         : "+v"(peers_lo) : "s"(static_cast<uint32_t>(m[b])), "v"(x[b]));
            asm volatile("v_bitop3_b32 %0, %0, %1, %2 bitop3:0x90"
                         : "+v"(peers_hi) : "s"(static_cast<uint32_t>(m[b] >> 32)), "v"(x[b]));
        }
        // Every lane reads its digit's counter; then the lowest lane of each group of peers adds the
        // group's size.  LDS accesses of one wavefront complete in order and the counters belong to
        // this wavefront alone, so the reads see the value from before this step.
        const uint32_t below = __builtin_amdgcn_mbcnt_hi(peers_hi, __builtin_amdgcn_mbcnt_lo(peers_lo, 0u));
        const uint32_t old = whist[wave][d];
        if (valid && below == 0u) whist[wave][d] = old + static_cast<uint32_t>(__popc(peers_lo) + __popc(peers_hi));
        rank[j] = old + below;
    }
    __syncthreads();
    {   // digit `tid` (the first 256 threads have one): exclusive over the waves, then over the digits of the tile
        const bool has_digit = THREADS == 256 || tid < 256;
        uint32_t tot = 0;
        if (has_digit) {
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const uint32_t c = whist[w][tid];
                whist[w][tid] = tot;
                tot += c;
            }
        }
        uint32_t tile_total;
        const uint32_t ds = block_exclusive_sum(tot, scratch, &tile_total);
        if (has_digit) dstart[tid] = ds;
        if (CHAINED) {
            // publish this tile's count of digit `tid`, then add up the tiles before it
            uint32_t* st = state + static_cast<size_t>(t) * tiles * 256 + tid;  // entry of tile k: st[k * 256]
            if (has_digit)
                __hip_atomic_store(st + static_cast<size_t>(tile) * 256, (tile == 0 ? ST_SUM : ST_COUNT) | tot,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // start of the digit's range in the table: exclusive scan of the digit totals
            uint32_t all;
            const uint32_t dbase = block_exclusive_sum(has_digit ? dtot[t * 256 + tid] : 0u, scratch, &all);
            if (has_digit) {
                uint32_t before = 0;
                int polls = 0;
                for (int k = tile - 1; k >= 0;) {
                    const uint32_t v = __hip_atomic_load(st + static_cast<size_t>(k) * 256, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT);
                    const uint32_t tag = v >> 30;
                    if (tag == 0u) {
                        if (++polls > spin_limit) {  // give up: positions stay inside the digit's range
                            atomicOr(err, 1u);
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                        continue;
                    }
                    before += v & ST_VALUE;
                    if (tag == 2u) break;
                    --k;
                }
                if (tile > 0)
                    __hip_atomic_store(st + static_cast<size_t>(tile) * 256, ST_SUM | (before + tot), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                gbase[tid] = dbase + before - ds;
            }
        } else if (has_digit) {
            gbase[tid] = hist_scanned[(static_cast<size_t>(t) * 256 + tid) * tiles + tile] - ds;
        }
    }
    __syncthreads();
    // Stage the tile in digit order in LDS so that the global stores below walk
    // consecutive addresses inside every digit run (full-line writes instead of 4-byte ones).
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int idx = base_idx + j * 64 + lane;
        if (idx < n) {
            const uint32_t d = (kw[j] >> shift) & 255u;
            const uint32_t lp = dstart[d] + whist[wave][d] + rank[j];
            if (ONE_WORD) {
                st_key[lp] = kw[j];
                st_row[lp] = rw[j];
            } else if (TWO_WORDS) {
                *reinterpret_cast<uint2*>(&st_key[2 * lp]) =
                    word == 0 ? make_uint2(kw[j], kw_other[j]) : make_uint2(kw_other[j], kw[j]);
                st_row[lp] = rw[j];
            } else {
                st_key[lp] = static_cast<uint32_t>(idx - tile0);
            }
        }
    }
    __syncthreads();
    const int cnt = min(TILE, n - tile0);
    for (int slot = tid; slot < cnt; slot += THREADS) {
        if (ONE_WORD) {
            const uint32_t k = st_key[slot];
            const uint32_t dst = gbase[(k >> shift) & 255u] + static_cast<uint32_t>(slot);
            tkeys_out[dst] = k;
            trows_out[dst] = st_row[slot];
        } else if (TWO_WORDS) {
            const uint2 v = *reinterpret_cast<const uint2*>(&st_key[2 * slot]);
            const uint32_t kd = word == 0 ? v.x : v.y;
            const uint32_t dst = gbase[(kd >> shift) & 255u] + static_cast<uint32_t>(slot);
            *reinterpret_cast<uint2*>(tkeys_out + dst * 2u) = v;
            trows_out[dst] = st_row[slot];
        } else {
            const uint32_t src = static_cast<uint32_t>(tile0) + st_key[slot];
            if (KW == 4) {
                const uint4 v = *reinterpret_cast<const uint4*>(tkeys_in + src * 4u);
                const uint32_t kd = word == 0 ? v.x : (word == 1 ? v.y : (word == 2 ? v.z : v.w));
                const uint32_t dst = gbase[(kd >> shift) & 255u] + static_cast<uint32_t>(slot);
                *reinterpret_cast<uint4*>(tkeys_out + dst * 4u) = v;
                trows_out[dst] = trows_in ? trows_in[src] : static_cast<int32_t>(src);
            } else if (KW == 2) {
                const uint2 v = *reinterpret_cast<const uint2*>(tkeys_in + src * 2u);
                const uint32_t kd = word == 0 ? v.x : v.y;
                const uint32_t dst = gbase[(kd >> shift) & 255u] + static_cast<uint32_t>(slot);
                *reinterpret_cast<uint2*>(tkeys_out + dst * 2u) = v;
                trows_out[dst] = trows_in ? trows_in[src] : static_cast<int32_t>(src);
            } else {
                const uint32_t* ks = tkeys_in + static_cast<size_t>(src) * W;
                const uint32_t dst = gbase[(ks[word] >> shift) & 255u] + static_cast<uint32_t>(slot);
                for (int w = 0; w < W; ++w) tkeys_out[static_cast<size_t>(dst) * W + w] = ks[w];
                trows_out[dst] = trows_in ? trows_in[src] : static_cast<int32_t>(src);
            }
        }
    }
}

}  // namespace

namespace {

// One scatter pass with the tile shape of its key width.
template <int KW, bool CHAINED, int THREADS, int ITEMS, typename... Args>
culsh_status launch_scatter(culsh_ctx* ctx, dim3 grid, Args... args) {
    constexpr size_t lds = scatter_lds_bytes(KW, TileShape{THREADS, ITEMS});
    static PerDeviceOnce configured;  // more LDS than a launch may ask for by default
    if (lds > 48 * 1024 && !configured.is_set(ctx->device)) {
        CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(radix_scatter_kernel<KW, CHAINED, THREADS, ITEMS>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        configured.set(ctx->device);
    }
    {
        static const char* const names[2][5] = {
            {"radix_scatter_kernel<0, false>", "radix_scatter_kernel<1, false>", "radix_scatter_kernel<2, false>", "",
             "radix_scatter_kernel<4, false>"},
            {"radix_scatter_kernel<0, true>", "radix_scatter_kernel<1, true>", "radix_scatter_kernel<2, true>", "",
             "radix_scatter_kernel<4, true>"}};
        StageTimer st(ctx, names[CHAINED ? 1 : 0][KW]);
        hipLaunchKernelGGL((radix_scatter_kernel<KW, CHAINED, THREADS, ITEMS>), grid, dim3(THREADS), lds, ctx->stream, args...);
    }
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

template <bool CHAINED, typename... Args>
culsh_status scatter_pass(culsh_ctx* ctx, dim3 grid, int W, bool fixed_width, Args... args) {
    if (W == 1)
        return fixed_width ? launch_scatter<1, CHAINED, SHAPE_W1.threads, SHAPE_W1.items>(ctx, grid, args...)
                           : launch_scatter<0, CHAINED, SHAPE_W1.threads, SHAPE_W1.items>(ctx, grid, args...);
    if (W == 2)
        return fixed_width ? launch_scatter<2, CHAINED, SHAPE_W2.threads, SHAPE_W2.items>(ctx, grid, args...)
                           : launch_scatter<0, CHAINED, SHAPE_W2.threads, SHAPE_W2.items>(ctx, grid, args...);
    return (W == 4 && fixed_width) ? launch_scatter<4, CHAINED, SHAPE_ANY.threads, SHAPE_ANY.items>(ctx, grid, args...)
                                   : launch_scatter<0, CHAINED, SHAPE_ANY.threads, SHAPE_ANY.items>(ctx, grid, args...);
}

}  // namespace

size_t sort_scratch_bytes(int n, int T, int W) {
    const size_t tiles = (static_cast<size_t>(n) + tile_shape(W).tile() - 1) / tile_shape(W).tile();
    return align_up(static_cast<size_t>(T) * 256 * tiles * sizeof(uint32_t), 256) +
           align_up(static_cast<size_t>(W) * sizeof(uint32_t), 256) + 512;
}

culsh_status sort_tables(culsh_ctx* ctx, uint32_t* keys_in, uint32_t* keys_tmp, int32_t* rows_tmp,
                         int32_t* rows_out, int n, int T, int W, const uint32_t* known_vary,
                         uint32_t** sorted_keys) {
    CULSH_REQUIRE(n > 0 && T > 0 && W > 0 && W <= 64, CULSH_ERR_INVALID, "sort: bad sizes (W must be <= 64 words)");
    CULSH_REQUIRE(T <= 65535, CULSH_ERR_LIMIT, "n_hash_tables > 65535 is not supported");
    const int tile_items = tile_shape(W).tile();
    const int tiles = (n + tile_items - 1) / tile_items;
    const size_t N = static_cast<size_t>(n) * T;

    // which byte positions differ anywhere (given by the caller, or measured on the keys)
    uint32_t vary[64];
    if (known_vary) {
        for (int w = 0; w < W; ++w) vary[w] = known_vary[w];
    } else {
        uint32_t* vary_dev = nullptr;
        CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(W), &vary_dev));
        CULSH_HIP(hipMemsetAsync(vary_dev, 0, W * sizeof(uint32_t), ctx->stream));
        const bool vec = (W == 1 || W == 2 || W == 4) && (static_cast<size_t>(n) * W) % 4 == 0 &&
                         reinterpret_cast<uintptr_t>(keys_in) % 16 == 0;
        if (vec) {
            const unsigned bx = std::max(1u, std::min(64u, div_up(static_cast<size_t>(n) * W / 4, 256 * 4)));
            CULSH_LAUNCH(ctx, varying_bits_vec_kernel, dim3(bx, T), dim3(256), 0, ctx->stream, keys_in, n, W, vary_dev);
        } else {
            const unsigned bx = std::max(1u, std::min(64u, div_up(n, 256 * 8)));
            CULSH_LAUNCH(ctx, varying_bits_kernel, dim3(bx, T), dim3(256), 0, ctx->stream, keys_in, n, W, vary_dev);
        }
        CULSH_LAUNCH_CHECK();
        CULSH_TRY(read_back_u32(ctx, vary_dev, W, vary));
    }

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

    uint32_t* kin = keys_in;
    uint32_t* kout = keys_tmp;
    const int np = static_cast<int>(passes.size());
    const char* env_unchained = std::getenv("CULSH_SORT_UNCHAINED");
    const bool chained = !ctx->sort_unchained && n < (1 << 30) && !(env_unchained && *env_unchained == '1') &&
                         static_cast<size_t>(tiles) * T < (1ull << 31);
    // zero-initialised words in one block, cleared by one memset: [pass][T][256] digit totals, then
    // (chained) the published words [pass][T][tiles][256] and 2 flag words
    const size_t dtot_words = static_cast<size_t>(np) * T * 256;
    const size_t state_words = static_cast<size_t>(T) * tiles * 256;
    const size_t zero_words = dtot_words + (chained ? 2 + static_cast<size_t>(np) * state_words : 0);
    uint32_t* dtot = nullptr;
    CULSH_TRY(arena_alloc_t(ctx, zero_words, &dtot));
    CULSH_HIP(hipMemsetAsync(dtot, 0, zero_words * sizeof(uint32_t), ctx->stream));
    uint32_t* hist = nullptr;   // unchained: [T][256][tiles]
    uint32_t* state = nullptr;
    uint32_t* err = nullptr;
    ctx->sort_err_dev = nullptr;
    if (chained) {
        state = dtot + dtot_words;  // rows of 256 words stay 1 KiB aligned
        err = state + static_cast<size_t>(np) * state_words;
        ctx->sort_err_dev = err;
        for (int p0 = 0; p0 < np; p0 += MAX_PASSES_PER_LAUNCH) {
            PassList pl;
            pl.count = std::min(MAX_PASSES_PER_LAUNCH, np - p0);
            for (int i = 0; i < MAX_PASSES_PER_LAUNCH; ++i) {
                pl.word[i] = i < pl.count ? passes[p0 + i].word : 0;
                pl.shift[i] = i < pl.count ? passes[p0 + i].shift : 0;
            }
            // about four workgroups per CU over all tables
            const int per_table = std::max(1, std::min((n + TOT_TILE - 1) / TOT_TILE, (4 * ctx->n_cus + T - 1) / T));
            // as many histogram copies as 60 KiB hold, eight at most
            const int copies = std::max(1, std::min(8, (60 * 1024) / (pl.count * TOT_ROW * 4)));
            const size_t lds = static_cast<size_t>(copies) * pl.count * TOT_ROW * sizeof(uint32_t);
            static PerDeviceOnce configured;  // more LDS than a launch may ask for by default
            if (lds > 48 * 1024 && !configured.is_set(ctx->device)) {
                CULSH_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(radix_totals_kernel),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, 60 * 1024));
                configured.set(ctx->device);
            }
            CULSH_LAUNCH(ctx, radix_totals_kernel, dim3(per_table, T), dim3(SORT_THREADS), lds, ctx->stream, keys_in, n, W, pl,
                         T, copies, dtot + static_cast<size_t>(p0) * T * 256);
            CULSH_LAUNCH_CHECK();
        }
    } else {
        CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(T) * 256 * tiles, &hist));
    }
    // polls of an unpublished predecessor before a workgroup gives up (CULSH_SORT_SPIN_LIMIT: tests
    // set it to 0 to reach the give-up path while every kernel still runs to its end)
    const char* env_spin = std::getenv("CULSH_SORT_SPIN_LIMIT");
    const int spin_limit = (env_spin && *env_spin) ? std::atoi(env_spin) : (1 << 20);
    const int32_t* rin = nullptr;
    for (int p = 0; p < np; ++p) {
        // the last pass must land in rows_out
        int32_t* rout = ((np - 1 - p) % 2 == 0) ? rows_out : rows_tmp;
        uint32_t* pass_dtot = dtot + static_cast<size_t>(p) * T * 256;
        // fixed-width variants use 32-bit element offsets inside a table and vector accesses
        const bool fixed_width = n < (1 << 30) && (W == 1 || (reinterpret_cast<uintptr_t>(kin) % 16 == 0 &&
                                                               reinterpret_cast<uintptr_t>(kout) % 16 == 0));
        if (chained) {
            const dim3 grid(static_cast<unsigned>(tiles) * T);
            uint32_t* pass_state = state + static_cast<size_t>(p) * state_words;
            CULSH_TRY(scatter_pass<true>(ctx, grid, W, fixed_width, static_cast<const uint32_t*>(kin), rin, kout, rout,
                                         static_cast<const uint32_t*>(nullptr), n, W, passes[p].word, passes[p].shift,
                                         tiles, T, static_cast<const uint32_t*>(pass_dtot), pass_state, err, spin_limit));
        } else {
            const dim3 grid(tiles, T);
            CULSH_LAUNCH(ctx, radix_hist_kernel, grid, dim3(SORT_THREADS), 0, ctx->stream, kin, n, W,
                         passes[p].word, passes[p].shift, tiles, tile_items, hist, pass_dtot);
            CULSH_LAUNCH_CHECK();
            CULSH_LAUNCH(ctx, radix_scan_kernel, dim3(T, SCAN_PARTS), dim3(256), 0, ctx->stream, hist, pass_dtot, tiles);
            CULSH_LAUNCH_CHECK();
            CULSH_TRY(scatter_pass<false>(ctx, grid, W, fixed_width, static_cast<const uint32_t*>(kin), rin, kout, rout,
                                          static_cast<const uint32_t*>(hist), n, W, passes[p].word, passes[p].shift,
                                          tiles, T, static_cast<const uint32_t*>(nullptr),
                                          static_cast<uint32_t*>(nullptr), static_cast<uint32_t*>(nullptr), 0));
        }
        std::swap(kin, kout);
        rin = rout;
    }
    *sorted_keys = kin;
    return CULSH_OK;
}

}  // namespace culsh_amd
