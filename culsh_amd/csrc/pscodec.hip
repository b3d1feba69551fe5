// Order-preserving key compression for p-stable signatures.
//
// A p-stable signature is H little-endian int32 hashes, and buckets are ordered by the
// raw bytes (core/fit.cuh:265-272), i.e. every hash is ordered by its byte-swapped value.
// Sorting those 4*H bytes directly needs up to 4*H radix passes over 4*H-byte keys.  The
// hashes of real data span a few dozen values per hash function, so each hash is replaced
// by its rank (1-based, 0 = "value never seen at fit time") in byte-swapped order among
// the values of [min, max] observed for that (table, hash).  Ranks of `bits` bits are
// concatenated most-significant first, which keeps the bucket order bit for bit and
// shrinks keys from 32*H to bits*H bits.  The inverse table restores the signatures of
// the buckets in the reference layout.
#include <algorithm>
#include <climits>
#include <vector>

#include "common.hpp"

namespace culsh_amd {
namespace {

// VEC4: H divides 1024 and is a multiple of 4, sig is 16-byte aligned: a thread reads 16 bytes at a time and
// always meets the same four hash positions.
template <bool VEC4>
__global__ __launch_bounds__(256) void ps_minmax_kernel(const int32_t* __restrict__ sig, int n, int H,
                                                       int32_t* __restrict__ mm /*[T*H][2]*/) {
    __shared__ int32_t smin[1024], smax[1024];
    const int t = blockIdx.y;
    for (int h = threadIdx.x; h < H; h += 256) { smin[h] = INT_MAX; smax[h] = INT_MIN; }
    __syncthreads();
    const int32_t* ts = sig + static_cast<size_t>(t) * n * H;
    const size_t total = static_cast<size_t>(n) * H;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    size_t e = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (VEC4) {
        const int4* t4 = reinterpret_cast<const int4*>(ts);  // table bases stay 16-byte aligned: n * H * 4 bytes each
        const size_t quads = total / 4;
        int4 lo = make_int4(INT_MAX, INT_MAX, INT_MAX, INT_MAX), hi = make_int4(INT_MIN, INT_MIN, INT_MIN, INT_MIN);
#pragma unroll 4
        for (; e < quads; e += stride) {
            const int4 v = t4[e];
            lo.x = min(lo.x, v.x); lo.y = min(lo.y, v.y); lo.z = min(lo.z, v.z); lo.w = min(lo.w, v.w);
            hi.x = max(hi.x, v.x); hi.y = max(hi.y, v.y); hi.z = max(hi.z, v.z); hi.w = max(hi.w, v.w);
        }
        const int h0 = static_cast<int>((4 * (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x)) % H);  // 4 * stride is a multiple of H
        if (lo.x <= hi.x) {
            atomicMin(&smin[h0], lo.x); atomicMax(&smax[h0], hi.x);
            atomicMin(&smin[h0 + 1], lo.y); atomicMax(&smax[h0 + 1], hi.y);
            atomicMin(&smin[h0 + 2], lo.z); atomicMax(&smax[h0 + 2], hi.z);
            atomicMin(&smin[h0 + 3], lo.w); atomicMax(&smax[h0 + 3], hi.w);
        }
    } else if (256 % H == 0) {  // the thread always meets the same hash position
        int32_t lo = INT_MAX, hi = INT_MIN;
#pragma unroll 4
        for (; e < total; e += stride) {
            const int32_t v = ts[e];
            lo = min(lo, v);
            hi = max(hi, v);
        }
        if (lo <= hi) {
            atomicMin(&smin[threadIdx.x % H], lo);
            atomicMax(&smax[threadIdx.x % H], hi);
        }
    } else {
        for (; e < total; e += stride) {
            const int32_t v = ts[e];
            const int h = static_cast<int>(e % H);
            if (v < smin[h]) atomicMin(&smin[h], v);
            if (v > smax[h]) atomicMax(&smax[h], v);
        }
    }
    __syncthreads();
    for (int h = threadIdx.x; h < H; h += 256) {
        if (smin[h] <= smax[h]) {
            atomicMin(&mm[(t * H + h) * 2 + 0], smin[h]);
            atomicMax(&mm[(t * H + h) * 2 + 1], smax[h]);
        }
    }
}

__global__ __launch_bounds__(256) void ps_minmax_reset_kernel(int32_t* __restrict__ mm, int columns) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c < columns) {
        mm[2 * c] = INT_MAX;
        mm[2 * c + 1] = INT_MIN;
    }
}

// Rank tables of one table's H hash functions fit in LDS when they have at most this many words.
// Looking ranks up in global memory costs a 64-address gather per wave and hash, which keeps the
// texture path busy for longer than everything else in these kernels together.
constexpr int PS_LUT_WORDS = 8192;

template <bool VEC4, typename F, typename V>
__device__ __forceinline__ void ps_compress_item(const int32_t* __restrict__ s, uint32_t* __restrict__ k, int H,
                                                 int bits, int rmax, F fwd, V vmin, V range) {
    unsigned long long acc = 0;
    int nbits = 0, w = 0;
    auto put = [&](int h, int32_t v) {
        const long long idx = static_cast<long long>(v) - vmin[h];
        const uint32_t code = (idx >= 0 && idx < range[h]) ? fwd[h * rmax + static_cast<int>(idx)] + 1u : 0u;
        acc = (acc << bits) | code;
        nbits += bits;
        if (nbits >= 32) {
            k[w++] = static_cast<uint32_t>(acc >> (nbits - 32));
            nbits -= 32;
            acc &= (1ull << nbits) - 1ull;
        }
    };
    if (VEC4) {
        for (int h = 0; h < H; h += 4) {
            const int4 v = *reinterpret_cast<const int4*>(s + h);
            put(h, v.x);
            put(h + 1, v.y);
            put(h + 2, v.z);
            put(h + 3, v.w);
        }
    } else {
        for (int h = 0; h < H; ++h) put(h, s[h]);
    }
    if (nbits > 0) k[w++] = static_cast<uint32_t>(acc << (32 - nbits));
}

// VEC4: H is a multiple of 4 and sig is 16-byte aligned, so the hashes of an item come in 16-byte loads.
// `use_lds`: the launch carries (H * rmax + 2 * H) words of LDS; a workgroup whose items all belong to
// one table (all but T - 1 of them) looks ranks up there.
template <bool VEC4>
__global__ __launch_bounds__(256) void ps_compress_kernel(const int32_t* __restrict__ sig, size_t rows, int T, int H,
                                                         int bits, int rmax, int W, int use_lds, int t0,
                                                         const int32_t* __restrict__ vmin,
                                                         const int32_t* __restrict__ range,
                                                         const uint32_t* __restrict__ fwd,
                                                         uint32_t* __restrict__ keys) {
    extern __shared__ uint32_t ps_lut[];  // [H * rmax] ranks, [H] minima, [H] ranges
    const size_t items = rows * T;
    const size_t item0 = static_cast<size_t>(blockIdx.x) * 256;
    const size_t item = item0 + threadIdx.x;
    const int t_first = t0 + static_cast<int>(item0 / rows);  // t0: number of the first table of `sig`
    const int t_last = t0 + static_cast<int>(min(item0 + 255, items - 1) / rows);
    const bool staged = use_lds && t_first == t_last;  // uniform over the workgroup
    if (staged) {
        const int lut = H * rmax;
        const uint32_t* f = fwd + static_cast<size_t>(t_first) * lut;
        for (int i = threadIdx.x; i < lut; i += 256) ps_lut[i] = f[i];
        for (int h = threadIdx.x; h < H; h += 256) {
            ps_lut[lut + h] = static_cast<uint32_t>(vmin[t_first * H + h]);
            ps_lut[lut + H + h] = static_cast<uint32_t>(range[t_first * H + h]);
        }
        __syncthreads();
    }
    if (item >= items) return;
    const int32_t* s = sig + item * H;
    uint32_t* k = keys + item * W;
    if (staged) {
        const int32_t* lv = reinterpret_cast<const int32_t*>(ps_lut + H * rmax);
        ps_compress_item<VEC4>(s, k, H, bits, rmax, ps_lut, lv, lv + H);
    } else {
        const int t = t0 + static_cast<int>(item / rows);
        ps_compress_item<VEC4>(s, k, H, bits, rmax, fwd + static_cast<size_t>(t) * H * rmax, vmin + t * H,
                               range + t * H);
    }
}

// A workgroup restores the signatures of `bpb` consecutive buckets (a multiple of 256 chosen by the
// host so that the key words fit in 16 KiB of LDS).  The tables of its first and last bucket are
// searched once; nearly every workgroup lies inside one table or across one boundary, and then a
// bucket's table follows from one comparison.  (bucket, hash) pairs are written by consecutive
// threads to consecutive addresses.  With `use_lds` the launch also carries 2 * H * rmax words of
// LDS for the value tables of two neighbouring hash tables.
constexpr int PS_BPB_MIN = 256;

// largest t in [lo, hi) with table_bucket_offsets[t] <= bucket
__device__ __forceinline__ int ps_table_of(const int32_t* __restrict__ table_bucket_offsets, int lo, int hi, size_t bucket) {
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (static_cast<size_t>(table_bucket_offsets[mid]) <= bucket) lo = mid; else hi = mid;
    }
    return lo;
}

__global__ __launch_bounds__(256) void ps_keys_to_sig_kernel(const uint32_t* __restrict__ keys, size_t count,
                                                            const uint64_t* __restrict__ count_dev,
                                                            const int32_t* __restrict__ table_bucket_offsets, int T,
                                                            int H, int bits, int rmax, int W, int use_lds, int bpb,
                                                            const int32_t* __restrict__ inv,
                                                            int32_t* __restrict__ sig,
                                                            const uint32_t* __restrict__ sort_gave_up) {
    extern __shared__ uint32_t ps_lds[];  // [2] first and last table, [bpb][W] key words, then the value tables
    if (sort_gave_up && *sort_gave_up) return;  // bucket keys of a failed sort may hold ranks beyond the tables
    uint32_t* trange = ps_lds;
    uint32_t* kw = ps_lds + 2;
    int32_t* lut = reinterpret_cast<int32_t*>(kw + static_cast<size_t>(bpb) * W);
    if (count_dev) count = min(count, static_cast<size_t>(*count_dev));
    const size_t b0 = static_cast<size_t>(blockIdx.x) * bpb;
    if (b0 >= count) return;
    const int nb = static_cast<int>(min(static_cast<size_t>(bpb), count - b0));
    if (threadIdx.x < 2)
        trange[threadIdx.x] = static_cast<uint32_t>(
            ps_table_of(table_bucket_offsets, 0, T, threadIdx.x == 0 ? b0 : b0 + static_cast<size_t>(nb) - 1));
    for (int i = threadIdx.x; i < nb * W; i += 256) kw[i] = keys[b0 * W + i];
    __syncthreads();
    const int t_first = static_cast<int>(trange[0]), t_last = static_cast<int>(trange[1]);
    const bool near = t_last - t_first <= 1;  // uniform over the workgroup
    const bool staged = use_lds && near;
    if (staged) {
        const int words = (t_last - t_first + 1) * H * rmax;  // one table's values, or two
        const int32_t* src = inv + static_cast<size_t>(t_first) * H * rmax;
        for (int i = threadIdx.x; i < words; i += 256) lut[i] = src[i];
        __syncthreads();
    }
    // first bucket of the second table (none: beyond every bucket)
    const size_t second = t_last > t_first ? static_cast<size_t>(table_bucket_offsets[t_first + 1]) : ~size_t(0);
    const uint32_t mask = (1u << bits) - 1u;
    auto value = [&](int bl, int t, int h) -> int32_t {
        const uint32_t* k = kw + bl * W;
        const int o = h * bits, w0 = o >> 5, sh = o & 31;
        const unsigned long long two = (static_cast<unsigned long long>(k[w0]) << 32) | (w0 + 1 < W ? k[w0 + 1] : 0u);
        const uint32_t code = static_cast<uint32_t>(two >> (64 - sh - bits)) & mask;
        if (!code) return 0;
        const int c = t * H + h;
        return staged ? lut[(c - t_first * H) * rmax + static_cast<int>(code - 1u)]
                      : inv[static_cast<size_t>(c) * rmax + (code - 1u)];
    };
    auto table = [&](int bl) -> int {
        const size_t bucket = b0 + bl;
        return near ? t_first + (bucket >= second ? 1 : 0) : ps_table_of(table_bucket_offsets, t_first, t_last + 1, bucket);
    };
    int32_t* out = sig + b0 * H;
    if (H % 4 == 0 && reinterpret_cast<uintptr_t>(sig) % 16 == 0) {  // four hashes of a bucket per thread and store
        const int qpb = H >> 2;
        for (int q = threadIdx.x; q < nb * qpb; q += 256) {
            const int bl = q / qpb, h = (q - bl * qpb) << 2;
            const int t = table(bl);
            *reinterpret_cast<int4*>(out + 4 * static_cast<size_t>(q)) =
                make_int4(value(bl, t, h), value(bl, t, h + 1), value(bl, t, h + 2), value(bl, t, h + 3));
        }
    } else {
        for (int i = threadIdx.x; i < nb * H; i += 256) {
            const int bl = i / H;
            out[i] = value(bl, table(bl), i - bl * H);
        }
    }
}

}  // namespace

void free_ps_codec(culsh_index* ix) {
    dev_free(ix->psc.vmin);  // one block: vmin | range | fwd | inv
    ix->psc = PsCodec();
}

culsh_status ps_minmax_prepare(culsh_ctx* ctx, int T, int H, int32_t** mm_dev) {
    const int TH = T * H;
    CULSH_TRY(arena_alloc_t(ctx, static_cast<size_t>(TH) * 2, mm_dev));
    CULSH_LAUNCH(ctx, ps_minmax_reset_kernel, dim3(div_up(static_cast<size_t>(TH), 256)), dim3(256), 0, ctx->stream,
                 *mm_dev, TH);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status ps_build_codec(culsh_ctx* ctx, const int32_t* sig, int n, int T, int H, culsh_index* ix,
                            bool* compressed, int32_t* mm_folded) {
    *compressed = false;
    const int TH = T * H;
    if (H > 1024) return CULSH_OK;
    int32_t* mm_dev = mm_folded;
    if (!mm_dev) {
        CULSH_TRY(ps_minmax_prepare(ctx, T, H, &mm_dev));
        const size_t per_table = static_cast<size_t>(n) * H;
        const bool vec4 = H % 4 == 0 && 1024 % H == 0 && reinterpret_cast<uintptr_t>(sig) % 16 == 0;
        const unsigned bx = std::max(1u, std::min(256u, div_up(per_table, 256 * (vec4 ? 64 : 16))));
        if (vec4)
            CULSH_LAUNCH(ctx, ps_minmax_kernel<true>, dim3(bx, T), dim3(256), 0, ctx->stream, sig, n, H, mm_dev);
        else
            CULSH_LAUNCH(ctx, ps_minmax_kernel<false>, dim3(bx, T), dim3(256), 0, ctx->stream, sig, n, H, mm_dev);
        CULSH_LAUNCH_CHECK();
    }
    std::vector<int32_t> mm(static_cast<size_t>(TH) * 2);
    CULSH_HIP(hipMemcpyAsync(mm.data(), mm_dev, mm.size() * sizeof(int32_t), hipMemcpyDeviceToHost, ctx->stream));
    CULSH_HIP(hipStreamSynchronize(ctx->stream));
    return ps_build_codec_from_ranges(ctx, mm.data(), T, H, ix, compressed);
}

culsh_status ps_build_codec_from_ranges(culsh_ctx* ctx, const int32_t* mm, int T, int H, culsh_index* ix, bool* compressed) {
    *compressed = false;
    const int TH = T * H;
    if (H > 1024) return CULSH_OK;
    long long rmax = 1;
    for (int c = 0; c < TH; ++c) rmax = std::max(rmax, static_cast<long long>(mm[2 * c + 1]) - mm[2 * c] + 1);
    int bits = 1;
    while ((1ll << bits) < rmax + 1) ++bits;  // codes 1..range, 0 reserved
    const int W = (H * bits + 31) / 32;
    if (bits > 12 || W >= H) return CULSH_OK;  // wide value ranges: keep the plain byte order keys
    if (W > 56) return CULSH_OK;               // the restore kernel keeps at least 256 keys of W words in LDS

    // one host block, one device block, one copy: vmin[TH] | range[TH] | fwd[TH][rmax] | inv[TH][rmax]
    const size_t lut = static_cast<size_t>(TH) * rmax;
    std::vector<int32_t> host(2 * static_cast<size_t>(TH) + 2 * lut, 0);
    int32_t* vmin = host.data();
    int32_t* range = vmin + TH;
    uint32_t* fwd = reinterpret_cast<uint32_t*>(range + TH);
    int32_t* inv = reinterpret_cast<int32_t*>(fwd + lut);
    std::vector<std::pair<uint32_t, int32_t>> order;
    for (int c = 0; c < TH; ++c) {
        vmin[c] = mm[2 * c];
        range[c] = static_cast<int32_t>(static_cast<long long>(mm[2 * c + 1]) - mm[2 * c] + 1);
        order.clear();
        for (int i = 0; i < range[c]; ++i) {
            const int32_t v = vmin[c] + i;
            order.emplace_back(__builtin_bswap32(static_cast<uint32_t>(v)), v);  // byte order of a little-endian int32
        }
        std::sort(order.begin(), order.end());
        for (int r = 0; r < range[c]; ++r) {
            fwd[static_cast<size_t>(c) * rmax + (order[r].second - vmin[c])] = static_cast<uint32_t>(r);
            inv[static_cast<size_t>(c) * rmax + r] = order[r].second;
        }
    }
    PsCodec& pc = ix->psc;
    pc.bits = bits;
    pc.rmax = static_cast<int>(rmax);
    int32_t* block = nullptr;
    CULSH_HIP(dev_malloc(&block, host.size() * sizeof(int32_t)));
    pc.vmin = block;
    pc.range = block + TH;
    pc.fwd = reinterpret_cast<uint32_t*>(block + 2 * static_cast<size_t>(TH));
    pc.inv = block + 2 * static_cast<size_t>(TH) + lut;
    CULSH_TRY(upload_async(ctx, host.data(), host.size() * sizeof(int32_t), block));  // staged: `host` may go
    ix->enc = ENC_PSC;
    ix->key_w = W;
    *compressed = true;
    return CULSH_OK;
}

culsh_status launch_ps_compress(culsh_ctx* ctx, const int32_t* sig, size_t rows, int T, int H, const culsh_index* ix,
                                uint32_t* keys, int t0) {
    const size_t items = rows * T;
    if (items == 0) return CULSH_OK;
    CULSH_REQUIRE(items / 256 < (1ull << 31), CULSH_ERR_LIMIT, "too many items");
    const PsCodec& pc = ix->psc;
    const size_t lut_words = static_cast<size_t>(H) * pc.rmax;
    const int use_lds = lut_words <= PS_LUT_WORDS;
    const size_t lds = use_lds ? (lut_words + 2 * static_cast<size_t>(H)) * sizeof(uint32_t) : 0;
    if (H % 4 == 0 && reinterpret_cast<uintptr_t>(sig) % 16 == 0)
        CULSH_LAUNCH(ctx, ps_compress_kernel<true>, dim3(div_up(items, 256)), dim3(256), lds, ctx->stream, sig, rows, T,
                     H, pc.bits, pc.rmax, ix->key_w, use_lds, t0, pc.vmin, pc.range, pc.fwd, keys);
    else
        CULSH_LAUNCH(ctx, ps_compress_kernel<false>, dim3(div_up(items, 256)), dim3(256), lds, ctx->stream, sig, rows, T,
                     H, pc.bits, pc.rmax, ix->key_w, use_lds, t0, pc.vmin, pc.range, pc.fwd, keys);
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status launch_ps_keys_to_sig(culsh_ctx* ctx, const culsh_index* ix, size_t count, const uint64_t* count_dev,
                                   uint8_t* sig) {
    if (count == 0) return CULSH_OK;
    const PsCodec& pc = ix->psc;
    const size_t lut_words = 2 * static_cast<size_t>(ix->n_hashes) * pc.rmax;
    // buckets per workgroup: as many as 16 KiB of key words hold, 256 to 2048
    const int bpb = std::max(PS_BPB_MIN, std::min(2048, (4096 / ix->key_w) / 256 * 256));
    // the value tables go to LDS when they are small and fit beside the key words
    const int use_lds = lut_words <= PS_LUT_WORDS &&
                        (2 + static_cast<size_t>(bpb) * ix->key_w + lut_words) * sizeof(uint32_t) <= 64 * 1024;
    CULSH_REQUIRE(count / bpb < (1ull << 31), CULSH_ERR_LIMIT, "too many buckets");
    const size_t lds = (2 + static_cast<size_t>(bpb) * ix->key_w + (use_lds ? lut_words : 0)) * sizeof(uint32_t);
    CULSH_REQUIRE(lds <= 64 * 1024, CULSH_ERR_LIMIT, "key width too large for the signature restore kernel");
    CULSH_LAUNCH(ctx, ps_keys_to_sig_kernel, dim3(div_up(count, bpb)), dim3(256), lds, ctx->stream, ix->bucket_keys,
                 count, count_dev, ix->table_bucket_offsets, ix->n_hash_tables, ix->n_hashes, pc.bits, pc.rmax,
                 ix->key_w, use_lds, bpb, pc.inv, reinterpret_cast<int32_t*>(sig), static_cast<const uint32_t*>(ctx->sort_err_dev));
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

}  // namespace culsh_amd
