// Projection hashing for RPLSH and p-stable LSH on gfx950.
//
// Replaces the reference's GEMM + elementwise pass (rplsh/hash.cuh:92-129,
// pslsh/hash.cuh:104-142): X * P^T is computed with fp32 MFMA tiles and the sign /
// floor epilogue is applied to the accumulators in registers, so the n x (T*H)
// projection matrix is never written to memory.
#include <climits>

#include "common.hpp"

namespace culsh_amd {

typedef float f32x16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int BM = 128;        // rows of X per workgroup
constexpr int BN = 128;        // (virtual) hash columns per workgroup
constexpr int NTHREADS = 256;  // 4 wavefronts as 2 x 2, each 64 x 64 of the tile

struct ProjArgs {
    const float* X;
    const float* P;
    const float* b;
    void* out;
    int n, d, T, H;
    int n_row_tiles, n_col_tiles;
    int vec_x, vec_p;  // 16-byte vector loads allowed
    int32_t* mm;       // EPI_FLOOR_I32_MM: [T*H][2] running minimum / maximum per column
};

// p-stable epilogue that also folds every column's smallest and largest hash into ProjArgs::mm
// (kernel-internal: callers ask for EPI_FLOOR_I32 and pass the array)
constexpr int EPI_FLOOR_I32_MM = 4;

// Column order of the sign-packing epilogue.  Columns are grouped in tiles of 32 so that
// one wavefront ballot over a 32-column MFMA tile yields key bits directly:
//   H <= 32: a tile holds floor(32/H) whole tables; table `sub` owns ballot bits
//            [sub*H, sub*H + H) with hash 0 at the top of that field
//   H  > 32: a tile is one 32-bit key word of one table, hash 32w + j at bit 31 - j
// Returns the row of P feeding virtual column vc, or -1 for a padding column.
__device__ __forceinline__ int sign_vcol_to_prow(int vc, int T, int H) {
    const int tile = vc >> 5, c = vc & 31;
    if (H <= 32) {
        const int tpt = 32 / H;
        const int sub = c / H;
        const int table = tile * tpt + sub;
        if (sub >= tpt || table >= T) return -1;
        return table * H + (H - 1 - (c - sub * H));
    }
    const int wt = (H + 31) >> 5;
    const int table = tile / wt, w = tile - table * wt;
    const int h = 32 * w + (31 - c);
    if (table >= T || h >= H) return -1;
    return table * H + h;
}

__device__ __forceinline__ float4 load4(const float* __restrict__ base, size_t row_off, int k,
                                        int d, bool row_ok, int vec_ok) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!row_ok) return v;
    const float* p = base + row_off + k;
    if (vec_ok && k + 3 < d) return *reinterpret_cast<const float4*>(p);
    if (k + 0 < d) v.x = p[0];
    if (k + 1 < d) v.y = p[1];
    if (k + 2 < d) v.z = p[2];
    if (k + 3 < d) v.w = p[3];
    return v;
}

// VEC: n_features is a multiple of 4 and X, P are 16-byte aligned, so a stage is fetched
// with unconditional 16-byte loads.  Rows past the end of X and padding columns read a
// valid row instead of zeros: their accumulators are never stored.
// FULLK (with VEC): n_features is a multiple of BK, so no stage needs zero filling.
// BK features per stage: fewer mean fewer registers (more workgroups per CU), more barriers.
template <int EPI, bool VEC, int BK, bool FULLK>
__global__ __launch_bounds__(NTHREADS, (BK <= 8 ? 5 : (BK <= 16 ? 4 : 3))) void project_f32_kernel(ProjArgs a) {
    constexpr int PITCH = BK + 4;  // LDS row pitch in floats (bank spread for 16-byte reads)
    constexpr int F4 = BK / 4;     // float4 per tile row and stage
    constexpr int NLD = BM * F4 / NTHREADS;  // float4 fetched per thread, tile and stage
    constexpr int RSTEP = NTHREADS / F4;     // tile rows covered by one fetch of all threads
    __shared__ __attribute__((aligned(16))) float As[BM * PITCH];
    __shared__ __attribute__((aligned(16))) float Bs[BN * PITCH];
    __shared__ uint32_t tw[(EPI == EPI_SIGN_KEYS) ? BM * (BN / 32) : 1];
    constexpr bool FLOOR = (EPI == EPI_FLOOR_I32 || EPI == EPI_FLOOR_I32_MM);
    constexpr bool FOLD_MM = (EPI == EPI_FLOOR_I32_MM);
    constexpr int MM_PITCH = BN + 4;
    __shared__ int32_t cmin[FOLD_MM ? 8 * MM_PITCH : 1], cmax[FOLD_MM ? 8 * MM_PITCH : 1];  // [8 copies][column of the tile]
    if (FOLD_MM) {
        for (int i = threadIdx.x; i < 8 * MM_PITCH; i += NTHREADS) { cmin[i] = INT_MAX; cmax[i] = INT_MIN; }
        // the barriers of the stage loop stand between this and the epilogue (n_features > 0)
    }

    // Workgroup -> (row tile, column tile).  Consecutive workgroup ids are dealt round
    // robin to the 8 XCDs; ids are arranged so that all column tiles of one row tile land
    // on the same XCD (same id mod 8) and close in time, so the X tile is fetched from HBM
    // once and served from that XCD's L2 afterwards.
    //
    // A workgroup takes the tiles w, w + G, w + 2G, ... of that numbering, G (the grid) being a multiple
    // of 8 * n_col_tiles: its column tile and XCD never change, and a tile's first stage is fetched under
    // the last stage of the tile before.  The host launches one workgroup per tile (G = all tiles) or, for
    // launches of a single column tile, as many workgroups as stay resident.
    const int nct = a.n_col_tiles;
    const int per_group = 8 * nct;
    const int g0 = blockIdx.x / per_group, rem = blockIdx.x - g0 * per_group;
    const int ct = rem >> 3, slot = rem & 7;
    const int g_step = gridDim.x / per_group;       // row-tile groups between two tiles of this workgroup
    int rt = g0 * 8 + slot;                           // the tile being multiplied
    if (rt >= a.n_row_tiles) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r32 = lane & 31, half = lane >> 5;
    const int n = a.n, d = a.d, T = a.T, H = a.H;
    const int TH = T * H;

    // global -> LDS staging: thread loads float4 number (tid + 256*i), i < 4, of each tile.
    // Addresses are a wavefront-uniform tile base plus a 32-bit element offset per thread.
    const int lrow = tid / F4, c4 = (tid % F4) * 4;
    const float* xbase = nullptr;  // of the tile being fetched (the next one during a tile's last stage)
    uint32_t xoff[NLD], poff[NLD];
    bool xok[NLD], pok[NLD];
    auto fetch_from_tile = [&](int rt_f) {
        xbase = a.X + static_cast<size_t>(rt_f) * BM * d;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int lr = lrow + RSTEP * i;  // row inside the tile
            xok[i] = rt_f * BM + lr < n;
            // VEC reads a valid row instead of predicating: the last row of X for rows past the end
            xoff[i] = static_cast<uint32_t>(VEC ? min(lr, n - 1 - rt_f * BM) : lr) * static_cast<uint32_t>(d);
        }
    };
    fetch_from_tile(rt);
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int lr = lrow + RSTEP * i;  // row inside the tile
        const int vc = ct * BN + lr;
        const int prow = (EPI == EPI_SIGN_KEYS) ? sign_vcol_to_prow(vc, T, H) : (vc < TH ? vc : -1);
        pok[i] = prow >= 0;
        poff[i] = static_cast<uint32_t>(prow < 0 ? 0 : prow) * static_cast<uint32_t>(d);
    }
    // stage fetch: 4 + 4 float4 per thread
    auto fetch = [&](int k, float4 (&ra)[NLD], float4 (&rb)[NLD]) {
        if (VEC && FULLK) {
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const float4 va = *reinterpret_cast<const float4*>(xbase + (xoff[i] + static_cast<uint32_t>(k)));
                const float4 vb = *reinterpret_cast<const float4*>(a.P + (poff[i] + static_cast<uint32_t>(k)));
                ra[i] = make_float4(va.x, va.y, va.z, va.w);
                rb[i] = make_float4(vb.x, vb.y, vb.z, vb.w);
            }
        } else if (VEC) {
            const int kk = min(k, d - 4);
            const bool inside = k < d;  // a float4 is entirely inside or entirely outside [0, d)
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const float4 va = *reinterpret_cast<const float4*>(xbase + (xoff[i] + static_cast<uint32_t>(kk)));
                const float4 vb = *reinterpret_cast<const float4*>(a.P + (poff[i] + static_cast<uint32_t>(kk)));
                ra[i] = inside ? va : make_float4(0.f, 0.f, 0.f, 0.f);
                rb[i] = inside ? vb : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                ra[i] = load4(xbase, xoff[i], k, d, xok[i], 0);
                rb[i] = load4(a.P, poff[i], k, d, pok[i], 0);
            }
        }
    };

    float4 ra[NLD], rb[NLD];
    auto stage_to_lds = [&]() {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            *reinterpret_cast<float4*>(&As[(lrow + RSTEP * i) * PITCH + c4]) = ra[i];
            *reinterpret_cast<float4*>(&Bs[(lrow + RSTEP * i) * PITCH + c4]) = rb[i];
        }
    };
    fetch(c4, ra, rb);
    stage_to_lds();
    __syncthreads();

    const int nk = (d + BK - 1) / BK;
    for (;;) {  // tiles of this workgroup
        const int rt_next = rt + 8 * g_step;
        const bool has_next = rt_next < a.n_row_tiles;
        f32x16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

        for (int kt = 0; kt < nk; ++kt) {
            // LDS holds stage kt.  The next stage is fetched under this one's products: the tile's own, or
            // after its last stage the first one of the workgroup's next tile.
            const bool more = kt + 1 < nk;
            if (more) {
                fetch((kt + 1) * BK + c4, ra, rb);
            } else if (has_next) {
                fetch_from_tile(rt_next);
                fetch(c4, ra, rb);
            }
            // The 32x32x2 MFMA takes, per lane, A[row = lane%32][k = lane/32] and
            // B[k = lane/32][col = lane%32].  Any pairing of k between A and B that covers each
            // feature once is a valid dot product, so lanes 0-31 walk features 0..15 of the
            // stage and lanes 32-63 features BK/2..BK-1: each lane reads BK/2 consecutive floats.
            constexpr int KH = BK / 2;  // features per lane and stage
            float af[2][KH], bf[2][KH];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const float* pa = &As[(wm * 64 + i * 32 + r32) * PITCH + half * KH];
                const float* pb = &Bs[(wn * 64 + i * 32 + r32) * PITCH + half * KH];
#pragma unroll
                for (int q = 0; q < KH / 4; ++q) {
                    const float4 va = *reinterpret_cast<const float4*>(pa + 4 * q);
                    const float4 vb = *reinterpret_cast<const float4*>(pb + 4 * q);
                    af[i][4 * q + 0] = va.x; af[i][4 * q + 1] = va.y;
                    af[i][4 * q + 2] = va.z; af[i][4 * q + 3] = va.w;
                    bf[i][4 * q + 0] = vb.x; bf[i][4 * q + 1] = vb.y;
                    bf[i][4 * q + 2] = vb.z; bf[i][4 * q + 3] = vb.w;
                }
            }
#pragma unroll
            for (int k = 0; k < KH; ++k)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        // The key epilogue wants a lane to hold one column of its tile, the others one row
                        // (four neighbouring hashes per register quad): those swap the operands and get
                        // the transposed tile.
                        acc[i][j] = (EPI == EPI_SIGN_KEYS)
                                        ? __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][k], bf[j][k], acc[i][j], 0, 0, 0)
                                        : __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j][k], af[i][k], acc[i][j], 0, 0, 0);
            __syncthreads();  // every wavefront has its fragments: the stage may be overwritten
            if (more || has_next) stage_to_lds();
            __syncthreads();
        }

        // The epilogue's indices are derived again for every tile from a value the compiler cannot see
        // through: hoisted out of the tile loop as the loop invariants they are, they would sit in registers
        // all through the stage loop, which has none to spare.
        int e_tid = tid;
        asm volatile("" : "+v"(e_tid));
        const int e_lane = e_tid & 63, e_wave = e_tid >> 6;
        const int e_wm = e_wave >> 1, e_wn = e_wave & 1;
        const int e_r32 = e_lane & 31, e_half = e_lane >> 5;
        // Accumulator layout of the 32x32 tile: register v of e_lane l holds
        // row 8*(v/4) + 4*(l/32) + v%4, column l%32 of (first operand) x (second operand).
        if (EPI == EPI_SIGN_KEYS) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    int mine = 0;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        // hash bit = 1 iff the sign bit is clear (rplsh/hash.cuh:47)
                        const unsigned long long m =
                            __builtin_amdgcn_ballot_w64((__float_as_uint(acc[i][j][v]) >> 31) == 0u);
                        // the low e_half of the ballot is the word of row rlo, the high e_half that of row
                        // rlo + 4: each goes to the e_lane of that number
                        const int rlo = 8 * (v >> 2) + (v & 3);
                        const uint32_t m_lo = static_cast<uint32_t>(m), m_hi = static_cast<uint32_t>(m >> 32);
                        // (on gfx950 a vector instruction may not read an SGPR in the two issue slots after
                        // the vector compare that wrote it; the compiler does not pad inline assembly)
                        asm("s_nop 1\n\tv_writelane_b32 %0, %1, %3\n\tv_writelane_b32 %0, %2, %4"
                            : "+v"(mine)
                            : "s"(m_lo), "s"(m_hi), "n"(rlo), "n"(rlo + 4));
                    }
                    if (e_lane < 32) tw[(e_wm * 64 + i * 32 + e_lane) * (BN / 32) + (e_wn * 2 + j)] = static_cast<uint32_t>(mine);
                }
            __syncthreads();
            uint32_t* keys = static_cast<uint32_t*>(a.out);
            if (H <= 32) {
                const int tpt = 32 / H;
                const uint32_t mask = (H == 32) ? 0xFFFFFFFFu : ((1u << H) - 1u);
                // (table slot tl, row) pairs, rows fastest: a thread keeps its row and steps tl by
                // NTHREADS / BM, carrying (tc, sub) = (tl / tpt, tl % tpt) along without dividing
                constexpr int TL_STEP = NTHREADS / BM;
                const int row = e_tid % BM, grow = rt * BM + row;
                int tl = e_tid / BM;
                int tc = tl / tpt, sub = tl - tc * tpt;
                for (; tl < (BN / 32) * tpt; tl += TL_STEP) {
                    const int table = (ct * (BN / 32) + tc) * tpt + sub;
                    if (table < T && grow < n) {
                        const uint32_t field = (tw[row * (BN / 32) + tc] >> (sub * H)) & mask;
                        keys[static_cast<size_t>(table) * n + grow] = field << (32 - H);
                    }
                    sub += TL_STEP;
                    while (sub >= tpt) { sub -= tpt; ++tc; }
                }
            } else {
                const int wt = (H + 31) >> 5;
                for (int idx = e_tid; idx < (BN / 32) * BM; idx += NTHREADS) {
                    const int tc = idx / BM, row = idx - tc * BM;
                    const int tile = ct * (BN / 32) + tc;
                    const int table = tile / wt, w = tile - table * wt;
                    const int grow = rt * BM + row;
                    if (table < T && grow < n) {
                        const int nbits = min(32, H - 32 * w);
                        const uint32_t mask = (nbits == 32) ? 0xFFFFFFFFu : (0xFFFFFFFFu << (32 - nbits));
                        keys[(static_cast<size_t>(table) * n + grow) * wt + w] = tw[row * (BN / 32) + tc] & mask;
                    }
                }
            }
        } else {
            // Transposed tiles: registers 4g..4g+3 of e_lane l hold row l%32, columns 8g + 4*(l/32) + 0..3.
            // When H is a multiple of 4 those are four neighbouring hashes of one table, stored at once;
            // the 32 lanes of a e_half wave then cover 32 consecutive rows, H * 4 bytes apart.
            const bool quad = (H & 3) == 0 && (reinterpret_cast<uintptr_t>(a.out) & 15) == 0 &&
                              (!FLOOR || (reinterpret_cast<uintptr_t>(a.b) & 15) == 0);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int cb = ct * BN + e_wn * 64 + j * 32 + 4 * e_half;  // column of register 0
                int t = cb / H, h = cb - t * H;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int c0 = cb + 8 * g;
                    if (quad) {
                        if (c0 < TH) {
                            float4 bias = make_float4(0.f, 0.f, 0.f, 0.f);
                            if (FLOOR) bias = *reinterpret_cast<const float4*>(a.b + c0);
                            int4 lo = make_int4(INT_MAX, INT_MAX, INT_MAX, INT_MAX), hi = make_int4(INT_MIN, INT_MIN, INT_MIN, INT_MIN);
#pragma unroll
                            for (int i = 0; i < 2; ++i) {
                                const int row = rt * BM + e_wm * 64 + i * 32 + e_r32;
                                if (row >= n) continue;
                                const size_t off = (static_cast<size_t>(t) * n + row) * H + h;
                                const float x0 = acc[i][j][4 * g], x1 = acc[i][j][4 * g + 1];
                                const float x2 = acc[i][j][4 * g + 2], x3 = acc[i][j][4 * g + 3];
                                if (EPI == EPI_SIGN_BYTES) {
                                    const uint32_t bytes = ((__float_as_uint(x0) >> 31) ^ 1u) |
                                                           (((__float_as_uint(x1) >> 31) ^ 1u) << 8) |
                                                           (((__float_as_uint(x2) >> 31) ^ 1u) << 16) |
                                                           (((__float_as_uint(x3) >> 31) ^ 1u) << 24);
                                    *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(a.out) + off) = bytes;
                                } else {  // pslsh/hash.cuh:46
                                    const int4 v = make_int4(static_cast<int32_t>(floorf(x0 + bias.x)),
                                                             static_cast<int32_t>(floorf(x1 + bias.y)),
                                                             static_cast<int32_t>(floorf(x2 + bias.z)),
                                                             static_cast<int32_t>(floorf(x3 + bias.w)));
                                    *reinterpret_cast<int4*>(static_cast<int32_t*>(a.out) + off) = v;
                                    if (FOLD_MM) {
                                        lo.x = min(lo.x, v.x); lo.y = min(lo.y, v.y); lo.z = min(lo.z, v.z); lo.w = min(lo.w, v.w);
                                        hi.x = max(hi.x, v.x); hi.y = max(hi.y, v.y); hi.z = max(hi.z, v.z); hi.w = max(hi.w, v.w);
                                    }
                                }
                            }
                            if (FOLD_MM) {
                                // the 32 lanes of a e_half wave hold 32 rows of the same four columns; eight copies of
                                // the ranges (one per row residue, rows of MM_PITCH words: different banks) keep the
                                // lanes that meet at one word down to four (sixteen copies measured no faster)
                                int32_t* mn = &cmin[(e_r32 & 7) * MM_PITCH + (c0 - ct * BN)];
                                int32_t* mx = &cmax[(e_r32 & 7) * MM_PITCH + (c0 - ct * BN)];
                                atomicMin(mn, lo.x); atomicMin(mn + 1, lo.y); atomicMin(mn + 2, lo.z); atomicMin(mn + 3, lo.w);
                                atomicMax(mx, hi.x); atomicMax(mx + 1, hi.y); atomicMax(mx + 2, hi.z); atomicMax(mx + 3, hi.w);
                            }
                        }
                    } else {
                        int tq = t, hq = h;
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            if (c0 + q < TH) {
                                const float bias = FLOOR ? a.b[c0 + q] : 0.f;
#pragma unroll
                                for (int i = 0; i < 2; ++i) {
                                    const int row = rt * BM + e_wm * 64 + i * 32 + e_r32;
                                    if (row >= n) continue;
                                    const size_t off = (static_cast<size_t>(tq) * n + row) * H + hq;
                                    const float x = acc[i][j][4 * g + q];
                                    if (EPI == EPI_SIGN_BYTES) {
                                        static_cast<uint8_t*>(a.out)[off] =
                                            static_cast<uint8_t>((__float_as_uint(x) >> 31) ^ 1u);
                                    } else {
                                        static_cast<int32_t*>(a.out)[off] = static_cast<int32_t>(floorf(x + bias));
                                    }
                                }
                            }
                            if (++hq == H) { hq = 0; ++tq; }
                        }
                    }
                    h += 8;
                    while (h >= H) { h -= H; ++t; }
                }
            }
        }
        if (!has_next) break;
        rt = rt_next;
    }
    if (FOLD_MM) {  // the tile's ranges into the table's, again only where they would change
        __syncthreads();
        const int c = ct * BN + tid;
        if (tid < BN && c < TH) {
            int32_t lo = INT_MAX, hi = INT_MIN;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                lo = min(lo, cmin[k * MM_PITCH + tid]);
                hi = max(hi, cmax[k * MM_PITCH + tid]);
            }
            if (lo <= hi) {
                if (lo < a.mm[2 * c]) atomicMin(&a.mm[2 * c], lo);
                if (hi > a.mm[2 * c + 1]) atomicMax(&a.mm[2 * c + 1], hi);
            }
        }
    }
}

// ---------------------------------------------------------------- fp64 (MFMA 16x16x4 tiles)
// Same tiling as the fp32 kernel: 128 x 128 outputs per workgroup, 2 x 2 wavefronts of 64 x 64,
// here as 4 x 4 MFMA tiles of 16 x 16 x 4.  Operand lane l supplies A[row l%16][k l/16] and
// B[k l/16][col l%16]; the four lane groups walk four consecutive features each per stage
// pair, so fragments are 16-byte LDS reads.  Accumulator register i of lane l holds
// row 4*i + l/16, column l%16 of its tile.
typedef double f64x4 __attribute__((ext_vector_type(4)));

struct ProjArgs64 {
    const double* X;
    const double* P;
    const double* b;
    void* out;
    int n, d, T, H;
    int n_row_tiles, n_col_tiles;
};

constexpr int DBK = 16;  // features per stage

template <int EPI, bool VEC>
__global__ __launch_bounds__(NTHREADS, 2) void project_f64_kernel(ProjArgs64 a) {
    constexpr int PITCH = DBK + 2;  // LDS row pitch in doubles
    constexpr int D2 = DBK / 2;     // double2 per tile row and stage
    constexpr int NLD = BM * D2 / NTHREADS;
    constexpr int RSTEP = NTHREADS / D2;
    __shared__ __attribute__((aligned(16))) double As[BM * PITCH];
    __shared__ __attribute__((aligned(16))) double Bs[BN * PITCH];
    __shared__ uint32_t tw[(EPI == EPI_SIGN_KEYS) ? BM * (BN / 32) : 1];

    // same workgroup -> (row tile, column tile) arrangement as the fp32 kernel
    const int nct = a.n_col_tiles;
    const int per_group = 8 * nct;
    const int grp = blockIdx.x / per_group, rem = blockIdx.x - grp * per_group;
    const int ct = rem >> 3, slot = rem & 7;
    const int rt = grp * 8 + slot;
    if (rt >= a.n_row_tiles) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r16 = lane & 15, g = lane >> 4;
    const int n = a.n, d = a.d, T = a.T, H = a.H;
    const int TH = T * H;

    const int lrow = tid / D2, c2 = (tid % D2) * 2;
    const double* xbase = a.X + static_cast<size_t>(rt) * BM * d;
    uint32_t xoff[NLD], poff[NLD];
    bool xok[NLD], pok[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int lr = lrow + RSTEP * i;
        xok[i] = rt * BM + lr < n;
        xoff[i] = static_cast<uint32_t>(VEC ? min(lr, n - 1 - rt * BM) : lr) * static_cast<uint32_t>(d);
        const int vc = ct * BN + lr;
        const int prow = (EPI == EPI_SIGN_KEYS) ? sign_vcol_to_prow(vc, T, H) : (vc < TH ? vc : -1);
        pok[i] = prow >= 0;
        poff[i] = static_cast<uint32_t>(prow < 0 ? 0 : prow) * static_cast<uint32_t>(d);
    }
    auto fetch = [&](int k, double2 (&ra)[NLD], double2 (&rb)[NLD]) {
        if (VEC) {
            const int kk = min(k, d - 2);
            const bool inside = k < d;  // a double2 is entirely inside or entirely outside [0, d)
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const double2 va = *reinterpret_cast<const double2*>(xbase + (xoff[i] + static_cast<uint32_t>(kk)));
                const double2 vb = *reinterpret_cast<const double2*>(a.P + (poff[i] + static_cast<uint32_t>(kk)));
                ra[i] = inside ? make_double2(va.x, va.y) : make_double2(0.0, 0.0);
                rb[i] = inside ? make_double2(vb.x, vb.y) : make_double2(0.0, 0.0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                double2 va = make_double2(0.0, 0.0), vb = make_double2(0.0, 0.0);
                if (xok[i]) {
                    if (k < d) va.x = xbase[xoff[i] + k];
                    if (k + 1 < d) va.y = xbase[xoff[i] + k + 1];
                }
                if (pok[i]) {
                    if (k < d) vb.x = a.P[poff[i] + k];
                    if (k + 1 < d) vb.y = a.P[poff[i] + k + 1];
                }
                ra[i] = va;
                rb[i] = vb;
            }
        }
    };

    f64x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.0;

    double2 ra[NLD], rb[NLD];
    fetch(c2, ra, rb);
    const int nk = (d + DBK - 1) / DBK;
    for (int kt = 0; kt < nk; ++kt) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            *reinterpret_cast<double2*>(&As[(lrow + RSTEP * i) * PITCH + c2]) = ra[i];
            *reinterpret_cast<double2*>(&Bs[(lrow + RSTEP * i) * PITCH + c2]) = rb[i];
        }
        __syncthreads();
        if (kt + 1 < nk) fetch((kt + 1) * DBK + c2, ra, rb);
        // lane group g walks features 4g .. 4g+3 of the stage, two at a time
#pragma unroll
        for (int kk = 0; kk < 4; kk += 2) {
            double2 af[4], bf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                af[i] = *reinterpret_cast<const double2*>(&As[(wm * 64 + i * 16 + r16) * PITCH + g * 4 + kk]);
                bf[i] = *reinterpret_cast<const double2*>(&Bs[(wn * 64 + i * 16 + r16) * PITCH + g * 4 + kk]);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[i].x, bf[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[i].y, bf[j].y, acc[i][j], 0, 0, 0);
                }
        }
        __syncthreads();
    }

    if (EPI == EPI_SIGN_KEYS) {
#pragma unroll
        for (int ti = 0; ti < 4; ++ti)
#pragma unroll
            for (int cp = 0; cp < 2; ++cp) {
                int mine = 0;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    // hash bit = 1 iff the sign bit is clear (rplsh/hash.cuh:47; narrowing to float keeps it)
                    const unsigned long long b0 =
                        __builtin_amdgcn_ballot_w64(__double_as_longlong(acc[ti][2 * cp][v]) >= 0);
                    const unsigned long long b1 =
                        __builtin_amdgcn_ballot_w64(__double_as_longlong(acc[ti][2 * cp + 1][v]) >= 0);
#pragma unroll
                    for (int gg = 0; gg < 4; ++gg) {
                        // lanes 16gg..16gg+15 of a ballot are columns 0..15 of row 4v + gg
                        const uint32_t word = static_cast<uint32_t>((b0 >> (16 * gg)) & 0xFFFFull) |
                                              (static_cast<uint32_t>((b1 >> (16 * gg)) & 0xFFFFull) << 16);
                        asm("s_nop 1\n\tv_writelane_b32 %0, %1, %2" : "+v"(mine) : "s"(word), "n"(4 * v + gg));
                    }
                }
                if (lane < 16) tw[(wm * 64 + ti * 16 + lane) * (BN / 32) + (wn * 2 + cp)] = static_cast<uint32_t>(mine);
            }
        __syncthreads();
        uint32_t* keys = static_cast<uint32_t*>(a.out);
        if (H <= 32) {
            const int tpt = 32 / H;
            const uint32_t mask = (H == 32) ? 0xFFFFFFFFu : ((1u << H) - 1u);
            constexpr int TL_STEP = NTHREADS / BM;
            const int row = tid % BM, grow = rt * BM + row;
            int tl = tid / BM;
            int tc = tl / tpt, sub = tl - tc * tpt;
            for (; tl < (BN / 32) * tpt; tl += TL_STEP) {
                const int table = (ct * (BN / 32) + tc) * tpt + sub;
                if (table < T && grow < n) {
                    const uint32_t field = (tw[row * (BN / 32) + tc] >> (sub * H)) & mask;
                    keys[static_cast<size_t>(table) * n + grow] = field << (32 - H);
                }
                sub += TL_STEP;
                while (sub >= tpt) { sub -= tpt; ++tc; }
            }
        } else {
            const int wt = (H + 31) >> 5;
            for (int idx = tid; idx < (BN / 32) * BM; idx += NTHREADS) {
                const int tc = idx / BM, row = idx - tc * BM;
                const int tile = ct * (BN / 32) + tc;
                const int table = tile / wt, w = tile - table * wt;
                const int grow = rt * BM + row;
                if (table < T && grow < n) {
                    const int nbits = min(32, H - 32 * w);
                    const uint32_t mask = (nbits == 32) ? 0xFFFFFFFFu : (0xFFFFFFFFu << (32 - nbits));
                    keys[(static_cast<size_t>(table) * n + grow) * wt + w] = tw[row * (BN / 32) + tc] & mask;
                }
            }
        }
    } else {
#pragma unroll
        for (int ti = 0; ti < 4; ++ti)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = ct * BN + wn * 64 + j * 16 + r16;
                if (col >= TH) continue;
                const int t = col / H, h = col - t * H;
                const double bias = (EPI == EPI_FLOOR_I32) ? a.b[col] : 0.0;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int row = rt * BM + wm * 64 + ti * 16 + 4 * v + g;
                    if (row >= n) continue;
                    const size_t off = (static_cast<size_t>(t) * n + row) * H + h;
                    const double x = acc[ti][j][v];
                    if (EPI == EPI_SIGN_BYTES) {
                        // narrowing to float keeps the sign (rplsh/hash.cuh:47)
                        static_cast<uint8_t*>(a.out)[off] = (__double_as_longlong(x) < 0) ? 0 : 1;
                    } else {
                        static_cast<int32_t*>(a.out)[off] = static_cast<int32_t>(floor(x + bias));
                    }
                }
            }
    }
}

}  // namespace

culsh_status launch_project_f32(culsh_ctx* ctx, const float* X, const float* P, const float* b,
                                int n, int d, int T, int H, ProjEpilogue epi, void* out, int32_t* minmax,
                                bool* minmax_folded) {
    if (minmax_folded) *minmax_folded = false;
    CULSH_REQUIRE(X && P && out, CULSH_ERR_INVALID, "projection: null pointer");
    CULSH_REQUIRE(n > 0 && d > 0 && T > 0 && H > 0, CULSH_ERR_INVALID, "projection: sizes must be positive");
    const bool floor_epi = (epi == EPI_FLOOR_I32);
    CULSH_REQUIRE(!floor_epi || b, CULSH_ERR_INVALID, "projection: bias is required");
    CULSH_REQUIRE(static_cast<long long>(T) * H < (1ll << 30), CULSH_ERR_LIMIT, "T*H too large");
    CULSH_REQUIRE(static_cast<long long>(T) * H * d < (1ll << 32) && static_cast<long long>(BM) * d < (1ll << 31),
                  CULSH_ERR_LIMIT, "projection: T*H*n_features must be below 2^32");
    long long n_vcols;
    if (epi == EPI_SIGN_KEYS) {
        const long long tiles = (H <= 32) ? (T + (32 / H) - 1) / (32 / H)
                                          : static_cast<long long>(T) * ((H + 31) / 32);
        n_vcols = tiles * 32;
    } else {
        n_vcols = static_cast<long long>(T) * H;
    }
    ProjArgs a;
    a.X = X; a.P = P; a.b = b; a.out = out;
    a.n = n; a.d = d; a.T = T; a.H = H;
    a.n_row_tiles = (n + BM - 1) / BM;
    a.n_col_tiles = static_cast<int>((n_vcols + BN - 1) / BN);
    a.vec_x = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(X) % 16 == 0);
    a.vec_p = (d % 4 == 0) && (reinterpret_cast<uintptr_t>(P) % 16 == 0);
    a.mm = minmax;
    const bool fold_mm = floor_epi && minmax && minmax_folded && H % 4 == 0 &&
                         reinterpret_cast<uintptr_t>(out) % 16 == 0 && reinterpret_cast<uintptr_t>(b) % 16 == 0;
    // With one column tile (T * H <= 128) workgroups stay and walk over row tiles (see the kernel): as many
    // as fit on the device at once, in whole groups of 8.  With several column tiles every tile gets a
    // workgroup of its own: the dispatch order then keeps the column tiles of a row tile close in time, which
    // workgroups that each go their own way over hundreds of tiles do not (4M x 768 x 1024: 0.87 of the fp32
    // MFMA peak against 0.83 with resident workgroups; 1M x 128 x 512: no difference; 1M x 128 x 128 with the
    // floor epilogue: 0.55 against 0.59).
    const long long groups = (a.n_row_tiles + 7) / 8;
    const long long per_group = 8ll * a.n_col_tiles;
    const long long resident_groups = std::max(1ll, (static_cast<long long>(ctx->n_cus) * 4) / per_group);
    const long long launched = a.n_col_tiles == 1 ? std::min(groups, resident_groups) : groups;
    CULSH_REQUIRE(launched * per_group < (1ll << 31), CULSH_ERR_LIMIT, "projection grid too large");
    dim3 grid(static_cast<unsigned>(launched * per_group)), block(NTHREADS);
    const bool vec = a.vec_x && a.vec_p;
    // 16 features per stage keep the kernel at 124 registers, i.e. 4 workgroups per CU instead of
    // the 3 that 32 features per stage allow: measured 1.06 ms against 1.14 ms at 1M x 128 x 512
#define PROJ_CASE(E)                                                                                              \
    case E:                                                                                                       \
        if (vec && d % 16 == 0) CULSH_LAUNCH(ctx, (project_f32_kernel<E, true, 16, true>), grid, block, 0, ctx->stream, a); \
        else if (vec) CULSH_LAUNCH(ctx, (project_f32_kernel<E, true, 16, false>), grid, block, 0, ctx->stream, a);         \
        else CULSH_LAUNCH(ctx, (project_f32_kernel<E, false, 16, false>), grid, block, 0, ctx->stream, a);                 \
        break;
    switch (fold_mm ? EPI_FLOOR_I32_MM : static_cast<int>(epi)) {
        PROJ_CASE(EPI_SIGN_KEYS)
        PROJ_CASE(EPI_SIGN_BYTES)
        PROJ_CASE(EPI_FLOOR_I32)
        PROJ_CASE(EPI_FLOOR_I32_MM)
    }
    if (fold_mm) *minmax_folded = true;
#undef PROJ_CASE
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

culsh_status launch_project_f64(culsh_ctx* ctx, const double* X, const double* P, const double* b,
                                int n, int d, int T, int H, ProjEpilogue epi, void* out) {
    CULSH_REQUIRE(X && P && out, CULSH_ERR_INVALID, "projection: null pointer");
    CULSH_REQUIRE(n > 0 && d > 0 && T > 0 && H > 0, CULSH_ERR_INVALID, "projection: sizes must be positive");
    CULSH_REQUIRE(epi != EPI_FLOOR_I32 || b, CULSH_ERR_INVALID, "projection: bias is required");
    CULSH_REQUIRE(static_cast<long long>(T) * H < (1ll << 30), CULSH_ERR_LIMIT, "T*H too large");
    CULSH_REQUIRE(static_cast<long long>(T) * H * d < (1ll << 32) && static_cast<long long>(BM) * d < (1ll << 31),
                  CULSH_ERR_LIMIT, "projection: T*H*n_features must be below 2^32");
    long long n_vcols;
    if (epi == EPI_SIGN_KEYS) {
        const long long tiles = (H <= 32) ? (T + (32 / H) - 1) / (32 / H)
                                          : static_cast<long long>(T) * ((H + 31) / 32);
        n_vcols = tiles * 32;
    } else {
        n_vcols = static_cast<long long>(T) * H;
    }
    ProjArgs64 a;
    a.X = X; a.P = P; a.b = b; a.out = out;
    a.n = n; a.d = d; a.T = T; a.H = H;
    a.n_row_tiles = (n + BM - 1) / BM;
    a.n_col_tiles = static_cast<int>((n_vcols + BN - 1) / BN);
    const bool vec = (d % 2 == 0) && (reinterpret_cast<uintptr_t>(X) % 16 == 0) && (reinterpret_cast<uintptr_t>(P) % 16 == 0);
    const long long groups = (a.n_row_tiles + 7) / 8;
    const long long blocks = groups * 8 * a.n_col_tiles;
    CULSH_REQUIRE(blocks < (1ll << 31), CULSH_ERR_LIMIT, "projection grid too large");
    dim3 grid(static_cast<unsigned>(blocks)), block(NTHREADS);
#define PROJ_CASE64(E)                                                                                  \
    case E:                                                                                             \
        if (vec) CULSH_LAUNCH(ctx, (project_f64_kernel<E, true>), grid, block, 0, ctx->stream, a);      \
        else CULSH_LAUNCH(ctx, (project_f64_kernel<E, false>), grid, block, 0, ctx->stream, a);         \
        break;
    switch (epi) {
        PROJ_CASE64(EPI_SIGN_KEYS)
        PROJ_CASE64(EPI_SIGN_BYTES)
        PROJ_CASE64(EPI_FLOOR_I32)
    }
#undef PROJ_CASE64
    CULSH_LAUNCH_CHECK();
    return CULSH_OK;
}

}  // namespace culsh_amd
