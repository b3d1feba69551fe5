// Wavefront (64 lanes) and workgroup scan / reduce helpers for gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace culsh_amd {

constexpr int WAVE = 64;

template <typename T>
__device__ __forceinline__ T wave_inclusive_sum(T v) {
    const int lane = threadIdx.x & (WAVE - 1);
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
        const T o = __shfl_up(v, d, WAVE);
        if (lane >= d) v += o;
    }
    return v;
}

template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
    for (int d = WAVE / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, WAVE);
    return v;
}

// Inclusive prefix sum over the 64 lanes with DPP row shifts and row broadcasts (VALU only,
// no LDS traffic).  All 64 lanes must be active.
__device__ __forceinline__ uint32_t wave_inclusive_sum_dpp(uint32_t v) {
    int x = static_cast<int>(v);
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false);  // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false);  // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false);  // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false);  // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
    return static_cast<uint32_t>(x);
}

// Sum over the 64 lanes, in every lane, without LDS traffic (DPP scan, then the last lane's value).
__device__ __forceinline__ uint32_t wave_sum_dpp(uint32_t v) {
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(wave_inclusive_sum_dpp(v)), 63));
}

// Exclusive prefix sum over the workgroup (blockDim.x a multiple of 64, at most 1024).
// `scratch` holds 17 words of type T in LDS.  Returns this thread's exclusive prefix and
// stores the workgroup total in *total.  Contains three barriers; all threads must call it.
template <typename T>
__device__ __forceinline__ T block_exclusive_sum(T v, T* scratch, T* total) {
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x >> 6;
    const int nwaves = (blockDim.x + WAVE - 1) >> 6;
    const T incl = wave_inclusive_sum(v);
    if (lane == WAVE - 1) scratch[wave] = incl;
    __syncthreads();
    if (wave == 0) {
        T w = (lane < nwaves) ? scratch[lane] : T(0);
        const T wi = wave_inclusive_sum(w);
        if (lane < nwaves) scratch[lane] = wi - w;  // exclusive wave offsets
        if (lane == nwaves - 1) scratch[16] = wi;   // total
    }
    __syncthreads();
    const T res = scratch[wave] + incl - v;
    *total = scratch[16];
    __syncthreads();  // scratch may be reused by the next call
    return res;
}

}  // namespace culsh_amd
