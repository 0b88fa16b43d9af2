// Shared helpers of the HIP sources: error reporting, wavefront primitives.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/bmtk_amd.h"

namespace bmtk {

constexpr int kWave = 64;    // gfx950 wavefront
constexpr int kBlock = 256;  // 4 wavefronts per workgroup

void set_error(const char *fmt, ...);

#define BMTK_REQUIRE(cond, ...)            \
    do {                                   \
        if (!(cond)) {                     \
            bmtk::set_error(__VA_ARGS__);  \
            return BMTK_E_ARG;             \
        }                                  \
    } while (0)

#define BMTK_CHECK_LAUNCH(name)                                                        \
    do {                                                                               \
        hipError_t err__ = hipGetLastError();                                          \
        if (err__ != hipSuccess) {                                                     \
            bmtk::set_error("%s: launch failed: %s", name, hipGetErrorString(err__)); \
            return BMTK_E_LAUNCH;                                                      \
        }                                                                              \
    } while (0)

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// number of set bits of `mask` below this lane
__device__ __forceinline__ int lane_prefix(unsigned long long mask)
{
    return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
}

// value of `v` in lane `src`; `src` must be the same in every lane
__device__ __forceinline__ int bcast_i(int v, int src) { return __builtin_amdgcn_readlane(v, src); }
__device__ __forceinline__ float bcast_f(float v, int src)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
__device__ __forceinline__ unsigned long long bcast_u64(unsigned long long v, int src)
{
    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)v, src);
    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(v >> 32), src);
    return ((unsigned long long)hi << 32) | lo;
}

// inclusive prefix sum over the 64 lanes
__device__ __forceinline__ unsigned wave_inclusive_scan(unsigned v)
{
    const int lane = lane_id();
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const unsigned o = __shfl_up(v, off, kWave);
        if (lane >= off) v += o;
    }
    return v;
}

// exclusive prefix sum over the 256 threads of a workgroup; *total gets the block sum
__device__ __forceinline__ unsigned block_exclusive_scan(unsigned v, unsigned *total)
{
    __shared__ unsigned wave_sum[kBlock / kWave];
    const unsigned inc = wave_inclusive_scan(v);
    const int wave = threadIdx.x / kWave;
    if (lane_id() == kWave - 1) wave_sum[wave] = inc;
    __syncthreads();
    unsigned base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) {
        const unsigned s = wave_sum[w];
        if (w < wave) base += s;
        tot += s;
    }
    __syncthreads();
    *total = tot;
    return base + inc - v;
}

}  // namespace bmtk
