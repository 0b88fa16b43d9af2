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

// 24-bit multiplies (full rate; the compiler turns __umul24 with a uniform operand into the quarter-rate 32-bit
// multiply).  Only bits 0-23 of a and b count.
__device__ __forceinline__ unsigned mul_u24(unsigned a, unsigned b)
{
    unsigned r;
    asm("v_mul_u32_u24 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ unsigned mad_u24(unsigned a, unsigned b, unsigned c)
{
    unsigned r;
    asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// inclusive prefix sum over the 64 lanes, with data-parallel-primitive moves (no LDS round trips): sums of 4
// by three one-lane shifts within a row of 16, then shifts by 4 and 8 confined to the lanes that have such a
// neighbour, then the last lane of row 0 (2) is added to row 1 (3) and lane 31 to the upper half
#define BMTK_DPP(src, ctrl, row_mask, bank_mask, bound) \
    ((unsigned)__builtin_amdgcn_update_dpp(0, (int)(src), (ctrl), (row_mask), (bank_mask), (bound)))
__device__ __forceinline__ unsigned wave_inclusive_scan(unsigned v)
{
    // lanes without a source read 0 (bound_ctrl), which lets the compiler fold each move into its addition
    unsigned t = v + BMTK_DPP(v, 0x111, 0xF, 0xF, true);  // row_shr:1
    t += BMTK_DPP(v, 0x112, 0xF, 0xF, true);              // row_shr:2
    t += BMTK_DPP(v, 0x113, 0xF, 0xF, true);              // row_shr:3
    t += BMTK_DPP(t, 0x114, 0xF, 0xE, false);             // row_shr:4, lanes 4..15 of each row
    t += BMTK_DPP(t, 0x118, 0xF, 0xC, false);             // row_shr:8, lanes 8..15
    t += BMTK_DPP(t, 0x142, 0xA, 0xF, false);             // row_bcast:15 into rows 1 and 3
    t += BMTK_DPP(t, 0x143, 0xC, 0xF, false);             // row_bcast:31 into rows 2 and 3
    return t;
}
#undef BMTK_DPP

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
