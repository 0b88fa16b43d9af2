// Synapse-table view and the row walk shared by the scatter kernel and the
// fused simulation kernels.
#pragma once

#include "common.hpp"

namespace bmtk {

struct Table {
    const int32_t *indptr, *indices;
    const float *weights;
    const uint8_t *delays, *receptors;
};

// deliver row j of `t` for trial b; all 64 lanes of the wavefront take part
__device__ __forceinline__ void deliver_row(const Table &t, int j, int b, int batch, float *__restrict__ ring,
                                            int L, int slot0, int64_t ne)
{
    const int p0 = t.indptr[j], p1 = t.indptr[j + 1];
    for (int p = p0 + lane_id(); p < p1; p += kWave) {
        const int i = t.indices[p];
        const float w = t.weights[p];
        int slot = slot0 + (int)t.delays[p];
        slot = slot >= L ? slot - L : slot;
        const int r = t.receptors[p];
        atomicAdd(ring + ((int64_t)(slot * GLIF3_NREC + r) * ne + (int64_t)i * batch + b), w);
    }
}

// spike bits of source `src` in trials tile0 .. tile0+width-1 (width <= 64) as a lane mask: bit b = trial tile0+b.
// Reads one or two words of a spike-bit row; rows carry a padding word so that the second read stays inside.
__device__ __forceinline__ unsigned long long source_mask(const uint64_t *__restrict__ zbits, int src, int batch,
                                                          int tile0, int width)
{
    const int64_t bit = (int64_t)src * batch + tile0;
    const int64_t w = bit >> 6;
    const int sh = (int)(bit & 63);
    unsigned long long m = zbits[w] >> sh;
    if (sh + width > 64) m |= zbits[w + 1] << (64 - sh);
    if (width < 64) m &= (1ull << width) - 1ull;
    return m;
}

}  // namespace bmtk
