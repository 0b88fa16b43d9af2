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

// walk one row of a packed table, four 64-synapse chunks in flight at a time
__device__ __forceinline__ void deliver_row_packed(const int32_t *__restrict__ indptr,
                                                   const bmtk_synapse *__restrict__ syn, int j, int b, int batch,
                                                   float *__restrict__ ring, int L, int slot0, int64_t ne,
                                                   int idx_bits)
{
    const unsigned idx_mask = (1u << idx_bits) - 1u;
    const int p0 = indptr[j], p1 = indptr[j + 1];
    if (p1 <= p0) return;
    const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(syn);
    for (int base = p0 + lane_id(); base < p1; base += 4 * kWave) {
        uint2 s[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) s[u] = rows[min(base + u * kWave, p1 - 1)];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (base + u * kWave < p1) {
                const unsigned tdr = s[u].x;
                int slot = slot0 + (int)(tdr >> (idx_bits + 2));
                slot = slot >= L ? slot - L : slot;
                const int r = (tdr >> idx_bits) & 3;
                const int64_t i = tdr & idx_mask;
                atomicAdd(ring + ((int64_t)(slot * GLIF3_NREC + r) * ne + i * batch + b), __uint_as_float(s[u].y));
            }
        }
    }
}

}  // namespace bmtk
