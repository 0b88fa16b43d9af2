// What the two pull-form kernels share (the stand-alone propagation of propagate_pull.hip and the fused batched
// driver of simulate_fused.hip): exact sums in 64-bit fixed point and the stream of row blocks a wavefront owns.
#pragma once

#include "common.hpp"

namespace bmtk {

// fp32 -> Q31.32 two's complement.  The size |w| is split with floor(): the integer part, and what is left, which
// lies in [0, 1) and is exact (for a negative w, w - floor(w) = w + 1 would round); times 2^32 it is an integer
// below 2^32 up to the bits under 2^-32, which the conversion drops.  The sign is applied to the integer.
__device__ __forceinline__ unsigned long long to_fixed(float w)
{
    const float size = fabsf(w);
    const float whole = floorf(size);
    const unsigned lo = (unsigned)((size - whole) * 4294967296.0f);
    const unsigned long long v = ((unsigned long long)(unsigned)whole << 32) | lo;
    return w < 0.0f ? 0ull - v : v;
}

__device__ __forceinline__ float from_fixed(unsigned long long v)
{
    return (float)((double)(long long)v * (1.0 / 4294967296.0));
}

// One block of a row's synapse stream: positions [base, min(base + kPullChunks*64, p1)) of the packed table.
constexpr int kPullChunks = 4;  // 64-synapse chunks per block
struct PullBlock {
    int64_t row;  // >= n_tgt: past the end
    int base, p1;
    bool last;    // last block of its row: the sums are stored after it
    bool first;   // first block of its row
    int col;      // the row's column of a per-row table (PullCursor::classes), or the row itself
};

// The rows a wavefront owns (first, first + stride, ...) as a stream of blocks.  The bounds of the row after the
// current one are fetched a row ahead.  Everything here is the same in all lanes (scalar registers and loads).
struct PullCursor {
    const int32_t *__restrict__ indptr;
    int64_t n_tgt, stride, row;
    int q, p1, np0, np1;
    bool at_start;
    const int32_t *__restrict__ classes;  // optional: a column index per row, fetched a row ahead like the bounds
    int col, ncol;

    __device__ __forceinline__ void start(const int32_t *ip, int64_t n, int64_t first, int64_t step,
                                          const int32_t *cls = nullptr)
    {
        classes = cls;
        col = ncol = 0;
        indptr = ip;
        n_tgt = n;
        stride = step;
        row = first;
        q = p1 = np0 = np1 = 0;
        at_start = true;
        if (row < n_tgt) {
            q = indptr[row];
            p1 = indptr[row + 1];
            col = classes ? classes[row] : (int)row;
        }
        if (row + stride < n_tgt) {
            np0 = indptr[row + stride];
            np1 = indptr[row + stride + 1];
            ncol = classes ? classes[row + stride] : (int)(row + stride);
        }
    }
    __device__ __forceinline__ PullBlock next()
    {
        if (row >= n_tgt) return PullBlock{row, 0, 0, false, false, 0};  // past the end: an empty block of no row
        PullBlock b{row, q, p1, false, at_start, col};
        at_start = false;
        {
            q += kPullChunks * kWave;
            if (q >= p1) {
                b.last = true;
                at_start = true;
                row += stride;
                q = np0;
                p1 = np1;
                col = ncol;
                if (row + stride < n_tgt) {
                    np0 = indptr[row + stride];
                    np1 = indptr[row + stride + 1];
                    ncol = classes ? classes[row + stride] : (int)(row + stride);
                }
            }
        }
        return b;
    }
};

}  // namespace bmtk
