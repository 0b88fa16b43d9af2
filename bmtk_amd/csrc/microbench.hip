// Three small measurements the design of the simulation kernels rests on, kept in the library so that they can be
// repeated (bench.py --kernels lds): what an addition into LDS costs in its different forms, how long a word
// takes from one workgroup to another through device memory, and how many scattered fp32 atomic additions into
// device memory the chip works off per second.
#include "common.hpp"

namespace bmtk {

constexpr int kUbCells = 23040;  // the resident kernel's ring slice: 6 slots x 4 receptors x 960 elements
constexpr int kUbThreads = 1024;

// Every round, `active` lanes of every wavefront add to a pseudo-random cell of a block-shared LDS array.
// kOp 0: float atomic add; 1: 32-bit integer atomic add; 2: 64-bit integer atomic add (half as many cells);
// 3: float add by a compare-and-swap loop; 4: plain store.
template <int kOp>
__global__ __launch_bounds__(kUbThreads) void lds_add_kernel(float *out, int rounds, int active, uint32_t seed)
{
    extern __shared__ float cells[];
    for (int i = threadIdx.x; i < kUbCells; i += kUbThreads) cells[i] = 0.0f;
    __syncthreads();
    uint64_t x = ((uint64_t)blockIdx.x * kUbThreads + threadIdx.x + seed) * 0x9E3779B97F4A7C15ull;
    const bool on = lane_id() < active;
    for (int r = 0; r < rounds; ++r) {
        x ^= x >> 29;
        x *= 0xBF58476D1CE4E5B9ull;
        x ^= x >> 32;
        const int key = (int)((x >> 8) % (kOp == 2 ? kUbCells / 2 : kUbCells));
        const float w = (float)(key & 7) * 0.25f + 0.25f;
        if (!on) continue;
        if (kOp == 0) {
            atomicAdd(cells + key, w);
        } else if (kOp == 1) {
            atomicAdd(reinterpret_cast<unsigned *>(cells) + key, (unsigned)(key & 7) + 1u);
        } else if (kOp == 2) {
            atomicAdd(reinterpret_cast<unsigned long long *>(cells) + key, (unsigned long long)(key & 7) + 1ull);
        } else if (kOp == 3) {
            unsigned *cell = reinterpret_cast<unsigned *>(cells) + key;
            unsigned old = *reinterpret_cast<volatile unsigned *>(cell);
            while (true) {
                const unsigned seen = atomicCAS(cell, old, __float_as_uint(__uint_as_float(old) + w));
                if (seen == old) break;
                old = seen;
            }
        } else {
            cells[key] = w;
        }
    }
    __syncthreads();
    float s = 0.0f;
    for (int i = threadIdx.x; i < kUbCells; i += kUbThreads) s += cells[i];
    out[(size_t)blockIdx.x * kUbThreads + threadIdx.x] = s;
}

__device__ __forceinline__ unsigned xcc_id()
{
    unsigned v;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
    return v & 0xFu;
}

// Workgroups `a` and `b` of the grid pass a counter back and forth, `rounds` times, through two words of device
// memory 256 bytes apart, with relaxed agent-scope loads and stores (what the resident kernel's grid barrier uses).
// Every wait is a bounded spin: when one runs out the workgroup notes it in xcc[2] and leaves, and the other one's
// wait runs out in turn.  xcc[0], xcc[1]: the XCD each ran on.
__global__ void hop_kernel(unsigned *flag, unsigned *xcc, int a, int b, int rounds, unsigned limit)
{
    const int me = blockIdx.x == (unsigned)a ? 0 : blockIdx.x == (unsigned)b ? 1 : -1;
    if (me < 0 || threadIdx.x != 0) return;
    xcc[me] = xcc_id();
    unsigned *mine = flag + me * 64, *other = flag + (1 - me) * 64;
    for (int k = 1; k <= rounds; ++k) {
        if (me == 0) __hip_atomic_store(mine, (unsigned)k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned spins = 0;
        while (__hip_atomic_load(other, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < (unsigned)k) {
            if (++spins > limit) {
                xcc[2] = 1;
                return;
            }
        }
        if (me == 1) __hip_atomic_store(mine, (unsigned)k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Every thread adds 1 to `per_thread` pseudo-random cells of a region of device memory with the global fp32 atomic
// (what the event-driven propagation does per synaptic event).  own_eighth: a workgroup's cells all lie in the eighth
// of the region that belongs to the XCD it runs on (read from the hardware register), so that no cache line is
// ever touched from two XCDs.
__global__ __launch_bounds__(kBlock) void atomic_add_kernel(float *cells, unsigned n_cells, int per_thread, int own_eighth)
{
    const unsigned part = n_cells >> 3;
    const unsigned base = own_eighth ? (xcc_id() & 7u) * part : 0u, range = own_eighth ? part : n_cells;
    unsigned x = (blockIdx.x * kBlock + threadIdx.x) * 2654435761u + 12345u;
    for (int k = 0; k < per_thread; ++k) {
        x = x * 1664525u + 1013904223u;
        atomicAdd(cells + base + (x >> 8) % range, 1.0f);
    }
}

}  // namespace bmtk

using namespace bmtk;

extern "C" int bmtk_microbench_atomics(float *cells, int64_t n_cells, int32_t per_thread, int32_t n_blocks,
                                       int32_t own_eighth, void *stream)
{
    BMTK_REQUIRE(cells && n_cells >= 8 && n_cells < (1ll << 32) && per_thread >= 1 && n_blocks >= 1,
                 "microbench_atomics: cells non-null, 8 <= n_cells < 2^32, per_thread and n_blocks positive");
    hipLaunchKernelGGL(atomic_add_kernel, dim3((unsigned)n_blocks), dim3(kBlock), 0, (hipStream_t)stream, cells,
                       (unsigned)n_cells, per_thread, own_eighth);
    BMTK_CHECK_LAUNCH("microbench_atomics");
    return BMTK_OK;
}

extern "C" int bmtk_microbench_lds(int32_t op, int32_t active_lanes, int32_t rounds, int32_t n_blocks, float *out,
                                   void *stream)
{
    BMTK_REQUIRE(op >= 0 && op <= 4 && active_lanes >= 1 && active_lanes <= kWave && rounds >= 1 && n_blocks >= 1 && out,
                 "microbench_lds: op 0..4, active_lanes 1..64, rounds and n_blocks positive, out non-null");
    const void *kernels[5] = {reinterpret_cast<const void *>(lds_add_kernel<0>), reinterpret_cast<const void *>(lds_add_kernel<1>),
                              reinterpret_cast<const void *>(lds_add_kernel<2>), reinterpret_cast<const void *>(lds_add_kernel<3>),
                              reinterpret_cast<const void *>(lds_add_kernel<4>)};
    const size_t lds = (size_t)kUbCells * sizeof(float);
    hipError_t err = hipFuncSetAttribute(kernels[op], hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) {
        set_error("microbench_lds: cannot reserve LDS: %s", hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    int r = rounds, act = active_lanes;
    uint32_t seed = 1u;
    void *params[] = {&out, &r, &act, &seed};
    err = hipLaunchKernel(kernels[op], dim3((unsigned)n_blocks), dim3(kUbThreads), params, lds, (hipStream_t)stream);
    if (err != hipSuccess) {
        set_error("microbench_lds: launch failed: %s", hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    return BMTK_OK;
}

extern "C" int bmtk_microbench_hop(uint32_t *flags, uint32_t *xcc, int32_t block_a, int32_t block_b, int32_t rounds,
                                   uint32_t spin_limit, void *stream)
{
    BMTK_REQUIRE(flags && xcc && block_a >= 0 && block_b >= 0 && block_a != block_b && block_a < 16 && block_b < 16 &&
                     rounds >= 1 && spin_limit >= 1,
                 "microbench_hop: flags and xcc non-null, two different workgroups of 0..15, rounds and spin_limit positive");
    hipLaunchKernelGGL(hop_kernel, dim3(16), dim3(kWave), 0, (hipStream_t)stream, flags, xcc, block_a, block_b, rounds,
                       spin_limit);
    BMTK_CHECK_LAUNCH("microbench_hop");
    return BMTK_OK;
}
