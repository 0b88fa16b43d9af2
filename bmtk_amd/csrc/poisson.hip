// Poisson spike sources generated on the device: the homogeneous case of bmtk's
// PoissonSpikeGenerator._build_fixed_fr (bmtk/utils/reports/spike_trains/spike_trains.py:166-206) without
// refractory thinning -- per source, starting at t_start, t += -ln(1 - U) / rate until t > t_stop, every t a
// spike -- with one independent counter-based random stream per (source, trial) instead of NumPy's one global
// stream, so that every source is a thread.  The spikes come out as (emitting step, element id) keys, which the
// host side sorts into the per-step event lists the simulation reads; nothing passes through host memory.
#include <math.h>

#include "common.hpp"

namespace bmtk {

// Philox4x32-10 (Salmon et al., SC'11): counter (c0..c3), key (k0, k1) -> four random words
struct Philox {
    uint32_t c[4];
    __device__ __forceinline__ void round(uint32_t k0, uint32_t k1)
    {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c[0], p1 = (uint64_t)0xCD9E8D57u * c[2];
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
        c[1] = (uint32_t)p1;
        c[3] = (uint32_t)p0;
        c[0] = n0;
        c[2] = n2;
    }
    __device__ __forceinline__ void run(uint32_t k0, uint32_t k1)
    {
#pragma unroll
        for (int i = 0; i < 10; ++i) {
            round(k0, k1);
            k0 += 0x9E3779B9u;
            k1 += 0xBB67AE85u;
        }
    }
};

// the draw number `k` of element `id` under `seed`: uniform in [0, 1) with 53 random bits
__device__ __forceinline__ double poisson_uniform(uint64_t seed, uint64_t id, uint32_t k)
{
    Philox p;
    p.c[0] = (uint32_t)id;
    p.c[1] = (uint32_t)(id >> 32);
    p.c[2] = k;
    p.c[3] = 0x504F4953u;  // stream tag
    p.run((uint32_t)seed, (uint32_t)(seed >> 32));
    const uint64_t bits = ((uint64_t)(p.c[0] >> 5) << 26) | (uint64_t)(p.c[1] >> 6);
    return (double)bits * (1.0 / 9007199254740992.0);
}

struct PoissonArgs {
    int64_t n_ids;
    int32_t batch;
    const float *rate_hz;  // [n_ids / batch]
    double t_start_s, t_stop_s, dt_ms;
    int64_t n_steps;
    uint64_t seed;
};

// Walk the spike train of element `id`; emit(k, step, t_ms) for every spike whose emitting step lies inside the
// run.  A spike at time t gets the stamp ceil(t / dt) steps (at least 1) and is emitted in step stamp - 1, which
// is how spike times are binned for the simulation elsewhere in this package.
template <class Emit>
__device__ __forceinline__ int poisson_walk(const PoissonArgs &a, int64_t id, Emit emit)
{
    const double rate = (double)a.rate_hz[a.batch == 1 ? id : id / a.batch];
    if (!(rate > 0.0)) return 0;
    double t = a.t_start_s;
    int n = 0;
    for (uint32_t k = 0; k < 0x7fffffffu; ++k) {
        t += -log1p(-poisson_uniform(a.seed, (uint64_t)id, k)) / rate;
        if (t > a.t_stop_s) break;
        const double t_ms = t * 1000.0;
        int64_t stamp = (int64_t)ceil(t_ms / a.dt_ms - 1e-6);
        stamp = stamp < 1 ? 1 : stamp;
        if (stamp - 1 >= a.n_steps) break;  // times only grow
        emit(n, stamp - 1, t_ms);
        ++n;
    }
    return n;
}

__global__ __launch_bounds__(kBlock) void poisson_count_kernel(PoissonArgs a, int32_t *__restrict__ counts)
{
    const int64_t id = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (id >= a.n_ids) return;
    counts[id] = poisson_walk(a, id, [](int, int64_t, double) {});
}

__global__ __launch_bounds__(kBlock) void poisson_fill_kernel(PoissonArgs a, const int64_t *__restrict__ offsets,
                                                              int64_t *__restrict__ keys, double *__restrict__ times_ms)
{
    const int64_t id = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (id >= a.n_ids) return;
    const int64_t at = offsets[id];
    poisson_walk(a, id, [&](int k, int64_t step, double t_ms) {
        keys[at + k] = step * a.n_ids + id;
        if (times_ms) times_ms[at + k] = t_ms;
    });
}

}  // namespace bmtk

using namespace bmtk;

static int poisson_args(PoissonArgs &a, int64_t n_sources, int32_t batch, const float *rate_hz, double t_start_ms,
                        double t_stop_ms, double dt_ms, int64_t n_steps, uint64_t seed)
{
    BMTK_REQUIRE(n_sources > 0 && batch > 0 && rate_hz, "poisson: sources, batch and rates are needed");
    BMTK_REQUIRE(n_sources * (int64_t)batch < (1ll << 31), "poisson: n_sources*batch must stay below 2^31");
    BMTK_REQUIRE(t_start_ms >= 0.0 && t_stop_ms > t_start_ms, "poisson: Invalid start and stop times.");
    BMTK_REQUIRE(dt_ms > 0.0 && n_steps > 0 && n_steps < (1ll << 31), "poisson: bad resolution or number of steps");
    a = PoissonArgs{n_sources * (int64_t)batch, batch, rate_hz, t_start_ms * 1e-3, t_stop_ms * 1e-3, dt_ms, n_steps, seed};
    return BMTK_OK;
}

extern "C" int bmtk_poisson_count(int64_t n_sources, int32_t batch, const float *rate_hz, double t_start_ms,
                                  double t_stop_ms, double dt_ms, int64_t n_steps, uint64_t seed, int32_t *counts,
                                  void *stream)
{
    PoissonArgs a;
    const int rc = poisson_args(a, n_sources, batch, rate_hz, t_start_ms, t_stop_ms, dt_ms, n_steps, seed);
    if (rc != BMTK_OK) return rc;
    BMTK_REQUIRE(counts, "poisson_count: counts is null");
    hipLaunchKernelGGL(poisson_count_kernel, dim3((unsigned)((a.n_ids + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, a, counts);
    BMTK_CHECK_LAUNCH("poisson_count");
    return BMTK_OK;
}

extern "C" int bmtk_poisson_fill(int64_t n_sources, int32_t batch, const float *rate_hz, double t_start_ms,
                                 double t_stop_ms, double dt_ms, int64_t n_steps, uint64_t seed, const int64_t *offsets,
                                 int64_t *keys, double *times_ms, void *stream)
{
    PoissonArgs a;
    const int rc = poisson_args(a, n_sources, batch, rate_hz, t_start_ms, t_stop_ms, dt_ms, n_steps, seed);
    if (rc != BMTK_OK) return rc;
    BMTK_REQUIRE(offsets && keys, "poisson_fill: offsets and keys must be non-null");
    hipLaunchKernelGGL(poisson_fill_kernel, dim3((unsigned)((a.n_ids + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, a, offsets, keys, times_ms);
    BMTK_CHECK_LAUNCH("poisson_fill");
    return BMTK_OK;
}
