// Forward simulation driver: one fused kernel per step.
//
// Workgroups [0, n_update) each advance 256 elements: read and clear the ring
// slot of this step, run the GLIF3 update, publish the wavefront's spike
// ballot, and -- because every delay is at least one step, so nothing written
// now is read before the next launch -- the wavefront that detected a spike
// walks that neuron's out-going synapses immediately and adds the weights into
// the future ring slots with fp32 atomics.  No compaction pass, no spike list
// round trip through memory.  The remaining workgroups deliver the external
// input events of the step the same way.
#include "common.hpp"
#include "glif3_update.hpp"
#include "propagate.hpp"

namespace bmtk {

constexpr int kInputBlocks = 32;

__global__ __launch_bounds__(kBlock) void sim_step_kernel(bmtk_glif3_sim s, int64_t t, int64_t out_row,
                                                          int n_update)
{
    const int batch = s.batch;
    const int64_t ne = s.n_neurons * (int64_t)batch;
    const int L = s.ring_slots;
    const int slot0 = (int)(t % L);
    const int lane = lane_id();

    if ((int)blockIdx.x >= n_update) {
        // external input events emitted in this step
        const Table inp{s.inp_indptr, s.inp_indices, s.inp_weights, s.inp_delays, s.inp_receptors};
        const int64_t k0 = s.in_ptr[t], k1 = s.in_ptr[t + 1];
        const int n_waves = ((int)gridDim.x - n_update) * (kBlock / kWave);
        const int wave = ((int)blockIdx.x - n_update) * (kBlock / kWave) + threadIdx.x / kWave;
        for (int64_t k = k0 + wave; k < k1; k += n_waves) {
            const int e = s.in_events[k];
            const int j = batch == 1 ? e : (int)((uint32_t)e / (uint32_t)batch);
            deliver_row(inp, j, e - j * batch, batch, s.ring, L, slot0, ne);
        }
        return;
    }

    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    bool spike = false;
    float frac = 0.0f;
    if (e < ne) {
        const int64_t n = batch == 1 ? e : (int64_t)((uint32_t)e / (uint32_t)batch);
        const int64_t col = s.class_id ? (int64_t)s.class_id[n] : n;
        Glif3Prop p;
        p.load(s.prop, s.prop_stride, col);
        Glif3Elem st;
        glif3_load(st, s.V, s.asc, s.y1, s.y2, s.ref, ne, e);
        float *cur = s.ring + (int64_t)slot0 * GLIF3_NREC * ne + e;
        float syn[GLIF3_NREC];
#pragma unroll
        for (int k = 0; k < GLIF3_NREC; ++k) {
            syn[k] = cur[k * ne];
            cur[k * ne] = 0.0f;
        }
        const float I = s.i_ext ? s.i_ext[e] : 0.0f;
        spike = glif3_update(st, p, s.h, syn, I, &frac);
        glif3_store(st, s.V, s.asc, s.y1, s.y2, s.ref, ne, e);
    }
    unsigned long long m = __ballot(spike);
    const int64_t wave_base = e & ~(int64_t)(kWave - 1);
    if (s.spike_bits && lane == 0 && wave_base < ne) s.spike_bits[out_row * s.spike_bits_stride + (e >> 6)] = m;
    if (m == 0ull) return;

    if (s.spike_count) {
        // one counter bump per wavefront, record slots handed out in lane order
        const int leader = __ffsll((long long)m) - 1;
        unsigned long long base = 0ull;
        if (lane == leader) base = atomicAdd(s.spike_count, (unsigned long long)__popcll(m));
        base = bcast_u64(base, leader);
        const unsigned long long idx = base + (unsigned long long)lane_prefix(m);
        if (spike && idx < (unsigned long long)s.spike_cap) {
            s.spike_step[idx] = (int32_t)t;
            s.spike_elem[idx] = (int32_t)e;
            if (s.spike_frac) s.spike_frac[idx] = frac;
        }
    }
    if (s.rec_indptr) {
        const Table rec{s.rec_indptr, s.rec_indices, s.rec_weights, s.rec_delays, s.rec_receptors};
        while (m) {
            const int l = __ffsll((long long)m) - 1;
            m &= m - 1ull;
            const int es = (int)wave_base + l;
            const int j = batch == 1 ? es : (int)((uint32_t)es / (uint32_t)batch);
            deliver_row(rec, j, es - j * batch, batch, s.ring, L, slot0, ne);
        }
    }
}

}  // namespace bmtk

using namespace bmtk;

extern "C" int bmtk_glif3_simulate_fwd(const bmtk_glif3_sim *sim, int64_t step0, int64_t n_steps, void *stream)
{
    BMTK_REQUIRE(sim != nullptr, "glif3_simulate_fwd: sim is null");
    const bmtk_glif3_sim &s = *sim;
    BMTK_REQUIRE(s.n_neurons > 0 && s.batch > 0, "glif3_simulate_fwd: n_neurons and batch must be positive");
    const int64_t ne = s.n_neurons * (int64_t)s.batch;
    BMTK_REQUIRE(ne < (1ll << 31), "glif3_simulate_fwd: n_neurons*batch must stay below 2^31");
    BMTK_REQUIRE(s.ring_slots > 1, "glif3_simulate_fwd: ring_slots must exceed the largest delay (>= 2)");
    BMTK_REQUIRE(s.h > 0.0f, "glif3_simulate_fwd: resolution h must be positive");
    BMTK_REQUIRE(s.V && s.asc && s.y1 && s.y2 && s.ref && s.prop && s.ring,
                 "glif3_simulate_fwd: state, prop and ring pointers must be non-null");
    BMTK_REQUIRE(s.prop_stride > 0 && (s.class_id || s.prop_stride >= s.n_neurons),
                 "glif3_simulate_fwd: prop_stride too small");
    const bool has_rec = s.rec_indptr != nullptr;
    BMTK_REQUIRE(!has_rec || (s.rec_indices && s.rec_weights && s.rec_delays && s.rec_receptors),
                 "glif3_simulate_fwd: recurrent table is incomplete");
    const bool has_inp = s.in_ptr != nullptr;
    BMTK_REQUIRE(!has_inp || (s.in_events && s.inp_indptr && s.inp_indices && s.inp_weights && s.inp_delays &&
                              s.inp_receptors),
                 "glif3_simulate_fwd: input event list or input table is incomplete");
    BMTK_REQUIRE(!s.spike_bits || s.spike_bits_stride >= (ne + 63) / 64,
                 "glif3_simulate_fwd: spike_bits_stride smaller than ceil(ne/64)");
    BMTK_REQUIRE(!s.spike_count || (s.spike_step && s.spike_elem && s.spike_cap > 0),
                 "glif3_simulate_fwd: spike record needs spike_step, spike_elem and a positive spike_cap");
    BMTK_REQUIRE(step0 >= 0 && n_steps >= 0, "glif3_simulate_fwd: step0 and n_steps must be non-negative");
    const int n_update = (int)((ne + kBlock - 1) / kBlock);
    const unsigned grid = (unsigned)(n_update + (has_inp ? kInputBlocks : 0));
    for (int64_t k = 0; k < n_steps; ++k) {
        hipLaunchKernelGGL(sim_step_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, s, step0 + k, k,
                           n_update);
    }
    BMTK_CHECK_LAUNCH("glif3_simulate_fwd");
    return BMTK_OK;
}
