// Forward simulation driver: one launch per step, update and delivery overlapped.
//
// Launch for step t, three kinds of workgroups side by side:
//   update   advance 1024 elements: fold the arrivals of ring slot t-1 into y1
//            (and clear the slot), run the GLIF3 update, publish the
//            wavefront's spike ballot;
//   deliver  read the spike ballots of step t-1 and walk the out-going
//            synapses of every neuron that fired, adding the weights into the
//            ring slots t..t+D-1 with fp32 atomics;
//   input    the same for the external events emitted in step t-1.
// With a delay offset B the tables hold delays shortened by B steps and the
// deliver/input workgroups of launch t take the spikes and events of step
// t-1-B from the history instead: same arrival slots, a ring B slots shorter.
//
// Folding arrivals one launch late is exact: NEST adds the weights that arrive
// in step t to y1 at the end of step t (y1 = y1*P11 + s*psc0) and nothing reads
// y1 before the update of step t+1, so storing y1*P11 and adding s*psc0 at the
// top of the next update performs the same two rounded operations.  It buys a
// launch of slack: slot t must be complete when launch t+1 starts, not when
// launch t starts, so the delivery of step t-1 runs concurrently with the
// update of step t instead of after it.
#include "common.hpp"
#include "glif3_update.hpp"
#include "propagate.hpp"
#include "sim_internal.hpp"

namespace bmtk {

constexpr int kSimBlock = 512;
constexpr int kSimWaves = kSimBlock / kWave;
constexpr int kLdsTableBytes = 48 * 1024;

struct SimLaunch {
    int64_t t;        // step being updated (closing launch: one past the last step)
    int64_t src;      // step whose spikes and input events are delivered: t - 1 - delay_offset
    int hist;         // rows of the spike-bit history
    int64_t out_row;  // row of spike_bits to write
    int n_update, n_deliver, n_input;
    int do_update;     // 0 in the closing launch: fold only
    int fold_prev;     // slot t-1 holds arrivals not yet folded into y1
    int deliver_prev;  // work_bits buffer (t-1)%3 holds spikes not yet delivered
    int lds_table;     // propagator table staged in LDS
    int pull;          // pull_syn holds the recurrent arrivals of step t-1, to be folded with slot t-1
    int pull_inp;      // pull_inp_syn holds the input arrivals of step t-1
    int repeats;       // the input workgroups deliver the repeat lists (in_repeat_*) instead of the event lists
    int idx_bits;      // width of the index field of the packed tables (24 in the standard packing)
    int64_t probe_row; // row of probe_v this step's potentials go to, -1: not a sampled step
};

__global__ __launch_bounds__(kSimBlock) void sim_step_kernel(bmtk_glif3_sim s, SimLaunch q)
{
    extern __shared__ __align__(16) float table[];  // [GLIF3_NPROP][class] when q.lds_table
    const int batch = s.batch;
    const int64_t ne = s.n_neurons * (int64_t)batch;
    const int64_t words = (ne + 63) >> 6;
    const int L = s.ring_slots;
    const int lane = lane_id();
    const int bid = (int)blockIdx.x;

    // Delivery workgroups take the lowest block ids so they are dispatched first and
    // their dependent-load chains run under the streaming update, not after it.
    if (bid < q.n_input) {
        // ---- external input events emitted in step t-1 (t-1-B with a delay offset B) ----
        // (not those of step t: with L = largest delay + 1 slots, a delay of L-1
        //  from step t would land in slot t-1, which this launch is clearing)
        const int slot0 = (int)((q.t - 1) % L);
        const int64_t *__restrict__ ptr = q.repeats ? s.in_repeat_ptr : s.in_ptr;
        const int32_t *__restrict__ events = q.repeats ? s.in_repeat_events : s.in_events;
        const int64_t k0 = ptr[q.src], k1 = ptr[q.src + 1];
        const int n_waves = q.n_input * kSimWaves;
        const int wave = bid * kSimWaves + threadIdx.x / kWave;
        for (int64_t k = k0 + wave; k < k1; k += n_waves) {
            const int e = events[k];
            const int j = batch == 1 ? e : (int)((uint32_t)e / (uint32_t)batch);
            deliver_row_packed(s.inp_indptr, s.inp_packed, j, e - j * batch, batch, s.ring, L, slot0, ne, q.idx_bits);
        }
        return;
    }

    if (bid < q.n_input + q.n_deliver) {
        // ---- spikes of step t-1 ----
        if (!q.deliver_prev) return;
        const int slot0 = (int)((q.t - 1) % L);
        const uint64_t *__restrict__ bits = s.work_bits + (q.src % q.hist) * (words + 1);
        const int64_t n_waves = (int64_t)q.n_deliver * kSimWaves;
        const int64_t wave = (int64_t)(bid - q.n_input) * kSimWaves + threadIdx.x / kWave;
        const int64_t per = (words + n_waves - 1) / n_waves;
        const int64_t w_end = min(words, (wave + 1) * per);
        for (int64_t w0 = wave * per; w0 < w_end; w0 += kWave) {
            const int64_t w = w0 + lane;
            unsigned long long v = w < w_end ? bits[w] : 0ull;
            unsigned long long act = __ballot(v != 0ull);
            while (act) {
                const int l = __ffsll((long long)act) - 1;
                act &= act - 1ull;
                unsigned long long vl = bcast_u64(v, l);
                const int64_t e0 = (w0 + l) << 6;
                while (vl) {
                    const int bit = __ffsll((long long)vl) - 1;
                    vl &= vl - 1ull;
                    const int es = (int)(e0 + bit);
                    const int j = batch == 1 ? es : (int)((uint32_t)es / (uint32_t)batch);
                    deliver_row_packed(s.rec_indptr, s.rec_packed, j, es - j * batch, batch, s.ring, L, slot0, ne, q.idx_bits);
                }
            }
        }
        return;
    }

    // ---- update (or, in the closing launch, fold only) ----
    // What an element reads from device memory -- its state, slot t-1 of the ring with the pulled sums, its current,
    // its class -- is asked for first; the class table is copied into LDS while those loads are on their way.
    const int n_cols = (int)s.prop_stride;
    const int64_t e = (int64_t)(bid - q.n_input - q.n_deliver) * kSimBlock + threadIdx.x;
    bool spike = false;
    float frac = 0.0f;
    const bool live = e < ne;
    float *prev = s.ring + (int64_t)((q.t + L - 1) % L) * GLIF3_NREC * ne + (live ? e : 0);
    int64_t col = 0;
    float arrived[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
    float I = 0.0f;
    Glif3Elem st;
    if (live) {
        const int64_t n = batch == 1 ? e : (int64_t)((uint32_t)e / (uint32_t)batch);
        col = s.class_id ? (int64_t)s.class_id[n] : n;
        if (q.fold_prev) {
#pragma unroll
            for (int k = 0; k < GLIF3_NREC; ++k) {
                float a = prev[k * ne];
                if (q.pull) a = a + s.pull_syn[k * ne + e];
                if (q.pull_inp) a = a + s.pull_inp_syn[k * ne + e];
                arrived[k] = a;
            }
        }
        if (q.do_update) {
            glif3_load(st, s.V, s.asc, s.y1, s.y2, s.ref, ne, e);
            I = s.i_ext ? s.i_ext[e] : 0.0f;
        }
    }
    if (q.lds_table) {
        stage_class_table<kSimBlock>(table, s.prop, n_cols * GLIF3_NPROP);
        __syncthreads();
    }
    if (live) {
        if (!q.do_update) {
            if (q.fold_prev) {
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) {
                    const float psc0 = q.lds_table ? table[(GLIF3_PSC0_0 + k) * n_cols + col]
                                                   : s.prop[(GLIF3_PSC0_0 + k) * s.prop_stride + col];
                    prev[k * ne] = 0.0f;
                    s.y1[k * ne + e] = s.y1[k * ne + e] + arrived[k] * psc0;
                }
            }
        } else {
            Glif3Prop p;
            if (q.lds_table)
                p.load(table, n_cols, col);
            else
                p.load(s.prop, s.prop_stride, col);
            if (q.fold_prev) {
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) {
                    prev[k * ne] = 0.0f;
                    st.y1[k] = st.y1[k] + arrived[k] * p.psc0[k];
                }
            }
            const float zero[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
            const int ref_before = st.ref;
            spike = glif3_update(st, p, s.h, zero, I, &frac);
            glif3_store(st, s.V, s.asc, s.y1, s.y2, s.ref, ne, e);
            if (q.probe_row >= 0) {
                const int col = s.probe_col[e];
                if (col >= 0) s.probe_v[q.probe_row * s.probe_stride + col] = st.V;
            }
            if (s.save_v) {
                s.save_v[q.out_row * ne + e] = st.V;
                s.save_flags[q.out_row * ne + e] = (uint8_t)((spike ? BMTK_F_SPIKE : 0) |
                                                              (ref_before == 0 ? BMTK_F_INTEGRATING : 0) |
                                                              (ref_before > 0 && st.ref == 0 ? BMTK_F_RESET : 0));
            }
        }
    }
    if (!q.do_update) return;
    const unsigned long long m = __ballot(spike);
    const int64_t wave_base = e & ~(int64_t)(kWave - 1);
    if (lane == 0 && wave_base < ne) {
        s.work_bits[(q.t % q.hist) * (words + 1) + (e >> 6)] = m;
        if (s.spike_bits) s.spike_bits[q.out_row * s.spike_bits_stride + (e >> 6)] = m;
    }
    if (s.spike_count && m != 0ull) {
        // one counter bump per wavefront, record slots handed out in lane order
        const int leader = __ffsll((long long)m) - 1;
        unsigned long long base = 0ull;
        // the record may be split into several lists with a counter each (spike_ways)
        const unsigned ways = s.spike_ways > 1 ? (unsigned)s.spike_ways : 1u;
        const unsigned long long way = (unsigned)bid & (ways - 1u), way_cap = (unsigned long long)s.spike_cap / ways;
        if (lane == leader)
            base = atomicAdd(s.spike_count + way * BMTK_RECORD_COUNT_STRIDE, (unsigned long long)__popcll(m));
        base = bcast_u64(base, leader);
        unsigned long long idx = base + (unsigned long long)lane_prefix(m);
        if (spike && idx < way_cap) {
            idx += way * way_cap;
            s.spike_step[idx] = (int32_t)q.t;
            s.spike_elem[idx] = (int32_t)e;
            if (s.spike_frac) s.spike_frac[idx] = frac;
        }
    }
}

// one row of the input-event history: bit (source*batch+trial) for every event of the step
__global__ __launch_bounds__(kBlock) void input_bits_kernel(const int64_t *__restrict__ in_ptr,
                                                            const int32_t *__restrict__ in_events, int64_t step,
                                                            unsigned long long *__restrict__ row)
{
    const int64_t k0 = in_ptr[step], k1 = in_ptr[step + 1];
    for (int64_t k = k0 + (int64_t)blockIdx.x * kBlock + threadIdx.x; k < k1; k += (int64_t)gridDim.x * kBlock) {
        const int e = in_events[k];
        atomicOr(row + (e >> 6), 1ull << (e & 63));
    }
}

__global__ __launch_bounds__(kBlock) void zero_row_kernel(unsigned long long *__restrict__ row, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) row[i] = 0ull;
}

__global__ __launch_bounds__(kBlock) void pack_kernel(int64_t nnz, const int32_t *__restrict__ indices,
                                                      const float *__restrict__ weights,
                                                      const uint8_t *__restrict__ delays,
                                                      const uint8_t *__restrict__ receptors,
                                                      bmtk_synapse *__restrict__ packed)
{
    const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (p >= nnz) return;
    bmtk_synapse o;
    o.tdr = (uint32_t)indices[p] | ((uint32_t)receptors[p] << 24) | ((uint32_t)delays[p] << 26);
    o.weight = weights[p];
    packed[p] = o;
}

__global__ __launch_bounds__(kBlock) void pack_wide_kernel(int64_t nnz, const int32_t *__restrict__ indices,
                                                           const float *__restrict__ weights,
                                                           const int32_t *__restrict__ delays,
                                                           const uint8_t *__restrict__ receptors, int idx_bits,
                                                           bmtk_synapse *__restrict__ packed)
{
    const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (p >= nnz) return;
    bmtk_synapse o;
    o.tdr = (uint32_t)indices[p] | ((uint32_t)receptors[p] << idx_bits) | ((uint32_t)delays[p] << (idx_bits + 2));
    o.weight = weights[p];
    packed[p] = o;
}

}  // namespace bmtk

using namespace bmtk;

extern "C" int bmtk_csr_pack_wide(int64_t nnz, const int32_t *indices, const float *weights, const int32_t *delays,
                                  const uint8_t *receptors, int32_t delay_bits, bmtk_synapse *packed, void *stream)
{
    BMTK_REQUIRE(nnz >= 0 && nnz < (1ll << 31), "csr_pack_wide: nnz must lie in 0..2^31-1");
    BMTK_REQUIRE(delay_bits >= 6 && delay_bits <= 14, "csr_pack_wide: delay_bits must lie in 6..14");
    if (nnz == 0) return BMTK_OK;
    BMTK_REQUIRE(indices && weights && delays && receptors && packed, "csr_pack_wide: pointers must be non-null");
    hipLaunchKernelGGL(pack_wide_kernel, dim3((unsigned)((nnz + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, nnz, indices, weights, delays, receptors, 30 - delay_bits, packed);
    BMTK_CHECK_LAUNCH("csr_pack_wide");
    return BMTK_OK;
}

extern "C" int bmtk_csr_pack(int64_t nnz, const int32_t *indices, const float *weights, const uint8_t *delays,
                             const uint8_t *receptors, bmtk_synapse *packed, void *stream)
{
    BMTK_REQUIRE(nnz >= 0 && nnz < (1ll << 31), "csr_pack: nnz must lie in 0..2^31-1");
    if (nnz == 0) return BMTK_OK;
    BMTK_REQUIRE(indices && weights && delays && receptors && packed, "csr_pack: pointers must be non-null");
    hipLaunchKernelGGL(pack_kernel, dim3((unsigned)((nnz + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, nnz, indices, weights, delays, receptors, packed);
    BMTK_CHECK_LAUNCH("csr_pack");
    return BMTK_OK;
}

extern "C" int bmtk_glif3_simulate_fwd(const bmtk_glif3_sim *sim, int64_t step0, int64_t n_steps, void *stream)
{
    BMTK_REQUIRE(sim != nullptr, "glif3_simulate_fwd: sim is null");
    const bmtk_glif3_sim &s = *sim;
    BMTK_REQUIRE(s.n_neurons > 0 && s.batch > 0, "glif3_simulate_fwd: n_neurons and batch must be positive");
    const int64_t ne = s.n_neurons * (int64_t)s.batch;
    BMTK_REQUIRE(ne < (1ll << 31), "glif3_simulate_fwd: n_neurons*batch must stay below 2^31");
    const int delay_bits = s.delay_bits ? s.delay_bits : 6;
    BMTK_REQUIRE(delay_bits >= 6 && delay_bits <= 14, "glif3_simulate_fwd: delay_bits must be 0 or lie in 6..14");
    BMTK_REQUIRE(delay_bits == 6 || (s.res_span == 0 && s.pull_packed == nullptr),
                 "glif3_simulate_fwd: wide delay fields are read by the launch-per-step driver without the pull form only");
    BMTK_REQUIRE(s.n_neurons < (1ll << (30 - delay_bits)) && (s.in_ptr == nullptr || s.n_inputs < (1ll << 24)),
                 "glif3_simulate_fwd: more neurons than the index field of the packed tables holds");
    BMTK_REQUIRE(s.ring_slots > 1 && s.ring_slots <= (1 << delay_bits),
                 "glif3_simulate_fwd: ring_slots must exceed the largest delay and stay within 2..2^delay_bits");
    BMTK_REQUIRE(s.h > 0.0f, "glif3_simulate_fwd: resolution h must be positive");
    BMTK_REQUIRE(s.V && s.asc && s.y1 && s.y2 && s.ref && s.prop && s.ring && s.work_bits,
                 "glif3_simulate_fwd: state, prop, ring and work_bits pointers must be non-null");
    BMTK_REQUIRE(s.prop_stride > 0 && (s.class_id || s.prop_stride >= s.n_neurons),
                 "glif3_simulate_fwd: prop_stride too small");
    const bool has_rec = s.rec_indptr != nullptr;
    BMTK_REQUIRE(!has_rec || s.rec_packed, "glif3_simulate_fwd: recurrent table needs rec_packed");
    const bool has_inp = s.in_ptr != nullptr;
    BMTK_REQUIRE(!has_inp || (s.in_events && s.inp_indptr && s.inp_packed),
                 "glif3_simulate_fwd: input event list needs in_events, inp_indptr and inp_packed");
    BMTK_REQUIRE(!s.spike_bits || s.spike_bits_stride >= (ne + 63) / 64,
                 "glif3_simulate_fwd: spike_bits_stride smaller than ceil(ne/64)");
    BMTK_REQUIRE(!s.spike_count || (s.spike_step && s.spike_elem && s.spike_cap > 0),
                 "glif3_simulate_fwd: spike record needs spike_step, spike_elem and a positive spike_cap");
    BMTK_REQUIRE(s.spike_ways >= 0 && s.spike_ways <= 256 && (s.spike_ways & (s.spike_ways - 1)) == 0 &&
                     (s.spike_ways <= 1 || !s.spike_count || s.spike_cap % s.spike_ways == 0),
                 "glif3_simulate_fwd: spike_ways must be 0 or a power of two up to 256 that divides spike_cap");
    BMTK_REQUIRE(step0 >= 0 && n_steps >= 0, "glif3_simulate_fwd: step0 and n_steps must be non-negative");
    const int hist = s.hist_slots ? s.hist_slots : 3;
    BMTK_REQUIRE(s.delay_offset >= 0 && (hist >= s.delay_offset + 3 || (s.pull_packed && s.res_span == 0)),
                 "glif3_simulate_fwd: hist_slots must be at least delay_offset + 3");
    if (n_steps == 0) return BMTK_OK;
    BMTK_REQUIRE((s.save_v == nullptr) == (s.save_flags == nullptr),
                 "glif3_simulate_fwd: save_v and save_flags go together");
    BMTK_REQUIRE(!(s.save_v && s.res_span > 0), "glif3_simulate_fwd: the per-step record needs launch-per-step mode");
    if (s.res_span > 0) {
        BMTK_REQUIRE(s.batch == 1, "glif3_simulate_fwd: resident mode runs batch 1 only");
        BMTK_REQUIRE(s.res_span % 64 == 0 && s.res_span <= 1024, "glif3_simulate_fwd: res_span must be a multiple of 64, at most 1024");
        BMTK_REQUIRE(s.res_groups == (ne + s.res_span - 1) / s.res_span, "glif3_simulate_fwd: res_groups must equal ceil(ne/res_span)");
        BMTK_REQUIRE(s.res_sync, "glif3_simulate_fwd: resident mode needs res_sync");
        BMTK_REQUIRE(!has_rec || s.rec_seg, "glif3_simulate_fwd: resident mode needs rec_seg");
        BMTK_REQUIRE(!has_inp || s.inp_seg, "glif3_simulate_fwd: resident mode needs inp_seg");
        BMTK_REQUIRE((size_t)s.ring_slots * GLIF3_NREC * s.res_span * sizeof(float) +
                             (s.res_groups == 1 ? solo_lds_extra(s.res_span) : kResLdsExtra) <= kResLdsBytes,
                     "glif3_simulate_fwd: ring slice does not fit in LDS beside the active-row list");
        bmtk_glif3_sim r = s;
        if (!has_rec) r.rec_seg = nullptr;
        if (!has_inp) r.inp_seg = nullptr;
        return simulate_resident(r, step0, n_steps, (hipStream_t)stream);
    }

    if (s.fuse_packed != nullptr) return simulate_fused(s, step0, n_steps, (hipStream_t)stream);

    const int64_t words = (ne + 63) / 64;
    const bool pull = has_rec && s.pull_packed != nullptr;
    if (pull) {
        BMTK_REQUIRE(s.pull_indptr && s.pull_syn && s.pull_work,
                     "glif3_simulate_fwd: the pull form needs pull_indptr, pull_syn and pull_work");
        BMTK_REQUIRE(s.delay_offset == 0 && hist == s.ring_slots,
                     "glif3_simulate_fwd: the pull form needs delay_offset 0 and hist_slots == ring_slots");
    }
    const bool pull_inp = pull && has_inp && s.pull_inp_packed != nullptr;
    if (pull_inp) {
        BMTK_REQUIRE(s.pull_inp_indptr && s.pull_inp_syn && s.pull_inp_work && s.in_hist,
                     "glif3_simulate_fwd: the pull form of the inputs needs pull_inp_indptr, pull_inp_syn, "
                     "pull_inp_work and in_hist");
        BMTK_REQUIRE(s.in_hist_stride >= (s.n_inputs * (int64_t)s.batch + 63) / 64 + 1,
                     "glif3_simulate_fwd: in_hist_stride must hold ceil(n_inputs*batch/64)+1 words");
    }
    BMTK_REQUIRE(!s.probe_col || (s.probe_v && s.probe_every >= 1 && s.probe_stride >= 1),
                 "glif3_simulate_fwd: probes need probe_v, probe_stride and probe_every >= 1");
    SimLaunch q{};
    q.n_update = (int)((ne + kSimBlock - 1) / kSimBlock);
    const int64_t max_deliver = (words + kSimWaves - 1) / kSimWaves;  // at least one word per wavefront
    q.n_deliver = (has_rec && !pull) ? (int)(max_deliver < 128 ? max_deliver : 128) : 0;
    BMTK_REQUIRE((s.in_repeat_ptr == nullptr) == (s.in_repeat_events == nullptr),
                 "glif3_simulate_fwd: in_repeat_ptr and in_repeat_events go together");
    // with the pull form of the inputs only the few repeated ids of a step are still delivered as events
    const bool repeats = pull_inp && s.in_repeat_ptr != nullptr;
    const int n_input = has_inp ? (!pull_inp ? 64 : (repeats ? 4 : 0)) : 0;
    const size_t table_bytes = (size_t)s.prop_stride * GLIF3_NPROP * sizeof(float);
    q.lds_table = (s.class_id && table_bytes <= (size_t)kLdsTableBytes && ((uintptr_t)s.prop & 15u) == 0) ? 1 : 0;
    const size_t lds = q.lds_table ? table_bytes : 0;
    for (int64_t k = 0; k <= n_steps; ++k) {
        const bool closing = k == n_steps;
        q.t = step0 + k;
        q.src = q.t - 1 - s.delay_offset;
        q.hist = hist;
        q.idx_bits = 30 - delay_bits;
        q.out_row = k;
        // sampled steps: (t + 1) % every == 0; row = how many of them the call has seen before
        q.probe_row = -1;
        if (s.probe_col && !closing && (q.t + 1) % s.probe_every == 0)
            q.probe_row = (q.t + 1) / s.probe_every - step0 / s.probe_every - 1;
        q.do_update = closing ? 0 : 1;
        q.fold_prev = k > 0;
        // the first launch of a call delivers nothing: the closing launch of the call before it did
        q.deliver_prev = (k > 0 && q.src >= 0 && has_rec && !pull) ? 1 : 0;
        q.pull = (pull && k > 0) ? 1 : 0;
        if (q.pull) {
            // everything that arrives in step t-1 over recurrent synapses, from the spikes of steps <= t-2
            const int rc = bmtk_csr_propagate_pull(s.work_bits, words + 1, s.ring_slots, s.n_neurons, s.batch,
                                                   s.pull_indptr, s.pull_packed, s.pull_syn, s.n_neurons, q.t - 1,
                                                   s.pull_work, stream);
            if (rc != BMTK_OK) return rc;
        }
        q.pull_inp = 0;
        if (pull_inp && q.t >= 1) {
            // the events of step t-1 become row (t-1) % L of the input history; what arrives in step t-1 is then
            // summed from the rows of the steps before it
            unsigned long long *row = reinterpret_cast<unsigned long long *>(s.in_hist) +
                                      ((q.t - 1) % s.ring_slots) * s.in_hist_stride;
            hipLaunchKernelGGL(zero_row_kernel, dim3((unsigned)((s.in_hist_stride + kBlock - 1) / kBlock)),
                               dim3(kBlock), 0, (hipStream_t)stream, row, s.in_hist_stride);
            hipLaunchKernelGGL(input_bits_kernel, dim3(16), dim3(kBlock), 0, (hipStream_t)stream, s.in_ptr,
                               s.in_events, q.t - 1, row);
            if (k > 0) {
                const int rc = bmtk_csr_propagate_pull(s.in_hist, s.in_hist_stride, s.ring_slots, s.n_inputs, s.batch,
                                                       s.pull_inp_indptr, s.pull_inp_packed, s.pull_inp_syn,
                                                       s.n_neurons, q.t - 1, s.pull_inp_work, stream);
                if (rc != BMTK_OK) return rc;
                q.pull_inp = 1;
            }
        }
        q.n_input = (k > 0 && q.src >= 0) ? n_input : 0;
        q.repeats = repeats ? 1 : 0;
        const unsigned grid = (unsigned)(q.n_update + q.n_deliver + q.n_input);
        hipLaunchKernelGGL(sim_step_kernel, dim3(grid), dim3(kSimBlock), lds, (hipStream_t)stream, s, q);
    }
    BMTK_CHECK_LAUNCH("glif3_simulate_fwd");
    return BMTK_OK;
}
