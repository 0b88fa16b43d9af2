// Resident forward simulation of a SMALL network: one workgroup holds all of it.
//
// Up to 1024 elements (batch 1) fit one workgroup of the resident scheme: state
// and propagators in registers, the whole delay ring in LDS.  Then nothing has
// to cross workgroups and the machinery the large form needs for that -- a grid
// barrier per step, spike ballots read back through the memory system, segment
// offsets per workgroup -- falls away: the ballots of a step are handed over in
// LDS, a workgroup barrier separates the steps, and a wavefront walks the whole
// synapse row of a neuron that fired (every target is its own workgroup's).
// bmtk's example networks (a few hundred cells, often at resolutions of a
// microsecond, i.e. millions of steps) are this case: a step costs about a
// microsecond instead of the three the grid barrier sets as a floor.
//
// Per step t:
//   1. fold the arrivals of slot t-1 into y1, update from registers, publish
//      the wavefront ballots (LDS for the next step, the history in device
//      memory for later steps and later calls, the output rows);
//   2. list the neurons that fired in step t-1-B (B = delay offset): from LDS
//      when B = 0, else from the history row written B+1 steps ago;
//   3. one wavefront per listed neuron or input event of that step streams the
//      row's synapses and adds the weights into the LDS ring.
// The closing pull and fold leave state and ring exactly as the other drivers
// leave them.
#include "glif3_update.hpp"
#include "sim_internal.hpp"

namespace bmtk {

constexpr int kSoloBlock = 1024;
constexpr int kSoloWaves = kSoloBlock / kWave;  // at most: a launch has as many wavefronts as the network needs

struct Solo {
    int64_t step0;
    int n_steps;
    int span;          // elements rounded up to whole wavefronts
    int offset, hist;  // delay offset B, rows of the ballot history
};

__global__ __launch_bounds__(kSoloBlock) void sim_solo_kernel(bmtk_glif3_sim s, Solo r)
{
    extern __shared__ float ring_l[];  // [L*4][span], then the list of fired neurons [kSoloBlock]
    __shared__ unsigned long long ballot_l[2][kSoloWaves];  // ballots of this step and the one before
    __shared__ unsigned n_act;
    __shared__ int go_on;
    const int tid = threadIdx.x, lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int n_threads = (int)blockDim.x, n_waves = n_threads / kWave;  // span threads, at least four wavefronts
    const int ne = (int)s.n_neurons, words = (ne + 63) >> 6;
    const int L = s.ring_slots, span = r.span, B = r.offset;
    const bool own = tid < ne;
    const int e = tid;
    unsigned *act = reinterpret_cast<unsigned *>(ring_l + L * GLIF3_NREC * span);
    unsigned long long *hist = reinterpret_cast<unsigned long long *>(s.work_bits);
    // an earlier resident run on this simulator gave up and nobody has looked yet: do nothing (the word is sticky)
    if (tid == 0) go_on = (s.res_sync == nullptr || __hip_atomic_load(s.res_sync + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u) ? 1 : 0;
    __syncthreads();
    if (!go_on) return;

    for (int c = tid; c < L * GLIF3_NREC * span; c += n_threads) {
        const int dr = c / span, i = c - dr * span;
        ring_l[c] = i < ne ? s.ring[(int64_t)dr * ne + i] : 0.0f;
    }
    Glif3Elem st{};
    Glif3Prop p{};
    float I = 0.0f;
    if (own) {
        const int64_t col = s.class_id ? (int64_t)s.class_id[e] : e;
        p.load(s.prop, s.prop_stride, col);
        glif3_load(st, s.V, s.asc, s.y1, s.y2, s.ref, ne, e);
        I = s.i_ext ? s.i_ext[e] : 0.0f;
    }
    const int probe_col = (own && s.probe_col) ? s.probe_col[e] : -1;
    int probe_phase = s.probe_col ? (int)((r.step0 + 1) % s.probe_every) : 1;  // 0: sample after this step
    int64_t probe_row = 0;
    const float zero[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
    const unsigned long long rec_cap = (unsigned long long)s.spike_cap / (s.spike_ways > 1 ? (unsigned)s.spike_ways : 1u);
    __syncthreads();

    // the spikes and input events of step u, handed over as if emitted in the step whose ring slot is slot0;
    // lds_row: where the ballots of step u lie in LDS, or -1 to take them from the history (all threads call this)
    auto deliver = [&](int64_t u, int slot0, int lds_row, int64_t ka, int64_t kb) {
        if (u < 0) return;
        if (wave == 0) {
            unsigned long long v = 0ull;
            if (lane < words && s.rec_indptr)
                v = lds_row >= 0 ? ballot_l[lds_row][lane]
                                 : __hip_atomic_load(hist + (u % r.hist) * (words + 1) + lane, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT);
            const unsigned cnt = (unsigned)__popcll(v);
            const unsigned inc = wave_inclusive_scan(cnt);
            unsigned pos = inc - cnt;
            while (v) {
                const int bit = __ffsll((long long)v) - 1;
                v &= v - 1ull;
                act[pos++] = (unsigned)(lane * kWave + bit);
            }
            if (lane == kWave - 1) n_act = inc;
        }
        __syncthreads();
        const int n_fired = (int)n_act;
        const int64_t total = n_fired + (kb - ka);
        const unsigned q_lo = (unsigned)slot0 * 4u, q_wrap = q_lo - 4u * (unsigned)L;
        for (int64_t i = wave; i < total; i += n_waves) {
            const bool is_input = i >= n_fired;
            const int row = is_input ? s.in_events[ka + (i - n_fired)] : (int)act[i];
            const int32_t *ip = is_input ? s.inp_indptr : s.rec_indptr;
            const uint2 *__restrict__ tab = reinterpret_cast<const uint2 *>(is_input ? s.inp_packed : s.rec_packed);
            const int p0 = ip[row], p1 = ip[row + 1];
            for (int q = p0 + lane; q < p1; q += kWave) {
                const uint2 sy = tab[q];
                // ring cell: the record's upper byte is delay*4 + receptor, so (slot0 + delay) % L * 4 + receptor
                // = min(x, x - 4L) with x = slot0*4 + that byte (unsigned)
                const unsigned dq = sy.x >> 24;
                const unsigned plane = min(dq + q_lo, dq + q_wrap);
                atomicAdd(ring_l + (plane * (unsigned)span + (sy.x & 0xFFFFFFu)), __uint_as_float(sy.y));
            }
        }
    };

    // bounds of the input events: in_ptr[i] for i > 0, 0 before (in_ptr[0] = 0 and steps before 0 have no events)
    int64_t ka = (s.in_ptr && r.step0 - B > 0) ? s.in_ptr[r.step0 - B] : 0;
    long long kb_lanes = 0;
    const int wait_every = B < 64 ? (B > 0 ? B : 1) : 64;
    int opaque_zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(opaque_zero));
    auto first_lane = [](long long v) -> int64_t {
        return ((int64_t)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
               (int64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)v);
    };
    for (int k = 0; k < r.n_steps; ++k) {
        const int64_t t = r.step0 + k;
        const int slot_prev = (int)((t + L - 1) % L);
        // The input events of the step delivered in step t, u = t-1-B, are in_events[ka, kb).  The bound the NEXT
        // step needs is asked for now and looked at a step later (through a vector load: the address gets a zero
        // the compiler cannot see through, or it would make this a scalar load, whose answer every wavefront then
        // waits for at its next LDS access, a few lines down).
        const int64_t u = t - 1 - B;
        long long next_lanes = 0;
        if (s.in_ptr && t - B + 1 > 0) next_lanes = s.in_ptr[t - B + 1 + opaque_zero];
        // 1. fold the arrivals of slot t-1 and update
        bool spike = false;
        float frac = 0.0f;
        if (own) {
            if (k > 0) {
                float *prev = ring_l + slot_prev * GLIF3_NREC * span + tid;
#pragma unroll
                for (int q = 0; q < GLIF3_NREC; ++q) {
                    const float a = prev[q * span];
                    prev[q * span] = 0.0f;
                    st.y1[q] = st.y1[q] + a * p.psc0[q];
                }
            }
            spike = glif3_update(st, p, s.h, zero, I, &frac);
        }
        if (s.probe_col) {
            if (probe_phase == 0) {
                if (probe_col >= 0) s.probe_v[probe_row * s.probe_stride + probe_col] = st.V;
                ++probe_row;
            }
            probe_phase = probe_phase + 1 == s.probe_every ? 0 : probe_phase + 1;
        }
        const unsigned long long m = __ballot(spike);
        // A history row is read again B+1 steps after it was written (B = 0 hands the ballots over in LDS and
        // reads no row inside a call): by then its store must have been acknowledged.  Every wavefront therefore
        // waits for its earlier stores once in B steps (at most 64), here, before this step's stores go out: a row
        // written in step t is then known to have arrived by step t+B at the latest, and workgroup barriers lie
        // between that point and the pull of step t+B+1, the first to read it.  A write-through store takes about
        // a step to be acknowledged, so waiting in every step would set the pace.
        if (B > 0 && k % wait_every == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (lane == 0) ballot_l[k & 1][wave] = m;
        if (lane == 0 && wave < words) {
            __hip_atomic_store(hist + (t % r.hist) * (words + 1) + wave, m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (s.spike_bits) s.spike_bits[k * s.spike_bits_stride + wave] = m;
        }
        if (s.spike_count && m != 0ull) {
            const int leader = __ffsll((long long)m) - 1;
            unsigned long long base = 0ull;
            if (lane == leader) base = atomicAdd(s.spike_count, (unsigned long long)__popcll(m));
            base = bcast_u64(base, leader);
            const unsigned long long idx = base + (unsigned long long)lane_prefix(m);
            if (spike && idx < rec_cap) {  // a single workgroup appends to the first list only
                s.spike_step[idx] = (int32_t)t;
                s.spike_elem[idx] = (int32_t)e;
                if (s.spike_frac) s.spike_frac[idx] = frac;
            }
        }
        __syncthreads();
        // 2. + 3. the spikes and events of step t-1-B (the first step of a call pulls nothing: the call before it
        //    closed with that pull)
        if (k > 0) {
            const int64_t kb = first_lane(kb_lanes);
            deliver(u, slot_prev, B == 0 ? (k - 1) & 1 : -1, ka, kb);
            ka = kb;
        }
        kb_lanes = next_lanes;
        __syncthreads();
    }
    if (r.n_steps > 0) {
        // closing: spikes and inputs of the last step (less the delay offset), then fold the last slot
        const int64_t tl = r.step0 + r.n_steps - 1;
        deliver(tl - B, (int)(tl % L), B == 0 ? (r.n_steps - 1) & 1 : -1, ka, first_lane(kb_lanes));
        __syncthreads();
        if (own) {
            float *prev = ring_l + (int)(tl % L) * GLIF3_NREC * span + tid;
#pragma unroll
            for (int q = 0; q < GLIF3_NREC; ++q) {
                const float a = prev[q * span];
                prev[q * span] = 0.0f;
                st.y1[q] = st.y1[q] + a * p.psc0[q];
            }
        }
        __syncthreads();
    }
    if (own) glif3_store(st, s.V, s.asc, s.y1, s.y2, s.ref, ne, e);
    for (int c = tid; c < L * GLIF3_NREC * span; c += n_threads) {
        const int dr = c / span, i = c - dr * span;
        if (i < ne) s.ring[(int64_t)dr * ne + i] = ring_l[c];
    }
}

int simulate_resident_solo(const bmtk_glif3_sim &s, int64_t step0, int64_t n_steps, hipStream_t stream)
{
    if (n_steps >= (1ll << 31)) {
        set_error("glif3_simulate_fwd: a resident call covers fewer than 2^31 steps");
        return BMTK_E_ARG;
    }
    const int hist = s.hist_slots ? s.hist_slots : 3;
    Solo r{step0, (int)n_steps, s.res_span, s.delay_offset, hist};
    const size_t lds = (size_t)s.ring_slots * GLIF3_NREC * s.res_span * sizeof(float) + kSoloBlock * sizeof(unsigned);
    const void *kernel = reinterpret_cast<const void *>(sim_solo_kernel);
    hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) {
        set_error("glif3_simulate_fwd: the single-workgroup form needs %zu bytes of LDS: %s", lds, hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    const int threads = kSoloBlock;  // wavefronts without elements still walk rows: a step's spikes and events in one round
    hipLaunchKernelGGL(sim_solo_kernel, dim3(1), dim3(threads), lds, stream, s, r);
    err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("glif3_simulate_fwd: launch of the single-workgroup form failed: %s", hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    return BMTK_OK;
}

}  // namespace bmtk
