// Resident forward simulation of a SMALL network: one workgroup holds all of it.
//
// Up to 1024 elements (batch 1) fit one workgroup of the resident scheme: state
// and propagators in registers, the whole delay ring in LDS.  Then nothing has
// to cross workgroups and the machinery the large form needs for that -- a grid
// barrier per step, spike ballots read back through the memory system, segment
// offsets per workgroup -- falls away: the ballots of a step are handed over in
// LDS, ONE workgroup barrier separates the steps, and a wavefront walks the
// whole synapse row of a neuron that fired (every target is its own
// workgroup's).  bmtk's example networks (a few hundred cells, often at
// resolutions of a microsecond, i.e. millions of steps) are this case: a step
// costs about a microsecond instead of the three the grid barrier sets as a
// floor.
//
// What sets the pace of such a step is the chain of things that must follow
// one another, not the amount of work: a wavefront issues an instruction every
// four cycles at best, so every instruction on the chain counts, serial
// sections that one wavefront runs for all count sixteenfold, and so does every
// wait for memory.  On this hardware a wavefront's vector memory operations
// complete in the order issued: a wavefront that waits for a load also waits
// for every store it issued before it, and a store is acknowledged only after
// a trip to the far side of L2, about as long as the whole step.  Hence:
//   * no serial section: after the barrier EVERY wavefront reads the step's
//     list (16 ballot words, the number of input events) from LDS, takes the
//     prefix sums of the popcounts itself and picks "its" item;
//   * the sixteen wavefronts divide the memory traffic by kind, so that none
//     waits for a load behind a store or behind a load only just asked for.
//     Every wavefront updates its 64 neurons from registers and leaves ballot,
//     spike offsets and probed potentials in LDS -- no device memory at all.
//     The STORE wavefront (the last) writes them out after the barrier: the
//     history row, the output row, the spike record (whose counter it keeps in
//     a register: nobody else appends while this kernel runs), the probes.
//     The FETCH wavefront (the last but one) reads the input events a step
//     ahead -- their bounds two steps ahead -- and hands their rows over in
//     LDS.  The other fourteen WALK rows: one fired neuron or input event
//     each, row bounds from a copy in LDS; the row's first 64 synapses are
//     asked for as soon as the list stands and added after the next update,
//     which covers their way from L2;
//   * running counters instead of 64-bit divisions and multiplications.
//
// Per step t, with B = the delay offset:
//   1. fold the arrivals of slot t-1 into y1, update, ballots etc. to LDS;
//      fetch wavefront: the events of step t-B, and for B > 0 the ballots of
//      step t-B (from LDS when B < 4, else from the history row written B
//      steps ago), become the list of this step;
//   2. add the synapses of the list of step t-1 into the LDS ring (slots t and
//      later: nobody folds those before the barrier);         -- barrier --
//   3. store wavefront: write out; walkers: "their" item of the list of step
//      t, its row bounds, the first synapses asked for.
// The closing pull and fold leave state and ring exactly as the other drivers
// leave them.
#include "glif3_update.hpp"
#include "sim_internal.hpp"

namespace bmtk {

constexpr int kSoloBlock = 1024;
constexpr int kSoloWaves = kSoloBlock / kWave;
constexpr int kStoreWave = kSoloWaves - 1, kFetchWave = kSoloWaves - 2, kWalkers = kSoloWaves - 2;
constexpr int kEvCap = 128;                  // input events of a step handed over in LDS; further ones are read in place
constexpr int kNearSteps = 4;                // the ballots of so many steps stay in LDS (delay offsets below that)
constexpr int kListWords = kSoloWaves + 2;   // a list: 16 ballot words, the number of events, where they begin
constexpr size_t kSoloStaticLds = 1024;      // the kernel's static LDS, rounded up
constexpr unsigned kNoSample = 0xFFFFFFFFu;  // a probe cell nobody writes (a NaN no update produces)

struct Solo {
    int64_t step0;
    int n_steps;
    int span;          // elements rounded up to whole wavefronts
    int offset, hist;  // delay offset B, rows of the ballot history
    int inp_lds;       // the input table's row bounds have room in LDS too
};

// dynamic LDS of the kernel below, the optional bounds of the input table aside
constexpr size_t solo_lds_bytes(int ring_slots, int span, int ne)
{
    return ((size_t)ring_slots * GLIF3_NREC + 4) * span * sizeof(float)  // the ring; spike offsets and probed
                                                                         // potentials of two steps
           + (size_t)(ne + 2) / 2 * 2 * sizeof(int)                      // row bounds of the recurrent table
           + 2 * kEvCap * sizeof(int);                                   // rows of the input events, two steps
}
static_assert(solo_lds_bytes(0, 1024, 1024) + kSoloStaticLds <= solo_lds_extra(1024), "solo_lds_extra must cover the kernel's LDS");

__global__ __launch_bounds__(kSoloBlock) void sim_solo_kernel(bmtk_glif3_sim s, Solo r)
{
    extern __shared__ float ring_l[];                             // [L*4][span], then the arrays of solo_lds_bytes
    __shared__ unsigned long long list_l[2][kListWords];          // the lists of this step and the one before
    __shared__ unsigned long long near_l[kNearSteps][kSoloWaves];  // B > 0: the ballots of the last steps
    __shared__ int n_cols;
    __shared__ int go_on;
    const int tid = threadIdx.x, lane = lane_id();
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int ne = (int)s.n_neurons, words = (ne + 63) >> 6;
    const int L = s.ring_slots, span = r.span, B = r.offset;
    const bool own = tid < ne;
    const int e = tid;
    float *frac_l = ring_l + L * GLIF3_NREC * span;  // [2][span]
    float *probe_l = frac_l + 2 * span;              // [2][span]
    int *rec_ip_l = reinterpret_cast<int *>(probe_l + 2 * span);
    int *ev_l = rec_ip_l + (ne + 2) / 2 * 2;         // [2][kEvCap]
    int *inp_ip_l = ev_l + 2 * kEvCap;
    unsigned long long *hist = reinterpret_cast<unsigned long long *>(s.work_bits);
    // an earlier resident run on this simulator gave up and nobody has looked yet: do nothing (the word is sticky)
    if (tid == 0) {
        go_on = (s.res_sync == nullptr || __hip_atomic_load(s.res_sync + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u) ? 1 : 0;
        n_cols = 0;
    }
    __syncthreads();
    if (!go_on) return;

    for (int c = tid; c < L * GLIF3_NREC * span; c += kSoloBlock) {
        const int dr = c / span, i = c - dr * span;
        ring_l[c] = i < ne ? s.ring[(int64_t)dr * ne + i] : 0.0f;
    }
    if (s.rec_indptr)
        for (int c = tid; c <= ne; c += kSoloBlock) rec_ip_l[c] = s.rec_indptr[c];
    if (r.inp_lds)
        for (int c = tid; c <= (int)s.n_inputs; c += kSoloBlock) inp_ip_l[c] = s.inp_indptr[c];
    for (int c = tid; c < 2 * span; c += kSoloBlock) probe_l[c] = __uint_as_float(kNoSample);
    if (tid < 2 * kListWords) (&list_l[0][0])[tid] = 0ull;
    if (B > 0 && B < kNearSteps && tid < B * kSoloWaves) {
        // the ballots of the B steps before this call, from the history the call before left
        const int64_t u = r.step0 - 1 - tid / kSoloWaves;
        const int w = tid % kSoloWaves;
        near_l[u & (kNearSteps - 1)][w] = (u >= 0 && w < words) ? hist[(u % r.hist) * (words + 1) + w] : 0ull;
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
    // probes: the potentials go to LDS cell probe_col and the store wavefront writes the cells out; a column beyond
    // the cells (a caller's table wider than the network) is written in place
    const int probe_col = (own && s.probe_col) ? s.probe_col[e] : -1;
    if (probe_col >= 0) atomicMax(&n_cols, min(probe_col + 1, span));
    int probe_phase = s.probe_col ? (int)((r.step0 + 1) % s.probe_every) : 1;  // 0: sample after this step
    float *probe_out = s.probe_v;                                              // the row of the next sample
    const float zero[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
    // the spike record: a single workgroup appends to the first list only, and alone
    const unsigned long long rec_cap = (unsigned long long)s.spike_cap / (s.spike_ways > 1 ? (unsigned)s.spike_ways : 1u);
    unsigned long long rec_count = (wave == kStoreWave && s.spike_count) ? s.spike_count[0] : 0ull;
    __syncthreads();
    const int probe_cells = n_cols;

    const uint2 *__restrict__ rec_tab = reinterpret_cast<const uint2 *>(s.rec_packed);
    const uint2 *__restrict__ inp_tab = reinterpret_cast<const uint2 *>(s.inp_packed);
    unsigned q_lo = 0u, q_wrap = 0u;  // ring planes of the delivering step, see add()
    auto add = [&](const uint2 sy) {
        // ring cell: the record's upper byte is delay*4 + receptor, so (slot0 + delay) % L * 4 + receptor
        // = min(x, x - 4L) with x = slot0*4 + that byte (unsigned)
        const unsigned dq = sy.x >> 24;
        const unsigned plane = min(dq + q_lo, dq + q_wrap);
        atomicAdd(ring_l + (plane * (unsigned)span + (sy.x & 0xFFFFFFu)), __uint_as_float(sy.y));
    };
    auto walk = [&](const uint2 *__restrict__ tab, int p0, int p1) {
        for (int q = p0 + lane; q < p1; q += kWave) add(tab[q]);
    };
    // a zero the compiler cannot see through: added to an address that is the same in all lanes it keeps the load a
    // vector load (a scalar load's answer would be waited for at the wavefront's next LDS access)
    int opaque_zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(opaque_zero));
    auto first_lane = [](long long v) -> int64_t {
        return ((int64_t)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
               (int64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)v);
    };
    // what LDS holds is pinned to a register here, so that the compiler does not merge an LDS read with a device
    // memory read of the other branch into one generic load (which waits for everything)
    auto pin = [](int v) -> int {
        asm volatile("" : "+v"(v));
        return v;
    };
    // The list delivered in the coming iteration: c_n_ev input events (rows in ev_l[c_buf], beyond kEvCap in
    // in_events[c_ka ..]), then c_n_fired neurons: the set bits of the 16 ballot words, of which lane i < 16 holds
    // word c_word, its popcount c_cnt and the popcounts before it c_before.  None in the first iteration: the call
    // before closed with that pull.
    int c_n_ev = 0, c_n_fired = 0, c_buf = 0;
    int64_t c_ka = 0;
    unsigned long long c_word = 0ull;
    unsigned c_cnt = 0u, c_before = 0u;
    int pre_p0 = 0, pre_p1 = 0;            // row bounds of this wavefront's item (the same in all lanes)
    uint2 pre_first = make_uint2(0u, 0u);  // ... and this lane's synapse of the row's first 64
    // the i-th neuron of the list (i the same in all lanes)
    auto fired = [&](int i) -> int {
        const unsigned long long holder = __ballot((unsigned)i - c_before < c_cnt);
        const int src = __ffsll((long long)holder) - 1;
        unsigned long long w = bcast_u64(c_word, src);
        for (int j = i - __builtin_amdgcn_readlane((int)c_before, src); j > 0; --j) w &= w - 1ull;
        return src * kWave + __ffsll((long long)w) - 1;
    };
    auto item_row = [&](int i) -> int {
        if (i >= c_n_ev) return fired(i - c_n_ev);
        if (i < kEvCap) return pin(ev_l[c_buf * kEvCap + i]);
        return s.in_events[c_ka + i + opaque_zero];
    };
    auto bounds = [&](bool is_input, int row, int &p0, int &p1) {
        if (!is_input) {
            p0 = pin(rec_ip_l[row]);
            p1 = pin(rec_ip_l[row + 1]);
        } else if (r.inp_lds) {
            p0 = pin(inp_ip_l[row]);
            p1 = pin(inp_ip_l[row + 1]);
        } else {
            p0 = s.inp_indptr[row + opaque_zero];
            p1 = s.inp_indptr[row + 1 + opaque_zero];
        }
    };
    // The carried list: this wavefront's item, whose first synapses are on their way, then items wave + kWalkers,
    // wave + 2 kWalkers, ... the plain way.  The additions go to slots t .. t+L-2, never to slot t-1, which other
    // wavefronts may still be folding: no barrier is needed before them.
    auto deliver = [&]() {
        const int total = c_n_ev + c_n_fired;
        if (wave >= kWalkers || wave >= total) return;
        const int p0 = __builtin_amdgcn_readfirstlane(pre_p0), p1 = __builtin_amdgcn_readfirstlane(pre_p1);
        if (p0 + lane < p1) add(pre_first);
        walk(wave < c_n_ev ? inp_tab : rec_tab, p0 + kWave, p1);
        for (int i = wave + kWalkers; i < total; i += kWalkers) {
            const bool is_input = i < c_n_ev;
            int q0, q1;
            bounds(is_input, item_row(i), q0, q1);
            walk(is_input ? inp_tab : rec_tab, q0, q1);
        }
    };
    // Fetch wavefront: the events of the list of iteration k (those of step u = step0+k-B) are
    // in_events[f_lo, f_hi); their first 128 rows and the bound after the next step's are asked for an iteration
    // ahead.  in_ptr[i] stands for 0 when i <= 0 (steps before 0 have no events); indices past the call's last
    // list are not touched.
    const int64_t u_end = r.step0 + r.n_steps - B;  // in_ptr[u_end] closes the last list
    int64_t f_lo = 0, f_hi = 0;
    long long f_req = 0;
    int f_row0 = 0, f_row1 = 0;
    auto ask_rows = [&]() {
        if (f_lo + lane < f_hi) f_row0 = s.in_events[f_lo + lane];
        if (f_lo + kWave + lane < f_hi) f_row1 = s.in_events[f_lo + kWave + lane];
    };
    auto ask_bound = [&](int64_t i) {
        f_req = f_hi;
        if (i > 0 && i <= u_end) f_req = s.in_ptr[i + opaque_zero];
    };
    if (wave == kFetchWave && s.in_ptr && r.n_steps > 0) {
        const int64_t u0 = r.step0 - B;
        f_lo = u0 > 0 ? s.in_ptr[u0] : 0;
        f_hi = u0 + 1 > 0 ? s.in_ptr[u0 + 1] : 0;
        ask_rows();
        ask_bound(u0 + 2);
    }
    // running counters (a 64-bit remainder is some hundred instructions)
    int slot_prev = (int)((r.step0 + L - 1) % L);  // ring slot of step t-1
    int near_row = (int)(r.step0 & (kNearSteps - 1));
    int hist_row = (int)(r.step0 % r.hist);        // store wavefront: history row of step t
    int64_t u = r.step0 - B;                       // the step whose spikes and events make this step's list
    int far_row = (int)(((u % r.hist) + r.hist) % r.hist);  // fetch wavefront, B >= kNearSteps: history row of step u
    unsigned t32 = (unsigned)r.step0;              // step number as the record holds it
    uint64_t *bits_out = s.spike_bits;             // store wavefront: output row of step t
    // A history row is read B steps after it was written, before the barrier of that step (B < kNearSteps reads no
    // row inside a call): by then its store must have been acknowledged.  The store wavefront therefore waits for
    // its earlier stores once in B-1 steps (at most 64), just before a barrier: a row written after the barrier of
    // step t is then known to have arrived before the barrier of step t+B-1 at the latest.  Waiting in every step
    // would set the pace.
    const int wait_every = B - 1 < 64 ? (B > 1 ? B - 1 : 1) : 64;
    int wait_in = 0;

    for (int k = 0; k < r.n_steps; ++k) {
        const int buf = k & 1;
        q_lo = (unsigned)slot_prev * 4u;
        q_wrap = q_lo - 4u * (unsigned)L;
        unsigned long long *cur = B == 0 ? list_l[buf] : near_l[near_row];  // where this step's ballots go
        // 1a. fetch wavefront: this step's list
        if (wave == kFetchWave) {
            const int n_ev = (int)(f_hi - f_lo);
            if (lane == 0) {
                list_l[buf][kSoloWaves] = (unsigned long long)(unsigned)n_ev;
                list_l[buf][kSoloWaves + 1] = (unsigned long long)f_lo;
            }
            if (lane < n_ev) ev_l[buf * kEvCap + lane] = f_row0;
            if (lane + kWave < n_ev) ev_l[buf * kEvCap + kWave + lane] = f_row1;
            if (B > 0) {
                unsigned long long v = 0ull;
                if (u >= 0 && lane < words) {
                    if (B < kNearSteps)
                        v = near_l[(near_row - B) & (kNearSteps - 1)][lane];
                    else
                        v = __hip_atomic_load(hist + far_row * (words + 1) + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                if (lane < kSoloWaves) list_l[buf][lane] = v;
                far_row = far_row + 1 == r.hist ? 0 : far_row + 1;
            }
            // a step on: the events of step u+1, the bound after those of step u+2
            if (s.in_ptr && k + 1 < r.n_steps) {
                f_lo = f_hi;
                f_hi = first_lane(f_req);
                ask_rows();
                ask_bound(u + 3);
            }
        }
        // 1b. fold the arrivals of slot t-1 and update
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
        const unsigned long long m = __ballot(spike);
        if (lane == 0) cur[wave] = m;
        if (spike && s.spike_frac) frac_l[buf * span + tid] = frac;
        const bool sample = probe_phase == 0;
        if (sample && probe_col >= 0) {
            if (probe_col < span)
                probe_l[buf * span + probe_col] = st.V;
            else
                probe_out[probe_col] = st.V;
        }
        if (wave == kStoreWave && B >= kNearSteps) {
            if (wait_in == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            wait_in = wait_in + 1 == wait_every ? 0 : wait_in + 1;
        }
        // 2. deliver the list of the step before
        deliver();
        __syncthreads();  // ballots, offsets, samples and the list are in LDS; the old list is done with
        // 3a. store wavefront: write out
        if (wave == kStoreWave) {
            unsigned long long v = lane < words ? cur[lane] : 0ull;
            if (lane < words) {
                __hip_atomic_store(hist + hist_row * (words + 1) + lane, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (bits_out) bits_out[lane] = v;
            }
            if (s.spike_count) {
                const unsigned cnt = (unsigned)__popcll(v);
                const unsigned inc = wave_inclusive_scan(cnt);
                unsigned long long idx = rec_count + (inc - cnt);
                while (v) {
                    const int bit = __ffsll((long long)v) - 1;
                    v &= v - 1ull;
                    const int elem = lane * kWave + bit;
                    if (idx < rec_cap) {
                        s.spike_step[idx] = (int32_t)t32;
                        s.spike_elem[idx] = (int32_t)elem;
                        if (s.spike_frac) s.spike_frac[idx] = frac_l[buf * span + elem];
                    }
                    ++idx;
                }
                rec_count += (unsigned long long)__builtin_amdgcn_readlane((int)inc, kWave - 1);
            }
            if (sample)
                for (int c = lane; c < probe_cells; c += kWave) {
                    const float x = probe_l[buf * span + c];
                    if (__float_as_uint(x) != kNoSample) probe_out[c] = x;
                }
            hist_row = hist_row + 1 == r.hist ? 0 : hist_row + 1;
            if (bits_out) bits_out += s.spike_bits_stride;
        }
        // 3b. every wavefront: the new list; walkers: their item of it, its bounds, the first synapses asked for
        {
            const unsigned long long v = lane < kListWords ? list_l[buf][lane] : 0ull;
            c_word = v;
            c_cnt = (lane < kSoloWaves && s.rec_indptr) ? (unsigned)__popcll(v) : 0u;
            const unsigned inc = wave_inclusive_scan(c_cnt);
            c_before = inc - c_cnt;
            c_n_fired = __builtin_amdgcn_readlane((int)inc, kSoloWaves - 1);
            c_n_ev = __builtin_amdgcn_readlane((int)(unsigned)v, kSoloWaves);
            c_ka = (int64_t)bcast_u64(v, kSoloWaves + 1);
            c_buf = buf;
            if (wave < kWalkers && wave < c_n_ev + c_n_fired) {
                const bool is_input = wave < c_n_ev;
                bounds(is_input, item_row(wave), pre_p0, pre_p1);
                if (pre_p0 + lane < pre_p1) pre_first = (is_input ? inp_tab : rec_tab)[pre_p0 + lane];
            }
        }
        if (s.probe_col) {
            if (sample) probe_out += s.probe_stride;
            probe_phase = probe_phase + 1 == s.probe_every ? 0 : probe_phase + 1;
        }
        slot_prev = slot_prev + 1 == L ? 0 : slot_prev + 1;
        near_row = (near_row + 1) & (kNearSteps - 1);
        ++u;
        ++t32;
    }
    if (r.n_steps > 0) {
        // closing: the list of the last iteration (spikes and inputs of the last step less the delay offset), then
        // fold the last slot
        q_lo = (unsigned)slot_prev * 4u;
        q_wrap = q_lo - 4u * (unsigned)L;
        deliver();
        __syncthreads();
        if (own) {
            float *prev = ring_l + slot_prev * GLIF3_NREC * span + tid;
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
    if (wave == kStoreWave && lane == 0 && s.spike_count) s.spike_count[0] = rec_count;
    for (int c = tid; c < L * GLIF3_NREC * span; c += kSoloBlock) {
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
    Solo r{step0, (int)n_steps, s.res_span, s.delay_offset, hist, 0};
    size_t lds = solo_lds_bytes(s.ring_slots, s.res_span, (int)s.n_neurons);
    const size_t inp_bounds = s.inp_indptr ? (size_t)(s.n_inputs + 1) * sizeof(int) : 0;
    if (inp_bounds && lds + inp_bounds + kSoloStaticLds <= kResLdsBytes) {
        r.inp_lds = 1;
        lds += inp_bounds;
    }
    const void *kernel = reinterpret_cast<const void *>(sim_solo_kernel);
    hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) {
        set_error("glif3_simulate_fwd: the single-workgroup form needs %zu bytes of LDS: %s", lds, hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    // always sixteen wavefronts: those without elements walk rows, fetch events, write out
    hipLaunchKernelGGL(sim_solo_kernel, dim3(1), dim3(kSoloBlock), lds, stream, s, r);
    err = hipGetLastError();
    if (err != hipSuccess) {
        set_error("glif3_simulate_fwd: launch of the single-workgroup form failed: %s", hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    return BMTK_OK;
}

}  // namespace bmtk
