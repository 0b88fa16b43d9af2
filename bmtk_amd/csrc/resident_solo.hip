// Resident forward simulation of a SMALL network: one workgroup holds all of it.
//
// Up to 1024 elements (batch 1) fit one workgroup of the resident scheme: state
// and propagators in registers, the whole delay ring in LDS.  Then nothing has
// to cross workgroups and the machinery the large form needs for that -- a grid
// barrier per step, spike ballots read back through the memory system, segment
// offsets per workgroup -- falls away: spikes are handed over in LDS, ONE
// workgroup barrier separates the steps, and a wavefront walks the whole
// synapse row of a neuron that fired (every target is its own workgroup's).
// bmtk's example networks (a few hundred cells, often at resolutions of a
// microsecond, i.e. millions of steps) are this case: a step costs about a
// microsecond instead of the two and a half the grid barrier sets as a floor.
//
// One compute unit runs it all, so what sets the pace of a step is how many
// instructions its sixteen wavefronts issue (a SIMD issues for one of its four
// wavefronts every four cycles; scalar bookkeeping counts like arithmetic), the
// chain of things that must follow one another -- LDS round trips, waits for
// memory, serial sections -- and, in a busy step, the one LDS unit.  On this
// hardware a wavefront's vector memory operations complete in the order
// issued: a wavefront that waits for a load also waits for every store it
// issued before it, and a store is acknowledged only after a trip to the far
// side of L2, about as long as the whole step.  Hence:
//   * a neuron that fires appends ITS OWN row (first synapse, length: two
//     registers of its thread) to the step's list of items in LDS; the input
//     events of the step arrive there the same way.  After the barrier a
//     walking wavefront reads the counts and "its" items in one LDS round trip
//     and asks for the rows' first 64 synapses at once; they are added after
//     the next update, which covers their way from L2;
//   * the sixteen wavefronts divide the memory traffic by kind, so that none
//     waits for a load behind a store or behind a load only just asked for.
//     Every wavefront updates its 64 neurons from registers and leaves ballot,
//     spike offsets and probed potentials in LDS -- no device memory at all.
//     The STORE wavefront (the last) writes them out after the barrier: the
//     history row, the output row, the spike record (whose counter it keeps in
//     a register: nobody else appends while this kernel runs), the probes.
//     The FETCH wavefront (the last but one) reads the input events a step
//     ahead -- their bounds two steps ahead -- and turns them into items.  The
//     other fourteen WALK rows: input events are dealt from the first walker
//     up, fired neurons from the last walker down, so that a walker seldom has
//     two;
//   * the loop over the steps is compiled once per role of a wavefront, so
//     that none steps through the branches and counters of the others, with
//     running counters instead of 64-bit divisions and multiplications;
//   * additions into the LDS ring are compare-and-swap loops: the LDS unit
//     works a float atomic off lane by lane.
// With a delay offset B > 0 the spikes handed over are B steps old: the fetch
// wavefront takes their ballots (from the last steps' ballots kept in LDS when
// B < 4, else from the history row written B steps ago) and turns them into
// items itself, a step's worth of time before the walkers want them.  Items
// beyond the 128 events and 512 neurons a step's lists hold take a slower way
// at delivery time: prefix sums over ballots' popcounts, row bounds from device
// memory.
//
// Per step t:
//   1. fetch wavefront: the events of step t-B become items; the others: fold
//      the arrivals of slot t-1 into y1, update, ballots etc. and items to LDS;
//   2. add the synapses of the items of step t-1 into the LDS ring (slots t and
//      later: nobody folds those before the barrier);         -- barrier --
//   3. store wavefront: write out; walkers: "their" items of step t, first
//      synapses asked for.
// The closing pull and fold leave state and ring exactly as the other drivers
// leave them.
#include <type_traits>

#include "glif3_update.hpp"
#include "sim_internal.hpp"

namespace bmtk {

constexpr int kSoloBlock = 1024;
constexpr int kSoloWaves = kSoloBlock / kWave;
constexpr int kStoreWave = kSoloWaves - 1, kFetchWave = kSoloWaves - 2, kWalkers = kSoloWaves - 2;
constexpr int kWalkRole = 0, kFetchRole = 1, kStoreRole = 2;  // what a wavefront does beside updating its neurons
constexpr int kEvCap = 128;                  // input events of a step that become items; further ones are read in place
constexpr int kFiredCap = 512;               // fired neurons of a step that become items; further ones: overflow ballot
constexpr int kNearSteps = 4;                // the ballots of so many steps stay in LDS (delay offsets below that)
constexpr size_t kSoloStaticLds = 2048;      // bound on the kernel's static LDS (1076 bytes and the compiler's padding)
constexpr unsigned kNoSample = 0xFFFFFFFFu;  // a probe cell nobody writes (a NaN no update produces)

struct Solo {
    int64_t step0;
    int n_steps;
    int span;          // elements rounded up to whole wavefronts
    int offset, hist;  // delay offset B, rows of the ballot history
    int inp_lds;       // the input table's row bounds have room in LDS
};

// dynamic LDS of the kernel below, the optional bounds of the input table aside
constexpr size_t solo_lds_bytes(int ring_slots, int span)
{
    return ((size_t)ring_slots * GLIF3_NREC + 4) * span * sizeof(float)  // the ring; spike offsets and probed
                                                                         // potentials of two steps
           + 2 * (kEvCap + kFiredCap) * sizeof(int2);                    // the items of two steps
}
static_assert(solo_lds_bytes(0, 1024) + kSoloStaticLds <= solo_lds_extra(1024), "solo_lds_extra must cover the kernel's LDS");

__global__ __launch_bounds__(kSoloBlock) void sim_solo_kernel(bmtk_glif3_sim s, Solo r)
{
    extern __shared__ float ring_l[];                              // [L*4][span], then the arrays of solo_lds_bytes
    __shared__ ulonglong2 pair_l[2][kSoloWaves];                   // per wavefront: ballot, ballot of the neurons without item
    __shared__ unsigned long long near_l[kNearSteps][kSoloWaves];  // B > 0: the ballots of the last steps
    __shared__ int4 meta_l[2];     // a step's events: how many, [B > 0: fired neurons], where they begin in in_events
    __shared__ unsigned count_l[3];  // B = 0: neurons that fired, three steps
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
    int2 *ev_items = reinterpret_cast<int2 *>(probe_l + 2 * span);  // [2][kEvCap]: first synapse, length
    int2 *fi_items = ev_items + 2 * kEvCap;                         // [2][kFiredCap]
    int *inp_ip_l = reinterpret_cast<int *>(fi_items + 2 * kFiredCap);
    unsigned long long *hist = reinterpret_cast<unsigned long long *>(s.work_bits);
    // an earlier resident run on this simulator gave up and nobody has looked yet: do nothing (the word is sticky)
    if (tid == 0) {
        go_on = (s.res_sync == nullptr || __hip_atomic_load(s.res_sync + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u) ? 1 : 0;
        n_cols = 0;
    }
    if (tid < 2 * kSoloWaves) (&pair_l[0][0])[tid] = make_ulonglong2(0ull, 0ull);
    if (tid < kNearSteps * kSoloWaves) (&near_l[0][0])[tid] = 0ull;
    if (tid < 3) count_l[tid] = 0u;
    if (tid < 2) meta_l[tid] = make_int4(0, 0, 0, 0);
    __syncthreads();
    if (!go_on) return;

    for (int c = tid; c < L * GLIF3_NREC * span; c += kSoloBlock) {
        const int dr = c / span, i = c - dr * span;
        ring_l[c] = i < ne ? s.ring[(int64_t)dr * ne + i] : 0.0f;
    }
    if (r.inp_lds)
        for (int c = tid; c <= (int)s.n_inputs; c += kSoloBlock) inp_ip_l[c] = s.inp_indptr[c];
    for (int c = tid; c < 2 * span; c += kSoloBlock) probe_l[c] = __uint_as_float(kNoSample);
    if (B > 0 && B < kNearSteps && tid < B * kSoloWaves) {
        // the ballots of the B steps before this call, from the history the call before left
        const int64_t u = r.step0 - 1 - tid / kSoloWaves;
        const int w = tid % kSoloWaves;
        near_l[u & (kNearSteps - 1)][w] = (u >= 0 && w < words) ? hist[(u % r.hist) * (words + 1) + w] : 0ull;
    }
    Glif3Elem st{};
    Glif3Prop p{};
    float I = 0.0f;
    int my_p0 = 0, my_len = 0;  // this neuron's row of the recurrent table
    if (own) {
        const int64_t col = s.class_id ? (int64_t)s.class_id[e] : e;
        p.load(s.prop, s.prop_stride, col);
        glif3_load(st, s.V, s.asc, s.y1, s.y2, s.ref, ne, e);
        I = s.i_ext ? s.i_ext[e] : 0.0f;
        if (s.rec_indptr) {
            my_p0 = s.rec_indptr[e];
            my_len = s.rec_indptr[e + 1] - my_p0;
        }
    }
    // probes: the potentials go to LDS cell probe_col and the store wavefront writes the cells out; a column beyond
    // the cells (a caller's table wider than the network) is written in place
    const int probe_col = (own && s.probe_col) ? s.probe_col[e] : -1;
    if (probe_col >= 0) atomicMax(&n_cols, min(probe_col + 1, span));
    int probe_phase = s.probe_col ? (int)((r.step0 + 1) % s.probe_every) : 1;  // 0: sample after this step
    float *probe_out = s.probe_v;                                              // the row of the next sample
    const float zero[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
    // the arrivals of a ring slot into y1; the slot is cleared (the four reads first: one wait instead of four)
    auto fold = [&](int slot) {
        float *cell = ring_l + slot * GLIF3_NREC * span + tid;
        float a[GLIF3_NREC];
#pragma unroll
        for (int q = 0; q < GLIF3_NREC; ++q) a[q] = cell[q * span];
#pragma unroll
        for (int q = 0; q < GLIF3_NREC; ++q) cell[q * span] = 0.0f;
#pragma unroll
        for (int q = 0; q < GLIF3_NREC; ++q) st.y1[q] = st.y1[q] + a[q] * p.psc0[q];
    };
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
        // An LDS float atomic is worked off lane by lane (about three clocks each: 135 for a row of 45 synapses), a
        // compare-and-swap in some 40 clocks per instruction whatever the number of lanes: the addition is a
        // compare-and-swap loop (a lane goes round again only if its cell changed in between: two synapses of
        // the row on one target and receptor, or another wavefront's row).  The one LDS unit is what a busy step of
        // this form is short of: 150 rows a step are 6,700 lanes.
        unsigned *cell = reinterpret_cast<unsigned *>(ring_l + (plane * (unsigned)span + (sy.x & 0xFFFFFFu)));
        const float w = __uint_as_float(sy.y);
        unsigned old = *cell;  // only seeds the loop: a stale value costs one more round
        while (true) {
            const unsigned seen = atomicCAS(cell, old, __float_as_uint(__uint_as_float(old) + w));
            if (seen == old) break;
            old = seen;
        }
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
    auto inp_bounds = [&](int row, int &p0, int &p1) {
        if (r.inp_lds) {
            p0 = pin(inp_ip_l[row]);
            p1 = pin(inp_ip_l[row + 1]);
        } else {
            p0 = s.inp_indptr[row];
            p1 = s.inp_indptr[row + 1];
        }
    };
    // The lists delivered in the coming iteration (none in the first: the call before closed with that pull):
    // c_n_ev input events, of which the first kEvCap are items ev_items[c_buf][..] and the others rows
    // in_events[c_ka + i]; c_n_fi fired neurons that are items fi_items[c_buf][..]; c_n_slow fired neurons marked in
    // the second ballots of pair_l[c_buf].  Walker w takes events w, w + 14, ... and neurons 13 - w, 27 - w, ...;
    // the first synapses of its first event and its first neuron are on their way (ev_first, fi_first).
    int c_n_ev = 0, c_n_fi = 0, c_n_slow = 0, c_buf = 0;
    int64_t c_ka = 0;
    int ev_p0 = 0, ev_len = 0, fi_p0 = 0, fi_len = 0;
    uint2 ev_first = make_uint2(0u, 0u), fi_first = make_uint2(0u, 0u);
    // The additions go to slots t .. t+L-2, never to slot t-1, which other wavefronts may still be folding: no
    // barrier is needed before them.
    // Items j, j + kWalkers, ... of a list (below n): a busy step has many more items than walkers, and a row taken
    // alone costs a whole trip to memory, so four rows' first synapses are asked for before any is added.
    auto rounds = [&](const int2 *__restrict__ items, const uint2 *__restrict__ tab, int j, int n)
                      __attribute__((always_inline)) {
        constexpr int kAhead = 4;
        for (; j < n; j += kAhead * kWalkers) {
            int p0[kAhead], len[kAhead];
            uint2 head[kAhead];
#pragma unroll
            for (int q = 0; q < kAhead; ++q) {
                const int2 it = j + q * kWalkers < n ? items[j + q * kWalkers] : make_int2(0, 0);
                p0[q] = __builtin_amdgcn_readfirstlane(it.x);
                len[q] = __builtin_amdgcn_readfirstlane(it.y);
            }
#pragma unroll
            for (int q = 0; q < kAhead; ++q)
                if (lane < len[q]) head[q] = tab[p0[q] + lane];
#pragma unroll
            for (int q = 0; q < kAhead; ++q) {
                if (lane < len[q]) add(head[q]);
                walk(tab, p0[q] + kWave, p0[q] + len[q]);
            }
        }
    };
    // (inlined by force: called out of line, everything it captures would live in memory)
    auto deliver = [&]() __attribute__((always_inline)) {
        if (wave >= kWalkers) return;
        const int n_evf = min(c_n_ev, kEvCap);
        if (wave < n_evf) {
            if (lane < ev_len) add(ev_first);
            walk(inp_tab, ev_p0 + kWave, ev_p0 + ev_len);
            rounds(ev_items + c_buf * kEvCap, inp_tab, wave + kWalkers, n_evf);
        }
        if (kWalkers - 1 - wave < c_n_fi) {
            if (lane < fi_len) add(fi_first);
            walk(rec_tab, fi_p0 + kWave, fi_p0 + fi_len);
            rounds(fi_items + c_buf * kFiredCap, rec_tab, 2 * kWalkers - 1 - wave, c_n_fi);
        }
        // the slower ways
        for (int i = kEvCap + wave; i < c_n_ev; i += kWalkers) {
            int p0, p1;
            inp_bounds(s.in_events[c_ka + i], p0, p1);
            walk(inp_tab, p0, p1);
        }
        if (c_n_slow > 0) {
            const unsigned long long word = lane < kSoloWaves ? pair_l[c_buf][lane].y : 0ull;
            const unsigned cnt = (unsigned)__popcll(word);
            const unsigned before = wave_inclusive_scan(cnt) - cnt;
            for (int i = wave; i < c_n_slow; i += kWalkers) {
                // the i-th marked neuron: the word that holds it, the bit within
                const unsigned long long holder = __ballot((unsigned)i - before < cnt);
                const int src = __ffsll((long long)holder) - 1;
                unsigned long long w = bcast_u64(word, src);
                for (int j = i - __builtin_amdgcn_readlane((int)before, src); j > 0; --j) w &= w - 1ull;
                const int id = src * kWave + __ffsll((long long)w) - 1;
                walk(rec_tab, s.rec_indptr[id], s.rec_indptr[id + 1]);
            }
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
    int cnt_row = 0;                               // count_l entry of this step
    int hist_row = (int)(r.step0 % r.hist);        // store wavefront: history row of step t
    int64_t u = r.step0 - B;                       // the step whose spikes and events are handed over in this step
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
    const bool has_rec = s.rec_indptr != nullptr;

    // The loop over the steps, compiled once per role of a wavefront -- what it does beside the barrier: walk rows,
    // fetch events or write out; whether it holds neurons; whether the delay offset is zero -- so that no wavefront
    // steps through the branches and counters of the others: the instructions issued per step, scalar ones
    // included, are what the sixteen wavefronts of the one compute unit compete for.
    auto steps = [&](auto role, auto neuron, auto zero_b) {
        constexpr int kRole = decltype(role)::value;
        constexpr bool kNeuron = decltype(neuron)::value, kZeroB = decltype(zero_b)::value;
        for (int k = 0; k < r.n_steps; ++k) {
            const int buf = k & 1;
            q_lo = (unsigned)slot_prev * 4u;
            q_wrap = q_lo - 4u * (unsigned)L;
            // 1a. fetch wavefront: this step's events become items
            if constexpr (kRole == kFetchRole) {
                const int n_ev = (int)(f_hi - f_lo);
                if (lane < n_ev) {
                    int p0, p1;
                    inp_bounds(f_row0, p0, p1);
                    ev_items[buf * kEvCap + lane] = make_int2(p0, p1 - p0);
                }
                if (lane + kWave < n_ev) {
                    int p0, p1;
                    inp_bounds(f_row1, p0, p1);
                    ev_items[buf * kEvCap + kWave + lane] = make_int2(p0, p1 - p0);
                }
                int n_slow = 0;
                if constexpr (!kZeroB) {
                    // the neurons that fired in step u
                    unsigned long long v = 0ull;
                    if (u >= 0 && lane < words && has_rec) {
                        if (B < kNearSteps)
                            v = near_l[(near_row - B) & (kNearSteps - 1)][lane];
                        else
                            v = __hip_atomic_load(hist + far_row * (words + 1) + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    const unsigned cnt = (unsigned)__popcll(v);
                    const bool any = __ballot(v != 0ull) != 0ull;  // (most steps of a fine resolution have none)
                    const unsigned upto = any ? wave_inclusive_scan(cnt) : 0u;
                    const int n_fired = any ? __builtin_amdgcn_readlane((int)upto, kWave - 1) : 0;
                    unsigned n_items = 0u;
                    if (!any) {
                    } else if (n_fired <= kFiredCap) {
                        // they become items here, a step's worth of time before the walkers want them: the neurons'
                        // numbers first (into the places of the items), then, 64 at a time, their rows' bounds
                        int2 *items = fi_items + buf * kFiredCap;
                        unsigned at = upto - cnt;
                        for (unsigned long long x = v; x; x &= x - 1ull)
                            items[at++].x = lane * kWave + (__ffsll((long long)x) - 1);
                        for (int i = lane; i < n_fired; i += kWave) {
                            const int id = items[i].x;
                            const int p0 = s.rec_indptr[id];
                            items[i] = make_int2(p0, s.rec_indptr[id + 1] - p0);
                        }
                        n_items = (unsigned)n_fired;
                        v = 0ull;
                    } else {
                        n_slow = n_fired;  // a volley beyond the list: all of them the slower way
                    }
                    if (lane == 0) count_l[cnt_row] = n_items;
                    if (lane < kSoloWaves) pair_l[buf][lane].y = v;
                    far_row = far_row + 1 == r.hist ? 0 : far_row + 1;
                }
                if (lane == 0) {
                    meta_l[buf] = make_int4(n_ev, n_slow, (int)(unsigned)f_lo, (int)(f_lo >> 32));
                    // B = 0: the neurons count themselves as they fire; the entry of the NEXT step is cleared here: it
                    // was last read before the barrier behind us and is added to after the barrier ahead
                    if (kZeroB) count_l[cnt_row == 2 ? 0 : cnt_row + 1] = 0u;
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
            const bool sample = probe_phase == 0;
            if constexpr (kNeuron) {  // wavefronts without neurons leave their ballot words as they are: zero
                bool spike = false;
                float frac = 0.0f;
                if (own) {
                    if (k > 0) fold(slot_prev);
                    spike = glif3_update(st, p, s.h, zero, I, &frac);
                }
                const unsigned long long m = __ballot(spike);
                if constexpr (kZeroB) {
                    unsigned long long no_item = 0ull;
                    if (m != 0ull && has_rec) {
                        unsigned at = kFiredCap;
                        if (spike) at = atomicAdd(&count_l[cnt_row], 1u);
                        if (at < kFiredCap) fi_items[buf * kFiredCap + at] = make_int2(my_p0, my_len);
                        no_item = __ballot(spike && at >= kFiredCap);
                    }
                    if (lane == 0) pair_l[buf][wave] = make_ulonglong2(m, no_item);
                } else if (lane == 0) {
                    near_l[near_row][wave] = m;
                }
                if (spike && s.spike_frac) frac_l[buf * span + tid] = frac;
                if (sample && probe_col >= 0 && probe_col < span) probe_l[buf * span + probe_col] = st.V;
                asm volatile("" ::: "memory");  // two stores, not one generic store to either place
                if (sample && probe_col >= span) probe_out[probe_col] = st.V;
            }
            if (kRole == kStoreRole && !kZeroB && B >= kNearSteps) {
                if (wait_in == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                wait_in = wait_in + 1 == wait_every ? 0 : wait_in + 1;
            }
            // 2. deliver the items of the step before
            if constexpr (kRole == kWalkRole) deliver();
            __syncthreads();  // ballots, offsets, samples and items are in LDS; the old items are done with
            // 3a. store wavefront: write out
            if constexpr (kRole == kStoreRole) {
                unsigned long long v = 0ull;
                if (lane < words) v = kZeroB ? pair_l[buf][lane].x : near_l[near_row][lane];
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
            // 3b. walkers: the new lists in one LDS round trip -- the counts, "my" event, "my" neuron -- and the first
            //     synapses asked for
            if constexpr (kRole == kWalkRole) {
                const int4 meta = meta_l[buf];
                const unsigned fired = count_l[cnt_row];
                const int2 ev = ev_items[buf * kEvCap + wave];
                const int2 fi = fi_items[buf * kFiredCap + kWalkers - 1 - wave];
                c_buf = buf;
                c_n_ev = __builtin_amdgcn_readfirstlane(meta.x);
                c_ka = ((int64_t)__builtin_amdgcn_readfirstlane(meta.w) << 32) | (int64_t)(unsigned)__builtin_amdgcn_readfirstlane(meta.z);
                const int n_fired = __builtin_amdgcn_readfirstlane((int)fired);
                c_n_fi = min(n_fired, kFiredCap);
                c_n_slow = kZeroB ? n_fired - c_n_fi : __builtin_amdgcn_readfirstlane(meta.y);
                if (wave < c_n_ev) {
                    ev_p0 = __builtin_amdgcn_readfirstlane(ev.x);
                    ev_len = __builtin_amdgcn_readfirstlane(ev.y);
                    if (lane < ev_len) ev_first = inp_tab[ev_p0 + lane];
                }
                if (kWalkers - 1 - wave < c_n_fi) {
                    fi_p0 = __builtin_amdgcn_readfirstlane(fi.x);
                    fi_len = __builtin_amdgcn_readfirstlane(fi.y);
                    if (lane < fi_len) fi_first = rec_tab[fi_p0 + lane];
                }
            }
            if constexpr (kNeuron || kRole == kStoreRole) {
                if (s.probe_col) {
                    if (sample) probe_out += s.probe_stride;
                    probe_phase = probe_phase + 1 == s.probe_every ? 0 : probe_phase + 1;
                }
            }
            slot_prev = slot_prev + 1 == L ? 0 : slot_prev + 1;
            if constexpr (!kZeroB) near_row = (near_row + 1) & (kNearSteps - 1);
            cnt_row = cnt_row == 2 ? 0 : cnt_row + 1;
            if constexpr (kRole == kFetchRole) ++u;
            if constexpr (kRole == kStoreRole) ++t32;
        }
    };
    auto with_offset = [&](auto role, auto neuron) {
        if (B == 0)
            steps(role, neuron, std::true_type{});
        else
            steps(role, neuron, std::false_type{});
    };
    auto with_neurons = [&](auto role) {
        if (wave < words)
            with_offset(role, std::true_type{});
        else
            with_offset(role, std::false_type{});
    };
    if (wave == kFetchWave)
        with_neurons(std::integral_constant<int, kFetchRole>{});
    else if (wave == kStoreWave)
        with_neurons(std::integral_constant<int, kStoreRole>{});
    else
        with_neurons(std::integral_constant<int, kWalkRole>{});
    if (r.n_steps > 0) {
        // closing: the items of the last iteration (spikes and inputs of the last step less the delay offset), then
        // fold the last slot
        q_lo = (unsigned)slot_prev * 4u;
        q_wrap = q_lo - 4u * (unsigned)L;
        deliver();
        __syncthreads();
        if (own) fold(slot_prev);
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
    size_t lds = solo_lds_bytes(s.ring_slots, s.res_span);
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
