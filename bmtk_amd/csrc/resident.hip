// Resident forward simulation: ONE cooperative launch for the whole run.
//
// Workgroup g owns elements [g*span, (g+1)*span): their state and propagators
// live in registers, their slice of the delay ring in LDS, from the first step
// to the last.  Per step a workgroup
//   1. folds the arrivals of slot t-1 (LDS) into y1 and runs the GLIF3 update
//      from registers, then publishes its wavefronts' spike ballots;
//   2. pulls the spikes of step t-1: it scans the ballots every workgroup
//      published before the previous barrier and, for each neuron that fired,
//      reads ITS OWN segment of that neuron's synapse row (rows are sorted by
//      target; a per-row offset table gives the segment bounds) and adds the
//      weights into its LDS ring slice with LDS atomics; external input events
//      of step t-1 are pulled the same way;
//   3. on the way, once every wavefront's ballot store of step t has been
//      acknowledged (an explicit wait on the vector memory counter, taken
//      together with the pull's first loads), signals the grid barrier of
//      step t, which then fills while the pull runs;
//   4. waits for the barrier where the spikes behind it are needed.
// Nothing but spike ballots, segment offsets and the synapses actually used
// crosses the memory system: no global atomics, no state traffic.
//
// Without slack (see below) a workgroup publishes, beside its ballots, the
// neurons that fired as a list of 16 places (res_fired: filled in LDS with one
// LDS atomic per spiking lane, written out by one wavefront once the workgroup
// has met after the update), and step 2 reads the lists -- four places per
// thread -- instead of taking the ballots of the whole network apart bit by
// bit, which every workgroup would do for itself; a step in which some list
// did not suffice is read from the ballots.  The same count gives a spike its
// place in the spike record when the workgroup has a record list of its own.
//
// Ballots live in a history of D rows, row t%D for step t.  With D = 3 a
// workgroup waits for the barrier of step t at the end of step t: row t%3 is
// read in step t+1 and next overwritten in step t+3, which a workgroup can only
// reach after the barrier of step t+2, i.e. after every workgroup finished
// reading it.  With a fourth row the wait moves to where the barrier is needed,
// just before the pull in step t+1: the update of step t+1 needs no spike newer
// than step t-1 (delays are at least one step, and arrivals enter y1 a step
// late), so it runs while the barrier of step t fills, and the wait is
// normally over before it begins.  A workgroup writing row t%4 is then at most
// two steps ahead of one still reading row (t-3)%4.
//
// With a delay offset B (tables hold delays shortened by B steps) step t pulls
// the spikes of step t-1-B from a history of D rows, and a workgroup only has
// to know that everybody has published step t-B before it starts step t+1: it
// waits for the barrier of S = min(B, D-3-B, 31) steps ago, so workgroups drift
// up to S steps apart and the wait is normally over before it begins.  Because
// of the drift one running count cannot tell who has arrived where: there is a
// counter per step, 64 of them used in turn (the fastest workgroup is at most
// 2S+1 < 64 steps ahead of a waiting one), each compared with the number of
// workgroups times the number of rounds it has served.  Row t%D is
// overwritten in step t+D; by then its writer has seen every workgroup arrive
// at the barrier of step t+D-1-S, hence finish the pull of step t+D-2-S, which
// read the spikes of step t+D-3-S-B >= t.
//
// Every wait is bounded: a workgroup that spins too long on the barrier raises
// the abort word, every other workgroup sees it and all leave the loop, so the
// grid always drains.
#include <stdlib.h>

#include "glif3_update.hpp"
#include "sim_internal.hpp"

namespace bmtk {

constexpr int kResBlock = 1024;
constexpr unsigned kMaxSpin = 4000000u;  // polls of the barrier word before giving up (seconds)
constexpr int kBarrierWords = 64;        // per-step arrival counters, used round-robin
// Words between two counters.  The arrivals of one step are a burst of one atomic per workgroup on one address,
// which the memory side works off one after the other (a few microseconds for 248 of them); a look at the
// counter of the step before must not queue up behind that burst, so every counter lives in a memory channel
// of its own rather than side by side in one cache line.
constexpr int kBarrierStride = BMTK_RES_SYNC_STRIDE;
// For the same reason a step's arrivals are spread over kWays counters (the workgroups of one XCD share one) and
// a look adds them up: the burst on one address is then an eighth as long, and so is the time the barrier takes
// to fill.  Counter (slot i, way x) is word (x * kBarrierWords + i) * kBarrierStride of the counter area.
constexpr int kWays = BMTK_RES_SYNC_WAYS;
constexpr int kWayStride = kBarrierWords * kBarrierStride;
static_assert(BMTK_RES_SYNC_WORDS >= (1 + kWays * kBarrierWords) * kBarrierStride, "res_sync too small");
constexpr int kMaxSlack = 31;

#ifdef BMTK_RES_PROFILE
__device__ unsigned long long g_prof[8];
__device__ unsigned long long g_prof_blk[256][4];  // per workgroup: update, pull, wait, segment pull
#define PROF_BLK(i, a, b) if (threadIdx.x == 0) atomicAdd(&g_prof_blk[blockIdx.x & 255][i], (unsigned long long)((b) - (a)))
#define PROF_T(var) const long long var = wall_clock64()
#define PROF_ADD(i, a, b) if (threadIdx.x == 0 && blockIdx.x == 0) atomicAdd(&g_prof[i], (unsigned long long)((b) - (a)))
#else
#define PROF_T(var)
#define PROF_ADD(i, a, b)
#define PROF_BLK(i, a, b)
#endif

struct Resident {
    int64_t step0, n_steps;
    int span, n_groups;
    int offset, hist, slack;  // B, D, S of the note above
    int check;                // the arrival counters are looked at every `check` steps (1 when S = 0)
};

__device__ __forceinline__ unsigned load_agent(const unsigned *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Wait until every vector memory operation this wavefront has issued is complete: its loads have returned and
// its stores -- the write-through, device-coherent ballot store among them -- have been acknowledged.  A release
// fence of workgroup scope does NOT do this: on this target it waits for LDS and scalar operations only, because
// the wavefronts of a workgroup share one vector cache.
//
// THE GRID BARRIER'S CONTRACT.  Four kinds of words in device memory are written by one workgroup and read by
// others during a launch; every such access is a relaxed atomic of AGENT scope (it passes the compute unit's
// vector cache and the XCD's L2 and is served where all XCDs see the same value), and the order between them is
// made by hand, because HIP's memory model offers no fence of the needed kind that does not also invalidate the
// XCD's L2 every step:
//   work_bits   (ballots)   written by: lane 0 of every wavefront that owns elements, right after its update of
//                           step t (row t % hist).  Read by: every workgroup's pull of step t, after it has seen
//                           the barrier of step t complete.
//   res_fired   (lists)     written by: the first 16 threads of a workgroup after the workgroup has met (row t %
//                           hist, the workgroup's 16 places).  Read by: every workgroup's pull of step t, as above.
//   arrival counters        written by: thread 0 of a workgroup, one increment per step, on the counter of (step,
//                           the workgroup's XCD), AFTER every wavefront of the workgroup has executed
//                           wait_vector_memory() and the workgroup has passed __syncthreads().  Read by: one look
//                           per workgroup and step (the eight counters of the step added up), repeated within a
//                           bounded spin.
//   abort word              written by: any workgroup whose spin ran out.  Read by: every workgroup inside its spin
//                           and at the start of a launch.  Sticky: only the host clears it.
// The one ordering that makes the barrier a barrier: a workgroup's ballot and list stores of step t are
// ACKNOWLEDGED (wait_vector_memory in every wavefront that stored, then the workgroup barrier) before its arrival
// for step t is sent.  A reader that has counted all arrivals of step t therefore loads ballots and lists that
// are already where agent-scope loads look.  Nothing else is assumed: readers do not rely on the order of two
// stores of another workgroup, and no acquire fence runs inside the loop (every read of another workgroup's words
// is an agent-scope load, which is not served from a copy that an earlier read left in the compute unit's cache).
// If the wait before the arrival were lost (a compiler that moved or dropped the asm, a fence mistaken for it),
// a reader could see the arrival before a ballot word and miss a spike of that step: the tests that run many
// workgroups for many steps against a driver without this barrier would differ in single synaptic segments --
// tests/test_gpu_simulate.py::test_v1_scale_resident_equals_per_step_launches and
// ::test_lists_of_fired_neurons_equal_the_ballots, tests/test_gpu_random_networks.py::
// test_many_workgroups_with_volleys_and_delay_offsets, tests/test_gpu_fullsize.py::
// test_v1_scale_forward_run_against_both_oracles.
__device__ __forceinline__ void wait_vector_memory()
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// add the weights of one row's synapses that target this workgroup's group,
// positions [seg_row[g], seg_row[g+1]) of the packed table, to the LDS ring
// slice.  Every lane of a wavefront reads a different cache line here, and the
// address unit serialises such requests, so the number of requests is what
// costs: the two bounds come in one 8-byte load, and only lanes that really
// have a k-th synapse issue the k-th load (a segment holds 1.2 on average).
struct __attribute__((packed, aligned(4))) SegBounds {
    uint32_t lo, hi;
};

__device__ __forceinline__ void pull_segment(const uint32_t *__restrict__ seg_row, int g,
                                             const bmtk_synapse *__restrict__ tab, float *ring_l, int span, int e0,
                                             int L, int slot0)
{
    const SegBounds sb = *reinterpret_cast<const SegBounds *>(seg_row + g);
    const uint32_t len = sb.hi - sb.lo;  // the offsets never decrease
    const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(tab) + sb.lo;
    // An LDS float atomic costs about three clocks per LANE on gfx950 (its lanes are worked off one after the
    // other), an integer compare-and-swap a few clocks per INSTRUCTION.  Where most lanes of a wavefront take
    // part -- the first synapse of the segments -- the addition is therefore a compare-and-swap loop (a
    // lane repeats only if another thread changed its cell in between, which is rare among 23,000 cells); the
    // thinly populated later ones keep the float atomic.  The sum is the same either way.
    // ring cell of a synapse: the record's upper byte is delay*4 + receptor, so (slot0 + delay) % L * 4 + receptor
    // = min(u, u - 4L) with u = slot0*4 + that byte (unsigned), times the span, plus the target's place in it.
    // Instruction issue is what the pull is short of (every lane walks its own segment, so each addition is a
    // wavefront instruction for a handful of lanes): the cell's address takes six instructions -- two byte adds, min,
    // mask, one 24-bit multiply-add, one shift-add onto the slice's origin less e0 -- and a synapse's load a compare
    // against the segment's length and an immediate offset.
    const unsigned q_lo = (unsigned)slot0 * 4u, q_wrap = q_lo - 4u * (unsigned)L;
    float *origin = ring_l - e0;
    unsigned span_v;  // in a vector register once, not before every multiply
    asm("v_mov_b32 %0, %1" : "=v"(span_v) : "s"(span));
    auto add = [&](const uint2 sy, bool crowded) {
        const unsigned dq = sy.x >> 24;
        const unsigned plane = min(dq + q_lo, dq + q_wrap);
        float *cell = origin + mad_u24(plane, span_v, sy.x & 0xFFFFFFu);
        const float w = __uint_as_float(sy.y);
        if (!crowded) {
            atomicAdd(cell, w);
            return;
        }
        unsigned *bits = reinterpret_cast<unsigned *>(cell);
        unsigned old = *bits;  // only seeds the loop: a stale value costs one more round
        while (true) {
            const unsigned seen = atomicCAS(bits, old, __float_as_uint(__uint_as_float(old) + w));
            if (seen == old) break;
            old = seen;
        }
    };
    // all of a segment's loads go out together: a loop of dependent loads for the few long segments would
    // hold up the whole wavefront (1 in 25 segments has more than 3 synapses, 1 in 5000 more than 6); measured at V1
    // scale: four together and the compare-and-swap for the first only, 5.35 us per step; six and two, 5.43
    constexpr int kTogether = 4;
    uint2 first[kTogether];
#pragma unroll
    for (int u = 0; u < kTogether; ++u)
        if ((uint32_t)u < len) first[u] = rows[u];
#pragma unroll
    for (int u = 0; u < kTogether; ++u)
        if ((uint32_t)u < len) add(first[u], u < 1);
    for (uint32_t q = (uint32_t)kTogether; q < len; ++q) add(rows[q], false);
}

constexpr int kScanWords = 4;   // ballot words per thread and round
constexpr unsigned kInputTag = 0x80000000u;

// Spikes and input events of one step, read from row `hist_row` of the ballot
// history and handed over as if emitted in the step whose ring slot is `slot0`
// (the step they were emitted in plus the delay offset) -> this workgroup's
// ring slice.
// Pass by pass: every thread reads kScanWords ballot words and one input
// event (independent loads), a workgroup-wide prefix sum packs the rows that
// fired into one LDS list, then one thread per listed row pulls this
// workgroup's segment of it.  Must be called by all threads of the workgroup.
// `arrival`, when not null, is the grid barrier counter this workgroup still has to bump for the step whose
// ballots its wavefronts have just stored: the bump may only happen once every one of those stores has been
// acknowledged, and the cheapest place to wait for that is where each wavefront waits for its scan loads anyway.
// Returns true when the bump has been made.
// kUnified: the input rows follow the recurrent rows in ONE table (inp_seg = rec_seg + n_neurons*(n_groups+1), both
// sets of offsets index rec_packed), so a listed row needs no choice between two tables.
// kLists: the workgroups publish the neurons that fired as short lists (res_fired) and a step is read from those
// when every list sufficed: two 8-byte loads per thread bring four places of the lists, the occupied ones go
// straight to the row list -- no ballot words to take apart bit by bit, which is the larger part of the
// instructions a quiet step costs.
template <bool kUnified, bool kLists>
__device__ __forceinline__ bool pull_step(const bmtk_glif3_sim &s, const Resident &r, int g, int hist_row, int slot0,
                                          float *ring_l, unsigned *act, unsigned *scan_l, int e0, int words,
                                          int64_t k0, int64_t k1, unsigned *arrival = nullptr)
{
    const int tid = threadIdx.x;
    const int L = s.ring_slots;
    const int wave = tid / kWave;
    const bool has_rec = s.rec_seg != nullptr;
    // one thread per listed row pulls this workgroup's segment of it
    auto pull_listed = [&](unsigned total) {
        for (unsigned a = tid; a < total; a += kResBlock) {
            // one code path for both kinds of rows: a wavefront nearly always holds some of each, and a
            // branch would make it walk the two chains of dependent loads one after the other
            const unsigned entry = act[a];
            if (kUnified) {  // rows * (n_groups + 1) stays below 2^32 (checked before the launch)
                pull_segment(s.rec_seg + mul_u24(entry, (unsigned)(r.n_groups + 1)), g, s.rec_packed, ring_l, r.span,
                             e0, L, slot0);
            } else {
                const int64_t row = entry & ~kInputTag;
                const bool is_input = (entry & kInputTag) != 0u;
                const uint32_t *seg = is_input ? s.inp_seg : s.rec_seg;
                const bmtk_synapse *tab = is_input ? s.inp_packed : s.rec_packed;
                pull_segment(seg + row * (r.n_groups + 1), g, tab, ring_l, r.span, e0, L, slot0);
            }
        }
    };
    bool arrived_above = false;
    if (kLists && s.res_fired && k1 - k0 <= kResBlock) {
        PROF_T(p0);
        constexpr unsigned kManyFlag = 1u << 20;  // in a count: some list did not suffice (1024 of them still fit 32 bits)
        static_assert(kManyFlag > (unsigned)kActCap && 5 * kResBlock <= kActCap, "a step read from the lists always fits the row list");
        const unsigned long long *lists = reinterpret_cast<const unsigned long long *>(
            s.res_fired + (int64_t)hist_row * r.n_groups * BMTK_RES_FIRED_SLOTS);
        unsigned long long w0 = 0ull, w1 = 0ull;  // four places: kResBlock threads cover 256 workgroups' lists
        if (has_rec && tid < r.n_groups * (BMTK_RES_FIRED_SLOTS / 4)) {
            w0 = __hip_atomic_load(lists + 2 * tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            w1 = __hip_atomic_load(lists + 2 * tid + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        const int64_t ke = k0 + tid;
        const bool has_event = ke < k1;
        const unsigned event_row = has_event ? (unsigned)s.in_events[ke] : 0u;
        const unsigned id[4] = {(unsigned)w0, (unsigned)(w0 >> 32), (unsigned)w1, (unsigned)(w1 >> 32)};
        unsigned cnt = has_event ? 1u : 0u;
#pragma unroll
        for (int u = 0; u < 4; ++u) cnt += id[u] != 0u ? 1u : 0u;
        if (id[0] == BMTK_RES_FIRED_MANY) cnt = kManyFlag;  // such a list is marked in every place
        const unsigned inc = wave_inclusive_scan(cnt);
        if (lane_id() == kWave - 1) scan_l[wave] = inc;
        if (arrival) wait_vector_memory();  // the loads are back already; this is for the stores of the update
        __syncthreads();
        if (arrival && tid == 0) __hip_atomic_fetch_add(arrival, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        PROF_T(p1);
        const unsigned part = wave_inclusive_scan(lane_id() < kResBlock / kWave ? scan_l[lane_id()] : 0u);
        const unsigned total = (unsigned)bcast_i((int)part, kResBlock / kWave - 1);
        const unsigned base = wave > 0 ? (unsigned)__shfl((int)part, wave - 1, kWave) : 0u;
        if (total <= (unsigned)kActCap) {  // workgroup-uniform: every list sufficed, and the row list holds them
            unsigned pos = base + inc - cnt;
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (id[u] != 0u) act[pos++] = id[u] - 1u;
            if (has_event) act[pos] = kUnified ? event_row + (unsigned)s.n_neurons : event_row | kInputTag;
            __syncthreads();
            PROF_T(p2);
            pull_listed(total);
            __syncthreads();
            PROF_T(p3);
            PROF_ADD(4, p0, p1);
            PROF_ADD(5, p1, p2);
            PROF_ADD(6, p2, p3);
            PROF_BLK(3, p2, p3);
            return arrival != nullptr;
        }
        // this step from the ballots (the arrival has been made)
        __syncthreads();  // scan_l is written again below
        arrived_above = arrival != nullptr;
        arrival = nullptr;
    }
    const unsigned long long *bits =
        reinterpret_cast<const unsigned long long *>(s.work_bits) + (int64_t)hist_row * (words + 1);
    // 32-bit counters wherever the sizes allow: the loop is short of scalar registers
    const int n_words = has_rec ? words : 0;
    const int word_rounds = (n_words + kScanWords * kResBlock - 1) / (kScanWords * kResBlock);
    const int event_rounds = (int)((k1 - k0 + kResBlock - 1) / kResBlock);  // a step's events are below 2^31
    const int rounds = word_rounds > event_rounds ? word_rounds : event_rounds;
    for (int round = 0; round < rounds; ++round) {
        const int w0 = round * kScanWords * kResBlock;
        PROF_T(p0);
        unsigned long long v[kScanWords];
        unsigned cnt = 0;
        // words past the end are read from the row's last word, which nothing ever writes (it stays zero):
        // no branch round the loads
        if (has_rec) {
#pragma unroll
            for (int u = 0; u < kScanWords; ++u) {
                const unsigned w = min((unsigned)w0 + (unsigned)(u * kResBlock + tid), (unsigned)words);
                v[u] = __hip_atomic_load(bits + w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        } else {
#pragma unroll
            for (int u = 0; u < kScanWords; ++u) v[u] = 0ull;
        }
        const int64_t ke = k0 + (round * kResBlock + tid);
        const bool has_event = ke < k1;
        const unsigned event_row = has_event ? (unsigned)s.in_events[ke] : 0u;
#pragma unroll
        for (int u = 0; u < kScanWords; ++u) cnt += (unsigned)__popcll(v[u]);
        cnt += has_event ? 1u : 0u;
        const unsigned inc = wave_inclusive_scan(cnt);
        if (lane_id() == kWave - 1) scan_l[wave] = inc;
        if (arrival && round == 0) wait_vector_memory();  // the loads are back already; this is for the ballot store
        __syncthreads();
        if (arrival && round == 0 && tid == 0)
            __hip_atomic_fetch_add(arrival, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        PROF_T(p1);
        // prefix over the 16 wavefront sums: one LDS read per lane and one more scan instead of 16 reads
        const unsigned part = wave_inclusive_scan(lane_id() < kResBlock / kWave ? scan_l[lane_id()] : 0u);
        const unsigned total = (unsigned)bcast_i((int)part, kResBlock / kWave - 1);
        const unsigned base = wave > 0 ? (unsigned)__shfl((int)part, wave - 1, kWave) : 0u;
        const bool listed = total <= (unsigned)kActCap;  // workgroup-uniform
        if (listed) {
            unsigned pos = base + inc - cnt;
#pragma unroll
            for (int u = 0; u < kScanWords; ++u) {
                unsigned long long x = v[u];
                const unsigned j0 = (unsigned)(w0 + u * kResBlock + tid) << 6;
                while (x) {
                    const int bit = __ffsll((long long)x) - 1;
                    x &= x - 1ull;
                    act[pos++] = j0 + (unsigned)bit;
                }
            }
            if (has_event) act[pos] = kUnified ? event_row + (unsigned)s.n_neurons : event_row | kInputTag;
        } else {
            // more rows than the list holds: every thread pulls what it found itself, unbalanced but correct
            for (int u = 0; u < kScanWords; ++u) {
                unsigned long long x = v[u];
                const int64_t j0 = (int64_t)(w0 + u * kResBlock + tid) << 6;
                while (x) {
                    const int bit = __ffsll((long long)x) - 1;
                    x &= x - 1ull;
                    pull_segment(s.rec_seg + (j0 + bit) * (r.n_groups + 1), g, s.rec_packed, ring_l, r.span, e0, L,
                                 slot0);
                }
            }
            if (has_event) {
                if (kUnified)
                    pull_segment(s.rec_seg + (s.n_neurons + (int64_t)event_row) * (r.n_groups + 1), g, s.rec_packed, ring_l,
                                 r.span, e0, L, slot0);
                else
                    pull_segment(s.inp_seg + (int64_t)event_row * (r.n_groups + 1), g, s.inp_packed, ring_l, r.span, e0,
                                 L, slot0);
            }
        }
        __syncthreads();
        PROF_T(p2);
        if (listed) pull_listed(total);
        __syncthreads();
        PROF_T(p3);
        PROF_ADD(4, p0, p1);
        PROF_ADD(5, p1, p2);
        PROF_ADD(6, p2, p3);
        PROF_BLK(3, p2, p3);
    }
    return arrived_above || (arrival != nullptr && rounds > 0);
}

// kLate: the run has slack (S > 0), see the loop body.  kForm: what the launch asks for beyond the simulation
// itself.  The loop is short of scalar registers (98 spilled in the general form; every use in the loop is a lane
// read), so the pointers and counters a launch does not use are taken out of it at compile time:
//   kFormLean    spike bits only, and the two tables are one (pull_step);
//   kFormRecord  the same with the spike record (what the PyNEST-shaped front end and the configuration runner
//                ask for), no membrane potential probes;
//   kFormAny     everything: probes, record, two tables.
enum { kFormAny = 0, kFormRecord = 1, kFormLean = 2 };
template <bool kLate, int kForm>
__global__ __launch_bounds__(kResBlock) void sim_resident_kernel(bmtk_glif3_sim s, Resident r)
{
    constexpr bool kUnifiedTables = kForm != kFormAny;
    constexpr bool kLists = !kLate;  // lists of fired neurons beside the ballots (res_fired), see pull_step
    if (kForm != kFormAny) {
        s.probe_col = nullptr;
        s.inp_seg = nullptr;
        s.inp_packed = nullptr;
    }
    if (kForm == kFormLean) s.spike_count = nullptr;
    extern __shared__ float ring_l[];  // [L*4][span], then the active-row list
    __shared__ int go_on;
    __shared__ unsigned scan_l[kResBlock / kWave];
    __shared__ unsigned fired_l[BMTK_RES_FIRED_SLOTS];  // this workgroup's list of the step: neuron + 1
    __shared__ unsigned fired_n[2];  // how many fired in this step and the one before
    const int tid = threadIdx.x;
    const int lane = lane_id();
    // Workgroups are dispatched round-robin over the 8 XCDs (block b runs on XCD
    // b % 8).  Give each XCD a run of consecutive groups so that the segments
    // of a synapse row its workgroups read -- and their offsets -- are
    // contiguous and are fetched into that XCD's L2 once.
    const int per_xcd = (int)gridDim.x >> 3;
    const int g = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    const int ne = (int)s.n_neurons;  // batch 1, at most 1024 elements per compute unit
    const int words = (ne + 63) >> 6;
    const int L = s.ring_slots;
    const int span = r.span;
    const int e0 = g * span;
    const int mine = max(0, min(span, ne - e0));  // groups past the end own nothing
    const bool own = tid < mine;
    const int e = e0 + tid;
    unsigned *act = reinterpret_cast<unsigned *>(ring_l + s.ring_slots * GLIF3_NREC * r.span);
    unsigned *abort_word = s.res_sync + 1;
    unsigned *arrivals = s.res_sync + kBarrierStride;  // [kBarrierWords] counters, kBarrierStride words apart
    // a run before this one gave up and nobody has looked yet: do nothing, so that the failure is still there to see
    // (one thread looks for the whole workgroup, so that all of its threads take the same way)
    if (tid == 0) {
        go_on = load_agent(abort_word) == 0u;
        fired_n[0] = fired_n[1] = 0u;
    }
    __syncthreads();
    if (!go_on) return;
    __syncthreads();  // go_on is written again in the loop

    for (int c = tid; c < L * GLIF3_NREC * span; c += kResBlock) {
        const int dr = c / span, i = c - dr * span;
        ring_l[c] = i < mine ? s.ring[(int64_t)dr * ne + e0 + i] : 0.0f;
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
    __syncthreads();

    // membrane potential probes: this thread's column, and where in the sampling period the call begins
    const int probe_col = (own && s.probe_col) ? s.probe_col[e] : -1;
    int probe_phase = s.probe_col ? (int)((r.step0 + 1) % s.probe_every) : 1;  // 0: sample after this step
    int64_t probe_row = 0;
    const float zero[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
    bool aborted = false;
    int done = 0;  // steps whose update has run
    // the spike record may be split into several lists, one per group of workgroups
    const unsigned rec_ways = s.spike_ways > 1 ? (unsigned)s.spike_ways : 1u;
    const unsigned long long rec_way = blockIdx.x & (rec_ways - 1u), rec_cap = (unsigned long long)s.spike_cap / rec_ways;
    // With as many lists as workgroups this one appends to its list alone: its count lives in a register of every
    // thread (first loaded, written back at the end), a spike's place is that count plus the spike's rank among the
    // workgroup's spikes of the step (the LDS atomic that also builds the list of fired neurons), and no wavefront
    // waits for an atomic on device memory, which the arrivals of a step would queue up behind.
    const bool own_record = !kLate && s.spike_count != nullptr && rec_ways >= gridDim.x;
    unsigned long long rec_count = own_record ? s.spike_count[rec_way * BMTK_RECORD_COUNT_STRIDE] : 0ull;
    const bool count_fired = own_record || (kLists && s.res_fired != nullptr);
    // the input events of the step pulled in step t, u = t-1-B, are in_events[ka, kb); the bound for the
    // next step is fetched a step ahead.  Steps before 0 have no events (in_ptr[0] = 0).
    const int B = r.offset;
    auto in_bound = [&](int64_t i) -> int64_t { return (s.in_ptr && i > 0) ? s.in_ptr[i] : 0; };
    int opaque_zero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(opaque_zero));
    int64_t ka = 0, kb = in_bound(r.step0 - B);
#ifdef BMTK_RES_PROFILE
    long long prof_prev = 0, prof_c1 = 0;
#endif
    // Wait until every workgroup has arrived at the barrier of step j of this call (all threads call it;
    // false = the run was given up).  No acquire fence: it would invalidate this XCD's L2 every step, and
    // the only data other workgroups write during the run are the ballots, which are read with agent-scope
    // loads that bypass the non-coherent caches.
    auto counter_of = [&](int j) { return arrivals + ((j < 0 ? 0 : j) & (kBarrierWords - 1)) * kBarrierStride; };
    auto poll = [&](int j) -> int {  // one thread: 1 = everybody arrived at step j, 0 = given up
        const unsigned *word = counter_of(j);
        const unsigned target = j < 0 ? 0u : gridDim.x * (unsigned)(j / kBarrierWords + 1);
        unsigned spins = 0;
        auto arrived = [&]() {  // the loads of a look travel together
            unsigned n[kWays];
#pragma unroll
            for (int x = 0; x < kWays; ++x) n[x] = load_agent(word + x * kWayStride);
            unsigned sum = 0;
#pragma unroll
            for (int x = 0; x < kWays; ++x) sum += n[x];
            return sum;
        };
        while (arrived() < target) {
            if (load_agent(abort_word) != 0u) return 0;
            if (++spins > (s.res_spin_limit ? s.res_spin_limit : kMaxSpin)) {
                __hip_atomic_store(abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return 0;
            }
            __builtin_amdgcn_s_sleep(2);
        }
        return 1;
    };
    auto wait_for = [&](int j) -> bool {
        if (tid == 0) go_on = poll(j);
        __syncthreads();
        return go_on != 0;
    };
    // Without slack, the pull of step t-1-B (in step t) is all that needs the barrier of step t-1, and the
    // update of step t needs neither: when the history has a row to spare (D >= B + 4) the wait for the barrier
    // of step t-1 moves from the end of step t-1 to just before that pull.  By then every workgroup arrived an
    // update and a pull ago, so the wait is over before it begins.  A workgroup writing row t%D may then be up
    // to two steps ahead of one still reading row (t-3-B)%D, hence the spare row.
    const bool defer = !kLate && r.hist >= B + 4;
    // The look itself is taken by the last wavefront, while the others update: its 64 threads own no elements
    // when the span is 960 or less, and the answer, a memory round trip away, is there when the workgroup meets
    // after the update.
    constexpr int kLooker = kResBlock - kWave;
    // ring slot of step t-1 and history rows of steps t and t-1-B, counted along instead of taking three
    // 64-bit remainders per step (every instruction of the loop costs all 16 wavefronts an issue slot)
    auto wrap = [](int64_t a, int m) { return (int)(((a % m) + m) % m); };
    int next_slot_prev = wrap(r.step0 - 1, L), next_row_t = wrap(r.step0, r.hist),
        next_row_p = wrap(r.step0 - 1 - B, r.hist);
    const int n_steps = (int)r.n_steps;
    for (int k = 0; k < n_steps; ++k) {
        const int64_t t = r.step0 + k;
        const int slot_prev = next_slot_prev, row_t = next_row_t, row_p = next_row_p;
        next_slot_prev = slot_prev + 1 == L ? 0 : slot_prev + 1;
        next_row_t = row_t + 1 == r.hist ? 0 : row_t + 1;
        next_row_p = row_p + 1 == r.hist ? 0 : row_p + 1;
        PROF_T(c0);
#ifdef BMTK_RES_PROFILE
        if (k > 0) PROF_ADD(1, prof_prev, c0);
#endif
        // The bound of the next step's events is asked for now and looked at after the pull.  The address gets a
        // zero the compiler cannot see through: a load it knows to be the same in every lane is moved to a scalar
        // register on the spot, and every wavefront would wait for the answer here, at the top of the step.
        const int64_t in_next = t + 1 - B;
        long long kn_lanes = 0;
        if (s.in_ptr && in_next > 0) kn_lanes = s.in_ptr[in_next + opaque_zero];
        if (defer && k > 0 && tid == kLooker) go_on = poll(k - 1);
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
        // only the wavefronts that cover this workgroup's span own a ballot word
        if (lane == 0 && tid < span && (e & ~(kWave - 1)) < ne) {
            __hip_atomic_store(reinterpret_cast<unsigned long long *>(s.work_bits) + (int64_t)row_t * (words + 1) + (e >> 6),
                               m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (s.spike_bits) s.spike_bits[k * s.spike_bits_stride + (e >> 6)] = m;
        }
        // Spike record: a wavefront with spikes takes its places in the list with ONE atomic, whose answer is a
        // memory round trip away.  It is only asked for here and looked at after the pull, so that no wavefront
        // stops for it in the update (which every other wavefront of the workgroup would wait out at the next
        // barrier).
        if (count_fired && m != 0ull && spike) {
            const unsigned at = atomicAdd(&fired_n[k & 1], 1u);
            if (kLists && s.res_fired && at < BMTK_RES_FIRED_SLOTS) fired_l[at] = (unsigned)e + 1u;
            if (own_record && rec_count + at < rec_cap) {
                const unsigned long long idx = rec_way * rec_cap + rec_count + at;
                s.spike_step[idx] = (int32_t)t;
                s.spike_elem[idx] = (int32_t)e;
                if (s.spike_frac) s.spike_frac[idx] = frac;
            }
        }
        unsigned long long rec_base = 0ull;
        if (s.spike_count && !own_record && m != 0ull && lane == __ffsll((long long)m) - 1)
            rec_base = atomicAdd(s.spike_count + rec_way * BMTK_RECORD_COUNT_STRIDE, (unsigned long long)__popcll(m));
        done = k + 1;
        // With no slack (S = 0) the arrival is signalled early in the pull so that the barrier fills while
        // the pull runs.  With slack nobody is waiting for this step yet: the arrival moves behind the pull,
        // which saves a workgroup barrier, and the counters are only looked at every `check` steps.
        constexpr bool late = kLate;
        const int check = late ? r.check : 1;
        unsigned *const my_counter = counter_of(k) + (blockIdx.x & (kWays - 1)) * kWayStride;
        if (!late) {
            // the workgroup meets, so that the looker's answer can be read
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __syncthreads();
            PROF_T(c1);
            PROF_ADD(0, c0, c1);
            PROF_BLK(0, c0, c1);
#ifdef BMTK_RES_PROFILE
            prof_c1 = c1;
#endif
            if (defer && k > 0 && !go_on) {  // written before the workgroup met above
                aborted = true;
                break;
            }
            // the list of this step, complete since the workgroup met: out with it, like the ballots (the arrival
            // waits for the store), and the count back to zero (it is added to again after the barriers of the pull)
            if (own_record) rec_count += fired_n[k & 1];
            if (kLists && s.res_fired && tid < BMTK_RES_FIRED_SLOTS && g < r.n_groups) {  // (the grid is rounded up)
                const unsigned n = fired_n[k & 1];
                const unsigned word = n > BMTK_RES_FIRED_SLOTS ? BMTK_RES_FIRED_MANY : ((unsigned)tid < n ? fired_l[tid] : 0u);
                __hip_atomic_store(s.res_fired + ((int64_t)row_t * r.n_groups + g) * BMTK_RES_FIRED_SLOTS + tid, word,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            // the other count, last read a barrier ago and next added to a barrier on, back to zero
            if (count_fired && tid == 0) fired_n[(k + 1) & 1] = 0u;
        }
        PROF_T(c2);
#ifdef BMTK_RES_PROFILE
        if (!kLate) PROF_ADD(7, prof_c1, c2);
#endif
        // 2. + 3. pull the spikes and input events of step t-1-B (the first step of a call pulls nothing: the
        //    call before it closed with that pull) and, without slack, arrive at the barrier of step t on the
        //    way, so that the barrier fills while the pull runs.  The arrival tells the other workgroups that
        //    this one's ballots of step t can be read: it must not move before every wavefront's ballot store
        //    (a write-through, device-coherent store) has been acknowledged, which each wavefront waits for
        //    together with the first loads of the pull.  No L2 write-back is needed: nothing else written
        //    inside the loop is read by another workgroup before the kernel ends.
        bool arrived = false;
        if (k > 0 && t - 1 - B >= 0 && mine > 0)
            arrived = pull_step<kUnifiedTables, kLists>(s, r, g, row_p, slot_prev, ring_l, act, scan_l, e0, words, ka, kb,
                                               late ? nullptr : my_counter);
        if (!late && !arrived) {
            wait_vector_memory();
            __syncthreads();
            if (tid == 0) __hip_atomic_fetch_add(my_counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        ka = kb;
        kb = ((int64_t)__builtin_amdgcn_readfirstlane((int)(kn_lanes >> 32)) << 32) |
             (int64_t)(unsigned)__builtin_amdgcn_readfirstlane((int)kn_lanes);
        if (s.spike_count && !own_record && m != 0ull) {  // the places asked for above: the answer has long arrived
            unsigned long long idx = bcast_u64(rec_base, __ffsll((long long)m) - 1) + (unsigned long long)lane_prefix(m);
            if (spike && idx < rec_cap) {
                idx += rec_way * rec_cap;  // this workgroup's list
                s.spike_step[idx] = (int32_t)t;
                s.spike_elem[idx] = (int32_t)e;
                if (s.spike_frac) s.spike_frac[idx] = frac;
            }
        }
        if (late) {
            // every wavefront's ballot store has been acknowledged before the workgroup meets and arrives
            wait_vector_memory();
            __syncthreads();
        }
        // (without slack no workgroup barrier is needed here: pull_step ends with one, and the word thread 0
        //  writes below was last read before the barrier that precedes the arrival)
        PROF_T(c3);
        if (late && tid == 0) __hip_atomic_fetch_add(my_counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // 4. every `check` steps (each step without slack) wait until every workgroup has published
        //    step k - S + (check - 1): enough for the steps up to the next look
        if (late && k % check != check - 1 && k + 1 < n_steps) continue;
        bool ok = true;
        if (!defer) {
            int j = late ? k - r.slack + (check - 1) : k;  // step of this call everybody must have published
            ok = wait_for(j < k ? j : k);
        }
        PROF_T(c4);
        PROF_ADD(2, c2, c3);
        PROF_ADD(3, c3, c4);
        PROF_BLK(1, c2, c3);
        PROF_BLK(2, c3, c4);
#ifdef BMTK_RES_PROFILE
        prof_prev = c4;
#endif
        if (!ok) {
            aborted = true;
            break;
        }
    }
    // with the deferred wait the closing pull is the first to need the barrier of the last step
    if (defer && !aborted && done > 0 && !wait_for(done - 1)) aborted = true;

    if (!aborted && done > 0) {
        // closing: spikes and inputs of the last step (less the delay offset), then fold the last slot
        const int64_t tl = r.step0 + done - 1;
        if (tl - B >= 0 && mine > 0)
            pull_step<kUnifiedTables, kLists>(s, r, g, wrap(tl - B, r.hist), wrap(tl, L), ring_l, act, scan_l, e0, words, ka,
                                              kb);
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
    if (own_record && tid == 0) s.spike_count[rec_way * BMTK_RECORD_COUNT_STRIDE] = rec_count;
    for (int c = tid; c < L * GLIF3_NREC * span; c += kResBlock) {
        const int dr = c / span, i = c - dr * span;
        if (i < mine) s.ring[(int64_t)dr * ne + e0 + i] = ring_l[c];
    }
}

__global__ void zero_words_kernel(unsigned *w, int n)
{
    if ((int)threadIdx.x < n) w[threadIdx.x] = 0u;
}

// abort flag and arrival counters of a resident run
__global__ void zero_sync_kernel(unsigned *sync)
{
    // word 1, the abort flag, is left alone: it stays set until the host has read and cleared it
    if (threadIdx.x == 0) sync[0] = 0u;
    for (int c = threadIdx.x; c < kWays * kBarrierWords; c += blockDim.x) sync[(1 + c) * kBarrierStride] = 0u;
}

__global__ __launch_bounds__(kBlock) void segment_offsets_kernel(int64_t n_rows, const int32_t *__restrict__ indptr,
                                                                 const int32_t *__restrict__ indices, int span,
                                                                 int n_groups, uint32_t *__restrict__ seg,
                                                                 int32_t *__restrict__ unsorted)
{
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int64_t total = n_rows * (int64_t)(n_groups + 1);
    if (idx >= total) return;
    const int64_t row = idx / (n_groups + 1);
    const int g = (int)(idx - row * (n_groups + 1));
    int lo = indptr[row], hi = indptr[row + 1];
    if (g == 0) {
        // one thread per row checks the ordering the binary searches rely on
        for (int p = lo + 1; p < hi; ++p)
            if (indices[p] < indices[p - 1]) {
                *unsorted = 1;
                break;
            }
    }
    const int64_t bound = (int64_t)g * span;  // first position with target >= bound
    while (lo < hi) {
        const int mid = lo + ((hi - lo) >> 1);
        if ((int64_t)indices[mid] < bound)
            lo = mid + 1;
        else
            hi = mid;
    }
    seg[idx] = (uint32_t)lo;
}

int simulate_resident(const bmtk_glif3_sim &s, int64_t step0, int64_t n_steps, hipStream_t stream)
{
    if (s.res_groups == 1) return simulate_resident_solo(s, step0, n_steps, stream);  // the whole network in one workgroup
    if (n_steps >= (1ll << 31)) {
        set_error("glif3_simulate_fwd: a resident call covers fewer than 2^31 steps");
        return BMTK_E_ARG;
    }
    const int hist = s.hist_slots ? s.hist_slots : 3;
    int slack = s.delay_offset < hist - 3 - s.delay_offset ? s.delay_offset : hist - 3 - s.delay_offset;
    slack = slack < kMaxSlack ? slack : kMaxSlack;
    Resident r{step0, n_steps, s.res_span, s.res_groups, s.delay_offset, hist, slack, slack / 2 + 1};
    const size_t lds = (size_t)s.ring_slots * GLIF3_NREC * s.res_span * sizeof(float) + kActCap * sizeof(int);
    // one table for recurrent and input rows lets the kernel drop the second set of pointers
    const bool has_inputs = s.in_ptr != nullptr;
    const int64_t rows = s.n_neurons + (has_inputs ? s.n_inputs : 0);
    const bool unified = s.rec_seg != nullptr && rows < (1ll << 24) && rows * (s.res_groups + 1) < (1ll << 32) &&
                         (!has_inputs || (s.inp_packed == s.rec_packed &&
                                          s.inp_seg == s.rec_seg + s.n_neurons * (int64_t)(s.res_groups + 1)));
    const int form = !unified || s.probe_col != nullptr ? kFormAny : (s.spike_count != nullptr ? kFormRecord : kFormLean);
    const void *const kernels[2][3] = {
        {reinterpret_cast<const void *>(sim_resident_kernel<false, kFormAny>),
         reinterpret_cast<const void *>(sim_resident_kernel<false, kFormRecord>),
         reinterpret_cast<const void *>(sim_resident_kernel<false, kFormLean>)},
        {reinterpret_cast<const void *>(sim_resident_kernel<true, kFormAny>),
         reinterpret_cast<const void *>(sim_resident_kernel<true, kFormRecord>),
         reinterpret_cast<const void *>(sim_resident_kernel<true, kFormLean>)}};
    const void *kernel = kernels[slack > 0 ? 1 : 0][form];
    hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (err != hipSuccess) {
        set_error("glif3_simulate_fwd: resident mode needs %zu bytes of LDS: %s", lds, hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    const unsigned grid = 8u * (unsigned)((s.res_groups + 7) / 8);
    // every workgroup must be on the device at once: the grid barrier has no other way to fill
    int dev = 0, n_cu = 0, per_cu = 0;
    (void)hipGetDevice(&dev);
    (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
    (void)hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kResBlock, lds);
    if ((int64_t)per_cu * n_cu < (int64_t)grid) {
        set_error("glif3_simulate_fwd: %u resident workgroups do not fit the device (%d compute units x %d)", grid,
                  n_cu, per_cu);
        return BMTK_E_LAUNCH;
    }
    hipLaunchKernelGGL(zero_sync_kernel, dim3(1), dim3(kBlock), 0, stream, s.res_sync);
    bmtk_glif3_sim s_copy = s;
    // BMTK_AMD_PLAIN_LAUNCH=1 uses an ordinary launch (co-residency then rests on the occupancy check
    // above and an otherwise idle device); for tools that cannot follow cooperative launches.
    const char *plain = getenv("BMTK_AMD_PLAIN_LAUNCH");
    void *args[] = {&s_copy, &r};
    if (plain && plain[0] == '1')
        err = hipLaunchKernel(kernel, dim3(grid), dim3(kResBlock), args, lds, stream);
    else
        err = hipLaunchCooperativeKernel(kernel, dim3(grid), dim3(kResBlock), args, lds, stream);
    if (err != hipSuccess) {
        set_error("glif3_simulate_fwd: launch of %u resident workgroups failed: %s", grid, hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    return BMTK_OK;
}

}  // namespace bmtk

using namespace bmtk;

#ifdef BMTK_RES_PROFILE
extern "C" void bmtk_debug_read_prof(unsigned long long *out)
{
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_prof), sizeof(g_prof));
}
extern "C" void bmtk_debug_read_prof_blocks(unsigned long long *out)
{
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_prof_blk), sizeof(g_prof_blk));
}
#endif

extern "C" int bmtk_csr_segment_offsets(int64_t n_rows, const int32_t *indptr, const int32_t *indices, int32_t span,
                                        int32_t n_groups, uint32_t *seg, int32_t *unsorted, void *stream)
{
    BMTK_REQUIRE(n_rows > 0 && indptr && indices && seg && unsorted, "csr_segment_offsets: bad sizes or null pointers");
    BMTK_REQUIRE(span > 0 && n_groups > 0, "csr_segment_offsets: span and n_groups must be positive");
    const int64_t total = n_rows * (int64_t)(n_groups + 1);
    BMTK_REQUIRE(total < (1ll << 40), "csr_segment_offsets: table too large");
    hipLaunchKernelGGL(segment_offsets_kernel, dim3((unsigned)((total + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, n_rows, indptr, indices, span, n_groups, seg, unsorted);
    BMTK_CHECK_LAUNCH("csr_segment_offsets");
    return BMTK_OK;
}
