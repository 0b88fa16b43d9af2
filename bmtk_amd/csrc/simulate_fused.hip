// Batched forward simulation: pull and update fused, TWO steps per pass over
// the synapse table.
//
// A wavefront advances 64 elements at a time: the 64 / batch neurons of a group
// with all their trials (batch 8, 16, 32 or 64), lane = (neuron of the group,
// trial).  In the launch for steps t and t+1 it
//   1. streams the rows of the group's neurons in the joint target-major table
//      (recurrent synapses and input synapses, lane = synapse) ONCE and asks of
//      every synapse two things: did its source fire in some trial of step
//      t-1-delay (then it contributes to what arrives in step t-1) and of step
//      t-delay (arrival in step t) -- two bit maps of the last L steps in LDS.
//      The synapses that pass fetch their sources' trial masks from the joint
//      history and add their weights into 64-bit fixed-point sums in LDS, one
//      per (arrival step, receptor, neuron of the group, trial): exact and
//      independent of the order of the additions.  Both questions only concern
//      spikes of steps <= t-1, which earlier launches left complete: delays are
//      at least one step, so nothing that fires in step t can arrive before
//      step t+1, whose arrivals the NEXT launch sums.  The table -- three
//      quarters of all bytes a step moves -- is thus read once per two steps;
//   2. folds the first sums into y1 and advances the 64 elements through step
//      t, folds the second sums and advances them through step t+1, state in
//      registers in between (NEST adds the arrivals of a step at the end of
//      that step and nothing reads y1 before the next update, so adding them at
//      the top of that update performs the same two rounded operations);
//   3. writes the spike bits of both steps -- one 64-bit word each -- into rows
//      t and t+1 of the history, where later launches find them.
// No arrival sum passes through device memory.  A workgroup owns a run of
// consecutive groups and its wavefronts take them one by one from a counter in
// LDS; two of them first turn the workgroup's share of the input events of
// steps t and t+1 into bits of the same history rows, and deliver the few ids
// that occur twice within a step (bits hold an id once) as events into the
// ring, which the update folds along.
#include "common.hpp"
#include "glif3_update.hpp"
#include "propagate.hpp"
#include "pull_common.hpp"
#include "sim_internal.hpp"

namespace bmtk {

constexpr int kFuseBlock = 1024;
constexpr int kFuseWaves = kFuseBlock / kWave;
constexpr int kFuseAhead = 2;  // table blocks of 2 KB per wavefront, in flight or at hand (4 and 5: no faster)
constexpr size_t kFuseLdsMax = 150u * 1024u;  // one workgroup per compute unit

struct FusedLaunch {
    int64_t t0;          // first step of the launch (closing launch: one past the last step)
    int64_t out_row;     // row of spike_bits / save_v / save_flags of the first step (the second: one further)
    int64_t probe_row0, probe_row1;  // rows of probe_v, -1: not a sampled step
    int64_t n_in_words;  // 64-bit words of the input part of a history row
    int n_main;          // workgroups
    int n_sub;           // steps the launch advances: 2, 1 (the odd one of a call), 0 (closing launch: fold only)
    int fold0;           // the arrivals of step t0-1 are pulled and folded first (every launch but a call's first)
    int use_ring;        // ring slots may hold arrivals (ids repeated within a step)
    int in_bits;         // the input events of the launch's steps become bits of their history rows
    int repeats;         // the repeated ids of the launch's steps are delivered as events
    int H;               // rows of the history (L + 4)
    int Lr;              // slots of the ring (L + 2)
    int n_w32;           // words per row of the activity map
    int shift;           // sources per bit of the activity map: 2^shift
};

// One block of the synapse stream a wavefront works through: positions [base, min(base + 256, p1)) of the packed
// table, all of one row.
struct FuseBlockDesc {
    int row;       // -1: past the end (an empty block of no row)
    int base, p1;
    bool first;    // first block of the first row of its group: the group's state is asked for
    bool last;     // last block of its row: the row's synapses are complete after it
    bool closes;   // ... and the row is the last of its group: the group is closed after it
};

// The groups a wavefront takes from its workgroup's counter, as a stream of blocks.  The bounds of the row after the
// current one (which may belong to the next group, taken from the counter a group ahead) are fetched a row ahead.
// Everything here is the same in all lanes.
template <int kRows>
struct GroupCursor {
    const int32_t *__restrict__ indptr;
    int *counter;
    int n, g_end;
    int grp, row, row_end;  // group and row at hand, one past the group's last row
    int q, p1;              // what is left of the row
    int ngrp;               // the group after (>= g_end: none)
    int nrow, np0, np1;     // the row after (-1: none) and its bounds
    bool at_start;

    __device__ __forceinline__ int grab()
    {
        int g = 0;
        if (lane_id() == 0) g = atomicAdd(counter, 1);
        return __builtin_amdgcn_readfirstlane(g);
    }
    __device__ __forceinline__ void look_ahead()
    {
        nrow = -1;
        if (row >= 0 && row + 1 < row_end)
            nrow = row + 1;
        else if (ngrp < g_end)
            nrow = ngrp * kRows;
        if (nrow >= 0) {
            np0 = indptr[nrow];
            np1 = indptr[nrow + 1];
        }
    }
    __device__ __forceinline__ void start(const int32_t *ip, int n_rows, int groups_end, int *ctr)
    {
        indptr = ip;
        counter = ctr;
        n = n_rows;
        g_end = groups_end;
        grp = grab();
        ngrp = grab();
        row = -1;
        row_end = q = p1 = np0 = np1 = 0;
        at_start = true;
        if (grp < g_end) {
            row = grp * kRows;
            row_end = min(n, row + kRows);
            q = indptr[row];
            p1 = indptr[row + 1];
        }
        look_ahead();
    }
    __device__ __forceinline__ FuseBlockDesc next()
    {
        if (row < 0) return FuseBlockDesc{-1, 0, 0, false, false, false};
        FuseBlockDesc b{row, q, p1, at_start, false, false};
        at_start = false;
        q += kPullChunks * kWave;
        if (q >= p1) {
            b.last = true;
            b.closes = row + 1 == row_end;
            const bool new_group = b.closes;
            row = nrow;
            q = np0;
            p1 = np1;
            if (new_group) {
                at_start = true;
                grp = ngrp;
                row_end = min(n, (grp + 1) * kRows);
                if (row >= 0) ngrp = grab();
            }
            look_ahead();
        }
        return b;
    }
};

template <int kBatch>
__global__ __launch_bounds__(kFuseBlock) void sim_fused_kernel(bmtk_glif3_sim s, FusedLaunch q)
{
    // accumulators [wavefront][arrival step][receptor][64], stages [wavefront][arrival step][64], then the activity
    // maps of the steps t0-1 .. t0-L
    extern __shared__ unsigned long long fuse_lds[];
    __shared__ int next_group;
    static_assert(kBatch == 8 || kBatch == 16 || kBatch == 32 || kBatch == 64, "whole neurons per wavefront");
    constexpr int kRows = kWave / kBatch;  // neurons of a group
    const int bid = (int)blockIdx.x;
    const int n = (int)s.n_neurons;
    const int64_t ne = (int64_t)n * kBatch;
    const int L = s.ring_slots, H = q.H, Lr = q.Lr;
    const unsigned lane = (unsigned)lane_id();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    const bool pull_a = q.fold0 != 0, pull_b = q.n_sub == 2;  // what arrives in step t0-1 / in step t0 is summed
    constexpr int kAccWave = 2 * GLIF3_NREC * kWave, kStageWave = 2 * kWave;
    unsigned long long *acc = fuse_lds + wave * kAccWave;
    uint2 *stage = reinterpret_cast<uint2 *>(fuse_lds + kFuseWaves * kAccWave) + wave * kStageWave;
    uint32_t *any_l = reinterpret_cast<uint32_t *>(fuse_lds + kFuseWaves * (kAccWave + kStageWave));
    // ring map: bit i of row (u % Lr) = some ring cell of neuron i in slot u % Lr holds an arrival (set where
    // repeated ids are delivered, cleared by the neuron's owner when it takes the cells along); behind the H rows
    // of the activity map
    const int ring_map_words = (n + 31) >> 5;
    uint32_t *__restrict__ ring_map = s.fuse_any + (int64_t)H * q.n_w32;

    // the workgroup's run of groups, and the counter its wavefronts take them from
    const int n_groups = (n + kRows - 1) / kRows;
    const int per_wg = (n_groups + q.n_main - 1) / q.n_main;
    const int g_first = bid * per_wg, g_end = min(n_groups, g_first + per_wg);
    if (threadIdx.x == 0) next_group = g_first;
    // the activity rows of the steps the NEXT launch writes start empty (no launch reads them before)
    for (int k = 0; k < 2; ++k) {
        uint32_t *__restrict__ next = s.fuse_any + ((q.t0 + q.n_sub + k) % H) * q.n_w32;
        for (int i = bid * kFuseBlock + (int)threadIdx.x; i < q.n_w32; i += q.n_main * kFuseBlock) next[i] = 0u;
    }
    if (pull_a || pull_b) {
        // the activity maps of the steps t0-1 .. t0-L, one after the other
        for (int k = 0; k < L; ++k) {
            const int64_t u = q.t0 - 1 - k;
            const uint32_t *__restrict__ src = s.fuse_any + (((u % H) + H) % H) * q.n_w32;
            for (int i = threadIdx.x; i < q.n_w32; i += kFuseBlock) any_l[k * q.n_w32 + i] = src[i];
        }
    }
    __syncthreads();

    if (wave == kFuseWaves - 1 && q.in_bits) {
        // ---- the workgroup's share of the input events of the launch's steps as bits of their history rows: a
        //      lane per 64-bit word; the events of a step are ascending, so a word's events are one run of the
        //      list, found by bisection.  (Read by later launches.)  The wavefront then takes groups like the
        //      others, which have taken a few more meanwhile. ----
        const int64_t in_word0 = s.fuse_in_base * kBatch / 64;
        for (int sub = 0; sub < q.n_sub; ++sub) {
            const int64_t t = q.t0 + sub;
            const int64_t k0 = s.in_ptr[t], k1 = s.in_ptr[t + 1];
            uint64_t *__restrict__ hist_row = s.work_bits + (t % H) * s.fuse_hist_stride;
            uint32_t *__restrict__ any_row = s.fuse_any + (t % H) * q.n_w32;
            for (int64_t w = (int64_t)bid * kWave + lane; w < q.n_in_words; w += (int64_t)q.n_main * kWave) {
                const int64_t lo = w * 64;
                int64_t a = k0, b = k1;
                while (a < b) {
                    const int64_t mid = (a + b) >> 1;
                    if ((int64_t)s.in_events[mid] < lo)
                        a = mid + 1;
                    else
                        b = mid;
                }
                unsigned long long bits = 0ull;
                for (; a < k1; ++a) {
                    const int64_t ev = s.in_events[a];
                    if (ev >= lo + 64) break;
                    bits |= 1ull << (ev - lo);
                }
                hist_row[in_word0 + w] = bits;
                if (bits != 0ull) {
                    const unsigned long long field = kBatch == 64 ? ~0ull : ((1ull << kBatch) - 1ull);
#pragma unroll
                    for (int f = 0; f < kRows; ++f) {
                        if ((bits >> (f * (kBatch & 63))) & field) {
                            const unsigned g = (unsigned)(s.fuse_in_base + w * kRows + f) >> q.shift;
                            atomicOr(any_row + (g >> 5), 1u << (g & 31u));
                        }
                    }
                }
            }
        }
    }
    if (wave == kFuseWaves - 2 && q.repeats) {
        // ---- ids that occur more than once among the input events of the launch's steps: the occurrences after
        //      the first, as events into the ring.  Those of step u land in slots u+1 .. u+L-1; this launch takes
        //      slots t0-1 and t0 along, which the launches before it completed (the ring has L+2 slots, so that
        //      slot t0+L is neither of the two) ----
        const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(s.inp_packed);
        for (int sub = 0; sub < q.n_sub; ++sub) {
            const int64_t t = q.t0 + sub;
            const int64_t k0 = s.in_repeat_ptr[t], k1 = s.in_repeat_ptr[t + 1];
            for (int64_t k = k0 + bid; k < k1; k += q.n_main) {
                const int e = s.in_repeat_events[k];
                const int j = (int)((uint32_t)e / (uint32_t)kBatch), b = e - j * kBatch;
                const int p1 = s.inp_indptr[j + 1];
                for (int p = s.inp_indptr[j] + (int)lane; p < p1; p += kWave) {
                    const uint2 sy = rows[p];
                    const int slot = (int)((t + (int64_t)(sy.x >> 26)) % Lr);
                    const int64_t i = sy.x & 0xFFFFFFu;
                    atomicAdd(s.ring + ((int64_t)(slot * GLIF3_NREC + (int)((sy.x >> 24) & 3u)) * ne + i * kBatch + b),
                              __uint_as_float(sy.y));
                    atomicOr(ring_map + (int64_t)slot * ring_map_words + (i >> 5), 1u << (i & 31));
                }
            }
        }
    }

    // ---- a group at a time: pull, fold, update, fold, update ----
    const unsigned uw32 = (unsigned)q.n_w32, ushift = (unsigned)q.shift, umax_dd = (unsigned)(L - 2);
    const unsigned sub_lane = lane / (unsigned)kBatch;  // this lane's neuron within a group
    // Asked for when a group's first block turns up, used when the group is closed: the state of its 64 elements,
    // their propagators (every lane its neuron's column) and the words of the ring map that hold the group's bits.
    Glif3Elem st;
    Glif3Prop pr;
    unsigned ring_word0 = 0u, ring_word1 = 0u;
    uint32_t *__restrict__ ring_map0 = ring_map + (int64_t)(((q.t0 - 1) % Lr + Lr) % Lr) * ring_map_words;
    uint32_t *__restrict__ ring_map1 = ring_map + (int64_t)(q.t0 % Lr) * ring_map_words;

    // Element accesses: a scalar base (array + plane k of ne elements) and this lane's 32-bit byte offset
    // (n_neurons * batch < 2^30, checked by the caller), the address form that needs no 64-bit lane arithmetic.
    const size_t plane = (size_t)ne * sizeof(float);
    auto ldf = [&](const float *base, int k, unsigned boff) {
        return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(base) + k * plane + boff);
    };
    auto stf = [&](float *base, int k, unsigned boff, float v) {
        *reinterpret_cast<float *>(reinterpret_cast<char *>(base) + k * plane + boff) = v;
    };
    // All lanes load, whatever they hold (the lanes past the last neuron of the network load the last neuron's
    // values and keep them to themselves): a load under a condition would have to be waited for at once, where the
    // two ways meet again.
    auto load_group = [&](int grp) {
        const int row = min(grp * kRows + (int)sub_lane, n - 1);
        const unsigned e = (unsigned)row * (unsigned)kBatch + (lane & (unsigned)(kBatch - 1));
        const unsigned boff = e * 4u;
        const int64_t col = s.class_id ? (int64_t)s.class_id[row] : (int64_t)row;
        pr.load(s.prop, s.prop_stride, col);
        if (q.use_ring) {
            ring_word0 = ring_map0[(grp * kRows) >> 5];
            ring_word1 = ring_map1[(grp * kRows) >> 5];
        }
        if (q.n_sub > 0) {
            st.V = ldf(s.V, 0, boff);
            st.ref = *reinterpret_cast<const int32_t *>(reinterpret_cast<const char *>(s.ref) + boff);
#pragma unroll
            for (int k = 0; k < GLIF3_NASC; ++k) st.asc[k] = ldf(s.asc, k, boff);
#pragma unroll
            for (int k = 0; k < GLIF3_NREC; ++k) {
                st.y1[k] = ldf(s.y1, k, boff);
                st.y2[k] = ldf(s.y2, k, boff);
            }
        }
    };
    // what is left to do for a group once its arrival sums are known: a0 what arrived in step t0-1, a1 in step t0
    auto finish_group = [&](int grp, float (&a0)[GLIF3_NREC], float (&a1)[GLIF3_NREC]) {
        const int row = grp * kRows + (int)sub_lane;
        const bool on = row < n;  // this lane holds an element
        const unsigned e = (unsigned)(grp * kRows) * (unsigned)kBatch + lane, boff = e * 4u;
        // the ring cells of one slot, where an id repeated within a step reached this neuron (rare)
        auto take_ring = [&](int64_t step, unsigned word, uint32_t *map_row, float (&a)[GLIF3_NREC]) {
            if (q.use_ring && on && ((word >> ((unsigned)row & 31u)) & 1u)) {
                float *cells = s.ring + (int64_t)((step % Lr + Lr) % Lr) * GLIF3_NREC * ne;
                float v[GLIF3_NREC];
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) v[k] = ldf(cells, k, boff);
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) {
                    stf(cells, k, boff, 0.0f);
                    a[k] = v[k] + a[k];
                }
                if ((lane & (unsigned)(kBatch - 1)) == 0u) atomicAnd(map_row + (row >> 5), ~(1u << ((unsigned)row & 31u)));
            }
        };
        if (q.fold0) take_ring(q.t0 - 1, ring_word0, ring_map0, a0);
        if (q.n_sub == 0) {
            // closing launch: what arrived in the last step enters y1, as at the end of that step
            if (on) {
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) stf(s.y1, k, boff, ldf(s.y1, k, boff) + a0[k] * pr.psc0[k]);
            }
            return;
        }
        // one step: fold, update, the step's outputs
        auto one_step = [&](int sub, bool fold, const float (&a)[GLIF3_NREC], int64_t probe_row) {
            const int64_t t = q.t0 + sub, out_row = q.out_row + sub;
            bool spike = false;
            float frac = 0.0f;
            if (on) {
                if (fold) {
#pragma unroll
                    for (int k = 0; k < GLIF3_NREC; ++k) st.y1[k] = st.y1[k] + a[k] * pr.psc0[k];
                }
                const float zero[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
                const float I = s.i_ext ? ldf(s.i_ext, 0, boff) : 0.0f;
                const int ref_before = st.ref;
                spike = glif3_update(st, pr, s.h, zero, I, &frac);
                if (probe_row >= 0) {
                    const int pc = *reinterpret_cast<const int32_t *>(reinterpret_cast<const char *>(s.probe_col) + boff);
                    if (pc >= 0) s.probe_v[probe_row * s.probe_stride + pc] = st.V;
                }
                if (s.save_v) {
                    stf(s.save_v + out_row * ne, 0, boff, st.V);
                    (s.save_flags + out_row * ne)[e] = (uint8_t)((spike ? BMTK_F_SPIKE : 0) |
                                                                  (ref_before == 0 ? BMTK_F_INTEGRATING : 0) |
                                                                  (ref_before > 0 && st.ref == 0 ? BMTK_F_RESET : 0));
                }
            }
            // the group's 64 elements are one word of spike bits
            const unsigned long long m = __ballot(spike);
            if (lane == 0) {
                s.work_bits[(t % H) * s.fuse_hist_stride + grp] = m;
                if (s.spike_bits) s.spike_bits[out_row * s.spike_bits_stride + grp] = m;
            }
            if (m != 0ull && on && (lane & (unsigned)(kBatch - 1)) == 0u) {
                const unsigned long long field = kBatch == 64 ? ~0ull : ((1ull << kBatch) - 1ull);
                if ((m >> (sub_lane * (unsigned)(kBatch & 63))) & field) {
                    const unsigned g = (unsigned)row >> ushift;
                    atomicOr(s.fuse_any + (t % H) * q.n_w32 + (g >> 5), 1u << (g & 31u));
                }
            }
            if (s.spike_count && m != 0ull) {
                // one counter bump per wavefront, record slots handed out in lane order
                const int leader = __ffsll((long long)m) - 1;
                unsigned long long base = 0ull;
                const unsigned ways = s.spike_ways > 1 ? (unsigned)s.spike_ways : 1u;
                const unsigned long long way = (unsigned)bid & (ways - 1u), way_cap = (unsigned long long)s.spike_cap / ways;
                if ((int)lane == leader)
                    base = atomicAdd(s.spike_count + way * BMTK_RECORD_COUNT_STRIDE, (unsigned long long)__popcll(m));
                base = bcast_u64(base, leader);
                unsigned long long idx = base + (unsigned long long)lane_prefix(m);
                if (spike && idx < way_cap) {
                    idx += way * way_cap;
                    s.spike_step[idx] = (int32_t)t;
                    s.spike_elem[idx] = (int32_t)e;
                    if (s.spike_frac) s.spike_frac[idx] = frac;
                }
            }
        };
        one_step(0, q.fold0 != 0, a0, q.probe_row0);
        if (q.n_sub == 2) {
            take_ring(q.t0, ring_word1, ring_map1, a1);
            one_step(1, true, a1, q.probe_row1);
        }
        if (on) {
            stf(s.V, 0, boff, st.V);
            *reinterpret_cast<int32_t *>(reinterpret_cast<char *>(s.ref) + boff) = st.ref;
#pragma unroll
            for (int k = 0; k < GLIF3_NASC; ++k) stf(s.asc, k, boff, st.asc[k]);
#pragma unroll
            for (int k = 0; k < GLIF3_NREC; ++k) {
                stf(s.y1, k, boff, st.y1[k]);
                stf(s.y2, k, boff, st.y2[k]);
            }
        }
    };

    if (!pull_a && !pull_b) {
        // one step as a call's first launch: the closing launch of the call before it has folded everything that
        // arrived, and nothing is summed here
        for (int grp = 0;;) {
            if (lane == 0) grp = atomicAdd(&next_group, 1);
            grp = __builtin_amdgcn_readfirstlane(grp);
            if (grp >= g_end) break;
            float a0[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f}, a1[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
            load_group(grp);
            finish_group(grp, a0, a1);
        }
        return;
    }

    const unsigned hrow_bytes = (unsigned)s.fuse_hist_stride * 8u;  // H * stride * 8 < 2^32 (checked by the caller)
    const unsigned uH = (unsigned)H;
    const char *__restrict__ hist_bytes = reinterpret_cast<const char *>(s.work_bits);
    const bmtk_synapse *__restrict__ packed = s.fuse_packed;
    // Block of the table: 64-bit words at a scalar base, 8 * (lane + u*64) bytes on.  Lanes past the end of the
    // row read its last synapse again (and are ignored later): no branch, the four loads go out back to back.
    // A block past the end or an empty one reads the table's first record the same way: every call issues exactly
    // four loads, which is what lets a turn wait for ITS block only and leave the younger ones in flight (the wait
    // is a count of loads still out, fixed at compile time).
    auto fetch = [&](unsigned long long *dst, const FuseBlockDesc &blk) {
        const bool some = blk.row >= 0 && blk.base < blk.p1;
        const char *__restrict__ src = reinterpret_cast<const char *>(packed) + (some ? (size_t)blk.base * 8u : (size_t)0);
        const unsigned last = some ? (unsigned)(blk.p1 - blk.base) - 1u : 0u;
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u)
            dst[u] = __builtin_nontemporal_load(
                reinterpret_cast<const unsigned long long *>(src + min(lane + u * kWave, last) * 8u));
    };
    // kFuseAhead table blocks per wavefront: the one at hand and the ones after it, whose loads stay in flight
    // while the wavefront works (a buffer is refilled, with the block kFuseAhead ahead, as soon as its turn is
    // over).  The buffers take turns in place -- a register copy of a block still on its way would wait for it --
    // (and a buffer chosen at run time would leave the compiler no way to tell which loads a turn may leave in
    // flight: it then waits for all of them), so the loop body holds one turn per buffer.
    GroupCursor<kRows> cursor;
    cursor.start(s.fuse_indptr, n, g_end, &next_group);
    FuseBlockDesc dq[kFuseAhead];
    unsigned long long d[kFuseAhead][kPullChunks];
#pragma unroll
    for (int k = 0; k < kFuseAhead; ++k) {
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) d[k][u] = 0ull;
        dq[k] = cursor.next();
        fetch(d[k], dq[k]);
    }
    if (dq[0].row < 0) return;
#pragma unroll
    for (int r = 0; r < 2 * GLIF3_NREC; ++r) acc[r * kWave + lane] = 0ull;
    // The sums of one arrival step.  A flush of the stage has two halves a turn apart, so that the masks travel
    // while the wavefront works on the next block: the first takes the staged synapses into registers and asks for
    // their sources' trial masks, the second converts the weights and adds.  A group's closing work waits for its
    // last flushes the same way and is done in the turn after the group's last block.  A flush holds synapses of
    // one row.
    struct Pull {
        unsigned long long *acc;  // [receptor][64]
        uint2 *stage;             // [64]
        unsigned arrive;          // history row of the arrival step: the emitting step of a synapse is `delay` rows back
        int staged;               // entries in the stage (same in all lanes)
        int pend_n;               // synapses of the flush under way (same in all lanes)
        unsigned pend_col;        // ... and the first column of their neuron in the accumulators
        uint2 pend_e;
        unsigned long long pend_m;
    };
    Pull pa{acc, stage, (unsigned)(((q.t0 - 1) % H + H) % H), 0, 0, 0u, make_uint2(0u, 0u), 0ull};
    Pull pb{acc + GLIF3_NREC * kWave, stage + kWave, (unsigned)(q.t0 % H), 0, 0, 0u, make_uint2(0u, 0u), 0ull};
    int fin_grp = -1;  // the group whose closing work is due
    auto flush_issue = [&](Pull &p, int row) {
        if (p.staged == 0) return;
        // every lane loads (the lanes without a synapse the mask of source 0 in the row of the arrival step, and
        // ignore it)
        const uint2 e = p.stage[lane];  // {source | receptor << 24 | delay << 26, weight}
        p.pend_e = (int)lane < p.staged ? e : make_uint2(0u, 0u);
        const unsigned src = p.pend_e.x & 0xFFFFFFu;
        const unsigned back = p.arrive - (p.pend_e.x >> 26);  // history row of the emitting step, by unsigned wrap-around
        const unsigned hrow = min(back, back + uH);
        const char *cell = hist_bytes + (hrow * hrow_bytes + src * (unsigned)(kBatch / 8));
        if (kBatch == 64)
            p.pend_m = *reinterpret_cast<const unsigned long long *>(cell);
        else if (kBatch == 32)
            p.pend_m = *reinterpret_cast<const uint32_t *>(cell);
        else if (kBatch == 16)
            p.pend_m = *reinterpret_cast<const uint16_t *>(cell);
        else
            p.pend_m = *reinterpret_cast<const uint8_t *>(cell);
        p.pend_n = p.staged;
        p.pend_col = (unsigned)(row % kRows) * (unsigned)kBatch;
        p.staged = 0;
    };
    auto flush_complete = [&](Pull &p) {
        if ((int)lane < p.pend_n) {
            unsigned long long *a = p.acc + ((p.pend_e.x >> 24) & 3u) * kWave + p.pend_col;
            const unsigned long long w = to_fixed(__uint_as_float(p.pend_e.y));
            unsigned long long mm = p.pend_m;
            while (mm) {
                const int b = __ffsll((long long)mm) - 1;
                mm &= mm - 1ull;
                atomicAdd(a + b, w);
            }
        }
        p.pend_n = 0;
    };
    // the flushes under way, then the closing work of the group they belonged to
    auto resolve = [&]() {
        flush_complete(pa);
        flush_complete(pb);
        float a0[GLIF3_NREC], a1[GLIF3_NREC];
#pragma unroll
        for (int r = 0; r < GLIF3_NREC; ++r) {
            a0[r] = from_fixed(pa.acc[r * kWave + lane]);
            a1[r] = from_fixed(pb.acc[r * kWave + lane]);
            pa.acc[r * kWave + lane] = 0ull;
            pb.acc[r * kWave + lane] = 0ull;
        }
        finish_group(fin_grp, a0, a1);
        fin_grp = -1;
    };
    auto stage_hits = [&](Pull &p, const unsigned long long (&who)[kPullChunks], const unsigned long long *cd, int row) {
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            const int cnt = __popcll(who[u]);
            if (cnt == 0) continue;
            if (p.staged + cnt > kWave) {
                flush_complete(p);
                flush_issue(p, row);
            }
            if ((who[u] >> lane) & 1ull)
                p.stage[p.staged + lane_prefix(who[u])] = make_uint2((unsigned)cd[u], (unsigned)(cd[u] >> 32));
            p.staged += cnt;
        }
    };
    // one turn: the block `cb` with its table words `cd`; afterwards the buffer takes the block kFuseAhead ahead
    auto turn = [&](FuseBlockDesc &cb, unsigned long long *cd) {
        const unsigned left = (cb.row >= 0 && cb.base < cb.p1) ? (unsigned)(cb.p1 - cb.base) : 0u;
        // activity bits of the four chunks, for both arrival steps (LDS reads, no branch between them): the map of
        // step t0-1-k is row k; a synapse of delay d sends what its source fired in step t0-1-d to arrival step
        // t0-1 (row d) and what it fired in step t0-d to arrival step t0 (row d-1)
        unsigned word_a[kPullChunks], word_b[kPullChunks], bit[kPullChunks];
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            const unsigned tdr = (unsigned)cd[u];
            const unsigned g = (tdr & 0xFFFFFFu) >> ushift;
            bit[u] = g & 31u;
            // delays are 1 .. L-1 (a buffer that was never filled holds delay 0: kept inside the map, ignored below)
            const unsigned at = __umul24(min((tdr >> 26) - 1u, umax_dd), uw32) + (g >> 5);
            word_b[u] = any_l[at];
            word_a[u] = any_l[at + uw32];
        }
        unsigned long long who_a[kPullChunks], who_b[kPullChunks];
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            const bool valid = lane + u * kWave < left;
            who_a[u] = __ballot(valid && pull_a && ((word_a[u] >> bit[u]) & 1u));
            who_b[u] = __ballot(valid && pull_b && ((word_b[u] >> bit[u]) & 1u));
        }
        // the group before: its last masks were asked for a turn ago, its closing work comes before any synapse of
        // this group is added (the one place of a turn where a group is closed)
        if (fin_grp >= 0) resolve();
        if (cb.first) load_group(cb.row / kRows);  // (after that group's closing work, which used the same registers)
        if (pull_a) stage_hits(pa, who_a, cd, cb.row);
        if (pull_b) stage_hits(pb, who_b, cd, cb.row);
        if (cb.last) {
            // (a flush of this row, or of the row before of the same group, may still be under way)
            flush_complete(pa);
            flush_issue(pa, cb.row);
            flush_complete(pb);
            flush_issue(pb, cb.row);
            if (cb.closes) fin_grp = cb.row / kRows;
        }
        cb = cursor.next();
        fetch(cd, cb);
    };
    // One way out of the loop, after a whole round of the buffers: with a way out after every turn the compiler
    // joins them in one block before the loop's head, and from there it looks as if a turn could follow directly
    // on the fetch of its own buffer -- every turn would then wait for all loads in flight.  The turns past a
    // wavefront's last block (at most kFuseAhead - 1) see empty blocks of no row.
    do {
#pragma unroll
        for (int k = 0; k < kFuseAhead; ++k) turn(dq[k], d[k]);
    } while (dq[0].row >= 0);
    if (fin_grp >= 0) resolve();
}

size_t fused_lds_bytes(int L, int n_w32)
{
    return (size_t)kFuseWaves * 2 * (GLIF3_NREC + 1) * kWave * sizeof(unsigned long long) + (size_t)L * n_w32 * 4u;
}

const void *fused_variant(int batch)
{
    switch (batch) {
    case 8: return reinterpret_cast<const void *>(sim_fused_kernel<8>);
    case 16: return reinterpret_cast<const void *>(sim_fused_kernel<16>);
    case 32: return reinterpret_cast<const void *>(sim_fused_kernel<32>);
    default: return reinterpret_cast<const void *>(sim_fused_kernel<64>);
    }
}

int simulate_fused(const bmtk_glif3_sim &s, int64_t step0, int64_t n_steps, hipStream_t stream)
{
    const int batch = s.batch, L = s.ring_slots;
    BMTK_REQUIRE(batch == 8 || batch == 16 || batch == 32 || batch == 64,
                 "glif3_simulate_fwd: the fused form runs batches of 8, 16, 32 or 64");
    BMTK_REQUIRE(s.fuse_indptr && s.fuse_any, "glif3_simulate_fwd: the fused form needs fuse_indptr and fuse_any");
    BMTK_REQUIRE(s.n_neurons * (int64_t)batch < (1ll << 30),
                 "glif3_simulate_fwd: the fused form addresses fewer than 2^30 elements");
    BMTK_REQUIRE(s.delay_offset == 0 && (s.delay_bits == 0 || s.delay_bits == 6) && s.hist_slots == L + 4,
                 "glif3_simulate_fwd: the fused form needs delay_offset 0, the standard packing and hist_slots == ring_slots + 4");
    BMTK_REQUIRE(s.fuse_shift >= 0 && s.fuse_shift <= 16, "glif3_simulate_fwd: fuse_shift must lie in 0..16");
    const int64_t in_base = ((s.n_neurons * batch + 63) / 64) * 64 / batch;
    BMTK_REQUIRE(s.fuse_in_base == in_base, "glif3_simulate_fwd: fuse_in_base must be ceil(n_neurons*batch/64)*64/batch");
    const bool has_inp = s.in_ptr != nullptr;
    BMTK_REQUIRE(s.n_inputs >= 0, "glif3_simulate_fwd: n_inputs must not be negative");
    const int64_t n_in = s.n_inputs;  // input sources of the joint space, with or without events in this call
    BMTK_REQUIRE(in_base + n_in < (1ll << 24),
                 "glif3_simulate_fwd: the fused form indexes fewer than 2^24 sources (neurons and inputs together)");
    const int64_t n_in_words = (n_in * batch + 63) / 64;
    BMTK_REQUIRE(s.fuse_hist_stride >= in_base * batch / 64 + n_in_words + 1,
                 "glif3_simulate_fwd: fuse_hist_stride too small");
    BMTK_REQUIRE((int64_t)(L + 4) * s.fuse_hist_stride < (1ll << 29), "glif3_simulate_fwd: joint history beyond 4 GiB");
    const int64_t groups = (in_base + n_in + (1ll << s.fuse_shift) - 1) >> s.fuse_shift;
    const int n_w32 = (int)((groups + 31) / 32);
    const size_t lds = fused_lds_bytes(L, n_w32);
    BMTK_REQUIRE(lds <= kFuseLdsMax, "glif3_simulate_fwd: the activity map does not fit in LDS; use a larger fuse_shift");
    BMTK_REQUIRE(!s.in_repeat_ptr || (s.in_repeat_events && s.inp_indptr && s.inp_packed),
                 "glif3_simulate_fwd: repeat lists need in_repeat_events and the source-major input table");
    BMTK_REQUIRE(!s.probe_col || (s.probe_v && s.probe_every >= 1 && s.probe_stride >= 1),
                 "glif3_simulate_fwd: probes need probe_v, probe_stride and probe_every >= 1");
    int dev = 0;
    (void)hipGetDevice(&dev);
    static int cu_count[64];  // compute units of every device seen so far
    int n_cu = (dev >= 0 && dev < 64) ? cu_count[dev] : 0;
    if (n_cu <= 0) {
        n_cu = 256;
        (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (dev >= 0 && dev < 64) cu_count[dev] = n_cu;
    }
    const void *kernel = fused_variant(batch);
    static bool asked[4][64];
    const int vi = batch == 8 ? 0 : batch == 16 ? 1 : batch == 32 ? 2 : 3;
    if (dev >= 0 && dev < 64 && !asked[vi][dev]) {
        const hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFuseLdsMax);
        if (err != hipSuccess) {
            set_error("glif3_simulate_fwd: cannot reserve %zu bytes of LDS: %s", kFuseLdsMax, hipGetErrorString(err));
            return BMTK_E_LAUNCH;
        }
        asked[vi][dev] = true;
    }
    FusedLaunch q{};
    const int per_cu = s.fuse_wg_per_cu > 0 ? s.fuse_wg_per_cu : 1;
    const int64_t n_groups = (s.n_neurons * batch + kWave - 1) / kWave;
    const int64_t want = (n_groups + kFuseWaves - 1) / kFuseWaves;
    const int64_t cap = (int64_t)n_cu * per_cu;
    q.n_main = (int)(want < cap ? want : cap);
    q.H = L + 4;
    q.Lr = L + 2;
    q.n_w32 = n_w32;
    q.shift = s.fuse_shift;
    q.n_in_words = n_in_words;
    q.use_ring = s.in_repeat_ptr != nullptr ? 1 : 0;
    // sampled steps: (t + 1) % every == 0; row = how many of them the call has seen before
    auto probe_row = [&](int64_t t) -> int64_t {
        if (!s.probe_col || (t + 1) % s.probe_every != 0) return -1;
        return (t + 1) / s.probe_every - step0 / s.probe_every - 1;
    };
    // two steps per launch; a call's first launch folds nothing (the closing launch of the call before it did), an
    // odd step count leaves one step for the last regular launch, the closing launch folds what arrived in the
    // last step
    for (int64_t k = 0; k <= n_steps;) {
        const bool closing = k == n_steps;
        q.n_sub = closing ? 0 : (int)(n_steps - k < 2 ? n_steps - k : 2);
        q.t0 = step0 + k;
        q.out_row = k;
        q.probe_row0 = closing ? -1 : probe_row(q.t0);
        q.probe_row1 = q.n_sub == 2 ? probe_row(q.t0 + 1) : -1;
        q.fold0 = k > 0 ? 1 : 0;
        q.in_bits = (has_inp && !closing && n_in_words > 0) ? 1 : 0;
        q.repeats = (s.in_repeat_ptr && !closing) ? 1 : 0;
        k += closing ? 1 : q.n_sub;
        bmtk_glif3_sim args = s;
        FusedLaunch launch = q;
        void *params[] = {&args, &launch};
        const hipError_t err = hipLaunchKernel(kernel, dim3((unsigned)q.n_main), dim3(kFuseBlock),
                                               params, lds, stream);
        if (err != hipSuccess) {
            set_error("glif3_simulate_fwd: launch failed: %s", hipGetErrorString(err));
            return BMTK_E_LAUNCH;
        }
    }
    return BMTK_OK;
}

}  // namespace bmtk
