// Batched forward simulation, one launch per step, pull and update fused.
//
// A wavefront owns a target neuron at a time and its lanes are the neuron's
// trials (batch 8, 16, 32 or 64).  For step t it
//   1. streams the neuron's row of the joint target-major table (recurrent
//      synapses and input synapses, lane = synapse), keeps the synapses whose
//      source fired in some trial of the emitting step t-1-delay (a bit map of
//      the last L-1 steps in LDS), fetches those sources' trial masks from the
//      joint history and adds the weights into 64-bit fixed-point sums in LDS,
//      one per (receptor, trial): everything that arrives at the neuron in
//      step t-1, exact and independent of the order of the additions;
//   2. folds the sums into y1 (NEST adds the arrivals of step t-1 at the end of
//      that step; nothing reads y1 before the update of step t, so adding them
//      at the top of that update performs the same two rounded operations);
//   3. advances the neuron's trials through step t (lane = trial; the
//      propagators are the same in all lanes) and writes its spike bits into
//      row t of the history, where the launches of steps t+2 .. t+L find them.
// No arrival sum passes through device memory and no launch stands between the
// pull and the update.  Other workgroups of the same launch turn the input
// events of step t into bits of the same history row, and deliver the few ids
// that occur twice within a step (bits hold an id once) as events into the
// ring, which the update folds along.
#include "common.hpp"
#include "glif3_update.hpp"
#include "propagate.hpp"
#include "pull_common.hpp"
#include "sim_internal.hpp"

namespace bmtk {

constexpr int kFuseBlock = 1024;
constexpr int kFuseAhead = 3;  // table blocks of 2 KB per wavefront, in flight or at hand (4 and 5: no faster)
constexpr int kFuseWaves = kFuseBlock / kWave;
constexpr size_t kFuseLdsMax = 80u * 1024u;  // half a compute unit's LDS: the few workgroups of the other roles fit beside

struct FusedLaunch {
    int64_t t;           // step being updated (closing launch: one past the last step)
    int64_t out_row;     // row of spike_bits / save_v / save_flags
    int64_t probe_row;   // row of probe_v, -1: not a sampled step
    int64_t n_in_words;  // 64-bit words of the input part of a history row
    int n_main, n_inb, n_rep;  // workgroups per role, in this order of block ids
    int do_update;       // 0 in the closing launch: pull and fold only
    int fold;            // the arrivals of step t-1 are pulled and folded (every launch but a call's first)
    int use_ring;        // ring slot t-1 may hold arrivals (ids repeated within a step)
    int H;               // rows of the history
    int n_w32;           // words per row of the activity map
    int shift;           // sources per bit of the activity map: 2^shift
};

// the spike bits of one neuron's trials: bits [row*kBatch, (row+1)*kBatch) of a history row
template <int kBatch>
__device__ __forceinline__ void store_trial_bits(uint64_t *__restrict__ words, int64_t row, unsigned long long m)
{
    if (kBatch == 64)
        words[row] = m;
    else if (kBatch == 32)
        reinterpret_cast<uint32_t *>(words)[row] = (uint32_t)m;
    else if (kBatch == 16)
        reinterpret_cast<uint16_t *>(words)[row] = (uint16_t)m;
    else
        reinterpret_cast<uint8_t *>(words)[row] = (uint8_t)m;
}

template <int kBatch>
__global__ __launch_bounds__(kFuseBlock) void sim_fused_kernel(bmtk_glif3_sim s, FusedLaunch q)
{
    extern __shared__ unsigned long long fuse_lds[];  // accumulators, stages, then the activity map [L-1][n_w32]
    static_assert(kBatch == 8 || kBatch == 16 || kBatch == 32 || kBatch == 64, "lane = trial, whole bytes of spike bits");
    const int bid = (int)blockIdx.x;
    const int64_t n = s.n_neurons, ne = n * kBatch;
    const int L = s.ring_slots, H = q.H;
    const unsigned lane = (unsigned)lane_id();
    uint64_t *__restrict__ hist_t = s.work_bits + (q.t % H) * s.fuse_hist_stride;  // the row this launch writes
    uint32_t *__restrict__ any_t = s.fuse_any + (q.t % H) * q.n_w32;

    if (bid >= q.n_main + q.n_inb) {
        // ---- ids that occur more than once among the input events of step t-1: the occurrences after the first,
        //      as events into the ring (slots t .. t+L-2; this launch folds and clears slot t-1) ----
        const int slot0 = (int)((q.t - 1) % L);
        const int64_t k0 = s.in_repeat_ptr[q.t - 1], k1 = s.in_repeat_ptr[q.t];
        const int n_waves = q.n_rep * kFuseWaves;
        const int wave = (bid - q.n_main - q.n_inb) * kFuseWaves + threadIdx.x / kWave;
        const int ring_map_words = (int)((n + 31) >> 5);
        uint32_t *__restrict__ ring_map = s.fuse_any + (int64_t)H * q.n_w32;
        const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(s.inp_packed);
        for (int64_t k = k0 + wave; k < k1; k += n_waves) {
            const int e = s.in_repeat_events[k];
            const int j = (int)((uint32_t)e / (uint32_t)kBatch), b = e - j * kBatch;
            const int p1 = s.inp_indptr[j + 1];
            for (int p = s.inp_indptr[j] + (int)lane; p < p1; p += kWave) {
                const uint2 sy = rows[p];
                int slot = slot0 + (int)(sy.x >> 26);
                slot = slot >= L ? slot - L : slot;
                const int64_t i = sy.x & 0xFFFFFFu;
                atomicAdd(s.ring + ((int64_t)(slot * GLIF3_NREC + (int)((sy.x >> 24) & 3u)) * ne + i * kBatch + b),
                          __uint_as_float(sy.y));
                atomicOr(ring_map + (int64_t)slot * ring_map_words + (i >> 5), 1u << (i & 31));
            }
        }
        return;
    }

    if (bid >= q.n_main) {
        // ---- the input events of step t as bits of history row t: one thread per 64-bit word; the events of a
        //      step are ascending, so a word's events are one run of the list, found by bisection ----
        const int64_t w = (int64_t)(bid - q.n_main) * kFuseBlock + threadIdx.x;
        if (w >= q.n_in_words) return;
        const int64_t k0 = s.in_ptr[q.t], k1 = s.in_ptr[q.t + 1];
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
        const int64_t in_word0 = s.fuse_in_base * kBatch / 64;
        hist_t[in_word0 + w] = bits;
        if (bits != 0ull) {
            constexpr int kPerWord = 64 / kBatch;  // sources per word
            const unsigned long long field = kBatch == 64 ? ~0ull : ((1ull << kBatch) - 1ull);
#pragma unroll
            for (int f = 0; f < kPerWord; ++f) {
                if ((bits >> (f * (kBatch & 63))) & field) {
                    const unsigned g = (unsigned)(s.fuse_in_base + w * kPerWord + f) >> q.shift;
                    atomicOr(any_t + (g >> 5), 1u << (g & 31u));
                }
            }
        }
        return;
    }

    // ---- a neuron at a time: pull, fold, update ----
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    constexpr int kAccWords = GLIF3_NREC * kBatch;  // per wavefront
    unsigned long long *acc = fuse_lds + wave * kAccWords;  // [receptor][trial]
    uint2 *stage = reinterpret_cast<uint2 *>(fuse_lds + kFuseWaves * kAccWords) + wave * kWave;
    uint32_t *any_l = reinterpret_cast<uint32_t *>(fuse_lds + kFuseWaves * (kAccWords + kWave));
    // the activity row of the step after this one starts empty (no launch reads it before it is written)
    {
        uint32_t *__restrict__ next = s.fuse_any + ((q.t + 1) % H) * q.n_w32;
        for (int i = bid * kFuseBlock + (int)threadIdx.x; i < q.n_w32; i += q.n_main * kFuseBlock) next[i] = 0u;
    }
    const bool on = kBatch == 64 || lane < (unsigned)kBatch;  // this lane holds a trial
    const unsigned uw32 = (unsigned)q.n_w32, ushift = (unsigned)q.shift, umax_dd = (unsigned)(L - 2);
    Glif3Elem st;  // the state of the row at hand, asked for when its first block turns up
    float prop_col = 0.0f;  // ... and its propagators: lane k holds row k of the neuron's column
    unsigned ring_word = 0u;  // ... and the word of the ring map that holds the row's bit
    const unsigned prop_row_bytes = (unsigned)(s.prop_stride * sizeof(float));
    // ring map: bit i of row (u % L) = some ring cell of neuron i in slot u % L holds an arrival (set by the
    // workgroups that deliver repeated ids, cleared by the neuron's owner when it takes the cells along); it lies
    // behind the H rows of the activity map
    const int ring_map_words = (int)((n + 31) >> 5);
    uint32_t *__restrict__ ring_map = s.fuse_any + (int64_t)H * q.n_w32;
    uint32_t *__restrict__ ring_map_prev = ring_map + (int64_t)((q.t + L - 1) % L) * ring_map_words;
    static_assert(GLIF3_NPROP <= kWave, "a column of the propagator table in one wavefront register");

    // Element accesses: a scalar base (array + plane k of ne elements) and this lane's 32-bit byte offset
    // (n_neurons * batch < 2^30, checked by the caller), which is the address form that needs no 64-bit lane arithmetic.
    const size_t plane = (size_t)ne * sizeof(float);
    auto ldf = [&](const float *base, int k, unsigned boff) {
        return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(base) + k * plane + boff);
    };
    auto stf = [&](float *base, int k, unsigned boff, float v) {
        *reinterpret_cast<float *>(reinterpret_cast<char *>(base) + k * plane + boff) = v;
    };
    // what is left to do for a neuron once its arrival sums are known
    auto finish_row = [&](int64_t row, float (&a)[GLIF3_NREC]) {
        const unsigned e = (unsigned)(row * kBatch) + lane, boff = e * 4u;
        if (q.use_ring && q.fold && ((ring_word >> ((unsigned)row & 31u)) & 1u)) {
            // an id repeated within a step reached this neuron's ring cells of step t-1 (rare): take them along
            if (on) {
                float *prev = s.ring + (int64_t)((q.t + L - 1) % L) * GLIF3_NREC * ne;
                float v[GLIF3_NREC];
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) v[k] = ldf(prev, k, boff);
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) {
                    stf(prev, k, boff, 0.0f);
                    a[k] = v[k] + a[k];
                }
            }
            if (lane == 0) atomicAnd(ring_map_prev + (row >> 5), ~(1u << ((unsigned)row & 31u)));
        }
        Glif3Prop p;  // the same in all lanes
        p.load_from_lanes(prop_col);
        if (!q.do_update) {
            if (on && q.fold) {
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) stf(s.y1, k, boff, ldf(s.y1, k, boff) + a[k] * p.psc0[k]);
            }
            return;
        }
        bool spike = false;
        float frac = 0.0f;
        if (on) {
            if (q.fold) {
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) st.y1[k] = st.y1[k] + a[k] * p.psc0[k];
            }
            const float zero[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
            const float I = s.i_ext ? ldf(s.i_ext, 0, boff) : 0.0f;
            const int ref_before = st.ref;
            spike = glif3_update(st, p, s.h, zero, I, &frac);
            stf(s.V, 0, boff, st.V);
            *reinterpret_cast<int32_t *>(reinterpret_cast<char *>(s.ref) + boff) = st.ref;
#pragma unroll
            for (int k = 0; k < GLIF3_NASC; ++k) stf(s.asc, k, boff, st.asc[k]);
#pragma unroll
            for (int k = 0; k < GLIF3_NREC; ++k) {
                stf(s.y1, k, boff, st.y1[k]);
                stf(s.y2, k, boff, st.y2[k]);
            }
            if (q.probe_row >= 0) {
                const int pc = *reinterpret_cast<const int32_t *>(reinterpret_cast<const char *>(s.probe_col) + boff);
                if (pc >= 0) s.probe_v[q.probe_row * s.probe_stride + pc] = st.V;
            }
            if (s.save_v) {
                stf(s.save_v + q.out_row * ne, 0, boff, st.V);
                (s.save_flags + q.out_row * ne)[e] = (uint8_t)((spike ? BMTK_F_SPIKE : 0) |
                                                              (ref_before == 0 ? BMTK_F_INTEGRATING : 0) |
                                                              (ref_before > 0 && st.ref == 0 ? BMTK_F_RESET : 0));
            }
        }
        const unsigned long long m = __ballot(spike);
        if (lane == 0) {
            store_trial_bits<kBatch>(hist_t, row, m);
            if (s.spike_bits) store_trial_bits<kBatch>(s.spike_bits + q.out_row * s.spike_bits_stride, row, m);
            if (m != 0ull) {
                const unsigned g = (unsigned)row >> ushift;
                atomicOr(any_t + (g >> 5), 1u << (g & 31u));
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
                s.spike_step[idx] = (int32_t)q.t;
                s.spike_elem[idx] = (int32_t)e;
                if (s.spike_frac) s.spike_frac[idx] = frac;
            }
        }
    };
    // Asked for when a row's first block turns up, used when the row is closed: its propagator column (lane k
    // fetches row k; the lanes beyond the table fetch the last row again), the state of its trials, and the word
    // of the map of ring cells that hold something.  All lanes load, whatever they hold: see flush_issue.
    auto load_row = [&](int64_t row, int64_t col) {
        prop_col = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(s.prop + col) +
                                                    min(lane, (unsigned)(GLIF3_NPROP - 1)) * prop_row_bytes);
        if (q.use_ring) ring_word = ring_map_prev[row >> 5];
        if (q.do_update) {
            const unsigned boff = ((unsigned)(row * kBatch) + (on ? lane : 0u)) * 4u;
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

    const int64_t first_row = (int64_t)bid * kFuseWaves + wave, row_stride = (int64_t)q.n_main * kFuseWaves;
    if (!q.fold) {
        // a call's first launch: the closing launch of the call before it has folded everything that arrived
        for (int64_t row = first_row; row < n; row += row_stride) {
            float a[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
            load_row(row, s.class_id ? (int64_t)s.class_id[row] : row);
            finish_row(row, a);
        }
        return;
    }

    // the activity maps of the steps t-2 .. t-L (delays 1 .. L-1), one after the other
    for (int dd = 0; dd < L - 1; ++dd) {
        const int64_t u = q.t - 2 - dd;
        const uint32_t *__restrict__ src = s.fuse_any + (((u % H) + H) % H) * q.n_w32;
        for (int i = threadIdx.x; i < q.n_w32; i += kFuseBlock) any_l[dd * q.n_w32 + i] = src[i];
    }
    __syncthreads();

    const unsigned hrow_bytes = (unsigned)s.fuse_hist_stride * 8u;  // H * stride * 8 < 2^32 (checked by the caller)
    const unsigned uH = (unsigned)H, uprev = (unsigned)((q.t - 1) % H);
    const char *__restrict__ hist_bytes = reinterpret_cast<const char *>(s.work_bits);
    const bmtk_synapse *__restrict__ packed = s.fuse_packed;
    // Block of the table: 64-bit words at a scalar base, 8 * (lane + u*64) bytes on.  Lanes past the end of the
    // row read its last synapse again (and are ignored later): no branch, the four loads go out back to back.
    // A block past the end or an empty one reads the table's first record the same way: every call issues exactly
    // four loads, which is what lets a turn wait for ITS block only and leave the younger ones in flight (the wait
    // is a count of loads still out, fixed at compile time).
    auto fetch = [&](unsigned long long *dst, const PullBlock &blk) {
        const bool some = blk.row < n && blk.base < blk.p1;
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
    PullCursor cursor;
    cursor.start(s.fuse_indptr, n, first_row, row_stride, s.class_id);
    PullBlock dq[kFuseAhead];
    unsigned long long d[kFuseAhead][kPullChunks];
#pragma unroll
    for (int k = 0; k < kFuseAhead; ++k) {
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) d[k][u] = 0ull;
        dq[k] = cursor.next();
        fetch(d[k], dq[k]);
    }
    if (dq[0].row >= n) return;
    if (on) {
#pragma unroll
        for (int r = 0; r < GLIF3_NREC; ++r) acc[r * kBatch + lane] = 0ull;
    }
    int staged = 0;  // entries in the stage (same in all lanes)
    // A flush of the stage has two halves a turn apart, so that the masks travel while the wavefront works on the
    // next block: the first takes the staged synapses into registers and asks for their sources' trial masks, the
    // second converts the weights and adds.  A row's closing work (sums, fold, update) waits for its last flush
    // the same way and is done in the turn after the row's last block.
    int pend_n = 0;           // synapses of the flush under way (same in all lanes)
    uint2 pend_e = make_uint2(0u, 0u);
    unsigned long long pend_m = 0ull;
    int64_t fin_row = -1;     // the row whose closing work is due
    auto flush_issue = [&]() {
        // every lane loads (the lanes without a synapse the mask of source 0 in the row of step t-1, and ignore it):
        // a load under a condition would have to be waited for at once, where the two ways meet again
        const uint2 e = stage[lane];  // {source | receptor << 24 | delay << 26, weight}
        pend_e = (int)lane < staged ? e : make_uint2(0u, 0u);
        const unsigned src = pend_e.x & 0xFFFFFFu;
        const unsigned back = uprev - (pend_e.x >> 26);  // history row of the emitting step, by unsigned wrap-around
        const unsigned hrow = min(back, back + uH);
        const char *cell = hist_bytes + (hrow * hrow_bytes + src * (unsigned)(kBatch / 8));
        if (kBatch == 64)
            pend_m = *reinterpret_cast<const unsigned long long *>(cell);
        else if (kBatch == 32)
            pend_m = *reinterpret_cast<const uint32_t *>(cell);
        else if (kBatch == 16)
            pend_m = *reinterpret_cast<const uint16_t *>(cell);
        else
            pend_m = *reinterpret_cast<const uint8_t *>(cell);
        pend_n = staged;
        staged = 0;
    };
    auto flush_complete = [&]() {
        if ((int)lane < pend_n) {
            unsigned long long *a = acc + ((pend_e.x >> 24) & 3u) * kBatch;
            const unsigned long long w = to_fixed(__uint_as_float(pend_e.y));
            unsigned long long mm = pend_m;
            while (mm) {
                const int b = __ffsll((long long)mm) - 1;
                mm &= mm - 1ull;
                atomicAdd(a + b, w);
            }
        }
        pend_n = 0;
    };
    // the flush under way, then the closing work of the row it belonged to
    auto resolve = [&]() {
        flush_complete();
        float a[GLIF3_NREC] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (on) {
#pragma unroll
            for (int r = 0; r < GLIF3_NREC; ++r) {
                a[r] = from_fixed(acc[r * kBatch + lane]);
                acc[r * kBatch + lane] = 0ull;
            }
        }
        finish_row(fin_row, a);
        fin_row = -1;
    };
    // one turn: the block `cb` with its table words `cd`; afterwards the buffer takes the block kFuseAhead ahead
    auto turn = [&](PullBlock &cb, unsigned long long *cd) {
        const unsigned left = cb.base < cb.p1 ? (unsigned)(cb.p1 - cb.base) : 0u;
        // activity bits of the four chunks (LDS reads, no branch between them)
        unsigned word[kPullChunks], bit[kPullChunks];
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            const unsigned tdr = (unsigned)cd[u];
            const unsigned g = (tdr & 0xFFFFFFu) >> ushift;
            bit[u] = g & 31u;
            // delays are 1 .. L-1 (a buffer that was never filled holds delay 0: kept inside the map, ignored below)
            word[u] = any_l[__umul24(min((tdr >> 26) - 1u, umax_dd), uw32) + (g >> 5)];
        }
        bool hit[kPullChunks];
        unsigned long long who[kPullChunks];
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            hit[u] = lane + u * kWave < left && ((word[u] >> bit[u]) & 1u);
            who[u] = __ballot(hit[u]);
        }
        // the row before: its last masks were asked for a turn ago, its closing work comes before any synapse of
        // this row is added (the one place of a turn where a row is closed)
        if (fin_row >= 0) resolve();
        if (cb.first) load_row(cb.row, cb.col);  // (after that row's closing work, which used the same registers)
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            const int cnt = __popcll(who[u]);
            if (cnt == 0) continue;
            if (staged + cnt > kWave) {
                flush_complete();
                flush_issue();
            }
            if (hit[u]) stage[staged + lane_prefix(who[u])] = make_uint2((unsigned)cd[u], (unsigned)(cd[u] >> 32));
            staged += cnt;
        }
        if (cb.last) {
            flush_complete();  // a flush of this row still under way
            flush_issue();
            fin_row = cb.row;
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
    } while (dq[0].row < n);
    if (fin_row >= 0) resolve();
}

size_t fused_lds_bytes(int batch, int L, int n_w32)
{
    return (size_t)kFuseWaves * (GLIF3_NREC * batch + kWave) * sizeof(unsigned long long) + (size_t)(L - 1) * n_w32 * 4u;
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
    BMTK_REQUIRE(s.n_neurons * (int64_t)batch < (1ll << 30) && GLIF3_NPROP * s.prop_stride < (1ll << 30),
                 "glif3_simulate_fwd: the fused form addresses fewer than 2^30 elements and propagator entries");
    BMTK_REQUIRE(s.delay_offset == 0 && (s.delay_bits == 0 || s.delay_bits == 6) && s.hist_slots == L + 2,
                 "glif3_simulate_fwd: the fused form needs delay_offset 0, the standard packing and hist_slots == ring_slots + 2");
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
    BMTK_REQUIRE((int64_t)(L + 2) * s.fuse_hist_stride < (1ll << 29), "glif3_simulate_fwd: joint history beyond 4 GiB");
    const int64_t groups = (in_base + n_in + (1ll << s.fuse_shift) - 1) >> s.fuse_shift;
    const int n_w32 = (int)((groups + 31) / 32);
    const size_t lds = fused_lds_bytes(batch, L, n_w32);
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
    const int64_t want = (s.n_neurons + kFuseWaves - 1) / kFuseWaves;
    const int64_t cap = (int64_t)n_cu * per_cu;
    q.n_main = (int)(want < cap ? want : cap);
    q.H = L + 2;
    q.n_w32 = n_w32;
    q.shift = s.fuse_shift;
    q.n_in_words = n_in_words;
    q.use_ring = s.in_repeat_ptr != nullptr ? 1 : 0;
    for (int64_t k = 0; k <= n_steps; ++k) {
        const bool closing = k == n_steps;
        q.t = step0 + k;
        q.out_row = k;
        q.probe_row = -1;
        if (s.probe_col && !closing && (q.t + 1) % s.probe_every == 0)
            q.probe_row = (q.t + 1) / s.probe_every - step0 / s.probe_every - 1;
        q.do_update = closing ? 0 : 1;
        q.fold = k > 0 ? 1 : 0;
        q.n_inb = (has_inp && !closing && n_in_words > 0) ? (int)((n_in_words + kFuseBlock - 1) / kFuseBlock) : 0;
        q.n_rep = (s.in_repeat_ptr && k > 0 && q.t >= 1) ? 4 : 0;
        bmtk_glif3_sim args = s;
        FusedLaunch launch = q;
        void *params[] = {&args, &launch};
        const hipError_t err = hipLaunchKernel(kernel, dim3((unsigned)(q.n_main + q.n_inb + q.n_rep)), dim3(kFuseBlock),
                                               params, lds, stream);
        if (err != hipSuccess) {
            set_error("glif3_simulate_fwd: launch failed: %s", hipGetErrorString(err));
            return BMTK_E_LAUNCH;
        }
    }
    return BMTK_OK;
}

}  // namespace bmtk
