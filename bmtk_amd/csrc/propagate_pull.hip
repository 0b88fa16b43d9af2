// Pull-mode propagation (batched runs): one pass over a packed target-major
// table computes everything that arrives in one step from the spike bits of
// the last L steps.
//
// A wavefront owns a target row at a time.  The row's synapses are streamed 64
// per load instruction (lane = synapse); a per-source "fired in any trial" bit
// map of the L steps, staged in LDS, filters the synapses whose source was
// silent, and the others fetch their source's trial mask.  Every lane then
// walks the set bits of its mask and adds its weight to the wavefront's LDS
// accumulators [receptor][trial].
//
// The accumulators are 64-bit fixed point (Q31.32) and the additions are
// 64-bit integer LDS atomics.  Two reasons, both measured on gfx950: an LDS
// float atomic costs about three clocks per LANE (its lanes are worked off one
// after the other), an integer one about nine clocks per 64-lane INSTRUCTION;
// and integer additions commute exactly, so the sums do not depend on the
// order in which lanes and wavefronts arrive: the result is deterministic and
// equals the exact sum of the weights, rounded to fp32 once at the end of the
// row.  An fp32 weight converts to Q31.32 without error down to 2^-32 pA
// (smaller bits are dropped); weights must be finite and below 2^31 in size.

#include "common.hpp"
#include "propagate.hpp"
#include "pull_common.hpp"

namespace bmtk {

// any_map[slot][j/32] bit (j%32): source neuron j fired in at least one trial in the step held by history row `slot`
__global__ __launch_bounds__(kBlock) void pull_anymap_kernel(const uint64_t *__restrict__ hist, int64_t hist_stride,
                                                             int L, int batch, int64_t n_src, int n_w32,
                                                             uint32_t *__restrict__ any_map)
{
    const int64_t idx = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const int slot = (int)(idx / ((int64_t)n_w32 * 32));
    const int64_t j = idx - (int64_t)slot * n_w32 * 32;
    bool any = false;
    if (slot < L && j < n_src) {
        const uint64_t *row = hist + (int64_t)slot * hist_stride;
        for (int t0 = 0; t0 < batch && !any; t0 += kWave)
            any = source_mask(row, (int)j, batch, t0, min(kWave, batch - t0)) != 0ull;
    }
    const unsigned long long m = __ballot(any);
    if (slot < L && (lane_id() & 31) == 0 && j < (int64_t)n_w32 * 32)
        any_map[(int64_t)slot * n_w32 + (j >> 5)] = (uint32_t)(m >> (lane_id() & 32));
}

// The same facts source-major for up to 8 history rows: any_rel[j] bit d = source j fired in at least one trial in
// the step held by history row (slot_now - d) mod L, d = 0 .. L-1.  One byte answers every question a synapse of
// that source can ask, whatever its delay and for both arrival steps of pull2_kernel, from an address that is the
// source itself.
// `pulled` (bmtk_csr_propagate_auto2), when not null: one word per history row, zero for rows whose spikes were
// pushed into the ring as events when they occurred -- the pull must not see those.
__global__ __launch_bounds__(kBlock) void pull_anyrel_kernel(const uint64_t *__restrict__ hist, int64_t hist_stride,
                                                             int L, int batch, int64_t n_src, int slot_now,
                                                             uint8_t *__restrict__ any_rel,
                                                             const int32_t *__restrict__ pulled)
{
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (j >= n_src) return;
    unsigned m = 0u;
    for (int d = 0; d < L; ++d) {
        const int r = (slot_now + L - d) % L;
        if (pulled && !pulled[r]) continue;
        const uint64_t *row = hist + (int64_t)r * hist_stride;
        bool any = false;
        for (int t0 = 0; t0 < batch && !any; t0 += kWave)
            any = source_mask(row, (int)j, batch, t0, min(kWave, batch - t0)) != 0ull;
        m |= (any ? 1u : 0u) << d;
    }
    any_rel[j] = (uint8_t)m;
}

constexpr int kPullBlock = 1024;  // 16 wavefronts share one staged activity map
// per wavefront: 4 x 64 accumulators of 8 bytes and a stage of 64 entries of 8 bytes
constexpr size_t kPullAccBytes = (size_t)(kPullBlock / kWave) * (GLIF3_NREC + 1) * kWave * sizeof(unsigned long long);
constexpr size_t kPullLdsMax = 80u * 1024u;  // two workgroups per compute unit: each may take half of the 160 KB of LDS

// kWords64: batch == 64, so that the trial mask of source j is word j of a history row; otherwise the general
// bit-field read (any batch, tiles of 64 trials over blockIdx.y).
//
// Below ~5 Hz this kernel is bound by instruction issue, not by bandwidth: most synapses have a silent source, and
// what is spent per 64-synapse chunk on the few that do not -- mask address, gather, weight conversion, bit walk --
// costs the same whether 4 or 64 lanes take part.  So the synapses with an event are first packed into a
// 64-entry stage in LDS (one ballot and one store per chunk), and the expensive part runs once per full stage:
// one gather of 64 masks, one conversion, one bit walk with every lane busy.  At 1 Hz that is once per row
// instead of sixteen times.  The per-synapse part uses 32-bit offsets against scalar base pointers and unsigned
// wrap-around for the history row of a delay.
//
// kAuto: the kernel serves bmtk_csr_propagate_auto.  `ctrl` then says, per history row, whether the row's spikes
// are left to this kernel at all (the others were pushed into the ring as events when they occurred): with no such
// row among the L-1 the arrival step looks back on, the kernel returns at once.  And `syn` is the ring slot of the
// arrival step, which may already hold what pushed spikes sent there: ctrl says so, and the sums are then added to
// the cells instead of replacing them.
constexpr int kAutoRows = 64;  // ctrl: int32 pulled[kAutoRows], then int32 slot_holds[kAutoRows]
template <bool kWords64, bool kAuto>
__global__ __launch_bounds__(kPullBlock, 8) void pull_kernel(const uint64_t *__restrict__ hist, int64_t hist_stride, int L,
                                                         int batch, const int32_t *__restrict__ indptr,
                                                         const bmtk_synapse *__restrict__ packed,
                                                         float *__restrict__ syn, int64_t n_tgt, int64_t ne,
                                                         int slot_now, const uint32_t *__restrict__ any_map, int n_w32,
                                                         const int32_t *__restrict__ ctrl)
{
    extern __shared__ unsigned long long pull_lds[];  // accumulators, stages, then the activity map [L][n_w32]
    bool add_to_cells = false;
    if (kAuto) {
        int pulled = 0;
        for (int d = 1; d < L; ++d) pulled |= ctrl[(slot_now + L - d) % L];
        if (!pulled) return;
        add_to_cells = ctrl[kAutoRows + slot_now] != 0;
    }
    // (the wavefront's number through a scalar register, so that rows, bounds and base pointers stay scalar)
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    unsigned long long(*acc)[kWave] = reinterpret_cast<unsigned long long(*)[kWave]>(pull_lds) + wave * GLIF3_NREC;
    uint2 *stage = reinterpret_cast<uint2 *>(pull_lds + (kPullBlock / kWave) * GLIF3_NREC * kWave) + wave * kWave;
    uint32_t *any_l = reinterpret_cast<uint32_t *>(pull_lds + (kPullBlock / kWave) * (GLIF3_NREC + 1) * kWave);
    const unsigned lane = (unsigned)lane_id();
    const int tile0 = kWords64 ? 0 : (int)blockIdx.y * kWave;
    const int width = kWords64 ? kWave : min(kWave, batch - tile0);
    const unsigned hstride = (unsigned)hist_stride;  // L * hist_stride * 8 < 2^32 bytes (checked by the caller)
    const unsigned uL = (unsigned)L, unow = (unsigned)slot_now, uw32 = (unsigned)n_w32;
    const char *__restrict__ hist_bytes = reinterpret_cast<const char *>(hist);
    // Block of the table: 64-bit words at a scalar base, 8 * (lane + u*64) bytes on.  Lanes past the end of the
    // row read its last synapse again (and are ignored later): no branch, the four loads go out back to back.
    // A block past the end or an empty one reads the table's first record the same way: every call issues exactly
    // four loads, which is what lets a turn wait for ITS block only and leave the younger ones in flight (the wait
    // is a count of loads still out, fixed at compile time).
    auto fetch = [&](unsigned long long *dst, const PullBlock &blk) {
        const bool some = blk.row < n_tgt && blk.base < blk.p1;
        const char *__restrict__ src = reinterpret_cast<const char *>(packed) + (some ? (size_t)blk.base * 8u : (size_t)0);
        const unsigned last = some ? (unsigned)(blk.p1 - blk.base) - 1u : 0u;
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u)
            // streamed once per step: keep it from displacing the spike history in L2
            dst[u] = __builtin_nontemporal_load(
                reinterpret_cast<const unsigned long long *>(src + min(lane + u * kWave, last) * 8u));
    };
    PullCursor cursor;
    cursor.start(indptr, n_tgt, (int64_t)blockIdx.x * (kPullBlock / kWave) + wave,
                 (int64_t)gridDim.x * (kPullBlock / kWave));
    // Three table blocks per wavefront: the one at hand and the two after it, whose loads stay in flight during
    // the whole turn (a buffer is refilled, with the block three ahead, as soon as its turn is over).
    PullBlock b0 = cursor.next();
    unsigned long long d0[kPullChunks] = {0ull, 0ull, 0ull, 0ull}, d1[kPullChunks] = {0ull, 0ull, 0ull, 0ull},
                       d2[kPullChunks] = {0ull, 0ull, 0ull, 0ull};
    fetch(d0, b0);
    PullBlock b1 = cursor.next();
    fetch(d1, b1);
    PullBlock b2 = cursor.next();
    fetch(d2, b2);
    // the activity map comes into LDS while the first table blocks are on their way
    for (int i = threadIdx.x; i < L * n_w32; i += kPullBlock) any_l[i] = any_map[i];
    __syncthreads();
    if (b0.row >= n_tgt) return;
#pragma unroll
    for (int r = 0; r < GLIF3_NREC; ++r) acc[r][lane] = 0ull;
    int staged = 0;  // entries in the stage (same in all lanes)
    // the staged synapses: gather their trial masks, convert their weights, add
    auto flush = [&]() {
        if ((int)lane < staged) {
            const uint2 e = stage[lane];  // {source | receptor << 24 | history row << 26, weight}
            const unsigned src = e.x & 0xFFFFFFu, row = e.x >> 26;
            unsigned long long mm;
            if (kWords64)
                mm = *reinterpret_cast<const unsigned long long *>(hist_bytes + (__umul24(row, hstride) + src) * 8u);
            else
                mm = source_mask(hist + (size_t)row * hstride, (int)src, batch, tile0, width);
            unsigned long long *a = acc[(e.x >> 24) & 3u];
            const unsigned long long w = to_fixed(__uint_as_float(e.y));
            while (mm) {
                const int b = __ffsll((long long)mm) - 1;
                mm &= mm - 1ull;
                atomicAdd(a + b, w);
            }
        }
        staged = 0;
    };
    // one turn: the block `cb` with its table words `cd`; afterwards the buffer takes the block three ahead
    auto turn = [&](PullBlock &cb, unsigned long long *cd) {
        const unsigned left = cb.base < cb.p1 ? (unsigned)(cb.p1 - cb.base) : 0u;
        // activity bits of the four chunks (LDS reads, no branch between them)
        unsigned slot[kPullChunks], word[kPullChunks];
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            const unsigned tdr = (unsigned)cd[u];
            // history row of the emitting step: (now - delay) mod L by unsigned wrap-around
            const unsigned back = unow - (tdr >> 26);
            slot[u] = min(back, back + uL);
            word[u] = any_l[__umul24(slot[u], uw32) + ((tdr & 0xFFFFFFu) >> 5)];
        }
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            const unsigned tdr = (unsigned)cd[u];
            const bool hit = lane + u * kWave < left && ((word[u] >> (tdr & 31u)) & 1u);
            const unsigned long long who = __ballot(hit);
            const int n = __popcll(who);
            if (n == 0) continue;
            if (staged + n > kWave) flush();
            if (hit) stage[staged + lane_prefix(who)] = make_uint2((tdr & 0x3FFFFFFu) | (slot[u] << 26), (unsigned)(cd[u] >> 32));
            staged += n;
        }
        if (cb.last) {
            flush();
#pragma unroll
            for (int r = 0; r < GLIF3_NREC; ++r) {
                if ((int)lane < width) {
                    float *cell = syn + ((int64_t)r * ne + cb.row * batch + tile0 + lane);
                    const float sum = from_fixed(acc[r][lane]);
                    *cell = (kAuto && add_to_cells) ? *cell + sum : sum;
                }
                acc[r][lane] = 0ull;
            }
        }
        cb = cursor.next();
        fetch(cd, cb);
    };
    // The buffers take turns in place, so that no register copy ties the arrival of a later block to the work on
    // this one.  One way out of the loop, after a whole round: with a way out after every turn the compiler joins
    // them in one block before the loop's head, from where it looks as if a turn could follow directly on the fetch
    // of its own buffer, and every turn would wait for all loads in flight.  The turns past a wavefront's last
    // block (at most two) see empty blocks of no row.
    do {
        turn(b0, d0);
        turn(b1, d1);
        turn(b2, d2);
    } while (b0.row < n_tgt);
}

// What arrives in TWO consecutive steps, t-1 and t, in one pass over the table.  Both sums only depend on the spikes
// of steps up to t-1 (delays are at least one step), so a caller that advances two steps between calls needs the
// table -- most of the bytes of a call at low rates -- half as often.  Per synapse two questions (did the source
// fire in step t-1-delay, in step t-delay), two stages, two sets of sums; otherwise pull_kernel.  One workgroup of
// 1024 threads per compute unit (its two sets of accumulators and stages take 80 KB of LDS).
constexpr size_t kPull2AccBytes = 2 * kPullAccBytes;
constexpr size_t kPull2LdsMax = 150u * 1024u;
// kByteMap: L <= 8 and one byte per source fits the LDS: the activity map is pull_anyrel_kernel's, one LDS read and
// two shifts per synapse answer both questions (with the bit map: two reads at computed rows).
// out_a, out_b: [4][ne] each, the sums of steps t-1 and t.  kAuto (bmtk_csr_propagate_auto2): they are the two
// steps' ring slots, `ctrl` says which history rows are left to this kernel (with none it returns at once) and
// which of the two slots already hold what pushed spikes sent there (the sums are then added to the cells).
template <bool kWords64, bool kByteMap, bool kAuto>
__global__ __launch_bounds__(kPullBlock) void pull2_kernel(const uint64_t *__restrict__ hist, int64_t hist_stride, int L,
                                                           int batch, const int32_t *__restrict__ indptr,
                                                           const bmtk_synapse *__restrict__ packed,
                                                           float *__restrict__ out_a, float *__restrict__ out_b,
                                                           int64_t n_tgt, int64_t ne, int slot_now,
                                                           const uint32_t *__restrict__ any_map, int n_w32,
                                                           const int32_t *__restrict__ ctrl)
{
    extern __shared__ unsigned long long pull_lds[];  // accumulators [wave][step][4][64], stages [wave][step][64], map
    bool add_a = false, add_b = false;
    if (kAuto) {
        int pulled = 0;
        for (int r = 0; r < L; ++r) pulled |= ctrl[r];
        if (!pulled) return;
        add_a = ctrl[kAutoRows + (slot_now + L - 1) % L] != 0;
        add_b = ctrl[kAutoRows + slot_now] != 0;
    }
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / kWave));
    constexpr int kWaves = kPullBlock / kWave;
    unsigned long long *acc = pull_lds + wave * (2 * GLIF3_NREC * kWave);
    uint2 *stage = reinterpret_cast<uint2 *>(pull_lds + kWaves * 2 * GLIF3_NREC * kWave) + wave * 2 * kWave;
    uint32_t *any_l = reinterpret_cast<uint32_t *>(pull_lds + kWaves * 2 * (GLIF3_NREC + 1) * kWave);
    const unsigned lane = (unsigned)lane_id();
    const int tile0 = kWords64 ? 0 : (int)blockIdx.y * kWave;
    const int width = kWords64 ? kWave : min(kWave, batch - tile0);
    const unsigned hstride = (unsigned)hist_stride;  // L * hist_stride * 8 < 2^32 bytes (checked by the caller)
    const unsigned uL = (unsigned)L, uw32 = (unsigned)n_w32;
    const unsigned now_b = (unsigned)slot_now, now_a = (unsigned)((slot_now + L - 1) % L);  // rows of steps t and t-1
    const char *__restrict__ hist_bytes = reinterpret_cast<const char *>(hist);
    auto fetch = [&](unsigned long long *dst, const PullBlock &blk) {
        const bool some = blk.row < n_tgt && blk.base < blk.p1;
        const char *__restrict__ src = reinterpret_cast<const char *>(packed) + (some ? (size_t)blk.base * 8u : (size_t)0);
        const unsigned last = some ? (unsigned)(blk.p1 - blk.base) - 1u : 0u;
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u)
            dst[u] = __builtin_nontemporal_load(
                reinterpret_cast<const unsigned long long *>(src + min(lane + u * kWave, last) * 8u));
    };
    PullCursor cursor;
    cursor.start(indptr, n_tgt, (int64_t)blockIdx.x * kWaves + wave, (int64_t)gridDim.x * kWaves);
    PullBlock b0 = cursor.next();
    unsigned long long d0[kPullChunks] = {0ull, 0ull, 0ull, 0ull}, d1[kPullChunks] = {0ull, 0ull, 0ull, 0ull};
    fetch(d0, b0);
    PullBlock b1 = cursor.next();
    fetch(d1, b1);
    // the activity map comes into LDS while the first table blocks are on their way (n_w32 counts the byte map's
    // 16-byte pieces when kByteMap)
    if (kByteMap) {
        const uint4 *src16 = reinterpret_cast<const uint4 *>(any_map);
        uint4 *dst16 = reinterpret_cast<uint4 *>(any_l);
        for (int i = threadIdx.x; i < n_w32; i += kPullBlock) dst16[i] = src16[i];
    } else {
        for (int i = threadIdx.x; i < L * n_w32; i += kPullBlock) any_l[i] = any_map[i];
    }
    __syncthreads();
    if (b0.row >= n_tgt) return;
    const uint8_t *any_b = reinterpret_cast<const uint8_t *>(any_l);
#pragma unroll
    for (int r = 0; r < 2 * GLIF3_NREC; ++r) acc[r * kWave + lane] = 0ull;
    int staged[2] = {0, 0};  // entries in the two stages (same in all lanes)
    // the staged synapses of one arrival step: gather their trial masks, convert their weights, add
    auto flush = [&](int k) {
        if ((int)lane < staged[k]) {
            const uint2 e = stage[k * kWave + lane];  // {source | receptor << 24 | delay << 26, weight}
            const unsigned src = e.x & 0xFFFFFFu;
            const unsigned back = (k ? now_b : now_a) - (e.x >> 26);  // history row of the emitting step
            const unsigned row = min(back, back + uL);
            unsigned long long mm;
            if (kWords64)
                mm = *reinterpret_cast<const unsigned long long *>(hist_bytes + (__umul24(row, hstride) + src) * 8u);
            else
                mm = source_mask(hist + (size_t)row * hstride, (int)src, batch, tile0, width);
            unsigned long long *a = acc + (k * GLIF3_NREC + ((e.x >> 24) & 3u)) * kWave;
            const unsigned long long w = to_fixed(__uint_as_float(e.y));
            while (mm) {
                const int b = __ffsll((long long)mm) - 1;
                mm &= mm - 1ull;
                atomicAdd(a + b, w);
            }
        }
        staged[k] = 0;
    };
    auto turn = [&](PullBlock &cb, unsigned long long *cd) {
        const unsigned left = cb.base < cb.p1 ? (unsigned)(cb.p1 - cb.base) : 0u;
        // activity bits of the four chunks for both arrival steps (LDS reads, no branch between them): the map of a
        // step is the row of its history slot; a synapse of delay d looks at step t-1-d and at step t-d
        // (byte map: bit d of a source's byte = fired d steps before the step whose row is now_b, which holds step
        // t - L; a synapse of delay d asks for bit d on behalf of step t and bit d + 1, bit L being bit 0, for t - 1)
        unsigned word_a[kPullChunks], word_b[kPullChunks];
#pragma unroll
        for (int u = 0; u < kPullChunks; ++u) {
            const unsigned tdr = (unsigned)cd[u];
            if (kByteMap) {
                const unsigned m = any_b[tdr & 0xFFFFFFu];
                word_b[u] = (m | (m << uL)) >> (tdr >> 26);
                word_a[u] = word_b[u] >> 1;
            } else {
                const unsigned back_b = now_b - (tdr >> 26), back_a = now_a - (tdr >> 26);
                const unsigned at = (tdr & 0xFFFFFFu) >> 5;
                word_b[u] = any_l[__umul24(min(back_b, back_b + uL), uw32) + at] >> (tdr & 31u);
                word_a[u] = any_l[__umul24(min(back_a, back_a + uL), uw32) + at] >> (tdr & 31u);
            }
        }
#pragma unroll
        for (int k = 0; k < 2; ++k) {
#pragma unroll
            for (int u = 0; u < kPullChunks; ++u) {
                const unsigned tdr = (unsigned)cd[u];
                const bool hit = lane + u * kWave < left && ((k ? word_b[u] : word_a[u]) & 1u);
                const unsigned long long who = __ballot(hit);
                const int n = __popcll(who);
                if (n == 0) continue;
                if (staged[k] + n > kWave) flush(k);
                if (hit) stage[k * kWave + staged[k] + lane_prefix(who)] = make_uint2(tdr, (unsigned)(cd[u] >> 32));
                staged[k] += n;
            }
        }
        if (cb.last) {
            flush(0);
            flush(1);
#pragma unroll
            for (int k = 0; k < 2; ++k) {
#pragma unroll
                for (int r = 0; r < GLIF3_NREC; ++r) {
                    unsigned long long *cell = acc + (k * GLIF3_NREC + r) * kWave + lane;
                    if ((int)lane < width) {
                        float *out = (k ? out_b : out_a) + (int64_t)r * ne + cb.row * batch + tile0 + lane;
                        const float sum = from_fixed(*cell);
                        if (kAuto && (k ? add_b : add_a))
                            *out += sum;
                        else
                            *out = sum;
                    }
                    *cell = 0ull;
                }
            }
        }
        cb = cursor.next();
        fetch(cd, cb);
    };
    do {  // (one way out, after a whole round of the buffers: see pull_kernel)
        turn(b0, d0);
        turn(b1, d1);
    } while (b0.row < n_tgt);
}

// bmtk_csr_propagate_auto, first launch: the spikes of step `step` as events, if they are few.  Every workgroup
// reads the number of active elements and decides the same way; up to cnt_max the elements' rows are walked and
// their weights pushed into the ring (fp32 atomics), above it nothing happens here and the step is left to the
// pull kernel.  One thread records the decision: ctrl[row] = 1 when the history row of the step is to be pulled,
// and which ring slots hold pushed arrivals (the slot of the step itself, consumed by now, holds none).
// consumed: how many ring slots the caller has read and cleared since the launch before this one, counted back from
// slot0 (1 in the one-step form: the step's own slot; in the two-step form 2 for the first of a call's two steps --
// its own slot and the one before -- and 0 for the second, whose own slot this call is about to complete).
__global__ __launch_bounds__(kBlock) void auto_push_kernel(const int32_t *__restrict__ active,
                                                           const int32_t *__restrict__ n_active, int batch, Table t,
                                                           float *__restrict__ ring, int L, int64_t ne, int slot0,
                                                           int cnt_max, int32_t *__restrict__ ctrl, int consumed)
{
    const int n_waves = gridDim.x * (kBlock / kWave);
    const int cnt = *n_active;
    const bool push = cnt <= cnt_max;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        ctrl[slot0] = push ? 0 : 1;
        for (int c = 0; c < consumed; ++c) ctrl[kAutoRows + (slot0 + L - c) % L] = 0;
        if (push && cnt > 0)
            for (int d = 1; d < L; ++d) ctrl[kAutoRows + (slot0 + d) % L] = 1;
    }
    if (!push) return;
    for (int k = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave; k < cnt; k += n_waves) {
        const int e = active[k];
        const int j = batch == 1 ? e : (int)((uint32_t)e / (uint32_t)batch);
        deliver_row(t, j, e - j * batch, batch, ring, L, slot0, ne);
    }
}

// ... second launch: the row of the step in the activity map -- from the history row when the step is to be
// pulled, empty when its spikes were pushed (the pull kernel then finds nothing of that step)
__global__ __launch_bounds__(kBlock) void auto_anymap_kernel(const uint64_t *__restrict__ hist_row, int batch,
                                                             int64_t n_src, int n_w32, uint32_t *__restrict__ any_row,
                                                             const int32_t *__restrict__ pulled)
{
    const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    bool any = false;
    if (*pulled && j < n_src) {
        for (int t0 = 0; t0 < batch && !any; t0 += kWave)
            any = source_mask(hist_row, (int)j, batch, t0, min(kWave, batch - t0)) != 0ull;
    }
    const unsigned long long m = __ballot(any);
    if ((lane_id() & 31) == 0 && j < (int64_t)n_w32 * 32) any_row[j >> 5] = (uint32_t)(m >> (lane_id() & 32));
}

}  // namespace bmtk

extern "C" int64_t bmtk_csr_propagate_pull_workspace_bytes(int32_t L, int64_t n_src)
{
    if (L <= 0 || n_src <= 0) return 0;
    // one bit per (row, source), or one byte per source (the two-step form with up to 8 rows): the larger of the two
    const int64_t bits = (int64_t)L * ((n_src + 31) / 32) * 4, bytes = (n_src + 15) / 16 * 16;
    return bits > bytes ? bits : bytes;
}

extern "C" int bmtk_csr_propagate_pull(const uint64_t *spike_hist, int64_t hist_stride, int32_t L, int64_t n_src,
                                       int32_t batch, const int32_t *indptr, const bmtk_synapse *packed, float *syn,
                                       int64_t n_tgt, int64_t t_arrive, void *workspace, void *stream)
{
    using namespace bmtk;
    BMTK_REQUIRE(spike_hist && indptr && packed && syn && workspace, "csr_propagate_pull: pointers must be non-null");
    BMTK_REQUIRE(batch > 0 && n_tgt > 0 && n_src > 0 && t_arrive >= 0, "csr_propagate_pull: bad batch, sizes or step");
    BMTK_REQUIRE(L > 1 && L <= 64, "csr_propagate_pull: L must lie in 2..64");
    BMTK_REQUIRE(hist_stride >= (n_src * (int64_t)batch + 63) / 64 + 1,
                 "csr_propagate_pull: hist_stride must hold ceil(n_src*batch/64)+1 words");
    BMTK_REQUIRE(n_tgt * (int64_t)batch < (1ll << 31) && n_src < (1ll << 24), "csr_propagate_pull: network too large");
    BMTK_REQUIRE((int64_t)L * hist_stride < (1ll << 29) && hist_stride < (1ll << 24),
                 "csr_propagate_pull: spike history beyond 4 GiB");
    const int n_w32 = (int)((n_src + 31) / 32);
    const size_t lds = (size_t)L * n_w32 * 4 + kPullAccBytes;
    BMTK_REQUIRE(lds <= kPullLdsMax, "csr_propagate_pull: L * n_src too large for the activity map in LDS");
    uint32_t *any_map = (uint32_t *)workspace;
    const int64_t map_threads = (int64_t)L * n_w32 * 32;
    hipLaunchKernelGGL(pull_anymap_kernel, dim3((unsigned)((map_threads + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, spike_hist, hist_stride, L, batch, n_src, n_w32, any_map);
    const unsigned rows_per_block = kPullBlock / kWave;
    int dev = 0;
    (void)hipGetDevice(&dev);
    static int cu_count[64];  // compute units of every device seen so far
    int n_cu = (dev >= 0 && dev < 64) ? cu_count[dev] : 0;
    if (n_cu <= 0) {
        n_cu = 256;
        (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (dev >= 0 && dev < 64) cu_count[dev] = n_cu;
    }
    const unsigned want = (unsigned)((n_tgt + rows_per_block - 1) / rows_per_block);
    const unsigned cap = (unsigned)n_cu * 2u;  // persistent workgroups: the activity map is staged once per workgroup
    const dim3 grid(want < cap ? want : cap, (unsigned)((batch + kWave - 1) / kWave));
    BMTK_REQUIRE(grid.y <= 65535, "csr_propagate_pull: batch too large");
    // more than 64 KB of dynamic LDS has to be asked for, once per kernel and device
    static bool asked[2][64];
    if (dev >= 0 && dev < 64 && !asked[batch == kWave][dev]) {
        const hipError_t err = hipFuncSetAttribute(
            batch == kWave ? reinterpret_cast<const void *>(pull_kernel<true, false>)
                           : reinterpret_cast<const void *>(pull_kernel<false, false>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPullLdsMax);
        if (err != hipSuccess) {
            set_error("csr_propagate_pull: cannot reserve %zu bytes of LDS: %s", kPullLdsMax, hipGetErrorString(err));
            return BMTK_E_LAUNCH;
        }
        asked[batch == kWave][dev] = true;
    }
    if (batch == kWave)
        hipLaunchKernelGGL((pull_kernel<true, false>), grid, dim3(kPullBlock), lds, (hipStream_t)stream, spike_hist,
                           hist_stride, L, batch, indptr, packed, syn, n_tgt, n_tgt * (int64_t)batch, (int)(t_arrive % L),
                           any_map, n_w32, (const int32_t *)nullptr);
    else
        hipLaunchKernelGGL((pull_kernel<false, false>), grid, dim3(kPullBlock), lds, (hipStream_t)stream, spike_hist,
                           hist_stride, L, batch, indptr, packed, syn, n_tgt, n_tgt * (int64_t)batch, (int)(t_arrive % L),
                           any_map, n_w32, (const int32_t *)nullptr);
    BMTK_CHECK_LAUNCH("csr_propagate_pull");
    return BMTK_OK;
}

extern "C" int64_t bmtk_csr_propagate_auto_workspace_bytes(int32_t L, int64_t n_src)
{
    if (L <= 0 || n_src <= 0) return 0;
    return (int64_t)L * ((n_src + 31) / 32) * 4 + 2 * bmtk::kAutoRows * 4;
}

extern "C" int bmtk_csr_propagate_auto(const int32_t *active, const int32_t *n_active, int64_t max_active,
                                       const uint64_t *spike_hist, int64_t hist_stride, int32_t L, int64_t n_src,
                                       int32_t batch, const int32_t *src_indptr, const int32_t *src_indices,
                                       const float *src_weights, const uint8_t *src_delays, const uint8_t *src_receptors,
                                       const int32_t *tgt_indptr, const bmtk_synapse *tgt_packed, float *ring,
                                       int64_t n_tgt, int64_t step, int64_t scatter_max_active, void *workspace,
                                       void *stream)
{
    using namespace bmtk;
    BMTK_REQUIRE(active && n_active && spike_hist && ring && workspace, "csr_propagate_auto: pointers must be non-null");
    BMTK_REQUIRE(src_indptr && src_indices && src_weights && src_delays && src_receptors && tgt_indptr && tgt_packed,
                 "csr_propagate_auto: both forms of the table are needed");
    BMTK_REQUIRE(batch > 0 && n_tgt > 0 && n_src > 0 && step >= 0, "csr_propagate_auto: bad batch, sizes or step");
    BMTK_REQUIRE(L > 1 && L <= kAutoRows, "csr_propagate_auto: L must lie in 2..64");
    BMTK_REQUIRE(hist_stride >= (n_src * (int64_t)batch + 63) / 64 + 1,
                 "csr_propagate_auto: hist_stride must hold ceil(n_src*batch/64)+1 words");
    BMTK_REQUIRE(n_tgt * (int64_t)batch < (1ll << 31) && n_src < (1ll << 24), "csr_propagate_auto: network too large");
    BMTK_REQUIRE((int64_t)L * hist_stride < (1ll << 29) && hist_stride < (1ll << 24),
                 "csr_propagate_auto: spike history beyond 4 GiB");
    BMTK_REQUIRE(scatter_max_active >= 0 && scatter_max_active < (1ll << 31) && max_active >= 0,
                 "csr_propagate_auto: bad threshold or bound");
    const int n_w32 = (int)((n_src + 31) / 32);
    const size_t lds = (size_t)L * n_w32 * 4 + kPullAccBytes;
    BMTK_REQUIRE(lds <= kPullLdsMax, "csr_propagate_auto: L * n_src too large for the activity map in LDS");
    hipStream_t st = (hipStream_t)stream;
    uint32_t *any_map = (uint32_t *)workspace;
    int32_t *ctrl = (int32_t *)(any_map + (size_t)L * n_w32);
    const int64_t ne = n_tgt * (int64_t)batch;
    const int slot0 = (int)(step % L);
    {   // the step's spikes as events, if they are few (the launch also records the decision)
        const int64_t bound = max_active < scatter_max_active ? max_active : scatter_max_active;
        const int64_t waves = bound < 1 ? 1 : (bound < 8192 ? bound : 8192);
        const unsigned grid = (unsigned)((waves + kBlock / kWave - 1) / (kBlock / kWave));
        Table t{src_indptr, src_indices, src_weights, src_delays, src_receptors};
        hipLaunchKernelGGL(auto_push_kernel, dim3(grid), dim3(kBlock), 0, st, active, n_active, batch, t, ring, L, ne, slot0,
                           (int)scatter_max_active, ctrl, 1);
    }
    hipLaunchKernelGGL(auto_anymap_kernel, dim3((unsigned)(((int64_t)n_w32 * 32 + kBlock - 1) / kBlock)), dim3(kBlock), 0, st,
                       spike_hist + (int64_t)slot0 * hist_stride, batch, n_src, n_w32, any_map + (size_t)slot0 * n_w32,
                       ctrl + slot0);
    int dev = 0;
    (void)hipGetDevice(&dev);
    static int cu_count[64];
    int n_cu = (dev >= 0 && dev < 64) ? cu_count[dev] : 0;
    if (n_cu <= 0) {
        n_cu = 256;
        (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (dev >= 0 && dev < 64) cu_count[dev] = n_cu;
    }
    const unsigned rows_per_block = kPullBlock / kWave;
    const unsigned want = (unsigned)((n_tgt + rows_per_block - 1) / rows_per_block);
    const unsigned cap = (unsigned)n_cu * 2u;
    const dim3 grid(want < cap ? want : cap, (unsigned)((batch + kWave - 1) / kWave));
    BMTK_REQUIRE(grid.y <= 65535, "csr_propagate_auto: batch too large");
    static bool asked[2][64];
    if (dev >= 0 && dev < 64 && !asked[batch == kWave][dev]) {
        const hipError_t err = hipFuncSetAttribute(
            batch == kWave ? reinterpret_cast<const void *>(pull_kernel<true, true>)
                           : reinterpret_cast<const void *>(pull_kernel<false, true>),
            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPullLdsMax);
        if (err != hipSuccess) {
            set_error("csr_propagate_auto: cannot reserve %zu bytes of LDS: %s", kPullLdsMax, hipGetErrorString(err));
            return BMTK_E_LAUNCH;
        }
        asked[batch == kWave][dev] = true;
    }
    // everything that arrives in step + 1 from the steps that were not pushed, into the ring slot of that step
    const int slot_arrive = (int)((step + 1) % L);
    float *cells = ring + (int64_t)slot_arrive * GLIF3_NREC * ne;
    if (batch == kWave)
        hipLaunchKernelGGL((pull_kernel<true, true>), grid, dim3(kPullBlock), lds, st, spike_hist, hist_stride, L, batch,
                           tgt_indptr, tgt_packed, cells, n_tgt, ne, slot_arrive, any_map, n_w32, (const int32_t *)ctrl);
    else
        hipLaunchKernelGGL((pull_kernel<false, true>), grid, dim3(kPullBlock), lds, st, spike_hist, hist_stride, L, batch,
                           tgt_indptr, tgt_packed, cells, n_tgt, ne, slot_arrive, any_map, n_w32, (const int32_t *)ctrl);
    BMTK_CHECK_LAUNCH("csr_propagate_auto");
    return BMTK_OK;
}

extern "C" int64_t bmtk_csr_propagate_auto2_workspace_bytes(int32_t L, int64_t n_src)
{
    if (L <= 0 || n_src <= 0) return 0;
    return 2 * bmtk::kAutoRows * 4 + (n_src + 15) / 16 * 16;  // the record of pushed steps, then one byte per source
}

extern "C" int bmtk_csr_propagate_auto2(const int32_t *active_a, const int32_t *n_active_a, const int32_t *active_b,
                                        const int32_t *n_active_b, int64_t max_active, const uint64_t *spike_hist,
                                        int64_t hist_stride, int32_t L, int64_t n_src, int32_t batch,
                                        const int32_t *src_indptr, const int32_t *src_indices, const float *src_weights,
                                        const uint8_t *src_delays, const uint8_t *src_receptors,
                                        const int32_t *tgt_indptr, const bmtk_synapse *tgt_packed, float *ring,
                                        int64_t n_tgt, int64_t step, int64_t scatter_max_active, void *workspace,
                                        void *stream)
{
    using namespace bmtk;
    BMTK_REQUIRE(active_a && n_active_a && active_b && n_active_b && spike_hist && ring && workspace,
                 "csr_propagate_auto2: pointers must be non-null");
    BMTK_REQUIRE(src_indptr && src_indices && src_weights && src_delays && src_receptors && tgt_indptr && tgt_packed,
                 "csr_propagate_auto2: both forms of the table are needed");
    BMTK_REQUIRE(batch > 0 && n_tgt > 0 && n_src > 0 && step >= 1, "csr_propagate_auto2: bad batch, sizes or step");
    BMTK_REQUIRE(L > 1 && L <= 8, "csr_propagate_auto2: L must lie in 2..8 (longer histories: bmtk_csr_propagate_auto)");
    BMTK_REQUIRE(hist_stride >= (n_src * (int64_t)batch + 63) / 64 + 1,
                 "csr_propagate_auto2: hist_stride must hold ceil(n_src*batch/64)+1 words");
    BMTK_REQUIRE(n_tgt * (int64_t)batch < (1ll << 31) && n_src < (1ll << 24), "csr_propagate_auto2: network too large");
    BMTK_REQUIRE((int64_t)L * hist_stride < (1ll << 29) && hist_stride < (1ll << 24),
                 "csr_propagate_auto2: spike history beyond 4 GiB");
    BMTK_REQUIRE(scatter_max_active >= 0 && scatter_max_active < (1ll << 31) && max_active >= 0,
                 "csr_propagate_auto2: bad threshold or bound");
    const int n_16 = (int)((n_src + 15) / 16);
    const size_t lds = (size_t)n_16 * 16 + kPull2AccBytes;
    BMTK_REQUIRE(lds <= kPull2LdsMax, "csr_propagate_auto2: n_src too large for the activity map in LDS");
    hipStream_t st = (hipStream_t)stream;
    int32_t *ctrl = (int32_t *)workspace;
    uint8_t *any_rel = (uint8_t *)(ctrl + 2 * kAutoRows);
    int64_t ne = n_tgt * (int64_t)batch;
    {   // the two new steps' spikes as events where they are few (each launch records its decision)
        const int64_t bound = max_active < scatter_max_active ? max_active : scatter_max_active;
        const int64_t waves = bound < 1 ? 1 : (bound < 8192 ? bound : 8192);
        const unsigned grid = (unsigned)((waves + kBlock / kWave - 1) / (kBlock / kWave));
        Table t{src_indptr, src_indices, src_weights, src_delays, src_receptors};
        hipLaunchKernelGGL(auto_push_kernel, dim3(grid), dim3(kBlock), 0, st, active_a, n_active_a, batch, t, ring, L, ne,
                           (int)((step - 1) % L), (int)scatter_max_active, ctrl, 2);
        hipLaunchKernelGGL(auto_push_kernel, dim3(grid), dim3(kBlock), 0, st, active_b, n_active_b, batch, t, ring, L, ne,
                           (int)(step % L), (int)scatter_max_active, ctrl, 0);
    }
    int slot_now = (int)((step + 1) % L);  // the row the spikes of step + 1 will take: it holds step + 1 - L
    hipLaunchKernelGGL(pull_anyrel_kernel, dim3((unsigned)((n_src + kBlock - 1) / kBlock)), dim3(kBlock), 0, st, spike_hist,
                       hist_stride, L, batch, n_src, slot_now, any_rel, (const int32_t *)ctrl);
    int dev = 0;
    (void)hipGetDevice(&dev);
    static int cu_count[64];
    int n_cu = (dev >= 0 && dev < 64) ? cu_count[dev] : 0;
    if (n_cu <= 0) {
        n_cu = 256;
        (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (dev >= 0 && dev < 64) cu_count[dev] = n_cu;
    }
    const unsigned rows_per_block = kPullBlock / kWave;
    const unsigned want = (unsigned)((n_tgt + rows_per_block - 1) / rows_per_block);
    const dim3 grid(want < (unsigned)n_cu ? want : (unsigned)n_cu, (unsigned)((batch + kWave - 1) / kWave));
    BMTK_REQUIRE(grid.y <= 65535, "csr_propagate_auto2: batch too large");
    const void *kernel = batch == kWave ? reinterpret_cast<const void *>(pull2_kernel<true, true, true>)
                                        : reinterpret_cast<const void *>(pull2_kernel<false, true, true>);
    static bool asked[2][64];
    if (dev >= 0 && dev < 64 && !asked[batch == kWave][dev]) {
        const hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPull2LdsMax);
        if (err != hipSuccess) {
            set_error("csr_propagate_auto2: cannot reserve %zu bytes of LDS: %s", kPull2LdsMax, hipGetErrorString(err));
            return BMTK_E_LAUNCH;
        }
        asked[batch == kWave][dev] = true;
    }
    // what the steps not pushed send to steps `step` and `step + 1`, into (or onto) those steps' ring slots
    float *out_a = ring + (int64_t)(step % L) * GLIF3_NREC * ne, *out_b = ring + (int64_t)slot_now * GLIF3_NREC * ne;
    const uint32_t *map_arg = (const uint32_t *)any_rel;
    const int32_t *ctrl_arg = ctrl;
    int64_t stride_arg = hist_stride;
    int32_t L_arg = L, batch_arg = batch;
    int n_map = n_16;
    void *args[] = {&spike_hist, &stride_arg, &L_arg, &batch_arg, &tgt_indptr, &tgt_packed, &out_a, &out_b, &n_tgt, &ne,
                    &slot_now, &map_arg, &n_map, &ctrl_arg};
    const hipError_t err = hipLaunchKernel(kernel, grid, dim3(kPullBlock), args, lds, st);
    if (err != hipSuccess) {
        set_error("csr_propagate_auto2: launch failed: %s", hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    BMTK_CHECK_LAUNCH("csr_propagate_auto2");
    return BMTK_OK;
}

extern "C" int bmtk_csr_propagate_pull2(const uint64_t *spike_hist, int64_t hist_stride, int32_t L, int64_t n_src,
                                        int32_t batch, const int32_t *indptr, const bmtk_synapse *packed, float *syn2,
                                        int64_t n_tgt, int64_t t_arrive, void *workspace, void *stream)
{
    using namespace bmtk;
    BMTK_REQUIRE(spike_hist && indptr && packed && syn2 && workspace, "csr_propagate_pull2: pointers must be non-null");
    BMTK_REQUIRE(batch > 0 && n_tgt > 0 && n_src > 0 && t_arrive >= 1, "csr_propagate_pull2: bad batch, sizes or step");
    BMTK_REQUIRE(L > 1 && L <= 64, "csr_propagate_pull2: L must lie in 2..64");
    BMTK_REQUIRE(hist_stride >= (n_src * (int64_t)batch + 63) / 64 + 1,
                 "csr_propagate_pull2: hist_stride must hold ceil(n_src*batch/64)+1 words");
    BMTK_REQUIRE(n_tgt * (int64_t)batch < (1ll << 31) && n_src < (1ll << 24), "csr_propagate_pull2: network too large");
    BMTK_REQUIRE((int64_t)L * hist_stride < (1ll << 29) && hist_stride < (1ll << 24),
                 "csr_propagate_pull2: spike history beyond 4 GiB");
    // the activity map: one byte per source when the history has at most 8 rows and the bytes fit the LDS (the
    // kernel then asks one question per synapse instead of two), else one bit per row and source
    const int n_16 = (int)((n_src + 15) / 16);
    const bool byte_map = L <= 8 && (size_t)n_16 * 16 + kPull2AccBytes <= kPull2LdsMax;
    const int n_w32 = byte_map ? n_16 : (int)((n_src + 31) / 32);
    const size_t lds = (byte_map ? (size_t)n_16 * 16 : (size_t)L * n_w32 * 4) + kPull2AccBytes;
    BMTK_REQUIRE(lds <= kPull2LdsMax, "csr_propagate_pull2: L * n_src too large for the activity map in LDS");
    uint32_t *any_map = (uint32_t *)workspace;
    if (byte_map) {
        hipLaunchKernelGGL(pull_anyrel_kernel, dim3((unsigned)((n_src + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                           (hipStream_t)stream, spike_hist, hist_stride, L, batch, n_src, (int)(t_arrive % L),
                           (uint8_t *)workspace, (const int32_t *)nullptr);
    } else {
        const int64_t map_threads = (int64_t)L * n_w32 * 32;
        hipLaunchKernelGGL(pull_anymap_kernel, dim3((unsigned)((map_threads + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                           (hipStream_t)stream, spike_hist, hist_stride, L, batch, n_src, n_w32, any_map);
    }
    int dev = 0;
    (void)hipGetDevice(&dev);
    static int cu_count[64];
    int n_cu = (dev >= 0 && dev < 64) ? cu_count[dev] : 0;
    if (n_cu <= 0) {
        n_cu = 256;
        (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (dev >= 0 && dev < 64) cu_count[dev] = n_cu;
    }
    const unsigned rows_per_block = kPullBlock / kWave;
    const unsigned want = (unsigned)((n_tgt + rows_per_block - 1) / rows_per_block);
    const dim3 grid(want < (unsigned)n_cu ? want : (unsigned)n_cu, (unsigned)((batch + kWave - 1) / kWave));
    BMTK_REQUIRE(grid.y <= 65535, "csr_propagate_pull2: batch too large");
    const void *const kernels[2][2] = {
        {reinterpret_cast<const void *>(pull2_kernel<false, false, false>), reinterpret_cast<const void *>(pull2_kernel<false, true, false>)},
        {reinterpret_cast<const void *>(pull2_kernel<true, false, false>), reinterpret_cast<const void *>(pull2_kernel<true, true, false>)}};
    const void *kernel = kernels[batch == kWave][byte_map];
    static bool asked[2][2][64];
    if (dev >= 0 && dev < 64 && !asked[batch == kWave][byte_map][dev]) {
        const hipError_t err = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kPull2LdsMax);
        if (err != hipSuccess) {
            set_error("csr_propagate_pull2: cannot reserve %zu bytes of LDS: %s", kPull2LdsMax, hipGetErrorString(err));
            return BMTK_E_LAUNCH;
        }
        asked[batch == kWave][byte_map][dev] = true;
    }
    int64_t ne = n_tgt * (int64_t)batch;
    int slot_now = (int)(t_arrive % L), n_map = n_w32;
    const uint32_t *map_arg = any_map;
    int64_t stride_arg = hist_stride;
    int32_t L_arg = L, batch_arg = batch;
    float *out_a = syn2, *out_b = syn2 + GLIF3_NREC * ne;
    const int32_t *no_ctrl = nullptr;
    void *args[] = {&spike_hist, &stride_arg, &L_arg, &batch_arg, &indptr, &packed, &out_a, &out_b, &n_tgt, &ne, &slot_now,
                    &map_arg, &n_map, &no_ctrl};
    const hipError_t err = hipLaunchKernel(kernel, grid, dim3(kPullBlock), args, lds, (hipStream_t)stream);
    if (err != hipSuccess) {
        set_error("csr_propagate_pull2: launch failed: %s", hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    BMTK_CHECK_LAUNCH("csr_propagate_pull2");
    return BMTK_OK;
}
