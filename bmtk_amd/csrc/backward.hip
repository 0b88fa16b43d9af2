// Reverse-time adjoint of the forward simulation: transposed propagation,
// state adjoint, event-driven weight gradients.  The differentiable model
// these kernels transpose is stated in include/bmtk_amd.h (bmtk_glif3_bwd).
#include "common.hpp"
#include "glif3_update.hpp"

namespace bmtk {

struct BwdStep {
    int64_t t;    // absolute step being differentiated
    int64_t row;  // its row in the forward record
    int parts;    // partial sums gz[parts][ne] that the transposed propagation left (1, or 8 from the blocked form)
};

__device__ __forceinline__ float surrogate(float U, float th, float dampening)
{
    const float vhat = (U - th) / th;
    return dampening * fmaxf(0.0f, 1.0f - fabsf(vhat)) / th;
}

__device__ __forceinline__ unsigned long long trial_mask(const uint64_t *__restrict__ bits, int64_t j, int batch,
                                                         int tile0, int width)
{
    const int64_t bit = j * batch + tile0;
    const int64_t w = bit >> 6;
    const int sh = (int)(bit & 63);
    unsigned long long m = bits[w] >> sh;
    if (sh + width > 64) m |= bits[w + 1] << (64 - sh);
    if (width < 64) m &= (1ull << width) - 1ull;
    return m;
}

// gz[j*B+b] = sum over out-going synapses (j -> i, w, d, r) of w * lam_ring[(t+d)%L][r][i*B+b]:
// one wavefront per source neuron and trial tile.  A tile is `bp` trials wide
// (the batch rounded up to a power of two, at most 64) and the wavefront's 64
// lanes hold 64/bp synapses side by side, each lane reading one trial of one
// synapse's adjoint row (bp*4 contiguous bytes per synapse); four such groups
// are in flight before their products are added.  Rows whose every trial has
// a zero surrogate derivative in this step are skipped.
// kGrad (batches of one tile only): the recurrent weight gradient of the step rides along.  The wavefront has a
// synapse's adjoint row in registers anyway; where the source fired in some trial of this step, the entries of
// those trials are summed over the row's lanes and added to d_rec_w[p] -- this wavefront is the only writer of
// its row.  A separate kernel would fetch every such adjoint row a second time to use one or two words of it.
template <bool kGrad>
__global__ __launch_bounds__(kBlock) void bwd_gather_kernel(bmtk_glif3_bwd a, BwdStep q, int bp)
{
    const int batch = a.batch;
    const int64_t ne = a.n_neurons * (int64_t)batch;
    const int L = a.ring_slots;
    const int lane = lane_id();
    const int64_t j = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (j >= a.n_neurons) return;
    const int per = kWave / bp;  // synapses per wavefront instruction
    const int sub = lane / bp, b = lane - sub * bp;
    const int tile0 = blockIdx.y * kWave;
    const bool lane_on = tile0 + b < batch;
    const int64_t e = j * batch + tile0 + b;
    bool active = lane_on && a.save_flags == nullptr;  // without a forward record every element counts
    if (lane_on && a.save_flags) {
        const uint8_t f = a.save_flags[q.row * ne + e];
        if (f & BMTK_F_INTEGRATING) {
            const int64_t col = a.class_id ? (int64_t)a.class_id[j] : j;
            const float th = a.prop[GLIF3_TH * a.prop_stride + col];
            active = fabsf((a.save_v[q.row * ne + e] - th) / th) < 1.0f;
        }
    }
    // trials in which source j fired in this step (the same in all lanes)
    const unsigned long long fired = kGrad ? trial_mask(a.spike_bits + q.row * a.spike_bits_stride, j, batch, 0, batch) : 0ull;
    const bool mine = lane_on && ((fired >> b) & 1ull);
    if (__ballot(active) == 0ull && fired == 0ull) {
        if (lane_on && sub == 0) a.gz[e] = 0.0f;
        return;
    }
    const int slot0 = (int)(q.t % L);
    const int p0 = a.rec_indptr[j], p1 = a.rec_indptr[j + 1];
    const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(a.rec_packed);
    const float *__restrict__ ring = a.lam_ring + tile0 + b;
    constexpr int kInFlight = 4;
    float acc = 0.0f;
    for (int base = p0; base < p1; base += kWave) {
        const int p = base + lane;
        uint2 sy = make_uint2(0u, 0u);
        if (p < p1) sy = rows[p];
        const int n_here = min(kWave, p1 - base);
        for (int l0 = 0; l0 < n_here; l0 += per * kInFlight) {
            float w[kInFlight], v[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                const int idx = l0 + u * per + sub;
                const unsigned tdr = (unsigned)__shfl((int)sy.x, idx & (kWave - 1), kWave);
                w[u] = __uint_as_float((unsigned)__shfl((int)sy.y, idx & (kWave - 1), kWave));
                int slot = slot0 + (int)(tdr >> 26);
                slot = slot >= L ? slot - L : slot;
                const int r = (tdr >> 24) & 3;
                const int64_t i = tdr & 0xFFFFFFu;
                v[u] = ((active || mine) && idx < n_here) ? ring[(int64_t)(slot * GLIF3_NREC + r) * ne + i * batch] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) acc += active ? w[u] * v[u] : 0.0f;
            if (kGrad && fired != 0ull) {
#pragma unroll
                for (int u = 0; u < kInFlight; ++u) {
                    float g = mine ? v[u] : 0.0f;
                    for (int off = 1; off < bp; off <<= 1) g += __shfl_xor(g, off, kWave);
                    const int idx = l0 + u * per + sub;
                    if (b == 0 && idx < n_here) a.d_rec_w[base + idx] += g;
                }
            }
        }
    }
    for (int off = bp; off < kWave; off <<= 1) acc += __shfl_xor(acc, off, kWave);
    if (lane_on && sub == 0) a.gz[e] = acc;
}

// The same sums with four trials per lane, for batches that are a multiple of 4 and at most 64: a synapse's
// adjoint row (batch*4 contiguous bytes) is read by lp = bp/4 lanes as 16-byte pieces, so one wavefront
// instruction covers 64/lp synapses (8 at batch 32) and the address arithmetic and lane exchanges per synapse
// shrink fourfold.  Partial sums of the 64/lp synapse lanes are folded at the end.
template <bool kGrad>
__global__ __launch_bounds__(kBlock) void bwd_gather4_kernel(bmtk_glif3_bwd a, BwdStep q, int lp)
{
    const int batch = a.batch;
    const int64_t ne = a.n_neurons * (int64_t)batch;
    const int L = a.ring_slots;
    const int lane = lane_id();
    const int64_t j = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (j >= a.n_neurons) return;
    const int per = kWave / lp;  // synapses per wavefront instruction
    const int sub = lane / lp, b4 = (lane - sub * lp) * 4;
    const bool lane_on = b4 < batch;
    const int64_t e = j * batch + b4;
    unsigned act = (lane_on && a.save_flags == nullptr) ? 0xFu : 0u;  // bit c: trial b4+c has a non-zero surrogate derivative in this step
    if (lane_on && a.save_flags) {
        const uint32_t f4 = *reinterpret_cast<const uint32_t *>(a.save_flags + q.row * ne + e);
        const float4 v4 = *reinterpret_cast<const float4 *>(a.save_v + q.row * ne + e);
        const int64_t col = a.class_id ? (int64_t)a.class_id[j] : j;
        const float th = a.prop[GLIF3_TH * a.prop_stride + col];
        const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (((f4 >> (8 * c)) & BMTK_F_INTEGRATING) && fabsf((v[c] - th) / th) < 1.0f) act |= 1u << c;
    }
    // trials in which source j fired in this step (the same in all lanes), and this lane's four of them
    const unsigned long long fired = kGrad ? trial_mask(a.spike_bits + q.row * a.spike_bits_stride, j, batch, 0, batch) : 0ull;
    const unsigned mine = lane_on ? (unsigned)(fired >> b4) & 0xFu : 0u;
    if (__ballot(act != 0u) == 0ull && fired == 0ull) {
        if (lane_on && sub == 0) *reinterpret_cast<float4 *>(a.gz + e) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        return;
    }
    const int slot0 = (int)(q.t % L);
    const int p0 = a.rec_indptr[j], p1 = a.rec_indptr[j + 1];
    const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(a.rec_packed);
    const float *__restrict__ ring = a.lam_ring + b4;
    constexpr int kInFlight = 4;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int base = p0; base < p1; base += kWave) {
        const int p = base + lane;
        uint2 sy = make_uint2(0u, 0u);
        if (p < p1) sy = rows[p];
        const int n_here = min(kWave, p1 - base);
        for (int l0 = 0; l0 < n_here; l0 += per * kInFlight) {
            float w[kInFlight];
            float4 v[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                const int idx = l0 + u * per + sub;
                const unsigned tdr = (unsigned)__shfl((int)sy.x, idx & (kWave - 1), kWave);
                w[u] = __uint_as_float((unsigned)__shfl((int)sy.y, idx & (kWave - 1), kWave));
                int slot = slot0 + (int)(tdr >> 26);
                slot = slot >= L ? slot - L : slot;
                const int r = (tdr >> 24) & 3;
                const int64_t i = tdr & 0xFFFFFFu;
                v[u] = ((act | mine) != 0u && idx < n_here)
                           ? *reinterpret_cast<const float4 *>(ring + (int64_t)(slot * GLIF3_NREC + r) * ne + i * batch)
                           : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                acc[0] += w[u] * v[u].x;
                acc[1] += w[u] * v[u].y;
                acc[2] += w[u] * v[u].z;
                acc[3] += w[u] * v[u].w;
            }
            if (kGrad && fired != 0ull) {
#pragma unroll
                for (int u = 0; u < kInFlight; ++u) {
                    float g = ((mine & 1u) ? v[u].x : 0.0f) + ((mine & 2u) ? v[u].y : 0.0f) +
                              ((mine & 4u) ? v[u].z : 0.0f) + ((mine & 8u) ? v[u].w : 0.0f);
                    for (int off = 1; off < lp; off <<= 1) g += __shfl_xor(g, off, kWave);
                    const int idx = l0 + u * per + sub;
                    if (b4 == 0 && idx < n_here) a.d_rec_w[base + idx] += g;
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < 4; ++c)
        for (int off = lp; off < kWave; off <<= 1) acc[c] += __shfl_xor(acc[c], off, kWave);
    if (lane_on && sub == 0)
        *reinterpret_cast<float4 *>(a.gz + e) = make_float4((act & 1u) ? acc[0] : 0.0f, (act & 2u) ? acc[1] : 0.0f,
                                                            (act & 4u) ? acc[2] : 0.0f, (act & 8u) ? acc[3] : 0.0f);
}

// The same sums through the table regrouped by target range, for networks whose adjoint ring is far larger than an
// L2.  bwd_gather4_kernel visits the adjoint rows of a source's targets all over the ring: at 52k neurons x 32
// trials the ring is 133 MB, every 128-byte row misses the 4 MB L2 of its XCD and the kernel runs at the rate the
// fabric fills L2 lines (6.4 GB per step).  Here the targets are cut into blk_count ranges whose slice of the ring
// (all slots and receptors) fits an L2, and the table holds, range after range, a CSR over the sources of the
// synapses into that range.  Workgroup b runs on XCD b % 8 (workgroups are dealt to the XCDs in turn) and takes
// the ranges x*P .. x*P+P-1, one after the other, over a fixed share of the source rows, so that while an XCD
// works through a range its L2 holds that slice and each adjoint row is fetched from memory once per sweep
// instead of once per synapse.  A lane group of lp lanes (4 trials each) owns one source row; its partial sum
// over the ranges seen so far waits in LDS (16 bytes per lane and row, lane-private, so no barriers), which is
// what bounds the rows of a sweep: 16 wavefronts x gpw row groups x 64/lp rows.  The eight XCDs each see every
// row for their own ranges and write a partial sum of their own, gz[x][ne]; the state adjoint adds the eight.
__device__ __forceinline__ void bwd_inp_grad_waves(const bmtk_glif3_bwd &a, const BwdStep &q, int wave, int n_waves);
__device__ __forceinline__ void bwd_inp_grad2_waves(const bmtk_glif3_bwd &a, const BwdStep &q, int wave, int n_waves);
constexpr int kBlkThreads = 1024;
constexpr int kBlkWaves = kBlkThreads / kWave;
constexpr int kBlkMaxGroups = 8;  // row groups per wavefront and sweep: one byte of trial masks each in a 64-bit register
constexpr int kBlkInFlight = 8;   // synapses of a row in flight
static_assert(kBlkInFlight % 8 == 0 && 2 * kBlkInFlight <= BMTK_BLOCKED_PAD, "the kernel reads up to 2*kBlkInFlight - 1 records past a row's end");

// the value of `x` in the lane a data-parallel-primitive control word names (all of the ones used here have a source)
template <int kCtrl>
__device__ __forceinline__ float dpp_move(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), kCtrl, 0xF, 0xF, false));
}

// kNe24: n_neurons*batch < 2^24, so that the cell arithmetic can use 24-bit multiplies; kWide: lp >= 8
template <bool kGrad, bool kNe24, bool kWide>
__global__ __launch_bounds__(kBlkThreads) void bwd_gather_blocked_kernel(bmtk_glif3_bwd a, BwdStep q, int lp, int rows_cu,
                                                                         int sweeps, int gpw, int use_order, int do_inp)
{
    extern __shared__ float4 blk_acc[];  // [kBlkWaves][gpw][kWave], then the row order (uint16 per place)
    constexpr int kF = kBlkInFlight;
    const int batch = a.batch;
    const int64_t n = a.n_neurons, ne = n * batch;
    const int L = a.ring_slots;
    const int lane = lane_id(), wave = threadIdx.x / kWave;
    const int x = blockIdx.x & 7;
    const int P = a.blk_count >> 3;
    const int per = kWave / lp;  // rows a wavefront works on side by side
    const int grp = lane / lp, b4 = (lane - grp * lp) * 4;
    const bool lane_on = b4 < batch;
    const unsigned long long grp_lanes = (lp == kWave ? ~0ull : ((1ull << lp) - 1ull)) << (grp * lp);
    const int64_t row_lo = (int64_t)(blockIdx.x >> 3) * rows_cu;
    const int64_t row_hi = row_lo + rows_cu < n ? row_lo + rows_cu : n;
    const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(a.blk_packed);
    // byte offset of a synapse's adjoint cell from the start of the ring, in 32 bits: the record's upper byte is
    // delay*4 + receptor, so (slot0 + delay) % L * 4 + receptor = min(u, u - 4L) with u = slot0*4 + that byte
    const char *__restrict__ ring = reinterpret_cast<const char *>(a.lam_ring);
    const unsigned lane_off = (unsigned)b4 * 4u;
    const unsigned q_lo = (unsigned)(q.t % L) * 4u, q_wrap = q_lo - 4u * (unsigned)L;
    const unsigned ne32 = (unsigned)ne, batch32 = (unsigned)batch;
    auto cell_off = [&](unsigned tdr) -> unsigned {
        const unsigned dq = tdr >> 24;
        const unsigned plane = min(dq + q_lo, dq + q_wrap);
        const unsigned elem = mad_u24(tdr, batch32, kNe24 ? mul_u24(plane, ne32) : plane * ne32);  // bits 24-31 of tdr do not count
        return (elem << 2) + lane_off;
    };
    float4 *acc = blk_acc + (size_t)wave * gpw * kWave + lane;
    // Which row a lane group works on.  The workgroup's rows are taken in groups of `per` (a wavefront's lane groups
    // side by side), group g by wavefront g % 16 as its (g / 16)-th.  With the gradient riding along, the rows
    // whose source fired in this step come first in that order (a list in LDS, built once per launch): a wavefront
    // runs the gradient's extra work whenever ONE of its rows fired, so with a tenth of the rows firing and eight
    // rows side by side more than half of all visits ran it, seven eighths idle; gathered into the first groups
    // the fired rows fill a tenth of the visits, dealt out evenly over the wavefronts.
    uint16_t *order = reinterpret_cast<uint16_t *>(blk_acc + (size_t)kBlkWaves * gpw * kWave);
    const int places = sweeps * kBlkWaves * gpw * per;
    if (kGrad && use_order) {
        __shared__ unsigned scan_l[2][kBlkWaves];
        const uint64_t *__restrict__ bits = a.spike_bits + q.row * a.spike_bits_stride;
        // a thread looks at rows threadIdx.x, threadIdx.x + 1024, ... (at most 16): fired or not, one bit each
        unsigned fm = 0u, n_mine = 0u;
        for (int i = 0; (int)threadIdx.x + i * kBlkThreads < rows_cu; ++i) {
            const int64_t j = row_lo + threadIdx.x + i * kBlkThreads;
            if (j < row_hi && trial_mask(bits, j, batch, 0, batch) != 0ull) fm |= 1u << i;
            ++n_mine;
        }
        const unsigned c1 = (unsigned)__popc(fm), c0 = n_mine - c1;
        const unsigned in1 = wave_inclusive_scan(c1), in0 = wave_inclusive_scan(c0);
        if (lane == kWave - 1) {
            scan_l[0][wave] = in0;
            scan_l[1][wave] = in1;
        }
        __syncthreads();
        unsigned base0 = 0u, base1 = 0u, total1 = 0u;
#pragma unroll
        for (int w = 0; w < kBlkWaves; ++w) {
            if (w < wave) {
                base0 += scan_l[0][w];
                base1 += scan_l[1][w];
            }
            total1 += scan_l[1][w];
        }
        unsigned p1 = base1 + in1 - c1, p0 = total1 + base0 + in0 - c0;  // next place among the fired / the others
        for (unsigned i = 0; i < n_mine; ++i) {
            const unsigned local = threadIdx.x + i * kBlkThreads;
            if ((fm >> i) & 1u)
                order[p1++] = (uint16_t)local;
            else
                order[p0++] = (uint16_t)local;
        }
        for (int i = rows_cu + (int)threadIdx.x; i < places; i += kBlkThreads) order[i] = 0xFFFFu;  // places without a row
        __syncthreads();
    }
    // row of lane group `grp` in the wavefront's k-th group of sweep sw (row_hi and beyond: none)
    auto row_of = [&](int sw, int k) -> int64_t {
        const int place = ((sw * gpw + k) * kBlkWaves + wave) * per + grp;
        if (kGrad && use_order) {
            const unsigned local = order[place];
            return local == 0xFFFFu ? row_hi : row_lo + local;
        }
        return place < rows_cu ? row_lo + place : row_hi;
    };
    for (int sw = 0; sw < sweeps; ++sw) {
        // per row group one byte: bits 0-3 the lane's trials with a non-zero surrogate derivative in this step,
        // bits 4-7 those in which the source fired (kGrad)
        unsigned long long masks = 0ull;
        for (int k = 0; k < gpw; ++k) {
            const int64_t j = row_of(sw, k);
            unsigned act = 0u, mine = 0u;
            if (j < row_hi && lane_on) {
                const int64_t e = j * batch + b4;
                if (a.save_flags) {
                    const uint32_t f4 = *reinterpret_cast<const uint32_t *>(a.save_flags + q.row * ne + e);
                    const float4 v4 = *reinterpret_cast<const float4 *>(a.save_v + q.row * ne + e);
                    const int64_t col = a.class_id ? (int64_t)a.class_id[j] : j;
                    const float th = a.prop[GLIF3_TH * a.prop_stride + col];
                    const float v[4] = {v4.x, v4.y, v4.z, v4.w};
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        if (((f4 >> (8 * c)) & BMTK_F_INTEGRATING) && fabsf((v[c] - th) / th) < 1.0f) act |= 1u << c;
                } else {
                    act = 0xFu;
                }
                if (kGrad)
                    mine = (unsigned)(trial_mask(a.spike_bits + q.row * a.spike_bits_stride, j, batch, 0, batch) >> b4) & 0xFu;
            }
            masks |= (unsigned long long)(act | (mine << 4)) << (8 * k);
            acc[k * kWave] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
        // the synapses this lane's row of group k sends into range ph: [p, p1); empty for rows none of whose
        // trials needs them, and for rows past the end
        auto row_range = [&](int ph, int k, int &p, int &p1) {
            p = p1 = 0;
            if (ph >= P) return;
            const bool want = ((masks >> (8 * k)) & 0xFFull) != 0ull;
            const int64_t j = row_of(sw, k);
            if ((__ballot(want) & grp_lanes) != 0ull && j < row_hi) {
                const int32_t *__restrict__ ip = a.blk_indptr + (int64_t)(x * P + ph) * n + j;
                p = ip[0];
                p1 = ip[1];
            }
        };
        int p_next, p1_next;
        row_range(0, 0, p_next, p1_next);
        for (int ph = 0; ph < P; ++ph) {
            for (int k = 0; k < gpw; ++k) {
                int p = p_next;
                const int p1 = p1_next;
                row_range(k + 1 < gpw ? ph : ph + 1, k + 1 < gpw ? k + 1 : 0, p_next, p1_next);  // asked for a visit ahead
                if (__ballot(p < p1) == 0ull) continue;
                const unsigned mine = (unsigned)(masks >> (8 * k + 4)) & 0xFu;
                const int p1_lane = ((masks >> (8 * k)) & 0xFFull) != 0ull ? p1 : 0;  // lanes none of whose trials counts stay idle
                const bool row_fired = kGrad && (__ballot(mine != 0u) & grp_lanes) != 0ull;
                const float fired_f[4] = {(mine & 1u) ? 1.0f : 0.0f, (mine & 2u) ? 1.0f : 0.0f, (mine & 4u) ? 1.0f : 0.0f,
                                          (mine & 8u) ? 1.0f : 0.0f};
                const int in_row = lane - grp * lp;  // this lane's place among its row's lanes
                float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                // kF synapses of the row at a time: their adjoint rows are asked for, then the row's next kF
                // records (which arrive while the adjoint rows are on their way), then the products are added.
                // Lanes past the row's end read the ring's first cell with weight 0 -- no branches around loads.
                auto visit = [&](auto fetch, auto record) {
                    auto cur = fetch(0), nxt = cur;
                    auto work = [&](const decltype(cur) &have, decltype(cur) &ahead) {
                        float4 v[kF];
                        float w[kF];
#pragma unroll
                        for (int u = 0; u < kF; ++u) {
                            const uint2 sy = record(have, u);
                            const bool valid = p + u < p1_lane;
                            const unsigned off = valid ? cell_off(sy.x) : lane_off;
                            w[u] = valid ? __uint_as_float(sy.y) : 0.0f;
                            v[u] = *reinterpret_cast<const float4 *>(ring + off);
                        }
                        ahead = fetch(kF);
#pragma unroll
                        for (int u = 0; u < kF; ++u) {
                            s.x = fmaf(w[u], v[u].x, s.x);
                            s.y = fmaf(w[u], v[u].y, s.y);
                            s.z = fmaf(w[u], v[u].z, s.z);
                            s.w = fmaf(w[u], v[u].w, s.w);
                        }
                        if (kGrad && __ballot(row_fired && p < p1) != 0ull) {
                            if (kWide) {
                                // the gradient of record u is the sum, over the row's lanes, of the adjoint entries of
                                // the trials in which the source fired; every lane gets every sum (data-parallel
                                // moves within quads, half rows and rows of 16 lanes) and keeps the one of the
                                // record it then updates: one read-modify-write for the kF records of all rows
                                float keep = 0.0f;
#pragma unroll
                                for (int u = 0; u < kF; ++u) {
                                    float g = fmaf(fired_f[3], v[u].w, fmaf(fired_f[2], v[u].z, fmaf(fired_f[1], v[u].y, fired_f[0] * v[u].x)));
                                    g += dpp_move<0xB1>(g);   // quad_perm [1,0,3,2]
                                    g += dpp_move<0x4E>(g);   // quad_perm [2,3,0,1]
                                    g += dpp_move<0x141>(g);  // row_half_mirror: the other quad of these eight lanes
                                    if (lp > 8) g += dpp_move<0x140>(g);  // row_mirror: the other eight of these sixteen
                                    keep = in_row == u ? g : keep;
                                }
                                if (row_fired && in_row < kF && p + in_row < p1) a.d_blk_w[p + in_row] += keep;
                            } else {
#pragma unroll
                                for (int u = 0; u < kF; ++u) {
                                    float g = ((mine & 1u) ? v[u].x : 0.0f) + ((mine & 2u) ? v[u].y : 0.0f) +
                                              ((mine & 4u) ? v[u].z : 0.0f) + ((mine & 8u) ? v[u].w : 0.0f);
                                    for (int off = 1; off < lp; off <<= 1) g += __shfl_xor(g, off, kWave);
                                    if (row_fired && b4 == 0 && p + u < p1) a.d_blk_w[p + u] += g;
                                }
                            }
                        }
                        // a lane whose row segment has ended stays at its end: with p <= p1 at every fetch no lane
                        // reads a record at or beyond p1 + 2*kF, which is what BMTK_BLOCKED_PAD covers, however much
                        // longer the other rows of the visit are
                        p = min(p + kF, p1);
                    };
                    while (true) {
                        work(cur, nxt);
                        if (__ballot(p < p1) == 0ull) break;
                        work(nxt, cur);
                        if (__ballot(p < p1) == 0ull) break;
                    }
                };
                if (kWide) {
                    // a row's first eight lanes fetch one record in eight each (one wavefront instruction for eight
                    // records of every row) and pass them round; eight lanes fetching the same record eight times
                    // over kept the address unit busier than the adjoint rows did
                    struct Shared {
                        uint2 r[kF / 8];
                    };
                    const int c = (lane - grp * lp) & 7, first = grp * lp;
                    visit(
                        [&](int ahead) {
                            Shared f;
#pragma unroll
                            for (int i = 0; i < kF / 8; ++i) f.r[i] = rows[p + ahead + 8 * i + c];
                            return f;
                        },
                        [&](const Shared &have, int u) {
                            return make_uint2((unsigned)__shfl((int)have.r[u / 8].x, first + (u & 7), kWave),
                                              (unsigned)__shfl((int)have.r[u / 8].y, first + (u & 7), kWave));
                        });
                } else {
                    struct Records {
                        uint2 r[kF];
                    };
                    visit(
                        [&](int ahead) {
                            Records f;
#pragma unroll
                            for (int u = 0; u < kF; ++u) f.r[u] = rows[p + ahead + u];
                            return f;
                        },
                        [&](const Records &have, int u) { return have.r[u]; });
                }
                float4 t = acc[k * kWave];
                t.x += s.x;
                t.y += s.y;
                t.z += s.z;
                t.w += s.w;
                acc[k * kWave] = t;
            }
        }
        for (int k = 0; k < gpw; ++k) {
            const int64_t j = row_of(sw, k);
            if (j < row_hi && lane_on) {
                const unsigned act = (unsigned)(masks >> (8 * k)) & 0xFu;
                const float4 t = acc[k * kWave];
                *reinterpret_cast<float4 *>(a.gz + (int64_t)x * ne + j * batch + b4) =
                    make_float4((act & 1u) ? t.x : 0.0f, (act & 2u) ? t.y : 0.0f, (act & 4u) ? t.z : 0.0f,
                                (act & 8u) ? t.w : 0.0f);
            }
        }
    }
    // The input-weight gradient of the same step (it reads the same adjoint slots): a few thousand runs of events,
    // each a chain of dependent reads for one wavefront.  Done here by whichever wavefronts are through with their
    // rows, it disappears in this kernel's tail; beside the state adjoint it lengthened that launch by 20 us.
    if (do_inp) bwd_inp_grad_waves(a, q, (int)blockIdx.x * kBlkWaves + wave, (int)gridDim.x * kBlkWaves);
}

// TWO steps, t = q.t and t-1, in one pass over the blocked table (batches above 16: lp >= 8).  gz of step t reads
// the adjoint slots t+1 .. t+L-1, gz of step t-1 the slots t .. t+L-2, and slot t only depends on what the state
// adjoint of step t+1 left behind (it is psc0 times the adjoint of y1 BEFORE step t is undone): both sums can be taken
// before the state adjoint of step t runs.  Per synapse the record, its weight, the trip round the row's lanes, the
// row's bounds and the loop around them are paid once for two steps; the two adjoint rows (same target and
// receptor, neighbouring slots) are fetched side by side.  The weight gradient rides along for both steps with ONE
// read-modify-write per record.  Partial sums: gz[x] for step t, gz[8 + x] for step t-1.  Everything else as in
// bwd_gather_blocked_kernel, except that a row's two partial sums take 32 bytes of LDS per lane (half as many rows
// per sweep).
template <bool kGrad, bool kNe24>
__global__ __launch_bounds__(kBlkThreads) void bwd_gather_blocked2_kernel(bmtk_glif3_bwd a, BwdStep q, int lp, int rows_cu,
                                                                          int sweeps, int gpw, int use_order, int do_inp)
{
    extern __shared__ float4 blk_acc[];  // [kBlkWaves][gpw][2][kWave], then the row order (uint16 per place)
    constexpr int kF = kBlkInFlight;
    const int batch = a.batch;
    const int64_t n = a.n_neurons, ne = n * batch;
    const int L = a.ring_slots;
    const int lane = lane_id(), wave = threadIdx.x / kWave;
    const int x = blockIdx.x & 7;
    const int P = a.blk_count >> 3;
    const int per = kWave / lp;
    const int grp = lane / lp, b4 = (lane - grp * lp) * 4;
    const bool lane_on = b4 < batch;
    const unsigned long long grp_lanes = (lp == kWave ? ~0ull : ((1ull << lp) - 1ull)) << (grp * lp);
    const int64_t row_lo = (int64_t)(blockIdx.x >> 3) * rows_cu;
    const int64_t row_hi = row_lo + rows_cu < n ? row_lo + rows_cu : n;
    const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(a.blk_packed);
    const char *__restrict__ ring = reinterpret_cast<const char *>(a.lam_ring);
    const unsigned lane_off = (unsigned)b4 * 4u;
    const unsigned q_lo = (unsigned)(q.t % L) * 4u, q_wrap = q_lo - 4u * (unsigned)L;
    const unsigned ne32 = (unsigned)ne, batch32 = (unsigned)batch;
    // from a synapse's cell for step t to its cell for step t-1: one slot down, or L-1 slots up from slot 0 (bytes)
    const unsigned slot_down = 0u - 16u * ne32, slot_up = 16u * ne32 * (unsigned)(L - 1);
    auto cell_offs = [&](unsigned tdr, unsigned &off_t, unsigned &off_p) {
        const unsigned dq = tdr >> 24;
        const unsigned plane = min(dq + q_lo, dq + q_wrap);  // (slot of step t + delay) * 4 + receptor
        const unsigned elem = mad_u24(tdr, batch32, kNe24 ? mul_u24(plane, ne32) : plane * ne32);
        off_t = (elem << 2) + lane_off;
        off_p = off_t + (plane < 4u ? slot_up : slot_down);
    };
    float4 *acc = blk_acc + (size_t)wave * gpw * 2 * kWave + lane;
    const uint64_t *__restrict__ bits_t = a.spike_bits + q.row * a.spike_bits_stride;
    const uint64_t *__restrict__ bits_p = a.spike_bits + (q.row - 1) * a.spike_bits_stride;
    uint16_t *order = reinterpret_cast<uint16_t *>(blk_acc + (size_t)kBlkWaves * gpw * 2 * kWave);
    const int places = sweeps * kBlkWaves * gpw * per;
    if (kGrad && use_order) {  // rows whose source fired in one of the two steps first (see bwd_gather_blocked_kernel)
        __shared__ unsigned scan_l[2][kBlkWaves];
        unsigned fm = 0u, n_mine = 0u;
        for (int i = 0; (int)threadIdx.x + i * kBlkThreads < rows_cu; ++i) {
            const int64_t j = row_lo + threadIdx.x + i * kBlkThreads;
            if (j < row_hi && (trial_mask(bits_t, j, batch, 0, batch) | trial_mask(bits_p, j, batch, 0, batch)) != 0ull)
                fm |= 1u << i;
            ++n_mine;
        }
        const unsigned c1 = (unsigned)__popc(fm), c0 = n_mine - c1;
        const unsigned in1 = wave_inclusive_scan(c1), in0 = wave_inclusive_scan(c0);
        if (lane == kWave - 1) {
            scan_l[0][wave] = in0;
            scan_l[1][wave] = in1;
        }
        __syncthreads();
        unsigned base0 = 0u, base1 = 0u, total1 = 0u;
#pragma unroll
        for (int w = 0; w < kBlkWaves; ++w) {
            if (w < wave) {
                base0 += scan_l[0][w];
                base1 += scan_l[1][w];
            }
            total1 += scan_l[1][w];
        }
        unsigned at1 = base1 + in1 - c1, at0 = total1 + base0 + in0 - c0;
        for (unsigned i = 0; i < n_mine; ++i) {
            const unsigned local = threadIdx.x + i * kBlkThreads;
            if ((fm >> i) & 1u)
                order[at1++] = (uint16_t)local;
            else
                order[at0++] = (uint16_t)local;
        }
        for (int i = rows_cu + (int)threadIdx.x; i < places; i += kBlkThreads) order[i] = 0xFFFFu;
        __syncthreads();
    }
    auto row_of = [&](int sw, int k) -> int64_t {
        const int place = ((sw * gpw + k) * kBlkWaves + wave) * per + grp;
        if (kGrad && use_order) {
            const unsigned local = order[place];
            return local == 0xFFFFu ? row_hi : row_lo + local;
        }
        return place < rows_cu ? row_lo + place : row_hi;
    };
    // trials of this lane with a non-zero surrogate derivative in the step of record row `rec_row`
    auto active_trials = [&](int64_t rec_row, int64_t j) -> unsigned {
        if (!a.save_flags) return 0xFu;
        const int64_t e = j * batch + b4;
        const uint32_t f4 = *reinterpret_cast<const uint32_t *>(a.save_flags + rec_row * ne + e);
        const float4 v4 = *reinterpret_cast<const float4 *>(a.save_v + rec_row * ne + e);
        const int64_t col = a.class_id ? (int64_t)a.class_id[j] : j;
        const float th = a.prop[GLIF3_TH * a.prop_stride + col];
        const float v[4] = {v4.x, v4.y, v4.z, v4.w};
        unsigned act = 0u;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            if (((f4 >> (8 * c)) & BMTK_F_INTEGRATING) && fabsf((v[c] - th) / th) < 1.0f) act |= 1u << c;
        return act;
    };
    for (int sw = 0; sw < sweeps; ++sw) {
        // per row group one byte in each word: bits 0-3 the lane's trials with a non-zero surrogate derivative in
        // the step, bits 4-7 those in which the source fired (kGrad); masks_t for step t, masks_p for step t-1
        unsigned long long masks_t = 0ull, masks_p = 0ull;
        for (int k = 0; k < gpw; ++k) {
            const int64_t j = row_of(sw, k);
            unsigned at = 0u, ap = 0u, mt = 0u, mp = 0u;
            if (j < row_hi && lane_on) {
                at = active_trials(q.row, j);
                ap = active_trials(q.row - 1, j);
                if (kGrad) {
                    mt = (unsigned)(trial_mask(bits_t, j, batch, 0, batch) >> b4) & 0xFu;
                    mp = (unsigned)(trial_mask(bits_p, j, batch, 0, batch) >> b4) & 0xFu;
                }
            }
            masks_t |= (unsigned long long)(at | (mt << 4)) << (8 * k);
            masks_p |= (unsigned long long)(ap | (mp << 4)) << (8 * k);
            acc[(2 * k) * kWave] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            acc[(2 * k + 1) * kWave] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
        const unsigned long long masks_any = masks_t | masks_p;
        auto row_range = [&](int ph, int k, int &p, int &p1) {
            p = p1 = 0;
            if (ph >= P) return;
            const bool want = ((masks_any >> (8 * k)) & 0xFFull) != 0ull;
            const int64_t j = row_of(sw, k);
            if ((__ballot(want) & grp_lanes) != 0ull && j < row_hi) {
                const int32_t *__restrict__ ip = a.blk_indptr + (int64_t)(x * P + ph) * n + j;
                p = ip[0];
                p1 = ip[1];
            }
        };
        int p_next, p1_next;
        row_range(0, 0, p_next, p1_next);
        for (int ph = 0; ph < P; ++ph) {
            for (int k = 0; k < gpw; ++k) {
                int p = p_next;
                const int p1 = p1_next;
                row_range(k + 1 < gpw ? ph : ph + 1, k + 1 < gpw ? k + 1 : 0, p_next, p1_next);
                if (__ballot(p < p1) == 0ull) continue;
                const unsigned mine_t = (unsigned)(masks_t >> (8 * k + 4)) & 0xFu, mine_p = (unsigned)(masks_p >> (8 * k + 4)) & 0xFu;
                const int p1_lane = ((masks_any >> (8 * k)) & 0xFFull) != 0ull ? p1 : 0;
                const bool row_fired = kGrad && (__ballot((mine_t | mine_p) != 0u) & grp_lanes) != 0ull;
                const int in_row = lane - grp * lp;
                const int c8 = in_row & 7, first = grp * lp;
                float4 s_t = make_float4(0.0f, 0.0f, 0.0f, 0.0f), s_p = s_t;
                struct Shared {
                    uint2 r[kF / 8];
                };
                auto fetch = [&](int ahead) {
                    Shared f;
#pragma unroll
                    for (int i = 0; i < kF / 8; ++i) f.r[i] = rows[p + ahead + 8 * i + c8];
                    return f;
                };
                auto record = [&](const Shared &have, int u) {
                    return make_uint2((unsigned)__shfl((int)have.r[u / 8].x, first + (u & 7), kWave),
                                      (unsigned)__shfl((int)have.r[u / 8].y, first + (u & 7), kWave));
                };
                Shared cur = fetch(0), nxt = cur;
                auto work = [&](const Shared &have, Shared &ahead) {
                    float keep = 0.0f;
                    const bool grad_now = kGrad && __ballot(row_fired && p < p1) != 0ull;
                    float4 vt[kF], vp[kF];
                    float w[kF];
#pragma unroll
                    for (int u = 0; u < kF; ++u) {
                        const uint2 sy = record(have, u);
                        const bool valid = p + u < p1_lane;
                        // (lanes past their row's end take record 0 with weight 0: one select, then the same
                        // arithmetic and the same two loads for every lane.  With the select on the address instead,
                        // the compiler branched around the loads and waited for each of them.)
                        unsigned off_t, off_p;
                        cell_offs(valid ? sy.x : 0u, off_t, off_p);
                        w[u] = valid ? __uint_as_float(sy.y) : 0.0f;
                        vt[u] = *reinterpret_cast<const float4 *>(ring + off_t);
                        vp[u] = *reinterpret_cast<const float4 *>(ring + off_p);
                    }
                    ahead = fetch(kF);
#pragma unroll
                    for (int u = 0; u < kF; ++u) {
                        s_t.x = fmaf(w[u], vt[u].x, s_t.x);
                        s_t.y = fmaf(w[u], vt[u].y, s_t.y);
                        s_t.z = fmaf(w[u], vt[u].z, s_t.z);
                        s_t.w = fmaf(w[u], vt[u].w, s_t.w);
                        s_p.x = fmaf(w[u], vp[u].x, s_p.x);
                        s_p.y = fmaf(w[u], vp[u].y, s_p.y);
                        s_p.z = fmaf(w[u], vp[u].z, s_p.z);
                        s_p.w = fmaf(w[u], vp[u].w, s_p.w);
                    }
                    if (grad_now) {
                        // gradient of a record: over the row's lanes, the adjoint entries of the trials in which the
                        // source fired, of step t and of step t-1 (see bwd_gather_blocked_kernel)
#pragma unroll
                        for (int u = 0; u < kF; ++u) {
                            float g = ((mine_t & 1u) ? vt[u].x : 0.0f) + ((mine_t & 2u) ? vt[u].y : 0.0f) +
                                      ((mine_t & 4u) ? vt[u].z : 0.0f) + ((mine_t & 8u) ? vt[u].w : 0.0f);
                            g += ((mine_p & 1u) ? vp[u].x : 0.0f) + ((mine_p & 2u) ? vp[u].y : 0.0f) +
                                 ((mine_p & 4u) ? vp[u].z : 0.0f) + ((mine_p & 8u) ? vp[u].w : 0.0f);
                            g += dpp_move<0xB1>(g);
                            g += dpp_move<0x4E>(g);
                            g += dpp_move<0x141>(g);
                            if (lp > 8) g += dpp_move<0x140>(g);
                            keep = in_row == u ? g : keep;
                        }
                    }
                    if (grad_now && row_fired && in_row < kF && p + in_row < p1) a.d_blk_w[p + in_row] += keep;
                    p = min(p + kF, p1);  // (a lane whose segment has ended stays at its end: BMTK_BLOCKED_PAD)
                };
                while (true) {
                    work(cur, nxt);
                    if (__ballot(p < p1) == 0ull) break;
                    work(nxt, cur);
                    if (__ballot(p < p1) == 0ull) break;
                }
                float4 t = acc[(2 * k) * kWave];
                t.x += s_t.x;
                t.y += s_t.y;
                t.z += s_t.z;
                t.w += s_t.w;
                acc[(2 * k) * kWave] = t;
                t = acc[(2 * k + 1) * kWave];
                t.x += s_p.x;
                t.y += s_p.y;
                t.z += s_p.z;
                t.w += s_p.w;
                acc[(2 * k + 1) * kWave] = t;
            }
        }
        for (int k = 0; k < gpw; ++k) {
            const int64_t j = row_of(sw, k);
            if (j < row_hi && lane_on) {
                const unsigned at = (unsigned)(masks_t >> (8 * k)) & 0xFu, ap = (unsigned)(masks_p >> (8 * k)) & 0xFu;
                float4 t = acc[(2 * k) * kWave];
                *reinterpret_cast<float4 *>(a.gz + (int64_t)x * ne + j * batch + b4) =
                    make_float4((at & 1u) ? t.x : 0.0f, (at & 2u) ? t.y : 0.0f, (at & 4u) ? t.z : 0.0f, (at & 8u) ? t.w : 0.0f);
                t = acc[(2 * k + 1) * kWave];
                *reinterpret_cast<float4 *>(a.gz + (int64_t)(8 + x) * ne + j * batch + b4) =
                    make_float4((ap & 1u) ? t.x : 0.0f, (ap & 2u) ? t.y : 0.0f, (ap & 4u) ? t.z : 0.0f, (ap & 8u) ? t.w : 0.0f);
            }
        }
    }
    // the input-weight gradients of both steps, in the kernel's tail
    if (do_inp) bwd_inp_grad2_waves(a, q, (int)blockIdx.x * kBlkWaves + wave, (int)gridDim.x * kBlkWaves);
}

// One step of the state adjoint on registers: the adjoint of the state after the step comes in, that of the state
// before it goes out.  sg = surrogate derivative times the adjoint of the step's spike (only read where the
// element was integrating).
__device__ __forceinline__ void state_adjoint_step(float &lV, float (&lA)[GLIF3_NASC], float (&l1)[GLIF3_NREC],
                                                   float (&l2)[GLIF3_NREC], const Glif3Prop &p, float h, uint8_t f, float sg)
{
    // y1' = P11*y1 + psc0*s ; y2' = P21*y1 + P11*y2
    float n1[GLIF3_NREC], n2[GLIF3_NREC];
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        n1[k] = p.P11[k] * l1[k] + (h * p.P11[k]) * l2[k];
        n2[k] = p.P11[k] * l2[k];
    }
    float nV, nA[GLIF3_NASC];
    if (f & BMTK_F_INTEGRATING) {
        const float lU = lV + sg;
        nV = p.P33 * lU;
        const float lS = p.P30 * lU;
#pragma unroll
        for (int k = 0; k < GLIF3_NASC; ++k) nA[k] = p.c[k] * lS + p.d[k] * lA[k];
#pragma unroll
        for (int k = 0; k < GLIF3_NREC; ++k) {
            n1[k] += p.P31[k] * lU;
            n2[k] += p.P32[k] * lU;
        }
    } else if (f & BMTK_F_RESET) {
        nV = 0.0f;
#pragma unroll
        for (int k = 0; k < GLIF3_NASC; ++k) nA[k] = p.r[k] * lA[k];
    } else {
        nV = lV;
#pragma unroll
        for (int k = 0; k < GLIF3_NASC; ++k) nA[k] = lA[k];
    }
    lV = nV;
#pragma unroll
    for (int k = 0; k < GLIF3_NASC; ++k) lA[k] = nA[k];
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        l1[k] = n1[k];
        l2[k] = n2[k];
    }
}

// surrogate derivative times the adjoint of the spike of element e in the step of record row `row`: what comes back
// through the synapses (`parts` partial sums from plane `first` of gz on) plus the loss derivative
__device__ __forceinline__ float spike_adjoint(const bmtk_glif3_bwd &a, const Glif3Prop &p, int64_t row, int64_t e, int64_t ne,
                                               int first, int parts)
{
    float g = a.gz[(int64_t)first * ne + e];
    for (int x = 1; x < parts; ++x) g += a.gz[(int64_t)(first + x) * ne + e];
    if (a.dl_dz) g += a.dl_dz[row * ne + e];
    if (a.dl_dz_const) g += a.dl_dz_const[e];
    return surrogate(a.save_v[row * ne + e], p.th, a.dampening) * g;
}

// state adjoint of one step, one thread per element; writes the adjoint of
// this step's arrivals into ring slot t
__device__ __forceinline__ void bwd_state_block(const bmtk_glif3_bwd &a, const BwdStep &q, int64_t block)
{
    const int64_t ne = a.n_neurons * (int64_t)a.batch;
    const int64_t e = block * kBlock + threadIdx.x;
    if (e >= ne) return;
    const int64_t n = a.batch == 1 ? e : (int64_t)((uint32_t)e / (uint32_t)a.batch);
    const int64_t col = a.class_id ? (int64_t)a.class_id[n] : n;
    Glif3Prop p;
    p.load(a.prop, a.prop_stride, col);
    const uint8_t f = a.save_flags[q.row * ne + e];
    float lV = a.lam_V[e];
    float lA[GLIF3_NASC], l1[GLIF3_NREC], l2[GLIF3_NREC];
#pragma unroll
    for (int k = 0; k < GLIF3_NASC; ++k) lA[k] = a.lam_asc[k * ne + e];
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        l1[k] = a.lam_y1[k * ne + e];
        l2[k] = a.lam_y2[k * ne + e];
    }
    float *slot = a.lam_ring + (int64_t)(q.t % a.ring_slots) * GLIF3_NREC * ne + e;
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) slot[k * ne] = p.psc0[k] * l1[k];
    const float sg = (f & BMTK_F_INTEGRATING) ? spike_adjoint(a, p, q.row, e, ne, 0, q.parts) : 0.0f;
    state_adjoint_step(lV, lA, l1, l2, p, a.h, f, sg);
    a.lam_V[e] = lV;
#pragma unroll
    for (int k = 0; k < GLIF3_NASC; ++k) a.lam_asc[k * ne + e] = lA[k];
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        a.lam_y1[k * ne + e] = l1[k];
        a.lam_y2[k * ne + e] = l2[k];
    }
}

// The state adjoints of steps t = q.t and t-1 in one launch, the adjoint state in registers in between: the partial
// sums of step t are planes 0-7 of gz, those of step t-1 planes 8-15 (bwd_gather_blocked2_kernel).  Ring slots
// follow the rule of that kernel: slot s holds psc0 times the adjoint of y1 before step s is undone, so this launch
// writes slot t-1 between its two steps and, with write_after, slot t-2 from what it leaves (for the pair of steps
// that follows); slot t was written by the launch before, or by bwd_seed_slot_kernel at the start of a call.
__global__ __launch_bounds__(kBlock) void bwd_state2_kernel(bmtk_glif3_bwd a, BwdStep q, int write_after)
{
    const int64_t ne = a.n_neurons * (int64_t)a.batch;
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= ne) return;
    const int64_t n = a.batch == 1 ? e : (int64_t)((uint32_t)e / (uint32_t)a.batch);
    const int64_t col = a.class_id ? (int64_t)a.class_id[n] : n;
    Glif3Prop p;
    p.load(a.prop, a.prop_stride, col);
    const int L = a.ring_slots;
    float lV = a.lam_V[e];
    float lA[GLIF3_NASC], l1[GLIF3_NREC], l2[GLIF3_NREC];
#pragma unroll
    for (int k = 0; k < GLIF3_NASC; ++k) lA[k] = a.lam_asc[k * ne + e];
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        l1[k] = a.lam_y1[k * ne + e];
        l2[k] = a.lam_y2[k * ne + e];
    }
    const uint8_t f_t = a.save_flags[q.row * ne + e], f_p = a.save_flags[(q.row - 1) * ne + e];
    const float sg_t = (f_t & BMTK_F_INTEGRATING) ? spike_adjoint(a, p, q.row, e, ne, 0, 8) : 0.0f;
    const float sg_p = (f_p & BMTK_F_INTEGRATING) ? spike_adjoint(a, p, q.row - 1, e, ne, 8, 8) : 0.0f;
    state_adjoint_step(lV, lA, l1, l2, p, a.h, f_t, sg_t);
    float *slot = a.lam_ring + (int64_t)((q.t - 1) % L) * GLIF3_NREC * ne + e;
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) slot[k * ne] = p.psc0[k] * l1[k];
    state_adjoint_step(lV, lA, l1, l2, p, a.h, f_p, sg_p);
    if (write_after) {
        slot = a.lam_ring + (int64_t)((q.t + L - 2) % L) * GLIF3_NREC * ne + e;
#pragma unroll
        for (int k = 0; k < GLIF3_NREC; ++k) slot[k * ne] = p.psc0[k] * l1[k];
    }
    a.lam_V[e] = lV;
#pragma unroll
    for (int k = 0; k < GLIF3_NASC; ++k) a.lam_asc[k * ne + e] = lA[k];
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k) {
        a.lam_y1[k * ne + e] = l1[k];
        a.lam_y2[k * ne + e] = l2[k];
    }
}

// ring slot `slot` = psc0 times the present adjoint of y1: what the state adjoint of the step the slot belongs to
// would write first, done ahead for the two-step form, whose transposed propagation reads it before that
__global__ __launch_bounds__(kBlock) void bwd_seed_slot_kernel(bmtk_glif3_bwd a, int slot)
{
    const int64_t ne = a.n_neurons * (int64_t)a.batch;
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= ne) return;
    const int64_t n = a.batch == 1 ? e : (int64_t)((uint32_t)e / (uint32_t)a.batch);
    const int64_t col = a.class_id ? (int64_t)a.class_id[n] : n;
#pragma unroll
    for (int k = 0; k < GLIF3_NREC; ++k)
        a.lam_ring[((int64_t)slot * GLIF3_NREC + k) * ne + e] =
            a.prop[(GLIF3_PSC0_0 + k) * a.prop_stride + col] * a.lam_y1[k * ne + e];
}

// d_rec_w[p] += sum over trials b in which source j spiked in step t of
// lam_ring[(t+d)%L][r][i*B+b]: one wavefront owns the whole row of a source, so
// the accumulation needs no atomics; lane = synapse.
__global__ __launch_bounds__(kBlock) void bwd_rec_grad_kernel(bmtk_glif3_bwd a, BwdStep q)
{
    const int batch = a.batch;
    const int64_t ne = a.n_neurons * (int64_t)batch;
    const int L = a.ring_slots;
    const int64_t j = (int64_t)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave;
    if (j >= a.n_neurons) return;
    const uint64_t *__restrict__ bits = a.spike_bits + q.row * a.spike_bits_stride;
    const int slot0 = (int)(q.t % L);
    const int p0 = a.rec_indptr[j], p1 = a.rec_indptr[j + 1];
    const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(a.rec_packed);
    for (int tile0 = 0; tile0 < batch; tile0 += kWave) {
        const unsigned long long m = trial_mask(bits, j, batch, tile0, min(kWave, batch - tile0));
        if (m == 0ull) continue;
        for (int p = p0 + lane_id(); p < p1; p += kWave) {
            const uint2 sy = rows[p];
            int slot = slot0 + (int)(sy.x >> 26);
            slot = slot >= L ? slot - L : slot;
            const int r = (sy.x >> 24) & 3;
            const int64_t i = sy.x & 0xFFFFFFu;
            const float *cell = a.lam_ring + (int64_t)(slot * GLIF3_NREC + r) * ne + i * batch + tile0;
            float acc = 0.0f;
            unsigned long long mm = m;
            while (mm) {
                const int b = __ffsll((long long)mm) - 1;
                mm &= mm - 1ull;
                acc += cell[b];
            }
            a.d_rec_w[p] += acc;
        }
    }
}

// Input weights.  The events of a step are ascending in source*batch+trial, so the trials in
// which one source fired are adjacent: the wavefront that holds the first event of such a run
// takes the whole run, which makes it the only writer of that source's row -- no atomics.
constexpr int kInpGradGrid = 1024;  // workgroups of the input-gradient part of a launch
// (a workgroup of any size: wavefront `wave` of `n_waves`)
__device__ __forceinline__ void bwd_inp_grad_waves(const bmtk_glif3_bwd &a, const BwdStep &q, int wave, int n_waves);
__device__ __forceinline__ void bwd_inp_grad_block(const bmtk_glif3_bwd &a, const BwdStep &q, int block, int n_blocks)
{
    bwd_inp_grad_waves(a, q, block * (kBlock / kWave) + threadIdx.x / kWave, n_blocks * (kBlock / kWave));
}
// source of an input event
__device__ __forceinline__ int event_source(int ev, int batch)
{
    return batch == 1 ? ev : (int)((uint32_t)ev / (uint32_t)batch);
}

// d_inp_w of source j's row += the adjoint cells of the trials of two runs of events: [k, k_end) of a step whose
// adjoint slots start at slot0, and [m, m_end) of the step before it (slots start one lower); either may be empty
__device__ __forceinline__ void inp_grad_row(const bmtk_glif3_bwd &a, int j, int slot0, int64_t k, int64_t k_end,
                                             int slot0_before, int64_t m, int64_t m_end)
{
    const int batch = a.batch;
    const int64_t ne = a.n_neurons * (int64_t)batch;
    const int L = a.ring_slots;
    const uint2 *__restrict__ rows = reinterpret_cast<const uint2 *>(a.inp_packed);
    const int p0 = a.inp_indptr[j], p1 = a.inp_indptr[j + 1];
    // four synapses per lane at a time: their records, then their adjoint cells, travel together
    constexpr int kUnroll = 4;
    for (int base = p0 + lane_id(); base < p1; base += kUnroll * kWave) {
        uint2 sy[kUnroll];
        float old[kUnroll], acc[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int p = base + u * kWave;
            if (p < p1) {
                sy[u] = rows[p];
                old[u] = a.d_inp_w[p];
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            acc[u] = 0.0f;
            if (base + u * kWave < p1) {
                const int d = (int)(sy[u].x >> 26), r = (sy[u].x >> 24) & 3;
                const int64_t i = sy[u].x & 0xFFFFFFu;
                int slot = slot0 + d;
                slot = slot >= L ? slot - L : slot;
                const float *cell = a.lam_ring + (int64_t)(slot * GLIF3_NREC + r) * ne + i * batch;
                for (int64_t kk = k; kk < k_end; ++kk) acc[u] += cell[a.in_events[kk] - j * batch];
                if (m < m_end) {
                    slot = slot0_before + d;
                    slot = slot >= L ? slot - L : slot;
                    cell = a.lam_ring + (int64_t)(slot * GLIF3_NREC + r) * ne + i * batch;
                    for (int64_t kk = m; kk < m_end; ++kk) acc[u] += cell[a.in_events[kk] - j * batch];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u)
            if (base + u * kWave < p1) a.d_inp_w[base + u * kWave] = old[u] + acc[u];
    }
}

__device__ __forceinline__ void bwd_inp_grad_waves(const bmtk_glif3_bwd &a, const BwdStep &q, int wave, int n_waves)
{
    const int batch = a.batch;
    const int slot0 = (int)(q.t % a.ring_slots);
    const int64_t k0 = a.in_ptr[q.t], k1 = a.in_ptr[q.t + 1];
    for (int64_t k = k0 + wave; k < k1; k += n_waves) {
        const int j = event_source(a.in_events[k], batch);
        if (k > k0 && event_source(a.in_events[k - 1], batch) == j) continue;  // not the first event of its source's run
        int64_t k_end = k + 1;
        while (k_end < k1 && event_source(a.in_events[k_end], batch) == j) ++k_end;
        inp_grad_row(a, j, slot0, k, k_end, 0, 0, 0);
    }
}

// first event of [lo, hi) (ascending in source*batch+trial) whose source is at least j; called by a whole wavefront
// with the same arguments in every lane: 64 probes a round instead of one, two rounds for a step's few thousand
// events where a binary search is a chain of twelve dependent loads
__device__ __forceinline__ int64_t first_event_of(const int32_t *__restrict__ events, int64_t lo, int64_t hi, int j, int batch)
{
    const int lane = lane_id();
    while (hi - lo > kWave) {
        const int64_t stride = (hi - lo + kWave - 1) / kWave;
        const int64_t at = lo + lane * stride;
        const bool below = at < hi && event_source(events[at], batch) < j;  // ascending: the lanes below j are a prefix
        const int c = __popcll(__ballot(below));
        if (c == 0) return lo;
        const int64_t upto = lo + c * stride;
        lo = lo + (c - 1) * stride + 1;
        hi = upto < hi ? upto : hi;
    }
    const int64_t at = lo + lane;
    const unsigned long long at_least = __ballot(at < hi && event_source(events[at], batch) >= j);
    return at_least ? lo + (__ffsll((long long)at_least) - 1) : hi;
}

// The same for steps t = q.t and t-1 in ONE launch.  Two wavefronts must never update one source's row at a time, so
// a source with events in both steps belongs to the wavefront that holds the first event of its run in step t,
// which looks its run of step t-1 up (the events of a step are sorted) and adds both with one read-modify-write;
// runs of step t-1 whose source has no event in step t are taken by the holder of their first event.
__device__ __forceinline__ void bwd_inp_grad2_waves(const bmtk_glif3_bwd &a, const BwdStep &q, int wave, int n_waves)
{
    const int batch = a.batch;
    const int L = a.ring_slots;
    const int slot_t = (int)(q.t % L), slot_p = (int)((q.t - 1) % L);
    const int64_t k0 = a.in_ptr[q.t], k1 = a.in_ptr[q.t + 1];
    const int64_t m0 = a.in_ptr[q.t - 1], m1 = k0;  // (in_ptr[t-1] .. in_ptr[t]: the events of step t-1)
    for (int64_t k = k0 + wave; k < k1; k += n_waves) {
        const int j = event_source(a.in_events[k], batch);
        if (k > k0 && event_source(a.in_events[k - 1], batch) == j) continue;
        int64_t k_end = k + 1;
        while (k_end < k1 && event_source(a.in_events[k_end], batch) == j) ++k_end;
        const int64_t m = first_event_of(a.in_events, m0, m1, j, batch);
        int64_t m_end = m;
        while (m_end < m1 && event_source(a.in_events[m_end], batch) == j) ++m_end;
        inp_grad_row(a, j, slot_t, k, k_end, slot_p, m, m_end);
    }
    for (int64_t m = m0 + wave; m < m1; m += n_waves) {
        const int j = event_source(a.in_events[m], batch);
        if (m > m0 && event_source(a.in_events[m - 1], batch) == j) continue;
        const int64_t k = first_event_of(a.in_events, k0, k1, j, batch);
        if (k < k1 && event_source(a.in_events[k], batch) == j) continue;  // the source's run of step t takes it along
        int64_t m_end = m + 1;
        while (m_end < m1 && event_source(a.in_events[m_end], batch) == j) ++m_end;
        inp_grad_row(a, j, slot_p, m, m_end, 0, 0, 0);
    }
}

// The state adjoint of step t and the input-weight gradient of the same step in one launch, side by side: the
// gradient reads the adjoint slots t+1 .. t+L-1 and the step's events, the state adjoint writes slot t -- neither
// needs the other.  The gradient's workgroups (a chain of dependent reads per event run, few wavefronts) take the
// lowest block ids so that they start first and run under the streaming state adjoint instead of after it.
__global__ __launch_bounds__(kBlock) void bwd_state_kernel(bmtk_glif3_bwd a, BwdStep q, int n_inp_blocks)
{
    if ((int)blockIdx.x < n_inp_blocks)
        bwd_inp_grad_block(a, q, (int)blockIdx.x, n_inp_blocks);
    else
        bwd_state_block(a, q, (int64_t)blockIdx.x - n_inp_blocks);
}

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(float *x, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) x[i] = 0.0f;
}

__global__ __launch_bounds__(kBlock) void spike_counts_kernel(const uint64_t *__restrict__ bits, int64_t stride,
                                                              int64_t n_steps, int64_t ne,
                                                              int32_t *__restrict__ counts)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (e >= ne) return;
    const int64_t w = e >> 6;
    const int sh = (int)(e & 63);
    int c = 0;
    for (int64_t k = 0; k < n_steps; ++k) c += (int)((bits[k * stride + w] >> sh) & 1ull);
    counts[e] = c;
}

}  // namespace bmtk

using namespace bmtk;

namespace {

const void *blocked_variant(bool grad, bool ne24, bool wide)
{
#define BMTK_BLK(g, n, w) reinterpret_cast<const void *>(bwd_gather_blocked_kernel<g, n, w>)
    if (grad) {
        if (ne24) return wide ? BMTK_BLK(true, true, true) : BMTK_BLK(true, true, false);
        return wide ? BMTK_BLK(true, false, true) : BMTK_BLK(true, false, false);
    }
    if (ne24) return wide ? BMTK_BLK(false, true, true) : BMTK_BLK(false, true, false);
    return wide ? BMTK_BLK(false, false, true) : BMTK_BLK(false, false, false);
#undef BMTK_BLK
}

// launch geometry of bwd_gather_blocked_kernel for a network on the current device
struct BlockedPlan {
    unsigned grid;
    int lp, rows_cu, sweeps, gpw, use_order;
    size_t lds;
    // the two-step kernel: twice the LDS per row, hence half as many row groups per wavefront and sweep
    int sweeps2, gpw2, use_order2;
    size_t lds2;
};
constexpr size_t kBlkLdsMax = 160u * 1024u - 256u;  // a compute unit's LDS less the kernel's static part

int blocked_plan(const bmtk_glif3_bwd &a, BlockedPlan &pl)
{
    int dev = 0;
    (void)hipGetDevice(&dev);
    static int cu_count[64];
    int n_cu = (dev >= 0 && dev < 64) ? cu_count[dev] : 0;
    if (n_cu <= 0) {
        n_cu = 256;
        (void)hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev);
        if (dev >= 0 && dev < 64) cu_count[dev] = n_cu;
    }
    const int cus = n_cu >= 8 ? n_cu / 8 : 1;  // workgroups per XCD, one per compute unit
    int bp = 4;
    while (bp < a.batch) bp <<= 1;
    pl.lp = bp / 4;
    const int per = kWave / pl.lp;
    int64_t rows_cu = (a.n_neurons + cus - 1) / cus;
    rows_cu = (rows_cu + per - 1) / per * per;
    const int64_t cap = (int64_t)kBlkWaves * kBlkMaxGroups * per;  // rows of one sweep
    pl.sweeps = (int)((rows_cu + cap - 1) / cap);
    pl.gpw = (int)((rows_cu + (int64_t)pl.sweeps * kBlkWaves * per - 1) / ((int64_t)pl.sweeps * kBlkWaves * per));
    pl.rows_cu = (int)rows_cu;
    pl.grid = (unsigned)cus * 8u;
    pl.lds = (size_t)kBlkWaves * pl.gpw * kWave * sizeof(float4);
    // the row order list (gradient riding along): two bytes per place, where it fits (up to 16 rows per thread)
    const size_t order_bytes = (size_t)pl.sweeps * kBlkWaves * pl.gpw * per * sizeof(uint16_t);
    pl.use_order = (pl.lds + order_bytes <= kBlkLdsMax && rows_cu <= 16 * kBlkThreads && rows_cu < 0xFFFF) ? 1 : 0;
    if (pl.use_order) pl.lds += order_bytes;
    const int64_t cap2 = (int64_t)kBlkWaves * (kBlkMaxGroups / 2) * per;
    pl.sweeps2 = (int)((rows_cu + cap2 - 1) / cap2);
    pl.gpw2 = (int)((rows_cu + (int64_t)pl.sweeps2 * kBlkWaves * per - 1) / ((int64_t)pl.sweeps2 * kBlkWaves * per));
    pl.lds2 = (size_t)kBlkWaves * pl.gpw2 * 2 * kWave * sizeof(float4);
    const size_t order_bytes2 = (size_t)pl.sweeps2 * kBlkWaves * pl.gpw2 * per * sizeof(uint16_t);
    pl.use_order2 = (pl.lds2 + order_bytes2 <= kBlkLdsMax && rows_cu <= 16 * kBlkThreads && rows_cu < 0xFFFF) ? 1 : 0;
    if (pl.use_order2) pl.lds2 += order_bytes2;
    static bool asked[8][64];
    const void *variants[8];
    for (int g = 0; g < 8; ++g) variants[g] = blocked_variant(g & 4, g & 2, g & 1);
    for (int g = 0; g < 8; ++g) {
        if (dev < 0 || dev >= 64 || asked[g][dev]) continue;
        const hipError_t err = hipFuncSetAttribute(
            variants[g], hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBlkLdsMax);
        if (err != hipSuccess) {
            set_error("transposed propagation: cannot reserve LDS: %s", hipGetErrorString(err));
            return BMTK_E_LAUNCH;
        }
        asked[g][dev] = true;
    }
    static bool asked2[64];
    if (dev >= 0 && dev < 64 && !asked2[dev]) {
        const void *pair[4] = {reinterpret_cast<const void *>(bwd_gather_blocked2_kernel<true, true>),
                               reinterpret_cast<const void *>(bwd_gather_blocked2_kernel<true, false>),
                               reinterpret_cast<const void *>(bwd_gather_blocked2_kernel<false, true>),
                               reinterpret_cast<const void *>(bwd_gather_blocked2_kernel<false, false>)};
        for (int g = 0; g < 4; ++g) {
            const hipError_t err = hipFuncSetAttribute(pair[g], hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBlkLdsMax);
            if (err != hipSuccess) {
                set_error("transposed propagation: cannot reserve LDS: %s", hipGetErrorString(err));
                return BMTK_E_LAUNCH;
            }
        }
        asked2[dev] = true;
    }
    return BMTK_OK;
}

// what the blocked form of the table must satisfy
int blocked_check(const bmtk_glif3_bwd &a, const char *who)
{
    BMTK_REQUIRE(a.blk_count > 0 && a.blk_count % 8 == 0 && a.blk_indptr && a.blk_packed,
                 "%s: the blocked table needs blk_count (a multiple of 8), blk_indptr and blk_packed", who);
    BMTK_REQUIRE(a.batch % 4 == 0 && a.batch <= kWave, "%s: the blocked table serves batches that are a multiple of 4 up to 64",
                 who);
    BMTK_REQUIRE((int64_t)a.ring_slots * GLIF3_NREC * a.n_neurons * a.batch < (1ll << 30),
                 "%s: the adjoint ring must stay below 4 GB for the blocked table", who);
    return BMTK_OK;
}

int blocked_launch(const bmtk_glif3_bwd &a, const BwdStep &q, const BlockedPlan &pl, bool grad, bool inp_grad,
                   hipStream_t st)
{
    const bool ne24 = a.n_neurons * (int64_t)a.batch < (1ll << 24);
    bmtk_glif3_bwd args = a;
    BwdStep step = q;
    int lp = pl.lp, rows_cu = pl.rows_cu, sweeps = pl.sweeps, gpw = pl.gpw, use_order = pl.use_order;
    int do_inp = inp_grad ? 1 : 0;
    void *params[] = {&args, &step, &lp, &rows_cu, &sweeps, &gpw, &use_order, &do_inp};
    const hipError_t err = hipLaunchKernel(blocked_variant(grad, ne24, pl.lp >= 8), dim3(pl.grid), dim3(kBlkThreads),
                                           params, pl.lds, st);
    if (err != hipSuccess) {
        set_error("transposed propagation: launch failed: %s", hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    return BMTK_OK;
}

// the two-step kernel for steps q.t and q.t - 1
int blocked2_launch(const bmtk_glif3_bwd &a, const BwdStep &q, const BlockedPlan &pl, bool grad, bool inp_grad, hipStream_t st)
{
    const bool ne24 = a.n_neurons * (int64_t)a.batch < (1ll << 24);
    bmtk_glif3_bwd args = a;
    BwdStep step = q;
    int lp = pl.lp, rows_cu = pl.rows_cu, sweeps = pl.sweeps2, gpw = pl.gpw2, use_order = pl.use_order2;
    int do_inp = inp_grad ? 1 : 0;
    void *params[] = {&args, &step, &lp, &rows_cu, &sweeps, &gpw, &use_order, &do_inp};
    const void *fn = grad ? (ne24 ? reinterpret_cast<const void *>(bwd_gather_blocked2_kernel<true, true>)
                                  : reinterpret_cast<const void *>(bwd_gather_blocked2_kernel<true, false>))
                          : (ne24 ? reinterpret_cast<const void *>(bwd_gather_blocked2_kernel<false, true>)
                                  : reinterpret_cast<const void *>(bwd_gather_blocked2_kernel<false, false>));
    const hipError_t err = hipLaunchKernel(fn, dim3(pl.grid), dim3(kBlkThreads), params, pl.lds2, st);
    if (err != hipSuccess) {
        set_error("transposed propagation (two steps): launch failed: %s", hipGetErrorString(err));
        return BMTK_E_LAUNCH;
    }
    return BMTK_OK;
}

}  // namespace

namespace {

// what every entry point that takes the whole bmtk_glif3_bwd requires of it
int bwd_check(const bmtk_glif3_bwd *bwd, const char *who)
{
    BMTK_REQUIRE(bwd != nullptr, "%s: bwd is null", who);
    const bmtk_glif3_bwd &a = *bwd;
    BMTK_REQUIRE(a.n_neurons > 0 && a.batch > 0, "%s: n_neurons and batch must be positive", who);
    const int64_t ne = a.n_neurons * (int64_t)a.batch;
    BMTK_REQUIRE(ne < (1ll << 31) && a.n_neurons < (1ll << 24), "%s: network too large", who);
    BMTK_REQUIRE(a.ring_slots > 1 && a.ring_slots <= 64, "%s: ring_slots must lie in 2..64", who);
    BMTK_REQUIRE(a.h > 0.0f && a.dampening >= 0.0f, "%s: h must be positive, dampening non-negative", who);
    BMTK_REQUIRE(a.prop && a.prop_stride > 0 && (a.class_id || a.prop_stride >= a.n_neurons),
                 "%s: prop table missing or too small", who);
    BMTK_REQUIRE(a.save_v && a.save_flags && a.spike_bits, "%s: the forward record is incomplete", who);
    BMTK_REQUIRE(a.spike_bits_stride >= (ne + 63) / 64, "%s: spike_bits_stride too small", who);
    BMTK_REQUIRE(a.lam_V && a.lam_asc && a.lam_y1 && a.lam_y2 && a.lam_ring && a.gz,
                 "%s: adjoint state pointers must be non-null", who);
    BMTK_REQUIRE(!(a.dl_dz && a.dl_dz_const), "%s: give dl_dz or dl_dz_const, not both", who);
    const bool has_rec = a.rec_indptr != nullptr;
    BMTK_REQUIRE(!has_rec || a.rec_packed, "%s: recurrent table needs rec_packed", who);
    BMTK_REQUIRE(!a.d_rec_w || has_rec, "%s: d_rec_w without a recurrent table", who);
    BMTK_REQUIRE(!a.d_blk_w || a.blk_count != 0, "%s: d_blk_w without the blocked table", who);
    BMTK_REQUIRE(!a.d_inp_w || (a.in_ptr && a.in_events && a.inp_indptr && a.inp_packed),
                 "%s: d_inp_w needs the input events and the input table", who);
    return BMTK_OK;
}

}  // namespace

extern "C" int bmtk_glif3_simulate_bwd(const bmtk_glif3_bwd *bwd, int64_t step0, int64_t n_steps, void *stream)
{
    {
        const int rc = bwd_check(bwd, "glif3_simulate_bwd");
        if (rc != BMTK_OK) return rc;
    }
    const bmtk_glif3_bwd &a = *bwd;
    const int64_t ne = a.n_neurons * (int64_t)a.batch;
    const bool blocked = a.blk_count != 0;
    BlockedPlan pl{};
    if (blocked) {
        int rc = blocked_check(a, "glif3_simulate_bwd");
        if (rc == BMTK_OK) rc = blocked_plan(a, pl);
        if (rc != BMTK_OK) return rc;
    }
    const bool has_rec = a.rec_indptr != nullptr;
    const bool inp_grad = a.d_inp_w != nullptr;
    BMTK_REQUIRE(step0 >= 0 && n_steps >= 0, "glif3_simulate_bwd: step0 and n_steps must be non-negative");
    hipStream_t st = (hipStream_t)stream;
    const unsigned rows_grid = (unsigned)((a.n_neurons + kBlock / kWave - 1) / (kBlock / kWave));
    const unsigned tiles = (unsigned)((a.batch + kWave - 1) / kWave);
    const unsigned elem_grid = (unsigned)((ne + kBlock - 1) / kBlock);
    int bp = 1;  // trial-tile width: the batch rounded up to a power of two, at most one wavefront
    while (bp < a.batch && bp < kWave) bp <<= 1;
    int64_t k_top = n_steps - 1;
    // Two steps per pass over the blocked table where gz has room for both steps' partial sums and a lane holds
    // whole adjoint rows of eight lanes (batches above 16): pairs (k, k-1) from the top, a step left over at the
    // end goes the one-step way.
    if (blocked && a.gz_planes >= 16 && pl.lp >= 8 && n_steps >= 2) {
        hipLaunchKernelGGL(bwd_seed_slot_kernel, dim3(elem_grid), dim3(kBlock), 0, st, a, (int)((step0 + k_top) % a.ring_slots));
        for (; k_top >= 1; k_top -= 2) {
            BwdStep q{step0 + k_top, k_top, 8};
            const int rc = blocked2_launch(a, q, pl, a.d_blk_w != nullptr, inp_grad, st);
            if (rc != BMTK_OK) return rc;
            if (a.d_rec_w && !a.d_blk_w) {  // (before the state adjoint, which overwrites a slot step t-1's gradient reads)
                const BwdStep before{q.t - 1, q.row - 1, 8};
                hipLaunchKernelGGL(bwd_rec_grad_kernel, dim3(rows_grid), dim3(kBlock), 0, st, a, q);
                hipLaunchKernelGGL(bwd_rec_grad_kernel, dim3(rows_grid), dim3(kBlock), 0, st, a, before);
            }
            hipLaunchKernelGGL(bwd_state2_kernel, dim3(elem_grid), dim3(kBlock), 0, st, a, q, k_top - 1 > 0 ? 1 : 0);
        }
    }
    for (int64_t k = k_top; k >= 0; --k) {
        BwdStep q{step0 + k, k, blocked ? 8 : 1};
        // The recurrent weight gradient of step t reads the adjoint slots t+1 .. t+L-1, which the state adjoint of
        // this step (it writes slot t) leaves alone: it can ride along with the transposed propagation, which
        // reads the same slots before the state adjoint runs.  Batches of more than one tile keep the kernel of
        // their own (several wavefronts would share a row).
        const bool fused = blocked ? a.d_blk_w != nullptr : (a.d_rec_w && tiles == 1);
        if (blocked) {
            const int rc = blocked_launch(a, q, pl, fused, inp_grad, st);
            if (rc != BMTK_OK) return rc;
        } else if (has_rec && a.batch % 4 == 0 && a.batch <= kWave) {
            if (fused)
                hipLaunchKernelGGL(bwd_gather4_kernel<true>, dim3(rows_grid), dim3(kBlock), 0, st, a, q, bp / 4);
            else
                hipLaunchKernelGGL(bwd_gather4_kernel<false>, dim3(rows_grid), dim3(kBlock), 0, st, a, q, bp / 4);
        } else if (has_rec) {
            if (fused)
                hipLaunchKernelGGL(bwd_gather_kernel<true>, dim3(rows_grid, tiles), dim3(kBlock), 0, st, a, q, bp);
            else
                hipLaunchKernelGGL(bwd_gather_kernel<false>, dim3(rows_grid, tiles), dim3(kBlock), 0, st, a, q, bp);
        } else {
            hipLaunchKernelGGL(fill_zero_kernel, dim3(elem_grid), dim3(kBlock), 0, st, a.gz, ne);
        }
        const int n_inp_blocks = (inp_grad && !blocked) ? kInpGradGrid : 0;  // (the blocked kernel took it along)
        hipLaunchKernelGGL(bwd_state_kernel, dim3(elem_grid + n_inp_blocks), dim3(kBlock), 0, st, a, q, n_inp_blocks);
        if (a.d_rec_w && !fused) hipLaunchKernelGGL(bwd_rec_grad_kernel, dim3(rows_grid), dim3(kBlock), 0, st, a, q);
    }
    BMTK_CHECK_LAUNCH("glif3_simulate_bwd");
    return BMTK_OK;
}

extern "C" int bmtk_glif3_step_bwd(const bmtk_glif3_bwd *bwd, int64_t step0, int64_t k, int32_t gz_parts, void *stream)
{
    const int rc = bwd_check(bwd, "glif3_step_bwd");
    if (rc != BMTK_OK) return rc;
    BMTK_REQUIRE(step0 >= 0 && k >= 0, "glif3_step_bwd: step0 and k must be non-negative");
    BMTK_REQUIRE(gz_parts == 1 || gz_parts == 8, "glif3_step_bwd: gz holds 1 sum or 8 partial sums per element");
    const bmtk_glif3_bwd &a = *bwd;
    const int64_t ne = a.n_neurons * (int64_t)a.batch;
    BwdStep q{step0 + k, k, gz_parts};
    hipLaunchKernelGGL(bwd_state_kernel, dim3((unsigned)((ne + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, a, q, 0);
    BMTK_CHECK_LAUNCH("glif3_step_bwd");
    return BMTK_OK;
}

extern "C" int bmtk_csr_weight_grad(const bmtk_glif3_bwd *bwd, int64_t step0, int64_t k, void *stream)
{
    const int rc = bwd_check(bwd, "csr_weight_grad");
    if (rc != BMTK_OK) return rc;
    BMTK_REQUIRE(step0 >= 0 && k >= 0, "csr_weight_grad: step0 and k must be non-negative");
    const bmtk_glif3_bwd &a = *bwd;
    BMTK_REQUIRE(a.d_rec_w || a.d_inp_w, "csr_weight_grad: neither d_rec_w nor d_inp_w is given");
    BwdStep q{step0 + k, k, 1};
    if (a.d_rec_w)
        hipLaunchKernelGGL(bwd_rec_grad_kernel, dim3((unsigned)((a.n_neurons + kBlock / kWave - 1) / (kBlock / kWave))),
                           dim3(kBlock), 0, (hipStream_t)stream, a, q);
    if (a.d_inp_w)  // (bwd_state_kernel with nothing but gradient workgroups)
        hipLaunchKernelGGL(bwd_state_kernel, dim3(kInpGradGrid), dim3(kBlock), 0, (hipStream_t)stream, a, q, kInpGradGrid);
    BMTK_CHECK_LAUNCH("csr_weight_grad");
    return BMTK_OK;
}

extern "C" int bmtk_csr_propagate_bwd(const int32_t *indptr, const bmtk_synapse *packed, int64_t n_neurons,
                                      int32_t batch, const float *lam_ring, int32_t L, int64_t step, float *gz,
                                      int32_t trials_per_lane, void *stream)
{
    BMTK_REQUIRE(indptr && packed && lam_ring && gz, "csr_propagate_bwd: pointers must be non-null");
    BMTK_REQUIRE(n_neurons > 0 && batch > 0 && step >= 0, "csr_propagate_bwd: bad sizes or step");
    BMTK_REQUIRE(n_neurons * (int64_t)batch < (1ll << 31) && n_neurons < (1ll << 24), "csr_propagate_bwd: network too large");
    BMTK_REQUIRE(L > 1 && L <= 64, "csr_propagate_bwd: L must lie in 2..64");
    const bool can4 = batch % 4 == 0 && batch <= kWave;
    BMTK_REQUIRE(trials_per_lane == 0 || trials_per_lane == 1 || (trials_per_lane == 4 && can4),
                 "csr_propagate_bwd: trials_per_lane must be 0 (choose), 1, or 4 for batches that are a multiple of 4 up to 64");
    bmtk_glif3_bwd a{};
    a.n_neurons = n_neurons;
    a.batch = batch;
    a.ring_slots = L;
    a.rec_indptr = indptr;
    a.rec_packed = packed;
    a.lam_ring = const_cast<float *>(lam_ring);
    a.gz = gz;
    BwdStep q{step, 0, 1};
    const unsigned rows_grid = (unsigned)((n_neurons + kBlock / kWave - 1) / (kBlock / kWave));
    int bp = 1;
    while (bp < batch && bp < kWave) bp <<= 1;
    if (trials_per_lane == 4 || (trials_per_lane == 0 && can4))
        hipLaunchKernelGGL(bwd_gather4_kernel<false>, dim3(rows_grid), dim3(kBlock), 0, (hipStream_t)stream, a, q, bp / 4);
    else
        hipLaunchKernelGGL(bwd_gather_kernel<false>, dim3(rows_grid, (unsigned)((batch + kWave - 1) / kWave)), dim3(kBlock), 0,
                           (hipStream_t)stream, a, q, bp);
    BMTK_CHECK_LAUNCH("csr_propagate_bwd");
    return BMTK_OK;
}

extern "C" int bmtk_csr_propagate_bwd_blocked(const int32_t *blk_indptr, const bmtk_synapse *blk_packed, int32_t blk_count,
                                              int64_t n_neurons, int32_t batch, const float *lam_ring, int32_t L,
                                              int64_t step, float *gz_parts, void *stream)
{
    BMTK_REQUIRE(lam_ring && gz_parts, "csr_propagate_bwd_blocked: pointers must be non-null");
    BMTK_REQUIRE(n_neurons > 0 && batch > 0 && step >= 0, "csr_propagate_bwd_blocked: bad sizes or step");
    BMTK_REQUIRE(n_neurons * (int64_t)batch < (1ll << 31) && n_neurons < (1ll << 24),
                 "csr_propagate_bwd_blocked: network too large");
    BMTK_REQUIRE(L > 1 && L <= 64, "csr_propagate_bwd_blocked: L must lie in 2..64");
    bmtk_glif3_bwd a{};
    a.n_neurons = n_neurons;
    a.batch = batch;
    a.ring_slots = L;
    a.blk_count = blk_count;
    a.blk_indptr = blk_indptr;
    a.blk_packed = blk_packed;
    a.lam_ring = const_cast<float *>(lam_ring);
    a.gz = gz_parts;
    BlockedPlan pl{};
    int rc = blocked_check(a, "csr_propagate_bwd_blocked");
    if (rc == BMTK_OK) rc = blocked_plan(a, pl);
    if (rc != BMTK_OK) return rc;
    BwdStep q{step, 0, 8};
    rc = blocked_launch(a, q, pl, false, false, (hipStream_t)stream);
    if (rc != BMTK_OK) return rc;
    BMTK_CHECK_LAUNCH("csr_propagate_bwd_blocked");
    return BMTK_OK;
}

extern "C" int bmtk_csr_propagate_bwd_blocked_plan(int64_t n_neurons, int32_t batch, int32_t *plan_host)
{
    BMTK_REQUIRE(plan_host != nullptr, "csr_propagate_bwd_blocked_plan: plan_host is null");
    BMTK_REQUIRE(n_neurons > 0 && n_neurons < (1ll << 24) && batch > 0 && batch % 4 == 0 && batch <= kWave,
                 "csr_propagate_bwd_blocked_plan: n_neurons must lie in 1..2^24-1, batch be a multiple of 4 up to 64");
    bmtk_glif3_bwd a{};
    a.n_neurons = n_neurons;
    a.batch = batch;
    BlockedPlan pl{};
    const int rc = blocked_plan(a, pl);
    if (rc != BMTK_OK) return rc;
    plan_host[0] = (int32_t)pl.grid;
    plan_host[1] = pl.rows_cu;
    plan_host[2] = pl.sweeps;
    plan_host[3] = pl.gpw;
    return BMTK_OK;
}

extern "C" int bmtk_spike_counts(const uint64_t *spike_bits, int64_t stride, int64_t n_steps, int64_t ne,
                                 int32_t *counts, void *stream)
{
    BMTK_REQUIRE(spike_bits && counts && ne > 0 && n_steps >= 0 && stride >= (ne + 63) / 64,
                 "spike_counts: bad sizes or null pointers");
    hipLaunchKernelGGL(spike_counts_kernel, dim3((unsigned)((ne + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       (hipStream_t)stream, spike_bits, stride, n_steps, ne, counts);
    BMTK_CHECK_LAUNCH("spike_counts");
    return BMTK_OK;
}
