// HIP kernels and C entry points of the per-step operations: propagator
// precompute, fused GLIF3 state update, spike compaction, event-driven scatter
// and row-wise gather into the delay ring buffer.  gfx950 only.
#include <math.h>
#include <stdarg.h>

#include <mutex>

#include "common.hpp"
#include "glif3_update.hpp"
#include "propagate.hpp"

namespace bmtk {

static thread_local char g_error[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

// ---------------------------------------------------------------------------
// Propagators (NEST glif_psc::pre_run_hook + libnestutil/propagator_stability)
// ---------------------------------------------------------------------------

__device__ double propagator_32(double tau_syn, double tau, double C, double h)
{
    const double lin = 1.0 / (2.0 * C * tau * tau) * h * h * (tau_syn - tau) * exp(-h / tau);
    const double sing = h / C * exp(-h / tau);
    const double P32 = -tau / (C * (1.0 - tau / tau_syn)) * exp(-h / tau_syn) * expm1(h * (1.0 / tau_syn - 1.0 / tau));
    const double dev = fabs(P32 - sing);
    if (tau == tau_syn || (fabs(tau - tau_syn) < 0.1 && dev > 2.0 * fabs(lin))) return sing;
    return P32;
}

__device__ double propagator_31(double tau_syn, double tau, double C, double h)
{
    const double lin = 1.0 / (3.0 * C * tau * tau) * h * h * h * (tau_syn - tau) * exp(-h / tau);
    const double P31 = 1.0 / C *
                       (exp(-h / tau_syn) * expm1(-h / tau + h / tau_syn) / (tau / tau_syn - 1.0) * tau -
                        h * exp(-h / tau_syn)) /
                       (-1.0 - -tau / tau_syn) * tau;
    const double sing = h * h / 2.0 / C * exp(-h / tau);
    const double dev = fabs(P31 - sing);
    if (tau == tau_syn || (fabs(tau - tau_syn) < 0.1 && dev > 2.0 * fabs(lin))) return sing;
    return P31;
}

__global__ __launch_bounds__(kBlock) void precompute_kernel(int64_t n, const double *__restrict__ par, double h,
                                                            float *__restrict__ prop)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
#define PA(k) par[(int64_t)(k) * n + i]
#define PO(k) prop[(int64_t)(k) * n + i]
    const double C = PA(GLIF3_PAR_C_M), g = PA(GLIF3_PAR_G);
    const double tau = C / g;
    const double P33 = exp(-h / tau);
    PO(GLIF3_P33) = (float)P33;
    PO(GLIF3_P30) = (float)(1.0 / C * (1.0 - P33) * tau);
    PO(GLIF3_TH) = (float)(PA(GLIF3_PAR_V_TH) - PA(GLIF3_PAR_E_L));
    PO(GLIF3_UR) = (float)(PA(GLIF3_PAR_V_RESET) - PA(GLIF3_PAR_E_L));
    // NEST counts the refractory period down in floating point, one resolution per step
    const double t_ref = PA(GLIF3_PAR_T_REF);
    double rem = t_ref;
    int nref = 0;
    while (rem > 0.0 && nref < (1 << 24)) {
        rem -= h;
        ++nref;
    }
    PO(GLIF3_NREF) = (float)nref;
    for (int a = 0; a < GLIF3_NASC; ++a) {
        const double k = PA(GLIF3_PAR_ASC_DECAY0 + a);
        const double d = exp(-k * h);
        PO(GLIF3_D0 + a) = (float)d;
        PO(GLIF3_C0 + a) = (float)(((1.0 / k) / h) * (1.0 - d));
        PO(GLIF3_R0 + a) = (float)(PA(GLIF3_PAR_ASC_R0 + a) * exp(-k * t_ref));
        PO(GLIF3_AMP0 + a) = (float)PA(GLIF3_PAR_ASC_AMPS0 + a);
    }
    for (int r = 0; r < GLIF3_NREC; ++r) {
        const double ts = PA(GLIF3_PAR_TAU_SYN0 + r);
        PO(GLIF3_P11_0 + r) = (float)exp(-h / ts);
        PO(GLIF3_P31_0 + r) = (float)propagator_31(ts, tau, C, h);
        PO(GLIF3_P32_0 + r) = (float)propagator_32(ts, tau, C, h);
        PO(GLIF3_PSC0_0 + r) = (float)(2.718281828459045235360287 / ts);
    }
#undef PA
#undef PO
}

// ---------------------------------------------------------------------------
// Fused state update: one thread per element, every array access is a
// contiguous 256-byte row per wavefront.
// ---------------------------------------------------------------------------

struct StepArgs {
    int64_t ne;
    int32_t batch;
    float *V, *asc, *y1, *y2;
    int32_t *ref;
    const float *prop;
    int64_t stride;
    const int32_t *class_id;
    float h;
    float *syn;
    int32_t clear_syn;
    const float *i_ext;
    uint8_t *z;
    uint64_t *zbits;
    float *frac;
};

// kLdsTable: the propagators come from a class table small enough for LDS; the workgroup copies it there once
// and every thread reads its class's 29 values from there.  Read from device memory instead, those 29 scattered
// loads per thread, not the state traffic, set the pace (4.3 TB/s of algorithmic traffic against 6.1 with one
// parameter column per neuron).  At N = 2^20 with 111 classes, on two machines: 18.3 / 18.5 us with four tiles
// per workgroup, 18.1 / 19.5 with two, 24.4 with one; transposing the table on its way into LDS (an integer
// division per word, one word per load) took 19.8 / 20.2 with four tiles.  By measured bytes the launch then moves
// 5.95 TB/s where the form with a column per neuron moved 6.15 TB/s on the same machine.
constexpr int kStepTiles = 4;

template <bool kLdsTable>
__global__ __launch_bounds__(kBlock) void glif3_step_kernel(StepArgs a)
{
    extern __shared__ __align__(16) float step_table[];  // [GLIF3_NPROP][columns] when kLdsTable
    // with the table in LDS a workgroup takes kStepTiles tiles of 256 elements, so that staging the table is
    // shared by several tiles.  The state of all tiles is asked for first, before the table is staged: the loads
    // of the tiles travel together, and the staging runs while they are on their way.
    constexpr int kTiles = kLdsTable ? kStepTiles : 1;
    Glif3Elem s[kTiles];
    float syn[kTiles][GLIF3_NREC], I[kTiles];
    int64_t e[kTiles], col[kTiles];
#pragma unroll
    for (int t = 0; t < kTiles; ++t) {
        e[t] = ((int64_t)blockIdx.x * kTiles + t) * kBlock + threadIdx.x;
        col[t] = 0;
        I[t] = 0.0f;
        if (e[t] < a.ne) {
            const int64_t n = (a.batch == 1) ? e[t] : (int64_t)((uint32_t)e[t] / (uint32_t)a.batch);
            col[t] = a.class_id ? (int64_t)a.class_id[n] : n;
            glif3_load(s[t], a.V, a.asc, a.y1, a.y2, a.ref, a.ne, e[t]);
#pragma unroll
            for (int k = 0; k < GLIF3_NREC; ++k) syn[t][k] = a.syn ? a.syn[k * a.ne + e[t]] : 0.0f;
            I[t] = a.i_ext ? a.i_ext[e[t]] : 0.0f;
        }
    }
    if (kLdsTable) {
        stage_class_table<kBlock>(step_table, a.prop, (int)a.stride * GLIF3_NPROP);
        __syncthreads();
    }
#pragma unroll
    for (int t = 0; t < kTiles; ++t) {
        bool spike = false;
        if (e[t] < a.ne) {
            Glif3Prop p;
            if (kLdsTable)
                p.load(step_table, a.stride, col[t]);
            else
                p.load(a.prop, a.stride, col[t]);
            float frac = 0.0f;
            spike = glif3_update(s[t], p, a.h, syn[t], I[t], &frac);
            glif3_store(s[t], a.V, a.asc, a.y1, a.y2, a.ref, a.ne, e[t]);
            if (a.syn && a.clear_syn) {
#pragma unroll
                for (int k = 0; k < GLIF3_NREC; ++k) a.syn[k * a.ne + e[t]] = 0.0f;
            }
            if (a.z) a.z[e[t]] = spike ? 1 : 0;
            if (a.frac && spike) a.frac[e[t]] = frac;
        }
        if (a.zbits) {
            const unsigned long long m = __ballot(spike);
            if (lane_id() == 0 && (e[t] & ~(int64_t)(kWave - 1)) < a.ne) a.zbits[e[t] >> 6] = m;
        }
    }
}

// ---------------------------------------------------------------------------
// Compaction: flags -> bits -> per-block popcounts -> scan -> ordered ids
// ---------------------------------------------------------------------------

constexpr int kWordsPerBlock = kBlock;  // one 64-element word per thread

__global__ __launch_bounds__(kBlock) void pack_bits_kernel(const uint8_t *__restrict__ z, int64_t n,
                                                           uint64_t *__restrict__ bits)
{
    const int64_t e = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    const bool on = e < n && z[e] != 0;
    const unsigned long long m = __ballot(on);
    if (lane_id() == 0 && (e & ~(int64_t)(kWave - 1)) < n) bits[e >> 6] = m;
}

__device__ __forceinline__ unsigned long long load_word(const uint64_t *bits, int64_t w, int64_t n_words, int64_t n)
{
    if (w >= n_words) return 0ull;
    unsigned long long v = bits[w];
    const int tail = (int)(n & 63);
    if (w == n_words - 1 && tail) v &= (1ull << tail) - 1ull;
    return v;
}

__global__ __launch_bounds__(kBlock) void compact_count_kernel(const uint64_t *__restrict__ bits, int64_t n_words,
                                                               int64_t n, uint32_t *__restrict__ block_count)
{
    const int64_t w = (int64_t)blockIdx.x * kWordsPerBlock + threadIdx.x;
    unsigned total;
    block_exclusive_scan((unsigned)__popcll(load_word(bits, w, n_words, n)), &total);
    if (threadIdx.x == 0) block_count[blockIdx.x] = total;
}

// one workgroup: exclusive scan of block_count in place, total -> *count
__global__ __launch_bounds__(kBlock) void compact_scan_kernel(uint32_t *__restrict__ block_count, int n_blocks,
                                                              int32_t *__restrict__ count)
{
    const int per = (n_blocks + kBlock - 1) / kBlock;
    const int lo = threadIdx.x * per;
    const int hi = min(lo + per, n_blocks);
    unsigned sum = 0;
    for (int i = lo; i < hi; ++i) sum += block_count[i];
    unsigned total;
    unsigned run = block_exclusive_scan(sum, &total);
    for (int i = lo; i < hi; ++i) {
        const unsigned c = block_count[i];
        block_count[i] = run;
        run += c;
    }
    if (threadIdx.x == 0) *count = (int32_t)total;
}

__global__ __launch_bounds__(kBlock) void compact_write_kernel(const uint64_t *__restrict__ bits, int64_t n_words,
                                                               int64_t n, const uint32_t *__restrict__ block_offset,
                                                               int32_t *__restrict__ ids)
{
    const int64_t w = (int64_t)blockIdx.x * kWordsPerBlock + threadIdx.x;
    unsigned long long v = load_word(bits, w, n_words, n);
    unsigned total;
    unsigned pos = block_offset[blockIdx.x] + block_exclusive_scan((unsigned)__popcll(v), &total);
    const int32_t base = (int32_t)(w << 6);
    while (v) {
        const int b = __ffsll((long long)v) - 1;
        v &= v - 1ull;
        ids[pos++] = base + b;
    }
}

// Two launches instead of three or four, for up to kMaxFused blocks: the first counts (from flags it also packs
// the bits, 64 flags per thread), the second has every workgroup add up the counts of the workgroups before
// it by itself -- a few KB from L2 -- instead of waiting for a scan launch in between.
constexpr int kMaxFused = 4096;

// bits 0..3 = which of the four bytes of x are non-zero
__device__ __forceinline__ unsigned nonzero_bytes(unsigned x)
{
    const unsigned high = (((x & 0x7f7f7f7fu) + 0x7f7f7f7fu) | x) & 0x80808080u;  // bit 7 of every non-zero byte
    return (((high >> 7) * 0x00204081u) >> 21) & 0xFu;                             // bits 0, 8, 16, 24 -> 0..3
}

__global__ __launch_bounds__(kBlock) void compact_count_flags_kernel(const uint8_t *__restrict__ z, int64_t n,
                                                                     int64_t n_words, uint64_t *__restrict__ bits,
                                                                     uint32_t *__restrict__ block_count)
{
    const int64_t w = (int64_t)blockIdx.x * kWordsPerBlock + threadIdx.x;
    unsigned long long v = 0ull;
    if (w < n_words) {
        const int64_t e0 = w << 6;
        if (e0 + 64 <= n) {
            const uint4 *q = reinterpret_cast<const uint4 *>(z + e0);  // z is 16-byte aligned (checked by the caller)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint4 x = q[i];
                const unsigned long long part = nonzero_bytes(x.x) | (nonzero_bytes(x.y) << 4) |
                                                (nonzero_bytes(x.z) << 8) | (nonzero_bytes(x.w) << 12);
                v |= part << (16 * i);
            }
        } else {
            for (int64_t e = e0; e < n; ++e) v |= (unsigned long long)(z[e] != 0) << (e - e0);
        }
        bits[w] = v;
    }
    unsigned total;
    block_exclusive_scan((unsigned)__popcll(v), &total);
    if (threadIdx.x == 0) block_count[blockIdx.x] = total;
}

// block_count holds the plain per-block counts here
__global__ __launch_bounds__(kBlock) void compact_write_fused_kernel(const uint64_t *__restrict__ bits, int64_t n_words,
                                                                     int64_t n, const uint32_t *__restrict__ block_count,
                                                                     int32_t *__restrict__ ids,
                                                                     int32_t *__restrict__ count)
{
    unsigned before = 0;
    for (int b = threadIdx.x; b < (int)blockIdx.x; b += kBlock) before += block_count[b];
    unsigned offset;
    block_exclusive_scan(before, &offset);  // the block sum is what is wanted
    const int64_t w = (int64_t)blockIdx.x * kWordsPerBlock + threadIdx.x;
    unsigned long long v = load_word(bits, w, n_words, n);
    unsigned total;
    unsigned pos = offset + block_exclusive_scan((unsigned)__popcll(v), &total);
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) *count = (int32_t)(offset + total);
    const int32_t base = (int32_t)(w << 6);
    while (v) {
        const int b = __ffsll((long long)v) - 1;
        v &= v - 1ull;
        ids[pos++] = base + b;
    }
}

// ---------------------------------------------------------------------------
// Event-driven scatter: one wavefront per active element walks the source's
// out-going synapses 64 at a time (coalesced table reads), fp32 atomics into
// the ring.
// ---------------------------------------------------------------------------

__global__ __launch_bounds__(kBlock) void scatter_kernel(const int32_t *__restrict__ active,
                                                         const int32_t *__restrict__ n_active, int batch, Table t,
                                                         float *__restrict__ ring, int L, int64_t ne, int slot0)
{
    const int n_waves = gridDim.x * (kBlock / kWave);
    const int cnt = *n_active;
    for (int k = blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave; k < cnt; k += n_waves) {
        const int e = active[k];
        const int j = batch == 1 ? e : (int)((uint32_t)e / (uint32_t)batch);
        deliver_row(t, j, e - j * batch, batch, ring, L, slot0, ne);
    }
}

// ---------------------------------------------------------------------------
// Row-wise gather: one wavefront per target row, lane = trial.  The spike
// bits of a source over 64 trials are a native lane mask: a synapse whose
// source fired in any trial is broadcast to the wavefront and every lane whose
// trial fired adds the weight to its own accumulator (LDS, one column per
// lane, one row per (slot, receptor)).  Accumulators start from the ring cell
// on first touch and are stored back once, so every cell sees its additions
// in stored synapse order: deterministic and equal to a scalar loop.
// ---------------------------------------------------------------------------

__global__ __launch_bounds__(kBlock) void gather_kernel(const uint64_t *__restrict__ zbits, int batch, Table t,
                                                        float *__restrict__ ring, int L, int64_t n_tgt, int64_t ne,
                                                        int slot0)
{
    extern __shared__ float lds[];
    const int lane = lane_id();
    const int wave_in_block = threadIdx.x / kWave;
    float *acc = lds + (size_t)wave_in_block * L * GLIF3_NREC * kWave;
    const int64_t row = (int64_t)blockIdx.x * (kBlock / kWave) + wave_in_block;
    if (row >= n_tgt) return;
    const int tile0 = blockIdx.y * kWave;
    const int width = min(kWave, batch - tile0);
    const bool lane_on = lane < width;
    const int64_t cell0 = row * batch + tile0 + lane;
    unsigned long long touched = 0ull;  // bit (slot*4+r): accumulator row is live
    const int p0 = t.indptr[row], p1 = t.indptr[row + 1];
    for (int base = p0; base < p1; base += kWave) {
        const int p = base + lane;
        const bool valid = p < p1;
        float w = 0.0f;
        int dr = 0;
        unsigned long long m = 0ull;
        if (valid) {
            const int src = t.indices[p];
            w = t.weights[p];
            int slot = slot0 + (int)t.delays[p];
            slot = slot >= L ? slot - L : slot;
            dr = slot * GLIF3_NREC + (int)t.receptors[p];
            m = source_mask(zbits, src, batch, tile0, width);
        }
        unsigned long long act = __ballot(m != 0ull);
        while (act) {
            const int l = __ffsll((long long)act) - 1;
            act &= act - 1ull;
            const float wl = bcast_f(w, l);
            const int drl = bcast_i(dr, l);
            const unsigned long long ml = bcast_u64(m, l);
            float *a = acc + drl * kWave + lane;
            if (!((touched >> drl) & 1ull)) {
                touched |= 1ull << drl;
                *a = lane_on ? ring[(int64_t)drl * ne + cell0] : 0.0f;
            }
            if ((ml >> lane) & 1ull) *a += wl;
        }
    }
    while (touched) {
        const int drl = __ffsll((long long)touched) - 1;
        touched &= touched - 1ull;
        if (lane_on) ring[(int64_t)drl * ne + cell0] = acc[drl * kWave + lane];
    }
}

}  // namespace bmtk

// ===========================================================================
// C entry points
// ===========================================================================

using namespace bmtk;

extern "C" {

int bmtk_amd_abi_version(void) { return BMTK_AMD_ABI_VERSION; }

const char *bmtk_amd_last_error(void) { return g_error; }

int64_t bmtk_glif3_sim_sizeof(void) { return (int64_t)sizeof(bmtk_glif3_sim); }

int64_t bmtk_glif3_bwd_sizeof(void) { return (int64_t)sizeof(bmtk_glif3_bwd); }

int bmtk_glif3_precompute(int64_t n, const double *par, double h, float *prop, void *stream)
{
    BMTK_REQUIRE(n > 0 && par && prop, "glif3_precompute: n must be positive and pointers non-null");
    BMTK_REQUIRE(h > 0.0, "glif3_precompute: resolution h must be positive");
    const unsigned grid = (unsigned)((n + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(precompute_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, n, par, h, prop);
    BMTK_CHECK_LAUNCH("glif3_precompute");
    return BMTK_OK;
}

int bmtk_glif3_step_fwd(int64_t n_neurons, int32_t batch, float *V, float *asc, float *y1, float *y2, int32_t *ref,
                        const float *prop, int64_t prop_stride, const int32_t *class_id, float h, float *syn,
                        int32_t clear_syn, const float *i_ext, uint8_t *z, uint64_t *zbits, float *frac,
                        void *stream)
{
    BMTK_REQUIRE(n_neurons > 0 && batch > 0, "glif3_step_fwd: n_neurons and batch must be positive");
    BMTK_REQUIRE(V && asc && y1 && y2 && ref && prop, "glif3_step_fwd: state and prop pointers must be non-null");
    BMTK_REQUIRE(class_id || prop_stride >= n_neurons, "glif3_step_fwd: prop_stride smaller than n_neurons");
    BMTK_REQUIRE(prop_stride > 0, "glif3_step_fwd: prop_stride must be positive");
    BMTK_REQUIRE(h > 0.0f, "glif3_step_fwd: resolution h must be positive");
    const int64_t ne = n_neurons * (int64_t)batch;
    BMTK_REQUIRE(ne < (1ll << 31), "glif3_step_fwd: n_neurons*batch must stay below 2^31");
    StepArgs a{ne, batch, V, asc, y1, y2, ref, prop, prop_stride, class_id, h, syn, clear_syn, i_ext, z, zbits, frac};
    const unsigned grid = (unsigned)((ne + kBlock - 1) / kBlock);
    // a class table of up to 48 KB (423 classes) is staged in LDS by every workgroup (sixteen bytes per load: a
    // table that is not 16-byte aligned is read through the caches instead)
    const size_t table_bytes = (size_t)prop_stride * GLIF3_NPROP * sizeof(float);
    if (class_id && table_bytes <= 48u * 1024u && ((uintptr_t)prop & 15u) == 0)
        hipLaunchKernelGGL(glif3_step_kernel<true>, dim3((grid + kStepTiles - 1) / kStepTiles), dim3(kBlock), table_bytes,
                           (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL(glif3_step_kernel<false>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, a);
    BMTK_CHECK_LAUNCH("glif3_step_fwd");
    return BMTK_OK;
}

static int64_t n_words_of(int64_t n) { return (n + 63) / 64; }
static int64_t n_blocks_of(int64_t n) { return (n_words_of(n) + kWordsPerBlock - 1) / kWordsPerBlock; }

int64_t bmtk_spikes_compact_workspace_bytes(int64_t n)
{
    if (n <= 0) return 0;
    // bit words (+1 padding) followed by the per-block counters
    return 8 * (n_words_of(n) + 1) + 4 * (n_blocks_of(n) + 1);
}

static int compact_from_bits(const uint64_t *bits, int64_t n, int32_t *ids, int32_t *count, uint32_t *block_count,
                             hipStream_t stream)
{
    const int64_t n_words = n_words_of(n);
    const int n_blocks = (int)n_blocks_of(n);
    if (n_blocks <= kMaxFused) {
        hipLaunchKernelGGL(compact_count_kernel, dim3(n_blocks), dim3(kBlock), 0, stream, bits, n_words, n, block_count);
        hipLaunchKernelGGL(compact_write_fused_kernel, dim3(n_blocks), dim3(kBlock), 0, stream, bits, n_words, n,
                           (const uint32_t *)block_count, ids, count);
        BMTK_CHECK_LAUNCH("spikes_compact");
        return BMTK_OK;
    }
    hipLaunchKernelGGL(compact_count_kernel, dim3(n_blocks), dim3(kBlock), 0, stream, bits, n_words, n, block_count);
    hipLaunchKernelGGL(compact_scan_kernel, dim3(1), dim3(kBlock), 0, stream, block_count, n_blocks, count);
    hipLaunchKernelGGL(compact_write_kernel, dim3(n_blocks), dim3(kBlock), 0, stream, bits, n_words, n,
                       (const uint32_t *)block_count, ids);
    BMTK_CHECK_LAUNCH("spikes_compact");
    return BMTK_OK;
}

int bmtk_spikes_compact(const uint8_t *z, int64_t n, int32_t *ids, int32_t *count, void *workspace, void *stream)
{
    BMTK_REQUIRE(n > 0 && n < (1ll << 31), "spikes_compact: n must lie in 1..2^31-1");
    BMTK_REQUIRE(z && ids && count && workspace, "spikes_compact: pointers must be non-null");
    uint64_t *bits = (uint64_t *)workspace;
    uint32_t *block_count = (uint32_t *)(bits + n_words_of(n) + 1);
    const int n_blocks = (int)n_blocks_of(n);
    if (n_blocks <= kMaxFused && (reinterpret_cast<uintptr_t>(z) & 15u) == 0) {
        hipLaunchKernelGGL(compact_count_flags_kernel, dim3(n_blocks), dim3(kBlock), 0, (hipStream_t)stream, z, n,
                           n_words_of(n), bits, block_count);
        hipLaunchKernelGGL(compact_write_fused_kernel, dim3(n_blocks), dim3(kBlock), 0, (hipStream_t)stream,
                           (const uint64_t *)bits, n_words_of(n), n, (const uint32_t *)block_count, ids, count);
        BMTK_CHECK_LAUNCH("spikes_compact");
        return BMTK_OK;
    }
    const unsigned grid = (unsigned)((n + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(pack_bits_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, z, n, bits);
    return compact_from_bits(bits, n, ids, count, block_count, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------
// The same compaction with the workspace inside the library: a file-scope
// device array, so that the call allocates nothing.  In host code the array's
// name is only a handle; its device address is asked for once per device, with
// that device current, and kept.
// ---------------------------------------------------------------------------

constexpr int64_t kNoAllocBytes = 8 * (BMTK_COMPACT_NOALLOC_MAX_N / 64 + 1) +
                                  4 * (BMTK_COMPACT_NOALLOC_MAX_N / 64 / kWordsPerBlock + 2);
static __device__ __align__(256) unsigned char scratch[(kNoAllocBytes + 255) / 256 * 256];

constexpr int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];  // device address of `scratch` on every device seen so far
static std::mutex g_scratch_mutex;

// device address of this device's copy of `scratch`, or nullptr with the error message set
static void *scratch_of_current_device()
{
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("spikes_compact_noalloc: cannot tell the current device (%s)", hipGetErrorString(err));
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !ptr) {
            set_error("spikes_compact_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(err));
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

int bmtk_spikes_compact_noalloc(const uint8_t *z, int64_t n, int32_t *ids, int32_t *count, void *stream)
{
    BMTK_REQUIRE(n > 0, "spikes_compact_noalloc: n must be positive");
    BMTK_REQUIRE(n <= BMTK_COMPACT_NOALLOC_MAX_N,
                 "spikes_compact_noalloc: n = %lld exceeds the %lld elements the built-in workspace holds; use "
                 "bmtk_spikes_compact with a workspace of the caller's", (long long)n,
                 (long long)BMTK_COMPACT_NOALLOC_MAX_N);
    BMTK_REQUIRE(z && ids && count, "spikes_compact_noalloc: pointers must be non-null");
    static_assert(kNoAllocBytes >= 8 * ((BMTK_COMPACT_NOALLOC_MAX_N + 63) / 64 + 1) +
                                       4 * (((BMTK_COMPACT_NOALLOC_MAX_N + 63) / 64 + kWordsPerBlock - 1) / kWordsPerBlock + 1),
                  "scratch smaller than bmtk_spikes_compact_workspace_bytes(BMTK_COMPACT_NOALLOC_MAX_N)");
    void *ws = scratch_of_current_device();
    if (!ws) return BMTK_E_DEVICE;
    // every word of the workspace a kernel reads is written earlier in the same call, so what the call before
    // left behind does not matter and nothing has to be cleared
    return bmtk_spikes_compact(z, n, ids, count, ws, stream);
}

int bmtk_spikes_compact_bits(const uint64_t *zbits, int64_t n, int32_t *ids, int32_t *count, void *workspace,
                             void *stream)
{
    BMTK_REQUIRE(n > 0 && n < (1ll << 31), "spikes_compact_bits: n must lie in 1..2^31-1");
    BMTK_REQUIRE(zbits && ids && count && workspace, "spikes_compact_bits: pointers must be non-null");
    uint32_t *block_count = (uint32_t *)((uint64_t *)workspace + n_words_of(n) + 1);
    return compact_from_bits(zbits, n, ids, count, block_count, (hipStream_t)stream);
}

int bmtk_csr_propagate_scatter(const int32_t *active, const int32_t *n_active, int64_t max_active, int32_t batch,
                               const int32_t *indptr, const int32_t *indices, const float *weights,
                               const uint8_t *delays, const uint8_t *receptors, float *ring, int32_t L,
                               int64_t n_tgt, int64_t step, void *stream)
{
    BMTK_REQUIRE(active && n_active && indptr && indices && weights && delays && receptors && ring,
                 "csr_propagate_scatter: pointers must be non-null");
    BMTK_REQUIRE(batch > 0 && n_tgt > 0 && L > 1 && step >= 0, "csr_propagate_scatter: bad batch, n_tgt, L or step");
    BMTK_REQUIRE(n_tgt * (int64_t)batch < (1ll << 31), "csr_propagate_scatter: n_tgt*batch must stay below 2^31");
    if (max_active <= 0) return BMTK_OK;
    const int64_t waves = max_active < 8192 ? max_active : 8192;
    const unsigned grid = (unsigned)((waves + kBlock / kWave - 1) / (kBlock / kWave));
    Table t{indptr, indices, weights, delays, receptors};
    hipLaunchKernelGGL(scatter_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, active, n_active, batch, t,
                       ring, L, n_tgt * (int64_t)batch, (int)(step % L));
    BMTK_CHECK_LAUNCH("csr_propagate_scatter");
    return BMTK_OK;
}

int bmtk_csr_propagate_gather(const uint64_t *zbits, int64_t n_src, int32_t batch, const int32_t *indptr,
                              const int32_t *indices, const float *weights, const uint8_t *delays,
                              const uint8_t *receptors, float *ring, int32_t L, int64_t n_tgt, int64_t step,
                              void *stream)
{
    BMTK_REQUIRE(zbits && indptr && indices && weights && delays && receptors && ring,
                 "csr_propagate_gather: pointers must be non-null");
    BMTK_REQUIRE(batch > 0 && n_tgt > 0 && n_src > 0 && step >= 0, "csr_propagate_gather: bad batch, sizes or step");
    BMTK_REQUIRE(L > 1 && L <= 16, "csr_propagate_gather: ring_slots must lie in 2..16");
    BMTK_REQUIRE(n_tgt * (int64_t)batch < (1ll << 31), "csr_propagate_gather: n_tgt*batch must stay below 2^31");
    const unsigned rows_per_block = kBlock / kWave;
    const dim3 grid((unsigned)((n_tgt + rows_per_block - 1) / rows_per_block), (unsigned)((batch + kWave - 1) / kWave));
    BMTK_REQUIRE(grid.y <= 65535, "csr_propagate_gather: batch too large");
    const size_t lds = (size_t)rows_per_block * L * GLIF3_NREC * kWave * sizeof(float);
    Table t{indptr, indices, weights, delays, receptors};
    hipLaunchKernelGGL(gather_kernel, grid, dim3(kBlock), lds, (hipStream_t)stream, zbits, batch, t, ring, L, n_tgt,
                       n_tgt * (int64_t)batch, (int)(step % L));
    BMTK_CHECK_LAUNCH("csr_propagate_gather");
    return BMTK_OK;
}

}  // extern "C"
