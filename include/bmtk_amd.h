/*
 * C ABI of libbmtk_amd.so -- the GLIF3 point-neuron hot path on one MI355X.
 *
 * The reference (bmtk's PointNet driver) reaches this arithmetic through
 * PyNEST, a Python module, not through an FFI of its own: nest.Create
 * (bmtk/simulator/pointnet/sonata_adaptors.py:64-66), nest.Connect
 * (bmtk/simulator/pointnet/pointnetwork.py:229-232) and nest.Simulate
 * (bmtk/simulator/pointnet/pointsimulator.py:159-166).  The entry points below
 * are the per-step operations NEST performs behind those calls, one function
 * per operation, each citing the call it stands behind.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer unless the name ends in _host.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *    Calls enqueue work and return; they never synchronise and never allocate.
 *  - Element index e = neuron * batch + trial ("trial-minor"): a 64-lane
 *    wavefront covers 64 trials of one neuron when batch is a multiple of 64.
 *  - State, SoA fp32: V[ne] (membrane potential minus E_L), asc[2][ne],
 *    y1[4][ne], y2[4][ne], ref[ne] (int32 refractory steps left), ne = n*batch.
 *  - Ring buffer: ring[L][4][ne] fp32, slot (t mod L) holds the weight sums
 *    that arrive in step t; L must exceed the largest delay in steps.
 *  - Synapse table: indptr int32[rows+1], indices int32[nnz], weights
 *    fp32[nnz], delays uint8[nnz] in steps (>= 1), receptors uint8[nnz] 0-based.
 *    "source-major": rows are presynaptic, indices are targets.
 *    "target-major": rows are postsynaptic, indices are sources.
 *  - Spike bits: uint64 words, bit (e mod 64) of word (e / 64) is element e;
 *    arrays hold ceil(ne/64)+1 words (the last one is padding kernels may read).
 *  - Return value: 0 on success, a negative BMTK_E_* code otherwise;
 *    bmtk_amd_last_error() returns the message of the calling thread's last
 *    failure.  Arguments are validated on the host before any launch; values
 *    stored in device arrays (indices, delays, class ids) are NOT checked by
 *    the kernels and must have been validated by the caller.
 */
#ifndef BMTK_AMD_H
#define BMTK_AMD_H

#include <stdint.h>

#include "bmtk_amd_layout.h"

#ifdef __cplusplus
extern "C" {
#endif

#define BMTK_OK 0
#define BMTK_E_ARG (-1)    /* null pointer, non-positive size, unsupported combination */
#define BMTK_E_LAUNCH (-2) /* HIP reported an error for the launch */
#define BMTK_E_DEVICE (-3) /* no usable gfx950 device */

/* Bumped whenever a struct layout or a signature below changes; bmtk_amd_abi_version() returns the value the
 * library was built with. */
#define BMTK_AMD_ABI_VERSION 24
int bmtk_amd_abi_version(void);
const char *bmtk_amd_last_error(void);
/* sizeof(bmtk_glif3_sim) as the library was compiled, for bindings that mirror the struct */
int64_t bmtk_glif3_sim_sizeof(void);
int64_t bmtk_glif3_bwd_sizeof(void);

/* NEST glif_psc::pre_run_hook, run when bmtk calls nest.Create('glif_psc', n,
 * params) (bmtk/simulator/pointnet/sonata_adaptors.py:64-66): NEST-unit
 * parameters par[GLIF3_NPARAM][n] (fp64) and the resolution h (ms) ->
 * propagators prop[GLIF3_NPROP][n] (fp32).  Computed in fp64, rounded once. */
int bmtk_glif3_precompute(int64_t n, const double *par, double h, float *prop, void *stream);

/* One glif_psc::update step for all n_neurons*batch elements (what
 * nest.Simulate does per neuron per step, bmtk/simulator/pointnet/pointsimulator.py:159-166).
 * prop is [GLIF3_NPROP][prop_stride]; column = neuron when class_id is NULL,
 * else column = class_id[neuron].
 * syn: [4][ne] weight sums arriving this step (one ring slot), may be NULL;
 *      when clear_syn != 0 the slot is zeroed after it has been read.
 * i_ext: [ne] external current used in this step, may be NULL.
 * z (uint8[ne]), zbits (spike bits), frac (fp32[ne], fraction of the step at
 * which threshold was crossed, written only where a spike occurred): outputs,
 * each may be NULL. */
int bmtk_glif3_step_fwd(int64_t n_neurons, int32_t batch,
                        float *V, float *asc, float *y1, float *y2, int32_t *ref,
                        const float *prop, int64_t prop_stride, const int32_t *class_id, float h,
                        float *syn, int32_t clear_syn, const float *i_ext,
                        uint8_t *z, uint64_t *zbits, float *frac, void *stream);

/* Spike flags -> ascending list of active element ids (NEST keeps the same
 * information as its per-slice spike register; bmtk maps ids back through
 * GidPool, bmtk/simulator/pointnet/gids.py:24-107).
 * ids must hold n entries, count is one int32; workspace must hold
 * bmtk_spikes_compact_workspace_bytes(n) bytes.  Exactly numpy.flatnonzero. */
int64_t bmtk_spikes_compact_workspace_bytes(int64_t n);
int bmtk_spikes_compact(const uint8_t *z, int64_t n, int32_t *ids, int32_t *count, void *workspace, void *stream);
/* Same from spike bits (n elements, ceil(n/64) words are read). */
int bmtk_spikes_compact_bits(const uint64_t *zbits, int64_t n, int32_t *ids, int32_t *count, void *workspace,
                             void *stream);

/* bmtk_spikes_compact without a workspace argument and without any allocation.  No counterpart in the
 * reference: it exists for callers that cannot allocate device memory -- code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  The workspace is an array inside the library (about 2.1 MB
 * of device memory on every GPU the library runs on, held until the process ends), which bounds the input:
 * n <= BMTK_COMPACT_NOALLOC_MAX_N, larger n returns BMTK_E_ARG.  z, ids (n entries) and count (one int32) are
 * the caller's, as above; the result is the same as bmtk_spikes_compact's.  All calls on one GPU share that
 * GPU's array: calls that overlap on one GPU (different streams or threads) race and must be serialised by the
 * caller; calls on different GPUs are independent.  The first call on a device looks up the array's address
 * (hipGetSymbolAddress, no allocation). */
#define BMTK_COMPACT_NOALLOC_MAX_N (1ll << 24)
int bmtk_spikes_compact_noalloc(const uint8_t *z, int64_t n, int32_t *ids, int32_t *count, void *stream);

/* Event-driven delivery (NEST static_synapse::send -> RingBuffer::add_value,
 * wired by nest.Connect in bmtk/simulator/pointnet/pointnetwork.py:161-173,187-232):
 * for every active element id = source*batch + trial in active[0..*n_active)
 * and every synapse (source -> i, w, d, r) of the SOURCE-MAJOR table,
 * ring[(step+d) mod L][r][i*batch+trial] += w with fp32 atomics.
 * n_active is read on the device; max_active bounds it (grid sizing only). */
int bmtk_csr_propagate_scatter(const int32_t *active, const int32_t *n_active, int64_t max_active, int32_t batch,
                               const int32_t *indptr, const int32_t *indices, const float *weights,
                               const uint8_t *delays, const uint8_t *receptors,
                               float *ring, int32_t L, int64_t n_tgt, int64_t step, void *stream);

/* The same sums taken row by row over the TARGET-MAJOR table from the spike
 * bits of the emitting step: deterministic (each ring cell is updated by one
 * wavefront, additions in stored synapse order), no atomics. */
int bmtk_csr_propagate_gather(const uint64_t *zbits, int64_t n_src, int32_t batch,
                              const int32_t *indptr, const int32_t *indices, const float *weights,
                              const uint8_t *delays, const uint8_t *receptors,
                              float *ring, int32_t L, int64_t n_tgt, int64_t step, void *stream);

/* One packed synapse: tdr = index | receptor << 24 | delay << 26 (index < 2^24, delay < 64 steps). */
typedef struct bmtk_synapse {
    uint32_t tdr;
    float weight;
} bmtk_synapse;

/* Pull form of the same sums, for batched runs: instead of pushing weights
 * into future ring slots, keep the spike bits of the last L steps
 * (spike_hist[L][hist_stride] uint64 words, row (k mod L) = spike bits of step
 * k) and compute everything that ARRIVES in step t_arrive in one pass over a
 * packed TARGET-MAJOR table:
 *   syn[r][i*batch+b] = sum over synapses (j -> i, w, d, r) of w * bit(spike_hist[(t_arrive-d) mod L], j*batch+b)
 * syn ([4][n_tgt*batch]) is overwritten and is exactly the `syn` argument of
 * bmtk_glif3_step_fwd for step t_arrive.  A wavefront owns a target row at a time, lane = synapse; a per-source
 * "fired in any trial" bit map of the L steps (built into `workspace`,
 * bmtk_csr_propagate_pull_workspace_bytes bytes, and staged in LDS) filters the synapses whose source was
 * silent, the others are gathered 64 at a time, fetch their source's trial mask and add their weight once per
 * trial bit into LDS accumulators.  The accumulators are 64-bit fixed point (Q31.32) and the additions integer
 * atomics, so the result does not depend on the order of the additions: it is the exact sum of the weights,
 * rounded to fp32 once, the same in every run.  Weights must be finite and smaller than 2^31 in size; weight
 * bits below 2^-32 are dropped.  The cost is one read of the table per step plus one mask fetch per synapse with
 * an active source.  L must exceed the largest delay; L * hist_stride must stay below 2^29 words; the bit map,
 * L * ceil(n_src/32) * 4 bytes, must fit in 40 KB of LDS (n_src <= 54,000 at L = 6).  The workspace size is the
 * larger of that map and n_src bytes rounded up to 16 (the map of bmtk_csr_propagate_pull2). */
int64_t bmtk_csr_propagate_pull_workspace_bytes(int32_t L, int64_t n_src);
int bmtk_csr_propagate_pull(const uint64_t *spike_hist, int64_t hist_stride, int32_t L, int64_t n_src, int32_t batch,
                            const int32_t *indptr, const bmtk_synapse *packed, float *syn, int64_t n_tgt,
                            int64_t t_arrive, void *workspace, void *stream);

/* Delivery step by step with the form chosen ON THE DEVICE from the number of active elements, without a host
 * synchronisation -- the switch NEST does not need (it is always event-driven) and a GPU does: pushing events costs
 * one fp32 atomic each (about 2e10 per second on one MI355X, whatever the rate), the pull form a pass over the whole
 * table (about 100 us for 52 M synapses, whatever the rate), so few spikes are pushed and many are pulled.
 * Call once per step, in order, after the step's spikes are known:
 *   - spike_hist row (step mod L) holds the spike bits of `step` (the caller wrote them), active / *n_active the
 *     same spikes as a list (bmtk_spikes_compact*);
 *   - up to scatter_max_active active elements the spikes are pushed into `ring` through the SOURCE-major table
 *     (as bmtk_csr_propagate_scatter) and their history row is struck from the pull's view; above it they are left
 *     to the pull kernel, which sums, over the packed TARGET-major table, what the steps not pushed send to step
 *     + 1 and writes (or, where pushed spikes already sent something, adds) it into ring slot (step + 1) mod L.
 *     When none of the L-1 steps the arrival step looks back on was left to it, the pull kernel returns at once.
 *   After the call ring slot (step + 1) mod L holds everything that arrives in step + 1, whatever mix of forms
 *   delivered it; the caller consumes and CLEARS that slot before the next call (bmtk_glif3_step_fwd with
 *   clear_syn does), as with the event-driven form.  Later slots hold the pushed part only.
 * workspace: bmtk_csr_propagate_auto_workspace_bytes(L, n_src) bytes, zeroed before the first call and then left
 * to the library (the activity map of the last L steps and the record of which steps were pushed).  Limits as for
 * bmtk_csr_propagate_pull.  On one MI355X with 51,978 neurons, in-degree 1000 and batch 64 the two forms cost the
 * same near 2,000 active elements per step (0.6 Hz); for other shapes about 0.032 n_src + 4e5 n_src / nnz (events
 * leave at 2e10 per second, a pass streams the table at 5 TB/s after 20 us of launches and set-up). */
int64_t bmtk_csr_propagate_auto_workspace_bytes(int32_t L, int64_t n_src);
int bmtk_csr_propagate_auto(const int32_t *active, const int32_t *n_active, int64_t max_active,
                            const uint64_t *spike_hist, int64_t hist_stride, int32_t L, int64_t n_src, int32_t batch,
                            const int32_t *src_indptr, const int32_t *src_indices, const float *src_weights,
                            const uint8_t *src_delays, const uint8_t *src_receptors,
                            const int32_t *tgt_indptr, const bmtk_synapse *tgt_packed,
                            float *ring, int64_t n_tgt, int64_t step, int64_t scatter_max_active, void *workspace,
                            void *stream);

/* bmtk_csr_propagate_pull for TWO consecutive arrival steps in one pass over the table: syn2[0][r][..] is what arrives in step
 * t_arrive - 1, syn2[1][r][..] what arrives in step t_arrive ([2][4][n_tgt*batch], overwritten).  Both only depend
 * on the spikes of steps up to t_arrive - 1 (delays are at least one step): spike_hist must hold the steps
 * t_arrive - L .. t_arrive - 1 (row k mod L = step k).  A caller that advances two steps between calls -- sums of
 * t-1 into the update of t, sums of t into the update of t+1 -- reads the table, most of a call's bytes at low
 * rates, once per two steps (the batched simulation driver does the same inside its launches).  Workspace and
 * limits as bmtk_csr_propagate_pull, except that the map may take up to 70 KB of LDS.  With L <= 8 and n_src <=
 * 70 KB the map is kept source-major instead, one byte per source whose bit d says "fired d steps before the
 * step whose row t_arrive's spikes will take": one LDS read then answers both questions a synapse asks (6 % faster
 * at 0.2 Hz at 51,978 x batch 64); bmtk_csr_propagate_pull_workspace_bytes covers both forms of the map. */
int bmtk_csr_propagate_pull2(const uint64_t *spike_hist, int64_t hist_stride, int32_t L, int64_t n_src, int32_t batch,
                             const int32_t *indptr, const bmtk_synapse *packed, float *syn2, int64_t n_tgt,
                             int64_t t_arrive, void *workspace, void *stream);

/* bmtk_csr_propagate_auto for a caller that advances TWO steps between calls (what bmtk_csr_propagate_pull2 is to
 * bmtk_csr_propagate_pull): call after steps `step - 1` and `step` are known, with step = 1, 3, 5, ... (any start,
 * then every second step).  spike_hist rows (step - 1) mod L and step mod L hold the two steps' spike bits,
 * active_a / active_b the same spikes as lists.  Each of the two steps is pushed as events or left to the pull by its
 * own count; the pull then sums, in ONE pass over the target-major table, what the steps not pushed send to steps
 * `step` and `step + 1`.  After the call ring slots step mod L and (step + 1) mod L hold everything that arrives in
 * those two steps; the caller consumes and clears both before the next call.  L at most 8 (the activity map is one
 * byte per source) and n_src bytes within 70 KB of LDS; workspace of bmtk_csr_propagate_auto2_workspace_bytes bytes,
 * zeroed before the first call.  At 51,978 x batch 64 a pair of steps left to the pull costs one table pass, 116 -
 * 435 us at 0.2 - 20 Hz, against two passes of 100 - 275 us each with the one-step switch. */
int64_t bmtk_csr_propagate_auto2_workspace_bytes(int32_t L, int64_t n_src);
int bmtk_csr_propagate_auto2(const int32_t *active_a, const int32_t *n_active_a, const int32_t *active_b,
                             const int32_t *n_active_b, int64_t max_active, const uint64_t *spike_hist,
                             int64_t hist_stride, int32_t L, int64_t n_src, int32_t batch,
                             const int32_t *src_indptr, const int32_t *src_indices, const float *src_weights,
                             const uint8_t *src_delays, const uint8_t *src_receptors,
                             const int32_t *tgt_indptr, const bmtk_synapse *tgt_packed,
                             float *ring, int64_t n_tgt, int64_t step, int64_t scatter_max_active, void *workspace,
                             void *stream);

/* Packed synapse format used by the fused simulation: one 8-byte record per
 * synapse, {uint32 tdr, float weight} with tdr = index | receptor << 24 |
 * delay << 26 (index < 2^24, delay < 64 steps).  bmtk_csr_pack converts the
 * four plain arrays of a table; packed must hold nnz records. */
int bmtk_csr_pack(int64_t nnz, const int32_t *indices, const float *weights, const uint8_t *delays,
                  const uint8_t *receptors, bmtk_synapse *packed, void *stream);

/* The same with a wider delay field, for delay spreads beyond 63 steps: tdr = index | receptor << (30 - delay_bits)
 * | delay << (32 - delay_bits), delay_bits in 6..14, index < 2^(30 - delay_bits), delay < 2^delay_bits (int32
 * input).  Only the launch-per-step driver without the pull form reads such tables (bmtk_glif3_sim.delay_bits);
 * its ring then has up to 2^delay_bits slots in device memory. */
int bmtk_csr_pack_wide(int64_t nnz, const int32_t *indices, const float *weights, const int32_t *delays,
                       const uint8_t *receptors, int32_t delay_bits, bmtk_synapse *packed, void *stream);

/* Per-row segment offsets of a SOURCE-MAJOR table whose rows are sorted by
 * target: seg[row*(n_groups+1) + g] = position of the first synapse of the row
 * whose target is >= g*span (g = 0..n_groups; the last entry is the row end).
 * *unsorted (one int32) is set to 1 if some row is not sorted by target. */
int bmtk_csr_segment_offsets(int64_t n_rows, const int32_t *indptr, const int32_t *indices, int32_t span,
                             int32_t n_groups, uint32_t *seg, int32_t *unsorted, void *stream);

#define BMTK_RES_SYNC_STRIDE 1088                          /* words: 4 KiB + 256 B */
#define BMTK_RES_SYNC_WAYS 8                               /* counters a step's arrivals are spread over */
#define BMTK_RES_FIRED_SLOTS 16       /* places of a workgroup's list in bmtk_glif3_sim.res_fired */
#define BMTK_RES_FIRED_MANY 0xFFFFFFFFu /* ... more neurons fired than the list holds */
#define BMTK_RES_SYNC_WORDS ((1 + 64 * BMTK_RES_SYNC_WAYS) * BMTK_RES_SYNC_STRIDE) /* size of bmtk_glif3_sim.res_sync */

/* Everything nest.Simulate needs for a forward run (bmtk/simulator/pointnet/pointsimulator.py:159-166). */
typedef struct bmtk_glif3_sim {
    int64_t n_neurons;
    int32_t batch;
    int32_t ring_slots;          /* L */
    float h;                     /* resolution, ms */
    int32_t _pad0;
    float *V, *asc, *y1, *y2;    /* state, see above */
    int32_t *ref;
    const float *prop;           /* [GLIF3_NPROP][prop_stride] */
    int64_t prop_stride;
    const int32_t *class_id;     /* NULL: one column per neuron */
    float *ring;                 /* [L][4][ne] */
    /* recurrent synapses, source-major (may be all NULL) */
    const int32_t *rec_indptr, *rec_indices;
    const float *rec_weights;
    const uint8_t *rec_delays, *rec_receptors;
    const bmtk_synapse *rec_packed; /* same table packed (bmtk_csr_pack); required when rec_indptr is set */
    /* external spike sources: per-step event lists + source-major table */
    int64_t n_inputs;
    const int64_t *in_ptr;       /* [total steps + 1], indexed by absolute step */
    const int32_t *in_events;    /* element ids source*batch+trial, emitted in that step; ascending within a step
                                  * (the input-weight gradient relies on it).  An id may repeat within a step (two
                                  * spikes of one source inside one resolution step): every occurrence is
                                  * delivered.  The pull form of the inputs (pull_inp_* below) turns a step's
                                  * events into bits, which hold an id once: with it, the second and later
                                  * occurrences must also be listed in in_repeat_ptr / in_repeat_events. */
    const int32_t *inp_indptr, *inp_indices;
    const float *inp_weights;
    const uint8_t *inp_delays, *inp_receptors;
    const bmtk_synapse *inp_packed; /* required when in_ptr is set */
    const float *i_ext;          /* [ne] constant external current or NULL */
    uint64_t *work_bits;         /* history of spike bits, hist_slots rows of ceil(ne/64)+1 words: the spikes
                                  * of step t live in row t % hist_slots.  Zero it before the first run and
                                  * leave it alone between runs that continue one another (the last word of
                                  * every row is never written and must stay zero). */
    /* Long delays.  NEST networks have a minimum delay, often far above one step (1-2 ms at a 0.001-0.1 ms
     * resolution).  With delay_offset = B every delay stored in the two tables is the true delay minus B steps
     * (still >= 1) and the spikes and input events of step u are handed to the tables B steps late, from the
     * history, so the ring only has to span the residual delays.  Results are identical to B = 0 with the true
     * delays.  In resident mode workgroups may then run up to min(B, hist_slots - 3 - B) steps apart before
     * one waits for another (at most 31) (what NEST's min_delay communication interval does between ranks). */
    int32_t delay_offset;        /* B >= 0 */
    int32_t hist_slots;          /* rows of work_bits, at least delay_offset + 3; 0 stands for 3.  One row more
                                  * lets the resident mode, also with delay_offset 0, look at its grid barrier
                                  * only when the spikes behind it are needed (after the next update) instead of
                                  * stopping at it every step. */
    int32_t delay_bits;          /* width of the delay field of rec_packed / inp_packed: 0 or 6 = the standard
                                  * packing; 7..14 = bmtk_csr_pack_wide tables (launch-per-step mode without the
                                  * pull form only), ring_slots may then reach 2^delay_bits */
    uint32_t res_spin_limit;     /* resident mode: polls of the grid barrier before a workgroup gives up and raises
                                  * the abort word (0 = the built-in limit, a few seconds) */
    /* Resident mode (optional, batch 1 only; res_span == 0 disables it): the
     * network is split into res_groups = ceil(ne/res_span) workgroups that keep
     * their elements' state in registers and their slice of the ring in LDS for
     * the whole run.  rec_seg / inp_seg are bmtk_csr_segment_offsets tables
     * built with the same span over tables whose rows are sorted by target;
     * rec_packed / inp_packed are those same tables packed. */
    /* A network of up to 1024 elements may be given to ONE workgroup (res_span = n rounded up to a multiple of 64,
     * res_groups = 1, the whole ring within LDS): the library then runs a form without grid barrier that hands the
     * spikes of a step over in LDS and walks whole rows of rec_packed / inp_packed through rec_indptr /
     * inp_indptr (rec_seg / inp_seg are not read); a step costs about a third. */
    int32_t res_span;            /* elements per workgroup: multiple of 64, at most 1024 */
    int32_t res_groups;
    const uint32_t *rec_seg;     /* [neurons][res_groups+1] */
    const uint32_t *inp_seg;     /* [inputs][res_groups+1] */
    uint32_t *res_sync;          /* BMTK_RES_SYNC_WORDS words of scratch, zeroed by the caller once: word 1 =
                                  * abort flag, from word BMTK_RES_SYNC_STRIDE on 64 x BMTK_RES_SYNC_WAYS arrival
                                  * counters that many words apart, which every call zeroes again.  Word 1 != 0
                                  * after a run means a grid barrier timed out and the results are invalid.  The
                                  * flag is sticky: no call clears it, and a call that finds it set does nothing,
                                  * so a failure cannot be overwritten before the host has seen it; the host
                                  * clears it after reading. */
    uint32_t *res_fired;         /* optional, several workgroups only: [hist_slots][res_groups][BMTK_RES_FIRED_SLOTS]
                                  * words (3 rows when hist_slots is 0), zeroed by the caller once and then left to
                                  * the library.  Beside its
                                  * ballots a workgroup publishes the neurons that fired in a step as a short list
                                  * (number + 1; 0 = free place; all places BMTK_RES_FIRED_MANY when the list does not
                                  * hold them), and the other workgroups read the lists instead of expanding the
                                  * ballots of the whole network, each for itself; steps in which some list did not
                                  * suffice are read from the ballots.  NULL: always from the ballots (a simulation passes it in
                                  * every call or in none: the lists of a call's last steps are read by the next).  Used by runs
                                  * without slack only (largest delay offset: the others do not wait per step). */
    /* Pull form of the recurrent delivery for batched runs (optional; launch-per-step mode with delay_offset 0
     * and hist_slots == ring_slots): a TARGET-major packed copy of the recurrent table.  The recurrent arrivals
     * of step t-1 are then summed in one pass over that table from the spike-bit history
     * (bmtk_csr_propagate_pull) before the launch of step t, instead of being pushed into the ring with global
     * atomics as the spikes occur.  Recurrent arrivals still ahead at the end of a call then live in the
     * history (work_bits), not in `ring`, which holds the input arrivals only. */
    const int32_t *pull_indptr;      /* [n_neurons + 1] */
    const bmtk_synapse *pull_packed; /* rows = targets, index field = source */
    float *pull_syn;                 /* [4][ne] scratch */
    void *pull_work;                 /* bmtk_csr_propagate_pull_workspace_bytes(ring_slots, n_neurons) bytes */
    /* The same for the external inputs (optional, only together with the above): a target-major packed copy of
     * the input table and a history of input-event bits, row t % ring_slots = the events of step t as bits of
     * element ids source*batch+trial; the driver fills the rows from in_ptr/in_events as it goes. */
    const int32_t *pull_inp_indptr;      /* [n_neurons + 1] */
    const bmtk_synapse *pull_inp_packed; /* rows = targets, index field = input source */
    float *pull_inp_syn;                 /* [4][ne] scratch */
    void *pull_inp_work;                 /* bmtk_csr_propagate_pull_workspace_bytes(ring_slots, n_inputs) bytes */
    uint64_t *in_hist;                   /* [ring_slots][in_hist_stride], zeroed before the first run */
    int64_t in_hist_stride;              /* >= ceil(n_inputs*batch/64) + 1 */
    /* With the pull form of the inputs only (ignored otherwise; both NULL when no id repeats within a step):
     * per-step lists, laid out like in_ptr / in_events, of the second and later occurrences of an id within a
     * step.  The bit rows deliver every id of a step once; these few are delivered on top as events, into the
     * ring. */
    const int64_t *in_repeat_ptr;        /* [total steps + 1] */
    const int32_t *in_repeat_events;
    /* Fused form of the batched driver (optional; launch-per-step mode, batch 8, 16, 32 or 64, delay_offset 0,
     * hist_slots == ring_slots + 4, `ring` of ring_slots + 2 slots; takes precedence over pull_*): one launch per TWO
     * steps in which a wavefront takes 64 / batch target neurons at a time -- in one pass over a joint target-major
     * table it sums what arrives at them in step t-1 and in step t over recurrent AND input synapses (64-bit fixed
     * point in LDS, as bmtk_csr_propagate_pull; both only depend on spikes up to step t-1, delays being at least one
     * step), folds the first sums into y1, advances the neurons' trials through step t, folds the second and
     * advances them through step t+1, lane = (neuron, trial); no arrival sum passes through device memory and the
     * table is read once per two steps.  The joint table's index field names a source of the joint space: neuron j is j,
     * input source k is fuse_in_base + k, fuse_in_base = ceil(n_neurons*batch/64)*64/batch.  work_bits is then the
     * joint history [hist_slots][fuse_hist_stride]: bit j*batch+b of row t % hist_slots = source j fired (or had an
     * input event) in trial b of step t; a launch writes the input parts of the rows of its own two steps from in_ptr /
     * in_events, for the launches after it.  Repeated ids of a step go through the ring as events (in_repeat_*, with inp_indptr /
     * inp_packed), as in the pull form.  fuse_any is the "some trial fired" map of the joint sources, one bit per
     * group of 2^fuse_shift sources and history row; a coarser map (larger shift) costs mask fetches for silent
     * sources but is what lets any number of sources fit the LDS: ring_slots * fuse_any_words * 4 bytes beside
     * the 80 KB of accumulators must stay within 150 KB. */
    const int32_t *fuse_indptr;        /* [n_neurons + 1] */
    const bmtk_synapse *fuse_packed;   /* rows = targets, index field = joint source */
    uint32_t *fuse_any;                /* [hist_slots][fuse_any_words] followed by [ring_slots + 2][ceil(n_neurons/32)]
                                        * words (a bit per neuron and ring slot: the slot holds an arrival of a
                                        * repeated id for the neuron), zeroed with work_bits before the first run;
                                        * fuse_any_words = ceil(ceil((fuse_in_base + n_inputs) / 2^fuse_shift) / 32) */
    int64_t fuse_hist_stride;          /* words per row of work_bits: >= fuse_in_base*batch/64 + ceil(n_inputs*batch/64) + 1 */
    int64_t fuse_in_base;
    int32_t fuse_shift;                /* 0..16 */
    int32_t fuse_wg_per_cu;            /* persistent workgroups per compute unit, 0 = the library's choice */
    /* outputs */
    uint64_t *spike_bits;        /* [n_steps][words] spike bits per step, words = ceil(ne/64); or NULL.
                                  * Row k belongs to step step0+k of the call that wrote it. */
    int64_t spike_bits_stride;   /* words per row (>= ceil(ne/64)) */
    /* optional per-step record for the backward pass (launch-per-step mode only; both or neither):
     * save_v[k][e] = membrane potential after step step0+k, save_flags[k][e] = BMTK_F_* bits */
    float *save_v;
    uint8_t *save_flags;
    /* optional membrane potential probes (both modes; what a NEST multimeter connected to some neurons records):
     * probe_col[e] = column of element e in probe_v, or -1.  After every step t with (t + 1) % probe_every == 0
     * the potentials U = V_m - E_L of the probed elements go to the next row of probe_v, row 0 being the first
     * such step of the call; probe_v must hold as many rows of probe_stride floats as the call has such steps. */
    const int32_t *probe_col;    /* [ne] or NULL */
    float *probe_v;
    int64_t probe_stride;
    int32_t probe_every;         /* >= 1 */
    int32_t _pad1;
    /* optional spike record with sub-step crossing fractions, appended with
     * atomics (unordered within a step); all NULL to disable */
    int32_t *spike_step;
    int32_t *spike_elem;
    float *spike_frac;
    int64_t spike_cap;
    unsigned long long *spike_count; /* device counter, keeps counting past spike_cap */
    /* The record in several lists.  Every wavefront with a spike takes its places in the list with one atomic
     * on the counter; at V1 scale that is 600 atomics on ONE address per step, which the memory side works off
     * one after the other (1.5 us of a 5.5 us step).  With spike_ways = W > 1 (a power of two up to 256;
     * spike_cap a multiple of W) the record is W lists of spike_cap / W entries each, list w in entries
     * [w * spike_cap / W, (w + 1) * spike_cap / W) of spike_step / spike_elem / spike_frac with its counter in
     * spike_count[w * BMTK_RECORD_COUNT_STRIDE]; a workgroup appends to list (its number mod W).  A counter keeps
     * counting past its list's end.  0 or 1: one list, as above.  With at least as many lists as workgroups (the
     * resident mode launches at most 256) and no delay offset, a workgroup has a list of its own and keeps the count
     * in a register for the length of a call: no atomics on device memory at all. */
    int32_t spike_ways;
    int32_t _pad2;
} bmtk_glif3_sim;

#define BMTK_RECORD_COUNT_STRIDE 16 /* 64-bit words between two counters of a record in several lists */

#define BMTK_F_SPIKE 1       /* the element spiked in this step */
#define BMTK_F_INTEGRATING 2 /* it was not refractory when the step began */
#define BMTK_F_RESET 4       /* it left refractoriness in this step (U and ASC were reset) */

/* Run steps step0 .. step0+n_steps-1.  One launch per step plus one closing
 * launch.  A launch updates every element for step t while, in other
 * workgroups of the same launch, the spikes of step t-1 are delivered through
 * the packed recurrent table and the input events of step t-1 through the
 * packed input table (fp32 atomics into the ring).  The two halves can overlap
 * because weights arriving in step t only enter y1 at the end of that step and
 * move no membrane potential before step t+1: the update of step t+1 folds the
 * arrivals of slot t into y1 first (same two roundings as adding them at the
 * end of step t), so slot t need only be complete when launch t+1 starts.  The
 * closing launch delivers the spikes and input events of the last step (with delay_offset = B: of
 * step last-B; the B younger steps stay in the history for a run that continues) and folds the last
 * slot, after which state and ring are what a step-by-step evaluation gives.
 * Enqueues n_steps+1 launches on `stream` and returns.
 *
 * With res_span > 0 the whole run is ONE cooperative launch instead: each
 * workgroup updates its elements from registers, publishes its spike ballots,
 * passes a grid barrier (one per step) and pulls, for every neuron that fired
 * anywhere in the previous step, its own segment of that neuron's synapses
 * into its LDS ring slice with LDS atomics -- no global atomics and no state
 * traffic.  The barrier spins a bounded number of times; see res_sync. */
int bmtk_glif3_simulate_fwd(const bmtk_glif3_sim *sim, int64_t step0, int64_t n_steps, void *stream);

/* Poisson spike sources generated on the device: the homogeneous case of bmtk's
 * PoissonSpikeGenerator._build_fixed_fr (bmtk/utils/reports/spike_trains/spike_trains.py:166-206) without
 * refractory thinning -- per element (source, trial), from t_start on, t += -ln(1 - U) / rate until t > t_stop,
 * every t a spike.  Every element has a random stream of its own (Philox4x32-10, keyed by `seed`), where the
 * reference draws all sources from NumPy's one global stream; the trains are therefore not the reference's
 * numbers but independent samples of the same process.  rate_hz holds one rate per source.  A spike at time t is
 * stamped ceil(t / dt) steps (at least 1) and emitted in step stamp - 1; spikes whose emitting step is n_steps
 * or later are left out.
 *   bmtk_poisson_count:  counts[e] = spikes of element e = source*batch + trial.
 *   bmtk_poisson_fill:   with offsets = the exclusive prefix sum of counts, keys[offsets[e] + k] =
 *                        step * (n_sources*batch) + e for the k-th spike of element e, and its time in ms in
 *                        times_ms (may be NULL).  Sorting the keys gives the per-step event lists (in_ptr,
 *                        in_events) of bmtk_glif3_sim, ascending within each step. */
int bmtk_poisson_count(int64_t n_sources, int32_t batch, const float *rate_hz, double t_start_ms, double t_stop_ms,
                       double dt_ms, int64_t n_steps, uint64_t seed, int32_t *counts, void *stream);
int bmtk_poisson_fill(int64_t n_sources, int32_t batch, const float *rate_hz, double t_start_ms, double t_stop_ms,
                      double dt_ms, int64_t n_steps, uint64_t seed, const int64_t *offsets, int64_t *keys,
                      double *times_ms, void *stream);

/* ---------------------------------------------------------------------------
 * Backward pass (reverse-time adjoint) of the forward simulation.
 *
 * bmtk and NEST have no gradient code: this part has no counterpart in the
 * reference; its definition is this library's own and is stated here.
 *  - The spike z = H(U' - th) gets the surrogate derivative
 *      dz/dU' = dampening * max(0, 1 - |(U' - th)/th|) / th      (th = V_th - E_L)
 *    in steps where the element was integrating; 0 otherwise.
 *  - Refractory bookkeeping is not differentiated: the hold U' = U passes the
 *    adjoint through, the reset U' = V_reset - E_L stops it, the after-spike
 *    reset ASC' = amp + r*ASC passes r.
 *  - Everything else is the exact transpose of the linear forward update.
 * The loss enters through dl_dz[k][e] (its derivative with respect to the spike
 * of element e in step step0+k), or through dl_dz_const[e] when it is the same
 * in every step (a loss on time-averaged rates).
 * Outputs: gradients with respect to every weight of the recurrent and input
 * tables, in packed-table order, accumulated (+=) into d_rec_w / d_inp_w.
 */
#define BMTK_BLOCKED_PAD 16
typedef struct bmtk_glif3_bwd {
    int64_t n_neurons;
    int32_t batch;
    int32_t ring_slots;
    float h;
    float dampening;
    const float *prop;
    int64_t prop_stride;
    const int32_t *class_id;
    /* forward record of the steps being differentiated, row k = step step0+k */
    const float *save_v;           /* [n_steps][ne] */
    const uint8_t *save_flags;     /* [n_steps][ne] */
    const uint64_t *spike_bits;    /* [n_steps][spike_bits_stride] */
    int64_t spike_bits_stride;
    /* the tables the forward run used (source-major, packed) */
    const int32_t *rec_indptr;
    const bmtk_synapse *rec_packed;
    const int64_t *in_ptr;         /* absolute step index, as in the forward run */
    const int32_t *in_events;
    const int32_t *inp_indptr;
    const bmtk_synapse *inp_packed;
    /* loss derivative: at most one of the two, the other NULL */
    const float *dl_dz;            /* [n_steps][ne] */
    const float *dl_dz_const;      /* [ne] */
    /* adjoint state, in/out (zero before the last step of the whole run) */
    float *lam_V, *lam_asc, *lam_y1, *lam_y2; /* [ne], [2][ne], [4][ne], [4][ne] */
    float *lam_ring;               /* [L][4][ne]: adjoint of the arrivals of the steps still ahead */
    float *gz;                     /* [ne] scratch; [8][ne] when the blocked table is given, [16][ne] with gz_planes 16 */
    /* outputs */
    float *d_rec_w;                /* [rec nnz] or NULL */
    float *d_inp_w;                /* [inp nnz] or NULL */
    /* Optional, for batches that are a multiple of 4 up to 64: the recurrent table regrouped by target range,
     * which the transposed propagation then uses instead of rec_indptr / rec_packed.  The targets are cut into
     * blk_count equal ranges (a multiple of 8; range s holds targets s*span .. (s+1)*span-1) small enough that a
     * range's part of lam_ring fits one L2 (a few MB), and the table is, range after range, a CSR over the
     * SOURCES of the synapses into that range: blk_indptr[s*n_neurons + j] .. [s*n_neurons + j + 1] delimit the
     * synapses source j sends into range s (one flat array of blk_count*n_neurons + 1 offsets), blk_packed holds
     * the records in that order FOLLOWED BY BMTK_BLOCKED_PAD more records of any content (the kernel reads up to
     * that many records past a row's end and ignores them).  Needs a lam_ring below 4 GB. */
    int32_t blk_count;             /* 0 = no blocked table */
    int32_t gz_planes;             /* planes of n_neurons*batch floats gz holds: 0 = 8.  With 16 or more and a batch above
                                      16 the blocked form takes TWO steps per pass over its table (a step's eight partial
                                      sums in planes 0-7, those of the step before it in planes 8-15) */
    const int32_t *blk_indptr;
    const bmtk_synapse *blk_packed;
    float *d_blk_w;                /* [rec nnz] recurrent weight gradient in the order of blk_packed, accumulated,
                                      or NULL (then d_rec_w, if given, is filled through rec_indptr / rec_packed) */
} bmtk_glif3_bwd;

/* Differentiate steps step0+n_steps-1 down to step0.  Per step: the transposed propagation (the weight gradients
 * ride in it where a wavefront holds whole adjoint rows), the state adjoint, and for batches above 64 a launch for
 * the recurrent weight gradient; with the blocked table, gz_planes >= 16 and a batch above 16, two launches per TWO
 * steps.  Whatever the form, lam_V .. lam_ring leave as a step-by-step evaluation would leave them. */
int bmtk_glif3_simulate_bwd(const bmtk_glif3_bwd *bwd, int64_t step0, int64_t n_steps, void *stream);

/* One backward step in its three parts, for callers that put their own work between them (a loss that is computed
 * step by step, truncation, clipping of the adjoint); no counterpart in the reference.  Both take the same struct
 * as bmtk_glif3_simulate_bwd and differentiate step step0 + k, whose forward record is row k.
 *  - bmtk_glif3_step_bwd: the state adjoint.  bwd->gz must hold the adjoint of the step's spikes that comes back
 *    through the synapses, as bmtk_csr_propagate_bwd (gz_parts = 1) or bmtk_csr_propagate_bwd_blocked (gz_parts =
 *    8 partial sums) leave it, or zeros; the loss derivative of the step is added to it.  Updates lam_V, lam_asc,
 *    lam_y1, lam_y2 and writes slot (step0 + k) % ring_slots of lam_ring.
 *  - bmtk_csr_weight_grad: d_rec_w += and d_inp_w += the step's contributions (whichever is given; d_blk_w is not
 *    served).  Reads the slots of the steps ahead only, so it may run before or after the state adjoint of the
 *    same step, but before that of step step0 + k - 1.
 * One step of bmtk_glif3_simulate_bwd == bmtk_csr_propagate_bwd, bmtk_glif3_step_bwd, bmtk_csr_weight_grad. */
int bmtk_glif3_step_bwd(const bmtk_glif3_bwd *bwd, int64_t step0, int64_t k, int32_t gz_parts, void *stream);
int bmtk_csr_weight_grad(const bmtk_glif3_bwd *bwd, int64_t step0, int64_t k, void *stream);

/* The transposed propagation of the backward pass on its own (the adjoint of the delivery; no counterpart in the
 * reference): through a packed SOURCE-major table of n_neurons rows,
 *   gz[j*batch+b] = sum over synapses (j -> i, w, d, r) of w * lam_ring[(step+d) % L][r][i*batch+b],
 * lam_ring being [L][4][n_neurons*batch].  It is the exact transpose of the event-driven delivery: for spikes z
 * emitted in `step`, <ring delivered from z, lam_ring> = <z, gz>.  One wavefront per source row; trials_per_lane
 * picks the kernel: 1 = lane = (synapse, trial), any batch; 4 = four trials per lane and 16-byte reads of the
 * adjoint rows, for batches that are a multiple of 4 up to 64; 0 = the one bmtk_glif3_simulate_bwd would take.
 * Every element counts (bmtk_glif3_simulate_bwd skips rows whose surrogate derivative is zero in all trials). */
int bmtk_csr_propagate_bwd(const int32_t *indptr, const bmtk_synapse *packed, int64_t n_neurons, int32_t batch,
                           const float *lam_ring, int32_t L, int64_t step, float *gz, int32_t trials_per_lane,
                           void *stream);

/* The same sums through the blocked form of the table (bmtk_glif3_bwd: blk_count, blk_indptr, blk_packed), as
 * eight partial sums gz_parts[8][n_neurons*batch] whose sum over the first index is gz.  Batches that are a
 * multiple of 4 up to 64; every element counts. */
int bmtk_csr_propagate_bwd_blocked(const int32_t *blk_indptr, const bmtk_synapse *blk_packed, int32_t blk_count,
                                   int64_t n_neurons, int32_t batch, const float *lam_ring, int32_t L, int64_t step,
                                   float *gz_parts, void *stream);

/* The launch geometry the blocked form takes for a network on the current device, for callers and tests that want
 * to know which of its paths a size exercises: plan_host[0] = workgroups (one per compute unit, workgroup b on XCD
 * b mod 8), [1] = source rows per workgroup, [2] = sweeps over them (a sweep holds at most 16 wavefronts x 8 row
 * groups x 64*4/batch rows in LDS), [3] = row groups per wavefront and sweep.  plan_host is a HOST pointer to four
 * int32. */
int bmtk_csr_propagate_bwd_blocked_plan(int64_t n_neurons, int32_t batch, int32_t *plan_host);

/* Number of spikes of every element over n_steps rows of spike bits: counts[e] (int32). */
int bmtk_spike_counts(const uint64_t *spike_bits, int64_t stride, int64_t n_steps, int64_t ne, int32_t *counts,
                      void *stream);

/* ---------------------------------------------------------------------------
 * Three measurements the kernels' design rests on, kept in the library so that they can be repeated
 * (bench.py --kernels lds).  No counterpart in the reference.
 *
 * bmtk_microbench_lds: n_blocks workgroups of 1024 threads; in each of `rounds` rounds, `active_lanes` lanes of every
 * wavefront add to a pseudo-random cell of a 92,160-byte LDS array.  op 0: float atomic (ds_add_f32), 1: 32-bit
 * integer atomic, 2: 64-bit integer atomic, 3: float add by a compare-and-swap loop, 4: plain store.  out: n_blocks *
 * 1024 floats (checksums).  The caller times the launch; time * clock / (16 * rounds) = clocks per wavefront
 * instruction on a compute unit.
 * bmtk_microbench_hop: workgroups block_a and block_b (0..15; workgroups go round the XCDs, so 0 and 8 share one, 0
 * and 1 do not) pass a counter back and forth `rounds` times through two words of `flags` (at least 512 bytes,
 * zeroed by the caller) with relaxed agent-scope loads and stores; time / rounds = two hops.  xcc (3 words, zeroed
 * by the caller): the XCD each ran on, and 1 in xcc[2] if a wait ran out after spin_limit polls (both then leave).
 * bmtk_microbench_atomics: n_blocks workgroups of 256 threads; every thread adds 1 to per_thread pseudo-random cells
 * of `cells` (n_cells floats, zeroed by the caller) with the global fp32 atomic; own_eighth != 0: a workgroup only adds
 * into the eighth of the region that belongs to the XCD it runs on.  The caller times the launch; the cells then sum
 * to n_blocks * 256 * per_thread. */
int bmtk_microbench_atomics(float *cells, int64_t n_cells, int32_t per_thread, int32_t n_blocks, int32_t own_eighth,
                            void *stream);
int bmtk_microbench_lds(int32_t op, int32_t active_lanes, int32_t rounds, int32_t n_blocks, float *out, void *stream);
int bmtk_microbench_hop(uint32_t *flags, uint32_t *xcc, int32_t block_a, int32_t block_b, int32_t rounds,
                        uint32_t spin_limit, void *stream);

#ifdef __cplusplus
}
#endif
#endif

