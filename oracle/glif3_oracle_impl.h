/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the GLIF3 point-neuron hot path.
 *
 * This file is included twice by glif3_oracle.c, once with REAL=double
 * (suffix _f64, the truth the tolerances are measured against) and once with
 * REAL=float (suffix _f32, same operation order as the HIP kernels so that
 * deterministic kernels can be compared bit for bit).  Nothing in the shipped
 * package may call it; only tests, the smoke check and the CPU leg of the
 * benchmark do.
 *
 * What it restates.  bmtk drives NEST through PyNEST and NEST does all the
 * per-step arithmetic:
 *   - nest.Create('glif_psc', n, params)   bmtk/simulator/pointnet/sonata_adaptors.py:64-66
 *   - nest.Connect(.., 'one_to_one', {'weight','delay','receptor_type'})
 *                                          bmtk/simulator/pointnet/pointnetwork.py:161-173,229-232
 *   - nest.Simulate(tstop)                 bmtk/simulator/pointnet/pointsimulator.py:159-166
 * NEST (nest-simulator, pinned =3.3 in docker/environment.yml:15) is not part
 * of the reference tree, so the functions below restate its published
 * algorithm: models/glif_psc.cpp (update), libnestutil/propagator_stability.cpp
 * (P31/P32), models/static_synapse.h + nestkernel/ring_buffer.h (delivery).
 *
 * Time convention (NEST's, confirmed by the reference known-answer test, see
 * tests/test_oracle_kat.py): step k advances time from k*h to (k+1)*h.  A spike
 * detected in step k is stamped (k+1)*h.  A spike with stamp s (in steps) sent
 * through a synapse with delay d (in steps, d >= 1) is added to the target's
 * y1 at the END of step s+d-1, so it first moves the target's membrane
 * potential in step s+d.  A neuron spike emitted in step k therefore lands in
 * ring slot (k+d) mod L and is consumed by the update of step k+d.
 */

#ifndef REAL
#error "include from glif3_oracle.c"
#endif

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUFFIX)

/* One GLIF3 (glif_psc with after_spike_currents only) step for every
 * (neuron, trial) element.  Element index e = n*batch + b.
 *
 * prop: [GLIF3_NPROP][prop_stride] table, row = quantity, column = neuron
 *       (class_id == NULL) or parameter class (class_id[n]).
 * syn : [GLIF3_NREC][n*batch] weight sums arriving in this step (may be NULL).
 * i_ext: [n*batch] external current S_.I_ used in this step (may be NULL).
 * z   : [n*batch] spike flag out (may be NULL).
 * frac: [n*batch] fraction of the step at which U crossed threshold by linear
 *       interpolation, NEST's spike offset is (1-frac)*h; only written where z=1.
 *
 * Follows NEST glif_psc::update for has_asc_=true, has_theta_spike_=false,
 * has_theta_voltage_=false, which is how bmtk instantiates
 * nest:glif_lif_asc_psc (bmtk/simulator/pointnet/glif_utils.py:301-320).
 */
void FN(glif3_step)(int64_t n_neurons, int32_t batch,
                    REAL *V, REAL *asc, REAL *y1, REAL *y2, int32_t *ref,
                    const REAL *prop, int64_t prop_stride, const int32_t *class_id,
                    REAL h, const REAL *syn, const REAL *i_ext,
                    uint8_t *z, REAL *frac)
{
    const int64_t ne = n_neurons * (int64_t)batch;
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < n_neurons; ++n) {
        const int64_t col = class_id ? (int64_t)class_id[n] : n;
#define PR(k) prop[(int64_t)(k) * prop_stride + col]
        const REAL P33 = PR(GLIF3_P33), P30 = PR(GLIF3_P30), th = PR(GLIF3_TH), Ur = PR(GLIF3_UR);
        const int32_t n_ref = (int32_t)PR(GLIF3_NREF);
        for (int32_t b = 0; b < batch; ++b) {
            const int64_t e = n * batch + b;
            const REAL v_old = V[e];
            REAL U = v_old;
            uint8_t spk = 0;
            if (ref[e] > 0) {
                /* refractory: hold U at its last value; on leaving, reset U and ASC */
                ref[e] -= 1;
                if (ref[e] == 0) {
                    for (int a = 0; a < GLIF3_NASC; ++a)
                        asc[a * ne + e] = PR(GLIF3_AMP0 + a) + asc[a * ne + e] * PR(GLIF3_R0 + a);
                    U = Ur;
                }
            } else {
                REAL S = (REAL)0;
                for (int a = 0; a < GLIF3_NASC; ++a) {
                    S = S + PR(GLIF3_C0 + a) * asc[a * ne + e];
                    asc[a * ne + e] = asc[a * ne + e] * PR(GLIF3_D0 + a);
                }
                const REAL I = i_ext ? i_ext[e] : (REAL)0;
                U = v_old * P33 + (I + S) * P30;
                for (int r = 0; r < GLIF3_NREC; ++r)
                    U = U + (PR(GLIF3_P31_0 + r) * y1[r * ne + e] + PR(GLIF3_P32_0 + r) * y2[r * ne + e]);
                if (U > th) {
                    spk = 1;
                    ref[e] = n_ref;
                    if (frac) frac[e] = (th - v_old) / (U - v_old);
                }
            }
            V[e] = U;
            if (z) z[e] = spk;
            /* alpha-shaped PSCs advance every step, refractory or not */
            for (int r = 0; r < GLIF3_NREC; ++r) {
                const REAL P11 = PR(GLIF3_P11_0 + r);
                const REAL P21 = h * P11;
                const REAL a1 = y1[r * ne + e], a2 = y2[r * ne + e];
                y2[r * ne + e] = P21 * a1 + P11 * a2;
                REAL n1 = a1 * P11;
                if (syn) n1 = n1 + syn[r * ne + e] * PR(GLIF3_PSC0_0 + r);
                y1[r * ne + e] = n1;
            }
        }
#undef PR
    }
}

/* Event-driven delivery in NEST's form: walk the out-going synapse list of
 * every active (source, trial) element and add the weight into the target's
 * per-receptor ring buffer (static_synapse::send -> glif_psc::handle ->
 * RingBuffer::add_value).  Source-major CSR: indptr[n_src+1], indices = target
 * neuron, delays in steps (>=1), receptors 0-based.
 * ring: [L][GLIF3_NREC][n_tgt*batch].  Spikes emitted in step `step`.
 */
void FN(csr_deliver_events)(int64_t n_active, const int32_t *active_e, int32_t batch,
                            const int32_t *indptr, const int32_t *indices, const float *weights,
                            const int32_t *delays, const uint8_t *receptors,
                            REAL *ring, int32_t L, int64_t n_tgt, int64_t step)
{
    const int64_t ne = n_tgt * (int64_t)batch;
    if (omp_get_max_threads() == 1) {
        /* serial: additions happen in (active list, synapse) order */
        for (int64_t k = 0; k < n_active; ++k) {
            const int32_t j = active_e[k] / batch, b = active_e[k] % batch;
            for (int32_t p = indptr[j]; p < indptr[j + 1]; ++p) {
                const int64_t slot = (step + delays[p]) % L;
                ring[(slot * GLIF3_NREC + receptors[p]) * ne + (int64_t)indices[p] * batch + b] += (REAL)weights[p];
            }
        }
        return;
    }
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t k = 0; k < n_active; ++k) {
        const int32_t j = active_e[k] / batch, b = active_e[k] % batch;
        for (int32_t p = indptr[j]; p < indptr[j + 1]; ++p) {
            const int64_t slot = (step + delays[p]) % L;
            REAL *cell = ring + (slot * GLIF3_NREC + receptors[p]) * ne + (int64_t)indices[p] * batch + b;
#pragma omp atomic
            *cell += (REAL)weights[p];
        }
    }
}

/* The same sums taken row by row over a target-major CSR (indices = source
 * neuron), reading the spike flags of one emission step.  z: [n_src*batch].
 * Adds in stored synapse order, which is the order the deterministic HIP
 * gather kernel uses.
 */
void FN(csr_gather_rows)(int64_t n_tgt, int32_t batch, const uint8_t *z,
                         const int32_t *indptr, const int32_t *indices, const float *weights,
                         const int32_t *delays, const uint8_t *receptors,
                         REAL *ring, int32_t L, int64_t step)
{
    const int64_t ne = n_tgt * (int64_t)batch;
#pragma omp parallel for schedule(dynamic, 64)
    for (int64_t i = 0; i < n_tgt; ++i) {
        for (int32_t p = indptr[i]; p < indptr[i + 1]; ++p) {
            const int64_t slot = (step + delays[p]) % L;
            REAL *cell = ring + (slot * GLIF3_NREC + receptors[p]) * ne + i * batch;
            const uint8_t *zj = z + (int64_t)indices[p] * batch;
            for (int32_t b = 0; b < batch; ++b)
                if (zj[b]) cell[b] += (REAL)weights[p];
        }
    }
}

/* Whole forward simulation, NEST-algorithm form.  Per step: update every
 * neuron from ring slot step%L (then clear it), deliver the spikes of the
 * step through the recurrent source-major CSR, deliver the external input
 * spikes emitted in this step through the input CSR.
 *
 * in_ptr[T+1], in_events: element ids j*batch+b of input sources emitting in
 * each step (stamp = step+1), ascending within a step.
 * i_ext: [n*batch] constant external current or NULL.
 * spk_step/spk_elem/spk_frac: spike record (capacity spk_cap), ascending
 * (step, element).  Returns the number of spikes (may exceed spk_cap; excess
 * is not stored).
 */
int64_t FN(glif3_simulate)(int64_t n_neurons, int32_t batch, int64_t n_steps, int64_t step0,
                           REAL *V, REAL *asc, REAL *y1, REAL *y2, int32_t *ref,
                           const REAL *prop, int64_t prop_stride, const int32_t *class_id, REAL h,
                           REAL *ring, int32_t L,
                           const int32_t *r_indptr, const int32_t *r_indices, const float *r_weights,
                           const int32_t *r_delays, const uint8_t *r_receptors,
                           const int64_t *in_ptr, const int32_t *in_events,
                           const int32_t *i_indptr, const int32_t *i_indices, const float *i_weights,
                           const int32_t *i_delays, const uint8_t *i_receptors,
                           const REAL *i_ext,
                           int32_t *spk_step, int32_t *spk_elem, REAL *spk_frac, int64_t spk_cap,
                           uint8_t *raster)
{
    const int64_t ne = n_neurons * (int64_t)batch;
    uint8_t *z = (uint8_t *)malloc((size_t)ne);
    REAL *fr = (REAL *)malloc((size_t)ne * sizeof(REAL));
    REAL *syn = (REAL *)malloc((size_t)ne * GLIF3_NREC * sizeof(REAL));
    int32_t *act = (int32_t *)malloc((size_t)ne * sizeof(int32_t));
    int64_t n_spk = 0;
    for (int64_t t = step0; t < step0 + n_steps; ++t) {
        const int64_t slot = t % L;
        REAL *cur = ring + slot * GLIF3_NREC * ne;
        memcpy(syn, cur, (size_t)ne * GLIF3_NREC * sizeof(REAL));
        memset(cur, 0, (size_t)ne * GLIF3_NREC * sizeof(REAL));
        FN(glif3_step)(n_neurons, batch, V, asc, y1, y2, ref, prop, prop_stride, class_id, h,
                       syn, i_ext, z, fr);
        int64_t na = 0;
        for (int64_t e = 0; e < ne; ++e)
            if (z[e]) {
                act[na++] = (int32_t)e;
                if (n_spk < spk_cap) {
                    if (spk_step) spk_step[n_spk] = (int32_t)t;
                    if (spk_elem) spk_elem[n_spk] = (int32_t)e;
                    if (spk_frac) spk_frac[n_spk] = fr[e];
                }
                ++n_spk;
            }
        if (raster) memcpy(raster + (t - step0) * ne, z, (size_t)ne);
        if (r_indptr)
            FN(csr_deliver_events)(na, act, batch, r_indptr, r_indices, r_weights, r_delays, r_receptors,
                                   ring, L, n_neurons, t);
        if (in_ptr && i_indptr)
            FN(csr_deliver_events)(in_ptr[t + 1] - in_ptr[t], in_events + in_ptr[t], batch,
                                   i_indptr, i_indices, i_weights, i_delays, i_receptors,
                                   ring, L, n_neurons, t);
    }
    free(z); free(fr); free(syn); free(act);
    return n_spk;
}

#undef FN
#undef CAT
#undef CAT_
