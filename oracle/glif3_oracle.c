/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the GLIF3 point-neuron hot path
 * (see glif3_oracle_impl.h for what it restates and the time convention).
 * Built by oracle/Makefile into oracle/libglif3_oracle.so; loaded by
 * oracle/glif3_oracle.py.  Never linked into the shipped library.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <omp.h>

#include "../include/bmtk_amd_layout.h"

void oracle_set_threads(int n) { omp_set_num_threads(n); }
int oracle_max_threads(void) { return omp_get_max_threads(); }

/* NEST libnestutil/propagator_stability.cpp: exact propagator entries of the
 * (y1, y2, U) linear system with the numerically stable fallback to the
 * tau == tau_syn limit.  The fallback criterion is restated from memory of the
 * NEST 3.3 source and is not pinned by any reference vector.  */
static double propagator_32(double tau_syn, double tau, double C, double h)
{
    const double P32_linear = 1.0 / (2.0 * C * tau * tau) * h * h * (tau_syn - tau) * exp(-h / tau);
    const double P32_singular = h / C * exp(-h / tau);
    const double P32 = -tau / (C * (1.0 - tau / tau_syn)) * exp(-h / tau_syn) * expm1(h * (1.0 / tau_syn - 1.0 / tau));
    const double dev = fabs(P32 - P32_singular);
    if (tau == tau_syn || (fabs(tau - tau_syn) < 0.1 && dev > 2.0 * fabs(P32_linear)))
        return P32_singular;
    return P32;
}

static double propagator_31(double tau_syn, double tau, double C, double h)
{
    const double P31_linear = 1.0 / (3.0 * C * tau * tau) * h * h * h * (tau_syn - tau) * exp(-h / tau);
    const double P31 = 1.0 / C * (exp(-h / tau_syn) * expm1(-h / tau + h / tau_syn) / (tau / tau_syn - 1.0) * tau
                                  - h * exp(-h / tau_syn)) / (-1.0 - -tau / tau_syn) * tau;
    const double P31_singular = h * h / 2.0 / C * exp(-h / tau);
    const double dev = fabs(P31 - P31_singular);
    if (tau == tau_syn || (fabs(tau - tau_syn) < 0.1 && dev > 2.0 * fabs(P31_linear)))
        return P31_singular;
    return P31;
}

/* NEST glif_psc::pre_run_hook.  par: [GLIF3_NPARAM][n] in NEST units (the
 * dictionary bmtk passes to nest.Create, bmtk/simulator/pointnet/glif_utils.py:301-320),
 * prop: [GLIF3_NPROP][n].  n_ref is the number of refractory steps NEST's
 * floating-point count-down (t_ref_remaining -= h until <= 0) takes.  */
void glif3_precompute_f64(int64_t n, const double *par, double h, double *prop)
{
#define PA(k) par[(int64_t)(k) * n + i]
#define PO(k) prop[(int64_t)(k) * n + i]
    for (int64_t i = 0; i < n; ++i) {
        const double C = PA(GLIF3_PAR_C_M), g = PA(GLIF3_PAR_G);
        const double tau = C / g;
        const double P33 = exp(-h / tau);
        PO(GLIF3_P33) = P33;
        PO(GLIF3_P30) = 1.0 / C * (1.0 - P33) * tau;
        PO(GLIF3_TH) = PA(GLIF3_PAR_V_TH) - PA(GLIF3_PAR_E_L);
        PO(GLIF3_UR) = PA(GLIF3_PAR_V_RESET) - PA(GLIF3_PAR_E_L);
        double rem = PA(GLIF3_PAR_T_REF);
        int64_t nref = 0;
        while (rem > 0.0) { rem -= h; ++nref; }
        PO(GLIF3_NREF) = (double)nref;
        for (int a = 0; a < GLIF3_NASC; ++a) {
            const double k = PA(GLIF3_PAR_ASC_DECAY0 + a);
            const double d = exp(-k * h);
            PO(GLIF3_D0 + a) = d;
            PO(GLIF3_C0 + a) = ((1.0 / k) / h) * (1.0 - d);
            PO(GLIF3_R0 + a) = PA(GLIF3_PAR_ASC_R0 + a) * exp(-k * PA(GLIF3_PAR_T_REF));
            PO(GLIF3_AMP0 + a) = PA(GLIF3_PAR_ASC_AMPS0 + a);
        }
        for (int r = 0; r < GLIF3_NREC; ++r) {
            const double ts = PA(GLIF3_PAR_TAU_SYN0 + r);
            PO(GLIF3_P11_0 + r) = exp(-h / ts);
            PO(GLIF3_P31_0 + r) = propagator_31(ts, tau, C, h);
            PO(GLIF3_P32_0 + r) = propagator_32(ts, tau, C, h);
            PO(GLIF3_PSC0_0 + r) = 1.0 * M_E / ts;
        }
    }
#undef PA
#undef PO
}

#define REAL double
#define SUFFIX _f64
#include "glif3_oracle_impl.h"
#undef REAL
#undef SUFFIX

#define REAL float
#define SUFFIX _f32
#include "glif3_oracle_impl.h"
#undef REAL
#undef SUFFIX
