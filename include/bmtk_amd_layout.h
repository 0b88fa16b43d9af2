/*
 * Row indices of the two parameter tables the GLIF3 path exchanges.
 * Plain C, no dependencies; shared by the library, its Python host code
 * (mirrored in bmtk_amd/layout.py) and the test oracle.
 */
#ifndef BMTK_AMD_LAYOUT_H
#define BMTK_AMD_LAYOUT_H

#define GLIF3_NASC 2 /* after-spike currents per neuron */
#define GLIF3_NREC 4 /* alpha-PSC receptor ports per neuron */

/* NEST-unit parameter table par[GLIF3_NPARAM][n] (fp64): the glif_psc
 * dictionary bmtk builds in bmtk/simulator/pointnet/glif_utils.py:301-320
 * or reads from examples/point_components/cell_models/ (files <id>_glif_lif_asc_psc.json). */
enum {
    GLIF3_PAR_C_M = 0,    /* pF */
    GLIF3_PAR_G,          /* nS */
    GLIF3_PAR_E_L,        /* mV */
    GLIF3_PAR_V_TH,       /* mV */
    GLIF3_PAR_V_RESET,    /* mV */
    GLIF3_PAR_T_REF,      /* ms */
    GLIF3_PAR_ASC_DECAY0, /* 1/ms */
    GLIF3_PAR_ASC_DECAY1,
    GLIF3_PAR_ASC_AMPS0,  /* pA */
    GLIF3_PAR_ASC_AMPS1,
    GLIF3_PAR_ASC_R0,     /* NEST asc_r, 1.0 unless given */
    GLIF3_PAR_ASC_R1,
    GLIF3_PAR_TAU_SYN0,   /* ms */
    GLIF3_PAR_TAU_SYN1,
    GLIF3_PAR_TAU_SYN2,
    GLIF3_PAR_TAU_SYN3,
    GLIF3_NPARAM
};

/* Per-step propagator table prop[GLIF3_NPROP][stride] (fp32 on the GPU):
 * what NEST's glif_psc::pre_run_hook derives from the parameters and the
 * resolution h.  U is the membrane potential relative to E_L. */
enum {
    GLIF3_P33 = 0, /* exp(-h/tau_m) */
    GLIF3_P30,     /* (1-P33)*tau_m/C_m */
    GLIF3_TH,      /* V_th - E_L */
    GLIF3_UR,      /* V_reset - E_L */
    GLIF3_NREF,    /* refractory steps, integer valued */
    GLIF3_C0,      /* ASC step-mean coefficient (1/k)/h*(1-exp(-k h)) */
    GLIF3_C1,
    GLIF3_D0,      /* ASC decay exp(-k h) */
    GLIF3_D1,
    GLIF3_R0,      /* asc_r*exp(-k t_ref) */
    GLIF3_R1,
    GLIF3_AMP0,    /* asc_amps */
    GLIF3_AMP1,
    GLIF3_P11_0,   /* exp(-h/tau_syn_r), r = 0..3 */
    GLIF3_P11_1, GLIF3_P11_2, GLIF3_P11_3,
    GLIF3_P31_0,   /* y1 -> U */
    GLIF3_P31_1, GLIF3_P31_2, GLIF3_P31_3,
    GLIF3_P32_0,   /* y2 -> U */
    GLIF3_P32_1, GLIF3_P32_2, GLIF3_P32_3,
    GLIF3_PSC0_0,  /* e/tau_syn_r */
    GLIF3_PSC0_1, GLIF3_PSC0_2, GLIF3_PSC0_3,
    GLIF3_NPROP
};

#endif
