"""Row indices of the parameter and propagator tables (mirror of
``include/bmtk_amd_layout.h``; ``tests/test_layout.py`` checks the two agree)."""

NASC = 2
NREC = 4

PARAM_ROWS = (
    "C_M", "G", "E_L", "V_TH", "V_RESET", "T_REF",
    "ASC_DECAY0", "ASC_DECAY1", "ASC_AMPS0", "ASC_AMPS1", "ASC_R0", "ASC_R1",
    "TAU_SYN0", "TAU_SYN1", "TAU_SYN2", "TAU_SYN3",
)
PROP_ROWS = (
    "P33", "P30", "TH", "UR", "NREF",
    "C0", "C1", "D0", "D1", "R0", "R1", "AMP0", "AMP1",
    "P11_0", "P11_1", "P11_2", "P11_3",
    "P31_0", "P31_1", "P31_2", "P31_3",
    "P32_0", "P32_1", "P32_2", "P32_3",
    "PSC0_0", "PSC0_1", "PSC0_2", "PSC0_3",
)
PAR = {name: i for i, name in enumerate(PARAM_ROWS)}
PROP = {name: i for i, name in enumerate(PROP_ROWS)}
NPARAM = len(PARAM_ROWS)
NPROP = len(PROP_ROWS)
