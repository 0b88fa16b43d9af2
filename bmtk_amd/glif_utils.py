"""Allen-Institute GLIF parameter files -> NEST ``glif_psc`` dictionaries, and
those dictionaries -> the fp64 parameter table the GPU path consumes.

Host-side counterpart of ``convert_aibs2nest`` / ``converter_builtin`` in
bmtk/simulator/pointnet/glif_utils.py:259-320.  Only the two model variants the
GPU path implements are converted (LIF and LIF with after-spike currents, both
with alpha-shaped post-synaptic currents); the reset-rule and adaptive-threshold
variants raise ``NotImplementedError``.
"""
import numpy as np

from .layout import NPARAM, PAR

TAU_SYN_DEFAULT = (5.5, 8.5, 2.8, 5.8)  # ms, receptor ports 1..4

_SUPPORTED = {"nest:glif_lif_psc": False, "nest:glif_lif_asc_psc": True}
_UNSUPPORTED = ("nest:glif_lif_r_psc", "nest:glif_lif_r_asc_psc", "nest:glif_lif_r_asc_a_psc")


def _common(cfg):
    k = cfg["coeffs"]
    e_ref_mv = cfg["El_reference"] * 1.0e3
    e_l = cfg["El"] * 1.0e3 + e_ref_mv
    return {
        "V_m": e_l,
        "V_th": k["th_inf"] * cfg["th_inf"] * 1.0e3 + e_ref_mv,
        "g": k["G"] / cfg["R_input"] * 1.0e9,
        "E_L": e_l,
        "C_m": k["C"] * cfg["C"] * 1.0e12,
        "t_ref": cfg["spike_cut_length"] * cfg["dt"] * 1.0e3,
        "V_reset": e_ref_mv,
        "tau_syn": np.array(TAU_SYN_DEFAULT),
        "spike_dependent_threshold": False,
        "adapting_threshold": False,
    }


def converter_builtin(model_template, dynamics_params):
    """SI-unit Allen cell-types GLIF config -> ('nest:glif_psc', NEST-unit dict).
    Units: mV, nS, pF, ms, pA, 1/ms (bmtk/simulator/pointnet/glif_utils.py:262-320)."""
    if model_template in _UNSUPPORTED:
        raise NotImplementedError(
            "{}: reset-rule / adaptive-threshold GLIF variants are not implemented on the GPU path".format(
                model_template))
    if model_template not in _SUPPORTED:
        return model_template, dynamics_params
    cfg = dynamics_params
    out = _common(cfg)
    with_asc = _SUPPORTED[model_template]
    out["after_spike_currents"] = with_asc
    if with_asc:
        out["asc_init"] = np.array(cfg["init_AScurrents"]) * 1.0e12
        out["asc_decay"] = 1.0 / np.array(cfg["asc_tau_array"]) * 1.0e-3
        out["asc_amps"] = np.array(cfg["asc_amp_array"]) * np.array(cfg["coeffs"]["asc_amp_array"]) * 1.0e12
    return "nest:glif_psc", out


def convert_aibs2nest(model_template, dynamics_params):
    """Entry point bmtk calls when ``model_template`` starts with ``nest:glif``
    and ``dynamics_params['type'] == 'GLIF'``
    (bmtk/simulator/pointnet/sonata_adaptors.py:158-167)."""
    return converter_builtin(model_template, dynamics_params)


def check_glif_psc_params(p):
    """Reject glif_psc dictionaries the GLIF3 kernels do not cover, and the
    values NEST itself rejects."""
    if p.get("spike_dependent_threshold", False) or p.get("adapting_threshold", False):
        raise NotImplementedError("glif_psc with spike_dependent_threshold/adapting_threshold is not implemented")
    if p["C_m"] <= 0 or p["g"] <= 0:
        raise ValueError("C_m and g must be strictly positive")
    if p["t_ref"] <= 0:
        raise ValueError("Refractory time constant must be strictly positive")
    if p["V_reset"] >= p["V_th"]:
        raise ValueError("Reset potential must be smaller than threshold")
    tau_syn = np.atleast_1d(p.get("tau_syn", TAU_SYN_DEFAULT))
    if tau_syn.size > 4 or np.any(tau_syn <= 0):
        raise ValueError("tau_syn must hold at most 4 strictly positive time constants")
    if p.get("after_spike_currents", True) and np.any(np.asarray(p.get("asc_decay", (1.0, 1.0))) <= 0):
        raise ValueError("asc_decay must be strictly positive")


def params_table(cells):
    """List of NEST-unit ``glif_psc`` dicts -> (par[NPARAM][n], asc_init[2][n], u_init[n]) fp64.

    A dict without after-spike currents becomes a GLIF3 cell whose ASC
    amplitudes and initial values are zero (so the ASC terms vanish exactly).
    ``u_init`` is V_m - E_L, the membrane potential relative to rest.
    """
    n = len(cells)
    par = np.zeros((NPARAM, n), np.float64)
    asc_init = np.zeros((2, n), np.float64)
    u_init = np.zeros(n, np.float64)
    for i, p in enumerate(cells):
        check_glif_psc_params(p)
        par[PAR["C_M"], i] = p["C_m"]
        par[PAR["G"], i] = p["g"]
        par[PAR["E_L"], i] = p["E_L"]
        par[PAR["V_TH"], i] = p["V_th"]
        par[PAR["V_RESET"], i] = p["V_reset"]
        par[PAR["T_REF"], i] = p["t_ref"]
        has_asc = p.get("after_spike_currents", True)
        par[PAR["ASC_DECAY0"]:PAR["ASC_DECAY0"] + 2, i] = p.get("asc_decay", (1.0, 1.0)) if has_asc else (1.0, 1.0)
        par[PAR["ASC_AMPS0"]:PAR["ASC_AMPS0"] + 2, i] = p.get("asc_amps", (0.0, 0.0)) if has_asc else (0.0, 0.0)
        par[PAR["ASC_R0"]:PAR["ASC_R0"] + 2, i] = p.get("asc_r", (1.0, 1.0))
        ts = np.atleast_1d(np.asarray(p.get("tau_syn", TAU_SYN_DEFAULT), np.float64))
        par[PAR["TAU_SYN0"]:PAR["TAU_SYN0"] + 4, i] = np.concatenate([ts, np.full(4 - ts.size, 2.0)])
        if has_asc:
            asc_init[:, i] = p.get("asc_init", (0.0, 0.0))
        u_init[i] = p.get("V_m", p["E_L"]) - p["E_L"]
    return par, asc_init, u_init
