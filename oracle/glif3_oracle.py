"""TEST INFRASTRUCTURE ONLY -- Python face of the CPU oracle.

Loads ``oracle/libglif3_oracle.so`` (built from ``glif3_oracle.c`` by
``oracle/Makefile``) and wraps its functions for numpy arrays.  The shipped
package never imports this module; tests, the smoke check and the CPU leg of
the benchmark do.

The C functions restate NEST's ``glif_psc`` update, ``static_synapse``
delivery and ring buffer as bmtk drives them
(bmtk/simulator/pointnet/sonata_adaptors.py:64-66,
bmtk/simulator/pointnet/pointnetwork.py:161-173,229-232,
bmtk/simulator/pointnet/pointsimulator.py:159-166); see ``glif3_oracle_impl.h``.

Pinned by: the reference's GLIF known-answer spike times (GLIF3 14.46548367 ms
and GLIF1 14.77547828 ms, bmtk/tests/simulator/pointnet/test_glif_utils.py:16-21)
reproduced to 1e-6 ms; ``scipy.linalg.expm`` for every propagator entry; the
closed-form alpha-PSC peak; a dense-matrix brute force for delivery.
Parity unpinned: the tau_m ~ tau_syn singular-propagator fallback threshold
(restated from memory of NEST 3.3, no reference vector exercises it).
"""
import ctypes as C
import os
import re
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libglif3_oracle.so")
_lib = None


def build(force=False):
    """Compile the oracle with gcc (a few seconds)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])


def _layout():
    txt = open(os.path.join(_HERE, "..", "include", "bmtk_amd_layout.h")).read()
    out = {}
    for body in re.findall(r"enum\s*\{(.*?)\};", txt, flags=re.S):
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        k = 0
        for tok in body.split(","):
            tok = tok.strip()
            if not tok:
                continue
            if "=" in tok:
                name, val = [s.strip() for s in tok.split("=")]
                k = int(val)
            else:
                name = tok
            out[name] = k
            k += 1
    return out


L = _layout()
NPROP, NPARAM, NASC, NREC = L["GLIF3_NPROP"], L["GLIF3_NPARAM"], 2, 4

_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.glif3_precompute_f64.argtypes = [C.c_int64, _f64p, C.c_double, _f64p]
        _lib.glif3_simulate_f64.restype = C.c_int64
        _lib.glif3_simulate_f32.restype = C.c_int64
    return _lib


def set_threads(n):
    lib().oracle_set_threads(int(n))


def max_threads():
    return lib().oracle_max_threads()


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _real(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float64:
        return "_f64", C.c_double
    if dtype == np.float32:
        return "_f32", C.c_float
    raise TypeError(dtype)


def params_table(cells):
    """NEST-unit parameter dictionaries -> par[NPARAM][n] (fp64)."""
    n = len(cells)
    par = np.zeros((NPARAM, n), np.float64)
    for i, p in enumerate(cells):
        par[L["GLIF3_PAR_C_M"], i] = p["C_m"]
        par[L["GLIF3_PAR_G"], i] = p["g"]
        par[L["GLIF3_PAR_E_L"], i] = p["E_L"]
        par[L["GLIF3_PAR_V_TH"], i] = p["V_th"]
        par[L["GLIF3_PAR_V_RESET"], i] = p["V_reset"]
        par[L["GLIF3_PAR_T_REF"], i] = p["t_ref"]
        par[L["GLIF3_PAR_ASC_DECAY0"]:L["GLIF3_PAR_ASC_DECAY0"] + 2, i] = p.get("asc_decay", (1.0, 1.0))
        par[L["GLIF3_PAR_ASC_AMPS0"]:L["GLIF3_PAR_ASC_AMPS0"] + 2, i] = p.get("asc_amps", (0.0, 0.0))
        par[L["GLIF3_PAR_ASC_R0"]:L["GLIF3_PAR_ASC_R0"] + 2, i] = p.get("asc_r", (1.0, 1.0))
        par[L["GLIF3_PAR_TAU_SYN0"]:L["GLIF3_PAR_TAU_SYN0"] + 4, i] = p["tau_syn"]
    return par


def precompute(par, h):
    """par[NPARAM][n] fp64 -> prop[NPROP][n] fp64 (NEST glif_psc::pre_run_hook)."""
    par = np.ascontiguousarray(par, np.float64)
    n = par.shape[1]
    prop = np.zeros((NPROP, n), np.float64)
    lib().glif3_precompute_f64(n, par, float(h), prop)
    return prop


def new_state(n_neurons, batch, dtype=np.float64, asc_init=None, u_init=None):
    ne = n_neurons * batch
    st = dict(V=np.zeros(ne, dtype), asc=np.zeros((NASC, ne), dtype), y1=np.zeros((NREC, ne), dtype),
              y2=np.zeros((NREC, ne), dtype), ref=np.zeros(ne, np.int32))
    if asc_init is not None:
        st["asc"][:] = np.repeat(np.asarray(asc_init, dtype).reshape(NASC, n_neurons), batch, axis=1)
    if u_init is not None:
        st["V"][:] = np.repeat(np.asarray(u_init, dtype), batch)
    return st


def step(st, prop, h, batch=1, class_id=None, syn=None, i_ext=None, want_frac=False):
    """One glif_psc update step in place on ``st``.  Returns (z, frac)."""
    dtype = st["V"].dtype
    sfx, creal = _real(dtype)
    ne = st["V"].size
    n = ne // batch
    prop = np.ascontiguousarray(prop, dtype)
    z = np.zeros(ne, np.uint8)
    frac = np.zeros(ne, dtype) if want_frac else None
    if syn is not None:
        syn = np.ascontiguousarray(syn, dtype)
    if i_ext is not None:
        i_ext = np.ascontiguousarray(i_ext, dtype)
    if class_id is not None:
        class_id = np.ascontiguousarray(class_id, np.int32)
    getattr(lib(), "glif3_step" + sfx)(
        C.c_int64(n), C.c_int32(batch), _ptr(st["V"]), _ptr(st["asc"]), _ptr(st["y1"]), _ptr(st["y2"]),
        _ptr(st["ref"]), _ptr(prop), C.c_int64(prop.shape[1]), _ptr(class_id), creal(h),
        _ptr(syn), _ptr(i_ext), _ptr(z), _ptr(frac))
    return z, frac


def _wide(csr):
    """The C side reads delays as int32 (any number of steps); tables carry uint8 or wider columns."""
    if csr is None or csr[0] is None:
        return csr
    return (csr[0], csr[1], csr[2], np.ascontiguousarray(csr[3], np.int32), csr[4])


def deliver_events(active_e, batch, csr, ring, n_tgt, step_idx):
    """Event-driven delivery through a source-major CSR (indptr, indices=targets,
    weights f32, delays in steps, receptors u8) into ring[L][NREC][n_tgt*batch]."""
    sfx, _ = _real(ring.dtype)
    indptr, indices, weights, delays, receptors = _wide(csr)
    active_e = np.ascontiguousarray(active_e, np.int32)
    getattr(lib(), "csr_deliver_events" + sfx)(
        C.c_int64(active_e.size), _ptr(active_e), C.c_int32(batch), _ptr(indptr), _ptr(indices), _ptr(weights),
        _ptr(delays), _ptr(receptors), _ptr(ring), C.c_int32(ring.shape[0]), C.c_int64(n_tgt), C.c_int64(step_idx))


def gather_rows(z, batch, csr, ring, n_tgt, step_idx):
    """Row-by-row sums over a target-major CSR (indices=sources), stored order."""
    sfx, _ = _real(ring.dtype)
    indptr, indices, weights, delays, receptors = _wide(csr)
    z = np.ascontiguousarray(z, np.uint8)
    getattr(lib(), "csr_gather_rows" + sfx)(
        C.c_int64(n_tgt), C.c_int32(batch), _ptr(z), _ptr(indptr), _ptr(indices), _ptr(weights),
        _ptr(delays), _ptr(receptors), _ptr(ring), C.c_int32(ring.shape[0]), C.c_int64(step_idx))


def simulate(st, prop, h, n_steps, batch=1, class_id=None, ring=None, rec=None, inp=None, in_ptr=None,
             in_events=None, i_ext=None, spike_cap=None, raster=False, step0=0):
    """Whole forward run in NEST's algorithmic form.  ``rec``/``inp`` are
    source-major CSR tuples.  Returns dict(step, elem, frac, count, raster)."""
    dtype = st["V"].dtype
    sfx, creal = _real(dtype)
    ne = st["V"].size
    n = ne // batch
    prop = np.ascontiguousarray(prop, dtype)
    if class_id is not None:
        class_id = np.ascontiguousarray(class_id, np.int32)
    if spike_cap is None:
        spike_cap = max(1024, ne * n_steps // 8)
    s_step = np.zeros(spike_cap, np.int32)
    s_elem = np.zeros(spike_cap, np.int32)
    s_frac = np.zeros(spike_cap, dtype)
    ras = np.zeros((n_steps, ne), np.uint8) if raster else None
    rec = _wide(rec) or (None,) * 5
    inp = _wide(inp) or (None,) * 5
    if in_ptr is not None:
        in_ptr = np.ascontiguousarray(in_ptr, np.int64)
        in_events = np.ascontiguousarray(in_events, np.int32)
    if i_ext is not None:
        i_ext = np.ascontiguousarray(i_ext, dtype)
    assert ring is not None and ring.dtype == dtype
    cnt = getattr(lib(), "glif3_simulate" + sfx)(
        C.c_int64(n), C.c_int32(batch), C.c_int64(n_steps), C.c_int64(step0),
        _ptr(st["V"]), _ptr(st["asc"]), _ptr(st["y1"]), _ptr(st["y2"]), _ptr(st["ref"]),
        _ptr(prop), C.c_int64(prop.shape[1]), _ptr(class_id), creal(h),
        _ptr(ring), C.c_int32(ring.shape[0]),
        *[_ptr(a) for a in rec], _ptr(in_ptr), _ptr(in_events), *[_ptr(a) for a in inp], _ptr(i_ext),
        _ptr(s_step), _ptr(s_elem), _ptr(s_frac), C.c_int64(spike_cap), _ptr(ras))
    k = min(cnt, spike_cap)
    return dict(step=s_step[:k], elem=s_elem[:k], frac=s_frac[:k], count=int(cnt), raster=ras)


# ---------------------------------------------------------------------------
# Independent restatements used to pin the C code (small sizes only)
# ---------------------------------------------------------------------------

def dense_deliver_bruteforce(z, batch, src, tgt, w, d, r, L, n_tgt, step_idx, dtype=np.float64):
    """Delivery written as dense matrices: one (n_tgt x n_src) matrix per
    (delay, receptor), ring[(t+d)%L][r] += W_{d,r} @ z.  COO edge list in."""
    n_src = z.size // batch
    zz = z.reshape(n_src, batch).astype(dtype)
    ring = np.zeros((L, NREC, n_tgt * batch), dtype)
    for dd in np.unique(d):
        for rr in np.unique(r):
            m = (d == dd) & (r == rr)
            W = np.zeros((n_tgt, n_src), dtype)
            np.add.at(W, (tgt[m], src[m]), w[m].astype(dtype))
            ring[(step_idx + int(dd)) % L, int(rr)] += (W @ zz).reshape(-1)
    return ring
