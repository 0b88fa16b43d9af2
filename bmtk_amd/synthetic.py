"""Seeded synthetic GLIF3 networks of the benchmark shapes (host / NumPy).

Every generator draws from ``numpy.random.default_rng(seed)`` so the CPU
oracle and the GPU path can be fed identical arrays.  Parameter ranges: C_m
50-200 pF, g 3-12 nS, E_L -80..-65 mV, V_th -55..-40 mV, t_ref 2-5 ms,
after-spike decay 0.003-0.3 /ms, tau_syn 1-20 ms per receptor; after-spike
amplitudes span the range of the example cells (-292..-4 pA,
examples/point_components/cell_models).  Weights are lognormal(0, 1) pA, signed
by the presynaptic class (80 % excitatory, 20 % inhibitory); receptors follow
the pre/post class pairing of examples/point_components/synaptic_models
(e2e -> 0, i2e -> 1, e2i -> 2, i2i -> 3, external input -> 0).
"""
import numpy as np

from .glif_utils import params_table
from .layout import NPARAM, PAR
from . import network as net


def random_cells(rng, n):
    """n NEST-unit glif_psc parameter sets -> par[NPARAM][n] (fp64)."""
    par = np.zeros((NPARAM, n), np.float64)
    par[PAR["C_M"]] = rng.uniform(50, 200, n)
    par[PAR["G"]] = rng.uniform(3, 12, n)
    par[PAR["E_L"]] = rng.uniform(-80, -65, n)
    par[PAR["V_TH"]] = rng.uniform(-55, -40, n)
    par[PAR["V_RESET"]] = par[PAR["E_L"]]
    par[PAR["T_REF"]] = rng.uniform(2, 5, n)
    par[PAR["ASC_DECAY0"]:PAR["ASC_DECAY0"] + 2] = rng.uniform(0.003, 0.3, (2, n))
    par[PAR["ASC_AMPS0"]:PAR["ASC_AMPS0"] + 2] = rng.uniform(-292, -4, (2, n))
    par[PAR["ASC_R0"]:PAR["ASC_R0"] + 2] = 1.0
    par[PAR["TAU_SYN0"]:PAR["TAU_SYN0"] + 4] = rng.uniform(1, 20, (4, n))
    return par


def _receptor(pre_inh, post_inh):
    return (pre_inh.astype(np.uint8) + 2 * post_inh.astype(np.uint8)).astype(np.uint8)


def poisson_events(rng, n_in, rate_hz, dt_ms, steps, batch=1):
    """Bernoulli(rate*dt) input spikes per (step, source, trial) as step-sorted
    event lists (in_ptr int64[steps+1], in_events int32[] = source*batch+trial)."""
    p = rate_hz * dt_ms * 1e-3
    counts = rng.binomial(n_in * batch, p, steps)
    in_ptr = np.concatenate(([0], np.cumsum(counts))).astype(np.int64)
    ev = np.empty(in_ptr[-1], np.int32)
    for t in range(steps):
        ev[in_ptr[t]:in_ptr[t + 1]] = np.sort(rng.choice(n_in * batch, counts[t], replace=False))
    return in_ptr, ev


def small_glif3_network(n=450, n_in=1000, steps=1000, seed=0, p_conn=0.1, in_rate=10.0, in_fanout=50,
                        max_delay=4, n_classes=None, batch=1, w_scale=1.0, in_w_scale=1.0):
    """The 450-neuron shape: Erdos-Renyi recurrent connectivity without
    self-loops, ``n_in`` Poisson inputs each projecting to ``in_fanout`` random
    targets, integer delays uniform in 1..max_delay, dt = 1 ms."""
    rng = np.random.default_rng(seed)
    h = 1.0
    n_par = n_classes if n_classes else n
    par = random_cells(rng, n_par)
    class_id = rng.integers(0, n_classes, n).astype(np.int32) if n_classes else None
    inh = rng.random(n) < 0.2
    mask = rng.random((n, n)) < p_conn
    np.fill_diagonal(mask, False)
    tgt, src = np.nonzero(mask)
    nnz = src.size
    w = (rng.lognormal(0, 1, nnz) * w_scale * np.where(inh[src], -1.0, 1.0)).astype(np.float32)
    d = rng.integers(1, max_delay + 1, nnz).astype(np.uint8)
    r = _receptor(inh[src], inh[tgt])
    rec_src = net.coo_to_csr(src, tgt, w, d, r, n_rows=n, major="source")
    rec_tgt = net.coo_to_csr(src, tgt, w, d, r, n_rows=n, major="target")
    isrc = np.repeat(np.arange(n_in), in_fanout)
    itgt = np.concatenate([rng.choice(n, in_fanout, replace=False) for _ in range(n_in)]) if n_in else np.zeros(0, int)
    iw = (rng.lognormal(0, 1, isrc.size) * in_w_scale).astype(np.float32)
    idl = rng.integers(1, max_delay + 1, isrc.size).astype(np.uint8)
    ir = np.zeros(isrc.size, np.uint8)
    inp_src = net.coo_to_csr(isrc, itgt, iw, idl, ir, n_rows=max(n_in, 1), major="source")
    in_ptr, in_events = poisson_events(rng, max(n_in, 1), in_rate if n_in else 0.0, h, steps, batch)
    return dict(n=n, n_in=n_in, steps=steps, h=h, L=max_delay + 1, par=par, class_id=class_id, inh=inh,
                rec_src=rec_src, rec_tgt=rec_tgt, inp_src=inp_src, in_ptr=in_ptr, in_events=in_events, batch=batch)


def random_state(rng, par, n, batch, class_id=None, dtype=np.float32, h=1.0):
    """States uniform in their physiological ranges: U in [0, V_th-E_L), ASC in
    [-300, 0] pA, y1, y2 in [0, 1], refractory counter in 0..ceil(t_ref/h) (a
    quarter of the elements refractory)."""
    ne = n * batch
    col = (class_id if class_id is not None else np.arange(n)).repeat(batch)
    th = (par[PAR["V_TH"]] - par[PAR["E_L"]])[col]
    nref = np.ceil(par[PAR["T_REF"]] / h)[col]
    st = dict(V=(rng.random(ne) * th).astype(dtype), asc=rng.uniform(-300, 0, (2, ne)).astype(dtype),
              y1=rng.random((4, ne)).astype(dtype), y2=rng.random((4, ne)).astype(dtype),
              ref=np.where(rng.random(ne) < 0.25, rng.integers(1, 100, ne) % (nref + 1), 0).astype(np.int32))
    return st


def sparse_in_degree_network(rng, n, mean_in, degree="poisson", max_delay=5, inh_frac=0.2):
    """Target-major table with a Poisson or lognormal in-degree and uniformly
    random sources (repeats allowed), the shape of the 52k / 230k networks."""
    if degree == "poisson":
        deg = rng.poisson(mean_in, n)
    else:
        sigma = 0.5
        deg = np.rint(rng.lognormal(np.log(mean_in) - sigma * sigma / 2, sigma, n)).astype(np.int64)
    indptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int64)
    nnz = int(indptr[-1])
    inh = rng.random(n) < inh_frac
    src = rng.integers(0, n, nnz, dtype=np.int32)
    tgt = net.csr_rows(indptr.astype(np.int32)) if nnz < 2 ** 31 else None
    w = (rng.lognormal(0, 1, nnz).astype(np.float32)) * np.where(inh[src], np.float32(-1), np.float32(1))
    d = rng.integers(1, max_delay + 1, nnz, dtype=np.uint8)
    r = _receptor(inh[src], inh[tgt])
    return (indptr.astype(np.int32), src, w.astype(np.float32), d, r), inh


# ---------------------------------------------------------------------------
# Large networks, generated on the device with torch's generator (the host
# generators above would take minutes for 50-70 M synapses).
# ---------------------------------------------------------------------------

def _t_receptor(pre_inh, post_inh):
    import torch
    return (pre_inh.to(torch.uint8) + 2 * post_inh.to(torch.uint8)).to(torch.uint8)


def device_network(n, mean_in, degree="lognormal", seed=3, max_delay=5, inh_frac=0.2, w_scale=1.0,
                   inh_scale=1.0, device="cuda", sigma=0.5):
    """Random recurrent network on the device: in-degree Poisson(mean_in) or
    lognormal with mean ``mean_in``, uniformly random sources, weights
    lognormal(0,1)*w_scale pA signed by the source class (inhibitory ones
    also times ``inh_scale``), delays uniform 1..max_delay.
    Returns (target-major table, source-major table, inh flags), each table a
    tuple of device tensors (indptr, indices, weights, delays, receptors)."""
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    if degree == "poisson":
        deg = torch.poisson(torch.full((n,), float(mean_in), device=device), generator=g).to(torch.int64)
    else:
        mu = float(np.log(mean_in) - sigma * sigma / 2)
        deg = torch.exp(torch.randn(n, device=device, generator=g) * sigma + mu).round().to(torch.int64)
    indptr = torch.zeros(n + 1, dtype=torch.int64, device=device)
    indptr[1:] = torch.cumsum(deg, 0)
    nnz = int(indptr[-1].item())
    if nnz >= 2 ** 31:
        raise ValueError("more than 2^31-1 synapses")
    inh = torch.rand(n, device=device, generator=g) < inh_frac
    tgt = torch.repeat_interleave(torch.arange(n, device=device, dtype=torch.int32), deg)
    src = torch.randint(0, n, (nnz,), device=device, generator=g, dtype=torch.int32)
    w = torch.exp(torch.randn(nnz, device=device, generator=g)) * w_scale
    pre_inh = inh[src.long()]
    w = torch.where(pre_inh, -w * inh_scale, w).to(torch.float32)
    d = torch.randint(1, max_delay + 1, (nnz,), device=device, generator=g, dtype=torch.uint8)
    r = _t_receptor(pre_inh, inh[tgt.long()])
    by_tgt = (indptr.to(torch.int32), src, w, d, r)
    order = torch.sort(src.long(), stable=True).indices
    sp = torch.zeros(n + 1, dtype=torch.int64, device=device)
    sp[1:] = torch.cumsum(torch.bincount(src.long(), minlength=n), 0)
    by_src = (sp.to(torch.int32), tgt[order], w[order], d[order], r[order])
    return by_tgt, by_src, inh


def device_input_table(n_in, n, n_syn, seed=4, max_delay=5, w_scale=1.0, device="cuda"):
    """External sources -> neurons, source-major on the device: ``n_syn``
    synapses with uniformly random source and target, excitatory, receptor 0."""
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    src = torch.sort(torch.randint(0, n_in, (n_syn,), device=device, generator=g)).values
    sp = torch.zeros(n_in + 1, dtype=torch.int64, device=device)
    sp[1:] = torch.cumsum(torch.bincount(src, minlength=n_in), 0)
    tgt = torch.randint(0, n, (n_syn,), device=device, generator=g, dtype=torch.int32)
    w = (torch.exp(torch.randn(n_syn, device=device, generator=g)) * w_scale).to(torch.float32)
    d = torch.randint(1, max_delay + 1, (n_syn,), device=device, generator=g, dtype=torch.uint8)
    r = torch.zeros(n_syn, dtype=torch.uint8, device=device)
    return (sp.to(torch.int32), tgt, w, d, r)


def device_poisson_events(n_in, rate_hz, dt_ms, steps, batch=1, seed=5, device="cuda"):
    """Bernoulli(rate*dt) spikes per (step, source, trial) -> step-sorted event
    lists on the device (in_ptr int64[steps+1], in_events int32[])."""
    import torch
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    p = rate_hz * dt_ms * 1e-3
    ptr = [0]
    chunks = []
    block = max(1, (1 << 26) // max(1, n_in * batch))
    for t0 in range(0, steps, block):
        k = min(block, steps - t0)
        z = torch.rand(k, n_in * batch, device=device, generator=g) < p
        tt, ee = torch.nonzero(z, as_tuple=True)
        counts = torch.bincount(tt, minlength=k)
        ptr.append(counts)
        chunks.append(ee.to(torch.int32))
    counts = torch.cat([c if torch.is_tensor(c) else torch.zeros(0, dtype=torch.int64, device=device) for c in ptr[1:]])
    in_ptr = torch.zeros(steps + 1, dtype=torch.int64, device=device)
    in_ptr[1:] = torch.cumsum(counts, 0)
    return in_ptr, torch.cat(chunks) if chunks else torch.zeros(0, dtype=torch.int32, device=device)
