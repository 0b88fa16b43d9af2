"""TEST INFRASTRUCTURE ONLY -- reference gradients for the backward pass.

The reference (bmtk / NEST) has no gradient code, so this oracle is pinned by
no reference vector: PARITY UNPINNED.  It restates the forward model of
``glif3_oracle_impl.h`` step by step in torch (fp64, CPU) with the
differentiable conventions declared in ``include/bmtk_amd.h`` and lets
``torch.autograd`` produce the gradients the HIP adjoint kernels are compared
with.  It shares no code with those kernels.  Small networks only.
"""
import numpy as np
import torch

from . import glif3_oracle as orc

P = orc.L


class _Spike(torch.autograd.Function):
    """Heaviside forward, triangular pseudo-derivative backward."""

    @staticmethod
    def forward(ctx, U, th, dampening):
        ctx.save_for_backward(U, th)
        ctx.dampening = dampening
        return (U > th).to(U.dtype)

    @staticmethod
    def backward(ctx, g):
        U, th = ctx.saved_tensors
        vhat = (U - th) / th
        return g * ctx.dampening * torch.clamp(1.0 - vhat.abs(), min=0.0) / th, None, None


def smooth_spike(U, th, dampening):
    """The differentiable function whose derivative with respect to U IS the triangular pseudo-derivative
    dampening * max(0, 1 - |v|) / th, v = (U - th) / th: dampening times the piecewise quadratic
    0 (v <= -1), (v+1)^2/2 (-1..0), 1 - (1-v)^2/2 (0..1), 1 (v >= 1).  With it in place of the Heaviside step the
    model is smooth, so its autograd gradient can be held against central finite differences."""
    v = (U - th) / th
    rise = 0.5 * (torch.clamp(v, -1.0, 0.0) + 1.0) ** 2
    fall = 0.5 - 0.5 * (1.0 - torch.clamp(v, 0.0, 1.0)) ** 2
    return dampening * (rise + fall)


def simulate_with_grad(prop, h, n_steps, n, batch, ring_slots, rec, inp, in_ptr, in_events, loss_fn,
                       class_id=None, dampening=0.3, asc_init=None, i_ext=None, smooth=False, record=False,
                       init=None, rec_w=None, inp_w=None):
    """rec / inp: source-major tables (indptr, indices, weights, delays, receptors), numpy.
    loss_fn(z) takes the raster z [n_steps, n*batch] (float64 tensor) and returns a scalar; a loss_fn of two
    arguments also gets the final state, dict(V, asc, y1, y2) of tensors.
    smooth: graded spikes z = smooth_spike(U) and no refractoriness or reset (every element integrates in every
            step) -- the smooth model whose exact derivative the surrogate gradient of the spiking model uses.
    record: also return the state after every step, traj = dict(V [T, ne], asc [T, 2, ne], y1, y2 [T, 4, ne]).
    init:   dict with any of V [ne], asc [2, ne], y1, y2 [4, ne] (numpy): the state to start from; the gradient with
            respect to each comes back in d_init.
    rec_w / inp_w: weights to use instead of the tables' (float64 arrays; lets finite differences perturb them
            below fp32 resolution).
    Returns dict(raster, d_rec_w, d_inp_w, loss[, traj][, d_init])."""
    dd = torch.float64
    ne = n * batch
    col = np.arange(n) if class_id is None else np.asarray(class_id)
    col_e = torch.as_tensor(np.repeat(col, batch))
    pr = torch.as_tensor(np.asarray(prop, np.float64))

    def row(name):
        return pr[P["GLIF3_" + name]][col_e]

    P33, P30, th, Ur = row("P33"), row("P30"), row("TH"), row("UR")
    n_ref = row("NREF").to(torch.int64)
    c = [row("C0"), row("C1")]; d = [row("D0"), row("D1")]; r = [row("R0"), row("R1")]; amp = [row("AMP0"), row("AMP1")]
    P11 = [row("P11_%d" % k) for k in range(4)]; P31 = [row("P31_%d" % k) for k in range(4)]
    P32 = [row("P32_%d" % k) for k in range(4)]; psc0 = [row("PSC0_%d" % k) for k in range(4)]

    def edges(table, w_override):
        if table is None:
            return None
        indptr, indices, w, dl, rc = table
        src = np.repeat(np.arange(indptr.size - 1), np.diff(indptr))
        wt = torch.tensor(np.asarray(w if w_override is None else w_override, np.float64), requires_grad=True)
        return dict(src=torch.as_tensor(src), tgt=torch.as_tensor(indices.astype(np.int64)), w=wt,
                    d=np.asarray(dl, np.int64), r=torch.as_tensor(rc.astype(np.int64)))

    R, I_ = edges(rec, rec_w), edges(inp, inp_w)
    init = init or {}
    start = {}

    def first(name, shape, default):
        if name in init:
            t = torch.tensor(np.asarray(init[name], np.float64).reshape(shape), requires_grad=True)
            start[name] = t
            return t
        return default

    U = first("V", (ne,), torch.zeros(ne, dtype=dd))
    A0 = torch.zeros(2, ne, dtype=dd)
    if asc_init is not None:
        A0 = torch.as_tensor(np.repeat(np.asarray(asc_init, np.float64).reshape(2, n), batch, axis=1))
    A0 = first("asc", (2, ne), A0)
    A = [A0[0], A0[1]]
    Y1 = first("y1", (4, ne), torch.zeros(4, ne, dtype=dd))
    Y2 = first("y2", (4, ne), torch.zeros(4, ne, dtype=dd))
    y1 = [Y1[k] for k in range(4)]
    y2 = [Y2[k] for k in range(4)]
    ref = torch.zeros(ne, dtype=torch.int64)
    Iext = torch.zeros(ne, dtype=dd) if i_ext is None else torch.as_tensor(np.asarray(i_ext, np.float64))
    arrivals = {}   # step -> [4] tensors (ne)

    def deliver(E, t, z_src_elems_weight):
        """add w * z for every (synapse, trial) into arrivals[t+d][r]"""
        src_e, tgt_e, wv, dv, rv = z_src_elems_weight
        for dly in np.unique(dv):
            m = torch.as_tensor(dv == dly)
            if not bool(m.any()):
                continue
            slot = arrivals.setdefault(t + int(dly), [torch.zeros(ne, dtype=dd) for _ in range(4)])
            for k in range(4):
                mk = m & (rv == k)
                if bool(mk.any()):
                    slot[k] = slot[k].index_add(0, tgt_e[mk], wv[mk])

    zs = []
    traj = dict(V=[], asc=[], y1=[], y2=[])
    barange = torch.arange(batch)
    for t in range(n_steps):
        integrating = torch.ones(ne, dtype=torch.bool) if smooth else ref == 0
        S = c[0] * A[0] + c[1] * A[1]
        U_int = U * P33 + (Iext + S) * P30
        for k in range(4):
            U_int = U_int + (P31[k] * y1[k] + P32[k] * y2[k])
        if smooth:
            z = smooth_spike(U_int, th, dampening)
            U = U_int
            A = [A[a] * d[a] for a in range(2)]
        else:
            z = _Spike.apply(U_int, th, dampening) * integrating.to(dd)
            spiked = z.detach() > 0
            ref_new = torch.where(integrating, torch.where(spiked, n_ref, ref), ref - 1)
            reset = (~integrating) & (ref_new == 0)
            U = torch.where(integrating, U_int, torch.where(reset, Ur, U))
            A = [torch.where(integrating, A[a] * d[a], torch.where(reset, amp[a] + A[a] * r[a], A[a])) for a in range(2)]
            ref = ref_new
        s = arrivals.pop(t, [torch.zeros(ne, dtype=dd) for _ in range(4)])
        y2n = [(h * P11[k]) * y1[k] + P11[k] * y2[k] for k in range(4)]
        y1 = [P11[k] * y1[k] + psc0[k] * s[k] for k in range(4)]
        y2 = y2n
        zs.append(z)
        if record:
            traj["V"].append(U.detach().numpy().copy())
            traj["asc"].append(torch.stack(A).detach().numpy().copy())
            traj["y1"].append(torch.stack(y1).detach().numpy().copy())
            traj["y2"].append(torch.stack(y2).detach().numpy().copy())
        # recurrent delivery: every synapse, every trial, weighted by the (surrogate-differentiable) spike
        if R is not None and R["src"].numel():
            src_e = (R["src"].view(-1, 1) * batch + barange).reshape(-1)
            tgt_e = (R["tgt"].view(-1, 1) * batch + barange).reshape(-1)
            wv = (R["w"].view(-1, 1) * z[src_e].view(-1, batch)).reshape(-1)
            deliver(R, t, (src_e, tgt_e, wv, np.repeat(R["d"], batch), R["r"].repeat_interleave(batch)))
        if I_ is not None and in_ptr is not None:
            ev = np.asarray(in_events[in_ptr[t]:in_ptr[t + 1]], np.int64)
            if ev.size:
                ip = inp[0]
                js, bs = ev // batch, ev % batch
                idx = np.concatenate([np.arange(ip[j], ip[j + 1]) for j in js]) if js.size else np.zeros(0, np.int64)
                bb = np.concatenate([np.full(ip[j + 1] - ip[j], b) for j, b in zip(js, bs)])
                idx_t = torch.as_tensor(idx)
                tgt_e = I_["tgt"][idx_t] * batch + torch.as_tensor(bb)
                deliver(I_, t, (None, tgt_e, I_["w"][idx_t], I_["d"][idx], I_["r"][idx_t]))
    zmat = torch.stack(zs)
    final = dict(V=U, asc=torch.stack(A), y1=torch.stack(y1), y2=torch.stack(y2))
    loss = loss_fn(zmat, final) if loss_fn.__code__.co_argcount >= 2 else loss_fn(zmat)
    if loss.requires_grad:
        loss.backward()
    out = dict(raster=zmat.detach().numpy().astype(np.uint8), z=zmat.detach().numpy(), loss=float(loss.detach()),
               d_rec_w=None if R is None or R["w"].grad is None else R["w"].grad.numpy().copy(),
               d_inp_w=None if I_ is None or I_["w"].grad is None else I_["w"].grad.numpy().copy())
    if record:
        out["traj"] = {k: np.stack(v) for k, v in traj.items()}
    if start:
        out["d_init"] = {k: (None if t.grad is None else t.grad.numpy().copy()) for k, t in start.items()}
    return out
