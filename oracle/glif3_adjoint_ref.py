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


def simulate_with_grad(prop, h, n_steps, n, batch, ring_slots, rec, inp, in_ptr, in_events, loss_fn,
                       class_id=None, dampening=0.3, asc_init=None, i_ext=None):
    """rec / inp: source-major tables (indptr, indices, weights, delays, receptors), numpy.
    loss_fn(z) takes the raster z [n_steps, n*batch] (float64 tensor) and returns a scalar.
    Returns dict(raster, d_rec_w, d_inp_w, loss)."""
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

    def edges(table):
        if table is None:
            return None
        indptr, indices, w, dl, rc = table
        src = np.repeat(np.arange(indptr.size - 1), np.diff(indptr))
        wt = torch.tensor(np.asarray(w, np.float64), requires_grad=True)
        return dict(src=torch.as_tensor(src), tgt=torch.as_tensor(indices.astype(np.int64)), w=wt,
                    d=np.asarray(dl, np.int64), r=torch.as_tensor(rc.astype(np.int64)))

    R, I_ = edges(rec), edges(inp)
    U = torch.zeros(ne, dtype=dd)
    A = [torch.zeros(ne, dtype=dd) for _ in range(2)]
    if asc_init is not None:
        A = [torch.as_tensor(np.repeat(np.asarray(asc_init, np.float64)[a], batch)) for a in range(2)]
    y1 = [torch.zeros(ne, dtype=dd) for _ in range(4)]
    y2 = [torch.zeros(ne, dtype=dd) for _ in range(4)]
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
    barange = torch.arange(batch)
    for t in range(n_steps):
        integrating = ref == 0
        S = c[0] * A[0] + c[1] * A[1]
        U_int = U * P33 + (Iext + S) * P30
        for k in range(4):
            U_int = U_int + (P31[k] * y1[k] + P32[k] * y2[k])
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
    loss = loss_fn(zmat)
    loss.backward()
    return dict(raster=zmat.detach().numpy().astype(np.uint8), loss=float(loss.detach()),
                d_rec_w=None if R is None else R["w"].grad.numpy().copy(),
                d_inp_w=None if I_ is None or I_["w"].grad is None else I_["w"].grad.numpy().copy())
