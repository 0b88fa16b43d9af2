"""The torch restatement used as the gradient oracle: its forward pass must be
the C oracle's model, and its surrogate gradient must equal a closed form in a
case where one exists.  (Gradients have no counterpart in the reference:
parity unpinned; these checks pin the oracle to its own stated definition.)"""
import numpy as np
import torch

from oracle import glif3_oracle as orc
from oracle import glif3_adjoint_ref as adj
from bmtk_amd import synthetic
from bmtk_amd.glif_utils import params_table


def test_torch_forward_is_the_c_oracle_model():
    cfg = synthetic.small_glif3_network(n=40, n_in=30, steps=80, seed=2, in_rate=40.0, in_w_scale=15.0, w_scale=4.0,
                                        in_fanout=20, p_conn=0.2)
    prop = orc.precompute(cfg["par"], cfg["h"])
    st = orc.new_state(40, 1, np.float64)
    ring = np.zeros((cfg["L"], 4, 40))
    want = orc.simulate(st, prop, cfg["h"], 80, ring=ring, rec=cfg["rec_src"], inp=cfg["inp_src"], in_ptr=cfg["in_ptr"],
                        in_events=cfg["in_events"], raster=True)
    assert want["count"] > 50
    got = adj.simulate_with_grad(prop, cfg["h"], 80, 40, 1, cfg["L"], cfg["rec_src"], cfg["inp_src"], cfg["in_ptr"],
                                 cfg["in_events"], lambda z: z.sum())
    np.testing.assert_array_equal(got["raster"], want["raster"])


def test_surrogate_gradient_equals_closed_form_below_threshold():
    """One neuron, one input synapse of weight w, a few input events, no spike.
    Then U_t = w * K_t with K the unit-weight response (taken from the C
    oracle), z_t = H(U_t - th) and the surrogate gradient of L = sum a_t z_t is
    sum_t a_t * dampening * max(0, 1 - |(w K_t - th)/th|) / th * K_t."""
    cell = dict(C_m=100.0, g=6.0, E_L=-70.0, V_th=-52.0, V_reset=-70.0, t_ref=3.0, asc_decay=(0.05, 0.3),
                asc_amps=(-20.0, -60.0), tau_syn=(5.5, 8.5, 2.8, 5.8))
    par, _, _ = params_table([cell])
    h, T, w = 1.0, 60, 55.0
    prop = orc.precompute(par, h)
    inp = (np.array([0, 1], np.int32), np.array([0], np.int32), np.array([1.0], np.float32),
           np.array([2], np.uint8), np.array([2], np.uint8))
    in_ptr = np.zeros(T + 1, np.int64)
    for s in (3, 9, 10, 30):
        in_ptr[s + 1:] += 1
    ev = np.zeros(4, np.int32)
    st = orc.new_state(1, 1, np.float64)
    K = []
    ring = np.zeros((4, 4, 1))
    for t in range(T):
        syn = ring[t % 4].copy(); ring[t % 4] = 0
        orc.step(st, prop, h, syn=syn)
        orc.deliver_events(ev[in_ptr[t]:in_ptr[t + 1]], 1, inp, ring, 1, t)
        K.append(st["V"][0])
    K = np.array(K)
    th = prop[orc.L["GLIF3_TH"], 0]
    assert (w * K).max() < th and (w * K).max() > 0.3 * th          # sub-threshold, inside the surrogate's support
    a = np.random.default_rng(0).normal(size=T)
    damp = 0.3
    want = np.sum(a * damp * np.maximum(0, 1 - np.abs((w * K - th) / th)) / th * K)
    inp_w = (inp[0], inp[1], np.array([w], np.float32), inp[3], inp[4])
    at = torch.as_tensor(a)
    got = adj.simulate_with_grad(prop, h, T, 1, 1, 4, None, inp_w, in_ptr, ev, lambda z: (z[:, 0] * at).sum(),
                                 dampening=damp)
    assert got["raster"].sum() == 0
    np.testing.assert_allclose(got["d_inp_w"][0], want, rtol=1e-10)
    assert abs(want) > 1e-4


def _c_oracle_trajectory(cfg, prop, batch, asc_init):
    """State after every step from the C oracle (fp64), stepping it by hand: take the arrivals of slot t, update,
    deliver the spikes and the input events of the step."""
    n, L, h = cfg["n"], cfg["L"], cfg["h"]
    st = orc.new_state(n, batch, np.float64, asc_init=asc_init)
    ring = np.zeros((L, 4, n * batch))
    traj = dict(V=[], asc=[], y1=[], y2=[])
    ras = []
    for t in range(cfg["steps"]):
        syn = ring[t % L].copy()
        ring[t % L] = 0
        z, _ = orc.step(st, prop, h, batch=batch, class_id=cfg["class_id"], syn=syn)
        orc.deliver_events(np.flatnonzero(z), batch, cfg["rec_src"], ring, n, t)
        orc.deliver_events(cfg["in_events"][cfg["in_ptr"][t]:cfg["in_ptr"][t + 1]], batch, cfg["inp_src"], ring, n, t)
        ras.append(z.copy())
        for k in traj:
            traj[k].append(st[k].copy())
    return {k: np.stack(v) for k, v in traj.items()}, np.stack(ras)


def test_torch_trajectories_equal_the_c_oracle_with_batch_classes_and_initial_currents():
    """Potential, after-spike currents and both PSC states after EVERY step, three trials, seven parameter
    classes, non-zero initial after-spike currents: the torch restatement and the C oracle are the same model to
    1e-12 (relative to a unit), not only to the same raster."""
    batch = 3
    cfg = synthetic.small_glif3_network(n=40, n_in=30, steps=90, seed=6, in_rate=40.0, in_w_scale=15.0, w_scale=4.0,
                                        in_fanout=20, p_conn=0.2, n_classes=7, batch=batch)
    prop = orc.precompute(cfg["par"], cfg["h"])
    asc_init = np.random.default_rng(2).uniform(-60, 20, (2, 40))
    want, ras = _c_oracle_trajectory(cfg, prop, batch, asc_init)
    assert ras.sum() > 150
    got = adj.simulate_with_grad(prop, cfg["h"], 90, 40, batch, cfg["L"], cfg["rec_src"], cfg["inp_src"], cfg["in_ptr"],
                                 cfg["in_events"], lambda z: z.sum(), class_id=cfg["class_id"], asc_init=asc_init,
                                 record=True)
    np.testing.assert_array_equal(got["raster"], ras)
    for k in ("V", "asc", "y1", "y2"):
        scale = np.maximum(np.abs(want[k]), 1.0)
        assert np.max(np.abs(got["traj"][k] - want[k]) / scale) < 1e-12, k


def test_pseudo_derivative_is_the_derivative_of_the_smooth_spike():
    """The backward rule of the Heaviside spike and the derivative of `smooth_spike` are the same function of U."""
    rng = np.random.default_rng(0)
    th = torch.as_tensor(rng.uniform(10, 30, 400))
    U = (th * torch.as_tensor(rng.uniform(-0.5, 2.5, 400))).requires_grad_(True)
    g = torch.as_tensor(rng.normal(size=400))
    (adj._Spike.apply(U, th, 0.3) * g).sum().backward()
    rule = U.grad.clone()
    U.grad = None
    (adj.smooth_spike(U, th, 0.3) * g).sum().backward()
    np.testing.assert_allclose(rule.numpy(), U.grad.numpy(), rtol=1e-12, atol=1e-15)
    assert (rule != 0).sum() > 100 and (rule == 0).sum() > 50
    # and the closed form: dampening * max(0, 1 - |v|) / th
    v = ((U - th) / th).detach().numpy()
    np.testing.assert_allclose(rule.numpy(), g.numpy() * 0.3 * np.maximum(0, 1 - np.abs(v)) / th.numpy(), rtol=1e-12)


def test_autograd_through_the_recurrent_path_equals_central_differences():
    """With the smooth spike the model is differentiable, and its autograd gradient -- spike -> recurrent synapse ->
    delay -> y1 -> y2 -> U -> next spike, over 40 steps and two trials -- must equal central finite differences
    with respect to recurrent and input weights (perturbed in fp64).  This checks the graph the GPU kernels are
    compared with: a dropped term or a detached tensor in the restatement would show here."""
    batch, T = 2, 40
    cfg = synthetic.small_glif3_network(n=24, n_in=12, steps=T, seed=9, in_rate=60.0, in_w_scale=12.0, w_scale=25.0,
                                        in_fanout=12, p_conn=0.3, batch=batch)
    n, h = cfg["n"], cfg["h"]
    prop = orc.precompute(cfg["par"], h)
    a = torch.as_tensor(np.random.default_rng(4).normal(size=(T, n * batch)))
    w_rec = cfg["rec_src"][2].astype(np.float64)
    w_inp = cfg["inp_src"][2].astype(np.float64)

    def run(wr, wi):
        return adj.simulate_with_grad(prop, h, T, n, batch, cfg["L"], cfg["rec_src"], cfg["inp_src"], cfg["in_ptr"],
                                      cfg["in_events"], lambda z: (z * a).sum(), smooth=True, rec_w=wr, inp_w=wi)
    base = run(w_rec, w_inp)
    z = base["z"]
    assert ((z > 0.01) & (z < 0.29)).mean() > 0.2          # graded spikes: inside the surrogate's support
    assert np.abs(base["d_rec_w"]).max() > 0 and np.abs(base["d_inp_w"]).max() > 0
    rng = np.random.default_rng(1)
    for name, w0, grad in (("rec", w_rec, base["d_rec_w"]), ("inp", w_inp, base["d_inp_w"])):
        order = np.argsort(-np.abs(grad))
        picks = np.concatenate([order[:6], rng.choice(order[6:], 6, replace=False)])
        for p in picks:
            eps = 1e-5 * max(1.0, abs(w0[p]))
            up, dn = w0.copy(), w0.copy()
            up[p] += eps
            dn[p] -= eps
            lp = run(up, w_inp)["loss"] if name == "rec" else run(w_rec, up)["loss"]
            lm = run(dn, w_inp)["loss"] if name == "rec" else run(w_rec, dn)["loss"]
            fd = (lp - lm) / (2 * eps)
            assert abs(fd - grad[p]) <= 1e-6 * np.abs(grad).max() + 1e-5 * abs(grad[p]), (name, p, fd, grad[p])


def test_state_transition_of_the_c_oracle_and_its_torch_transpose_satisfy_the_adjoint_identity():
    """<J v, u> = <v, J^T u> for the linear part of the update (leak, after-spike currents, both PSC states) over
    five steps: J v from the C oracle (the map is affine below threshold, so a difference of two runs is exact),
    J^T u from torch's vector-Jacobian product through the restatement."""
    n, batch, T = 30, 2, 5
    ne = n * batch
    rng = np.random.default_rng(11)
    par = synthetic.random_cells(rng, n)
    prop = orc.precompute(par, 1.0)
    th = np.repeat(prop[orc.L["GLIF3_TH"]], batch)
    x0 = dict(V=0.05 * th * rng.random(ne), asc=rng.uniform(-1, 1, (2, ne)), y1=rng.uniform(0, 0.02, (4, ne)),
              y2=rng.uniform(0, 0.02, (4, ne)))
    v = {k: rng.normal(size=a.shape) * 0.01 * (np.abs(a).mean() + 1e-3) for k, a in x0.items()}
    u = {k: rng.normal(size=a.shape) for k, a in x0.items()}

    def c_run(x):
        st = orc.new_state(n, batch, np.float64)
        for k in x:
            st[k][...] = x[k]
        for _ in range(T):
            z, _ = orc.step(st, prop, 1.0, batch=batch)
            assert z.sum() == 0
        return st
    a, b = c_run(x0), c_run({k: x0[k] + v[k] for k in x0})
    lhs = sum(float(((b[k] - a[k]) * u[k]).sum()) for k in x0)
    got = adj.simulate_with_grad(prop, 1.0, T, n, batch, 4, None, None, None, None,
                                 lambda z, final: sum((final[k] * torch.as_tensor(u[k])).sum() for k in u), init=x0)
    assert got["raster"].sum() == 0
    rhs = sum(float((got["d_init"][k] * v[k]).sum()) for k in x0)
    assert abs(lhs) > 1e-6
    assert abs(lhs - rhs) <= 1e-10 * abs(lhs)
