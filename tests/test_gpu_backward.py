"""GPU adjoint (BPTT) kernels against torch.autograd over an independent fp64
restatement of the same model.  Gradients have no counterpart in the
reference (parity unpinned); the tolerance is the 1e-4 relative the build
states, taken relative to the largest gradient magnitude of the table."""
import numpy as np
import pytest
import torch

from oracle import glif3_oracle as orc
from oracle import glif3_adjoint_ref as adj
from bmtk_amd import synthetic, training
from bmtk_amd.simulator import Glif3Simulator

pytestmark = pytest.mark.gpu


def _quarter_weights(csr):
    indptr, indices, w, d, r = csr
    return indptr, indices, (np.round(w * 4.0) / 4.0 + np.sign(w) * 0.25).astype(np.float32), d, r


def _net(batch, seed, n=40, n_in=30, steps=70):
    cfg = synthetic.small_glif3_network(n=n, n_in=n_in, steps=steps, seed=seed, in_rate=40.0, in_w_scale=15.0,
                                        w_scale=4.0, in_fanout=n // 2, p_conn=0.2, batch=batch)
    # exact weights keep the fp32 and fp64 forward rasters identical, so both sides differentiate the same run
    cfg["rec_src"] = _quarter_weights(cfg["rec_src"])
    cfg["inp_src"] = _quarter_weights(cfg["inp_src"])
    return cfg


def _rel(got, want):
    return float(np.max(np.abs(got - want)) / max(np.max(np.abs(want)), 1e-30))


def _share_within_relative(got, want, rel=1e-4, floor=0.01):
    """Of the gradient entries that are at least ``floor`` of the table's largest, the share whose OWN relative
    error is within ``rel``.  (The table-wide norm of ``_rel`` is the tolerance that is asserted everywhere; an
    entry far below the largest is a sum of cancelling terms and has no relative accuracy of its own in fp32.)"""
    big = np.abs(want) >= floor * np.abs(want).max()
    return float(np.mean(np.abs(got[big] - want[big]) <= rel * np.abs(want[big]))), int(big.sum())


@pytest.mark.parametrize("batch,seed,loss_kind,n_blocks",
                         [(1, 2, "per_step", 0), (3, 4, "per_step", 0), (1, 5, "rates", 0), (4, 6, "rates", 0),
                          (8, 8, "per_step", 0), (32, 9, "rates", 0),  # multiples of 4: four trials per lane
                          # the recurrent table regrouped into n_blocks target ranges (more ranges than fit: empty ones)
                          (8, 8, "per_step", 8), (32, 9, "rates", 16), (4, 6, "per_step", 64), (64, 3, "per_step", 8)])
def test_weight_gradients_match_autograd(batch, seed, loss_kind, n_blocks):
    cfg = _net(batch, seed)
    n, T, h = cfg["n"], cfg["steps"], cfg["h"]
    ne = n * batch
    prop = orc.precompute(cfg["par"], h)
    rng = np.random.default_rng(seed)
    sim = Glif3Simulator(n, cfg["par"], h, batch=batch, rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"],
                         resident=False)
    sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
    fwd = sim.run(T, save_state=True)
    ras = sim.raster(fwd["bits"]).cpu().numpy()
    bptt = training.Glif3Bptt(sim, dampening=0.3, blocked=n_blocks > 0, n_blocks=n_blocks or None)
    assert (bptt.blk is not None) == (n_blocks > 0)
    if loss_kind == "per_step":
        a = rng.normal(size=(T, ne))
        loss_fn = lambda z: (z * torch.as_tensor(a)).sum()
        bptt.backward(fwd, dl_dz=torch.as_tensor(a.astype(np.float32), device="cuda"))
    else:
        pop = rng.integers(0, 3, n)
        targets = rng.uniform(0, 0.05, (batch, 3))
        pop_t = torch.as_tensor(pop)

        def loss_fn(z):
            c = z.sum(0).view(n, batch)
            size = torch.bincount(pop_t, minlength=3).to(z.dtype)
            rate = torch.zeros(3, batch, dtype=z.dtype).index_add_(0, pop_t, c) / (size.view(-1, 1) * T)
            return ((rate.t() - torch.as_tensor(targets)) ** 2).mean()
        counts = training.spike_counts(fwd["bits"], ne)
        np.testing.assert_array_equal(counts.cpu().numpy(), ras.sum(0))
        loss, g = training.rate_mse(counts, T, batch, pop_t.cuda(), torch.as_tensor(targets, dtype=torch.float32,
                                                                                    device="cuda"))
        bptt.backward(fwd, dl_dz_const=g)
    want = adj.simulate_with_grad(prop, h, T, n, batch, cfg["L"], cfg["rec_src"], cfg["inp_src"], cfg["in_ptr"],
                                  cfg["in_events"], loss_fn, dampening=0.3)
    np.testing.assert_array_equal(ras, want["raster"])
    assert ras.sum() > 30 * batch
    if loss_kind == "rates":
        assert float(loss) == pytest.approx(want["loss"], rel=1e-5)
    got_rec, got_inp = bptt.d_rec_w.cpu().numpy(), bptt.d_inp_w.cpu().numpy()
    assert np.abs(want["d_rec_w"]).max() > 0 and np.abs(want["d_inp_w"]).max() > 0
    assert _rel(got_rec, want["d_rec_w"]) < 1e-4
    assert _rel(got_inp, want["d_inp_w"]) < 1e-4
    # entry by entry, as the tolerance is worded: of the entries of at least 1 % of the largest, how many hold
    # 1e-4 relative
    for got, ref in ((got_rec, want["d_rec_w"]), (got_inp, want["d_inp_w"])):
        share, count = _share_within_relative(got, ref)
        print("entries >= 1 %% of the largest: %d, within 1e-4 relative: %.5f" % (count, share))
        assert count > 20 and share >= 0.99, (share, count)


@pytest.mark.parametrize("batch", [1, 8, 32])
def test_weight_gradients_with_input_ids_repeated_within_a_step(batch):
    """Two or three spikes of one source inside one step: the forward run delivers every occurrence (batched runs
    through the bit rows of the pull form plus the repeat lists), and the input-weight gradient counts every
    occurrence too.  Same autograd reference and tolerance as above."""
    from test_gpu_simulate import _with_duplicate_events
    cfg = _net(batch, 21 + batch, n=60, n_in=40, steps=60)
    n, T, h = cfg["n"], cfg["steps"], cfg["h"]
    in_ptr, in_events = _with_duplicate_events(cfg, np.random.default_rng(5), batch)
    assert in_events.size > 1.15 * cfg["in_events"].size
    prop = orc.precompute(cfg["par"], h)
    sim = Glif3Simulator(n, cfg["par"], h, batch=batch, rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"],
                         resident=False, pull=batch >= 8)
    sim.set_input_events(in_ptr, in_events)
    assert sim.in_duplicates and (batch < 8 or (sim.fuse_table is not None and sim.in_repeat_ptr is not None))
    fwd = sim.run(T, save_state=True)
    ras = sim.raster(fwd["bits"]).cpu().numpy()
    a = np.random.default_rng(6).normal(size=(T, n * batch))
    bptt = training.Glif3Bptt(sim, dampening=0.3)
    bptt.backward(fwd, dl_dz=torch.as_tensor(a.astype(np.float32), device="cuda"))
    want = adj.simulate_with_grad(prop, h, T, n, batch, cfg["L"], cfg["rec_src"], cfg["inp_src"], in_ptr, in_events,
                                  lambda z: (z * torch.as_tensor(a)).sum(), dampening=0.3)
    np.testing.assert_array_equal(ras, want["raster"])
    assert ras.sum() > 30 * batch
    assert _rel(bptt.d_rec_w.cpu().numpy(), want["d_rec_w"]) < 1e-4
    assert _rel(bptt.d_inp_w.cpu().numpy(), want["d_inp_w"]) < 1e-4


def test_chunked_backward_equals_one_call():
    cfg = _net(2, 7)
    n, T, h = cfg["n"], cfg["steps"], cfg["h"]
    a = torch.as_tensor(np.random.default_rng(1).normal(size=(T, n * 2)).astype(np.float32), device="cuda")
    grads = []
    for chunks in ([T], [30, 25, 15]):
        sim = Glif3Simulator(n, cfg["par"], h, batch=2, rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"],
                             resident=False)
        sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        runs, k0 = [], 0
        for c in chunks:
            runs.append((sim.run(c, save_state=True), k0, c)); k0 += c
        bptt = training.Glif3Bptt(sim)
        for fwd, k0, c in reversed(runs):
            bptt.backward(fwd, dl_dz=a[k0:k0 + c].contiguous())
        grads.append((bptt.d_rec_w.cpu().numpy(), bptt.d_inp_w.cpu().numpy()))
    np.testing.assert_allclose(grads[0][0], grads[1][0], rtol=0, atol=1e-6 * np.abs(grads[0][0]).max())
    np.testing.assert_allclose(grads[0][1], grads[1][1], rtol=0, atol=1e-6 * np.abs(grads[0][1]).max())


def test_backward_argument_errors():
    cfg = _net(1, 3)
    sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"],
                         resident=True)
    with pytest.raises(ValueError):
        training.Glif3Bptt(sim)
    with pytest.raises(ValueError):
        sim.run(5, save_state=True)
    sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"],
                         resident=False)
    sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
    bptt = training.Glif3Bptt(sim)
    with pytest.raises(ValueError):
        bptt.backward(sim.run(5))                                 # no record
    from bmtk_amd._lib import BmtkAmdError
    fwd = sim.run(5, save_state=True)
    z = torch.zeros(5, cfg["n"], device="cuda")
    with pytest.raises(BmtkAmdError):
        bptt.backward(fwd, dl_dz=z, dl_dz_const=z[0].contiguous())


def test_state_adjoint_kernel_transposes_the_state_update():
    """<J v, u> = <v, J^T u> on the device for the linear part of the update (leak, after-spike currents, both PSC
    states) over three steps: J v as the difference of two forward runs of the step kernels from states x and x + v
    that stay below threshold, J^T u from the backward pass started with the adjoint state u and no loss.  fp32
    throughout: the identity is held to 1e-4 of its size."""
    n, batch, T = 3000, 4, 3
    ne = n * batch
    rng = np.random.default_rng(21)
    par = synthetic.random_cells(rng, n)
    prop = orc.precompute(par, 1.0)
    th = np.repeat(prop[orc.L["GLIF3_TH"]], batch)
    x0 = dict(V=(0.3 * th * rng.random(ne)).astype(np.float32), asc=rng.uniform(-2, 2, (2, ne)).astype(np.float32),
              y1=rng.uniform(0, 0.05, (4, ne)).astype(np.float32), y2=rng.uniform(0, 0.05, (4, ne)).astype(np.float32))
    v = {k: (rng.normal(size=a.shape) * 0.25 * (np.abs(a).mean() + 1e-3)).astype(np.float32) for k, a in x0.items()}
    u = {k: rng.normal(size=a.shape).astype(np.float32) for k, a in x0.items()}

    def forward(x):
        sim = Glif3Simulator(n, par, 1.0, batch=batch, resident=False)
        for k in x:
            getattr(sim.state, k).copy_(torch.as_tensor(x[k], device="cuda").reshape(getattr(sim.state, k).shape))
        fwd = sim.run(T, save_state=True)
        assert int(sim.raster(fwd["bits"]).sum().item()) == 0
        return sim, fwd, {k: getattr(sim.state, k).double().cpu().numpy().reshape(x[k].shape) for k in x}
    sim, fwd, a = forward(x0)
    _, _, b = forward({k: x0[k] + v[k] for k in x0})
    lhs = sum(float(((b[k] - a[k]) * u[k].astype(np.float64)).sum()) for k in x0)
    bptt = training.Glif3Bptt(sim, dampening=0.3)
    for k, t in (("V", bptt.lam_V), ("asc", bptt.lam_asc), ("y1", bptt.lam_y1), ("y2", bptt.lam_y2)):
        t.copy_(torch.as_tensor(u[k], device="cuda").reshape(t.shape))
    bptt.backward(fwd, dl_dz=torch.zeros(T, ne, device="cuda"))
    jt_u = dict(V=bptt.lam_V, asc=bptt.lam_asc, y1=bptt.lam_y1, y2=bptt.lam_y2)
    rhs = sum(float((jt_u[k].double().cpu().numpy().reshape(v[k].shape) * v[k].astype(np.float64)).sum()) for k in x0)
    assert abs(lhs) > 1.0
    assert abs(lhs - rhs) <= 1e-4 * abs(lhs), (lhs, rhs)


@pytest.mark.parametrize("batch,seed", [(1, 2), (3, 4), (8, 8), (32, 9), (100, 12)])
def test_backward_pass_in_its_three_parts_equals_the_fused_driver(batch, seed):
    """``bmtk_csr_propagate_bwd`` + ``bmtk_glif3_step_bwd`` + ``bmtk_csr_weight_grad`` step by step ==
    ``bmtk_glif3_simulate_bwd`` (pinned against autograd above): the adjoint state bit for bit (the same kernels
    in the same order; the driver's skipped rows have a zero surrogate derivative), the gradients bit for bit where
    the driver uses the same gradient kernels (more than 64 trials) and to 1e-6 of the largest entry otherwise (the
    driver's gradient rides along with the transposed propagation there and adds a row's trials in another
    order).  ``between`` sees every step once, last step first."""
    cfg = _net(batch, seed)
    n, T, h = cfg["n"], cfg["steps"], cfg["h"]
    ne = n * batch
    sim = Glif3Simulator(n, cfg["par"], h, batch=batch, rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"],
                         resident=False)
    sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
    fwd = sim.run(T, save_state=True)
    dl = torch.as_tensor(np.random.default_rng(seed).normal(size=(T, ne)).astype(np.float32), device="cuda")
    whole = training.Glif3Bptt(sim, dampening=0.3, blocked=False)
    whole.backward(fwd, dl_dz=dl)
    parts = training.Glif3Bptt(sim, dampening=0.3, blocked=False)
    seen = []
    parts.backward_stepwise(fwd, dl_dz=dl, between=seen.append)
    assert seen == list(range(T - 1, -1, -1))
    for name in ("lam_V", "lam_asc", "lam_y1", "lam_y2", "lam_ring"):
        assert torch.equal(getattr(parts, name), getattr(whole, name)), name
    assert float(whole.lam_V.abs().max()) > 0 and float(whole.d_rec_w.abs().max()) > 0
    for name in ("d_rec_w", "d_inp_w"):
        got, want = getattr(parts, name), getattr(whole, name)
        if batch > 64:
            assert torch.equal(got, want), name
        else:
            assert float((got - want).abs().max()) <= 1e-6 * float(want.abs().max()), name


def test_backward_parts_argument_errors():
    cfg = _net(4, 6)
    sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], batch=4, rec=cfg["rec_src"], ring_slots=cfg["L"],
                         resident=False)
    fwd = sim.run(5, save_state=True)
    bptt = training.Glif3Bptt(sim, blocked=False)
    a, step0, _ = bptt._struct(fwd, None, None, False)
    import ctypes
    from bmtk_amd import _lib
    lib = _lib.load()
    assert lib.bmtk_glif3_step_bwd(ctypes.byref(a), step0, 0, 3, None) != 0          # 1 or 8 partial sums
    assert "partial sums" in lib.bmtk_amd_last_error().decode()
    assert lib.bmtk_glif3_step_bwd(ctypes.byref(a), step0, -1, 1, None) != 0
    a.d_rec_w = None
    assert lib.bmtk_csr_weight_grad(ctypes.byref(a), step0, 0, None) != 0             # nothing to fill
    assert "neither" in lib.bmtk_amd_last_error().decode()


@pytest.mark.parametrize("batch,seed,n_blocks,steps", [(32, 9, 16, 70), (64, 3, 8, 69), (20, 5, 8, 33), (32, 11, 8, 3),
                                                        (32, 12, 8, 4)])
def test_two_steps_per_pass_of_the_blocked_form_equal_one(batch, seed, n_blocks, steps):
    """The blocked transposed propagation taking two steps per pass over its table (``gz_planes`` 16, batches above
    16) against the same form step by step: every sum is added in the same order, so the adjoint state and the
    adjoint ring agree BIT FOR BIT after an even and an odd number of steps, in one call and in chunks; the weight
    gradients add the two steps' contributions in another order (1e-6 of the largest entry)."""
    cfg = _net(batch, seed, steps=steps)
    n, T, h = cfg["n"], cfg["steps"], cfg["h"]
    ne = n * batch
    sim = Glif3Simulator(n, cfg["par"], h, batch=batch, rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"],
                         resident=False)
    sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
    cut = max(1, T // 3)
    chunks = [sim.run(cut, save_state=True), sim.run(T - cut, save_state=True)]
    rng = np.random.default_rng(seed)
    dl = [torch.as_tensor(rng.normal(size=(c["bits"].shape[0], ne)).astype(np.float32), device="cuda") for c in chunks]
    one = training.Glif3Bptt(sim, dampening=0.3, blocked=True, n_blocks=n_blocks, two_steps=False)
    two = training.Glif3Bptt(sim, dampening=0.3, blocked=True, n_blocks=n_blocks, two_steps=True)
    assert one.gz_planes == 8 and two.gz_planes == 16
    for b in (one, two):
        for c, d in zip(reversed(chunks), reversed(dl)):       # chunks in reverse time order
            b.backward(c, dl_dz=d)
    for name in ("lam_V", "lam_asc", "lam_y1", "lam_y2", "lam_ring"):
        assert torch.equal(getattr(one, name), getattr(two, name)), name
    assert float(one.lam_V.abs().max()) > 0
    for name in ("d_rec_w", "d_inp_w"):
        got, want = getattr(two, name), getattr(one, name)
        assert float(want.abs().max()) > 0 or steps < 30        # (a few steps from rest: nothing has fired yet)
        assert float((got - want).abs().max()) <= 1e-6 * float(want.abs().max()), name


def test_blocked_form_with_the_gradient_in_source_major_order():
    """A caller of the C interface may give the blocked table for the transposed propagation and still ask for the
    recurrent gradient in the order of the source-major table (``d_rec_w`` without ``d_blk_w``): a launch of its
    own per step, which in the two-step form must come before the state adjoint.  Equal to the gradient that rides
    along, brought back through the sort permutation (1e-6 of the largest: other order of additions)."""
    import ctypes
    from bmtk_amd import _lib
    cfg = _net(32, 14, steps=41)
    n, T = cfg["n"], cfg["steps"]
    sim = Glif3Simulator(n, cfg["par"], cfg["h"], batch=32, rec=cfg["rec_src"], inp=cfg["inp_src"],
                         ring_slots=cfg["L"], resident=False)
    sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
    fwd = sim.run(T, save_state=True)
    dl = torch.as_tensor(np.random.default_rng(1).normal(size=(T, n * 32)).astype(np.float32), device="cuda")
    want = training.Glif3Bptt(sim, dampening=0.3, blocked=True, n_blocks=8)
    want.backward(fwd, dl_dz=dl)
    assert float(want.d_rec_w.abs().max()) > 0
    for two_steps in (True, False):
        b = training.Glif3Bptt(sim, dampening=0.3, blocked=True, n_blocks=8, two_steps=two_steps)
        a, step0, n_steps = b._struct(fwd, None, dl, True)
        a.d_blk_w = None
        a.d_rec_w = b.d_rec_w.data_ptr()
        _lib.check(_lib.load().bmtk_glif3_simulate_bwd(ctypes.byref(a), step0, n_steps, None))
        torch.cuda.synchronize()
        assert float((b.d_rec_w - want.d_rec_w).abs().max()) <= 1e-6 * float(want.d_rec_w.abs().max()), two_steps
        assert torch.equal(b.lam_V, want.lam_V) and torch.equal(b.lam_ring, want.lam_ring)


@pytest.mark.parametrize("seed", range(10))
def test_two_step_backward_on_randomly_shaped_networks(seed):
    """Networks of odd sizes (so that the last workgroups hold few rows or none, ranges are empty, rows end within a
    record group), batches that fill a lane group partly (20, 24, 28) or fully (32, 64), class tables, runs cut into
    chunks of odd and even lengths: the two-step form of the blocked backward pass leaves the same adjoint state as
    the one-step form, bit for bit, and the same gradients to 1e-6 of the largest."""
    rng = np.random.default_rng(1000 + seed)
    batch = int(rng.choice([20, 24, 28, 32, 64]))
    n = int(rng.integers(9, 400))
    n_in = int(rng.integers(3, 60))
    steps = int(rng.integers(20, 60))
    n_blocks = int(rng.choice([8, 16, 24, 64]))
    cfg = synthetic.small_glif3_network(n=n, n_in=n_in, steps=steps, seed=seed, in_rate=40.0, in_w_scale=15.0, w_scale=4.0,
                                        in_fanout=max(1, n // 3), p_conn=float(rng.uniform(0.02, 0.3)), batch=batch,
                                        n_classes=int(rng.integers(2, 7)) if seed % 2 else None)
    sim = Glif3Simulator(n, cfg["par"], cfg["h"], batch=batch, class_id=cfg.get("class_id"), rec=cfg["rec_src"],
                         inp=cfg["inp_src"], ring_slots=cfg["L"], resident=False)
    sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
    cuts = sorted(set(int(c) for c in rng.integers(1, steps, size=int(rng.integers(0, 4)))))
    lengths = np.diff([0] + cuts + [steps])
    chunks = [sim.run(int(m), save_state=True) for m in lengths]
    dl = [torch.as_tensor(rng.normal(size=(int(m), n * batch)).astype(np.float32), device="cuda") for m in lengths]
    one = training.Glif3Bptt(sim, dampening=0.3, blocked=True, n_blocks=n_blocks, two_steps=False)
    two = training.Glif3Bptt(sim, dampening=0.3, blocked=True, n_blocks=n_blocks, two_steps=True)
    for b in (one, two):
        for c, d in zip(reversed(chunks), reversed(dl)):
            b.backward(c, dl_dz=d)
    for name in ("lam_V", "lam_asc", "lam_y1", "lam_y2", "lam_ring"):
        assert torch.equal(getattr(one, name), getattr(two, name)), (name, batch, n, n_blocks, list(lengths))
    assert float(one.lam_V.abs().max()) > 0
    for name in ("d_rec_w", "d_inp_w"):
        got, want = getattr(two, name), getattr(one, name)
        assert float((got - want).abs().max()) <= 1e-6 * max(float(want.abs().max()), 1e-30), (name, batch, n)
