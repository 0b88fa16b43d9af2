"""GPU parity of the fused forward simulation against the CPU oracle."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import glif3_oracle as orc
from bmtk_amd import network as net, synthetic
from bmtk_amd.glif_utils import convert_aibs2nest, params_table
from bmtk_amd.simulator import Glif3Simulator
from gpu_util import rel_err

pytestmark = pytest.mark.gpu


def _oracle_run(cfg, dtype, steps=None, batch=1, in_ptr=None, in_events=None):
    prop = orc.precompute(cfg["par"], cfg["h"])
    n = cfg["n"]
    st = orc.new_state(n, batch, dtype)
    ring = np.zeros((cfg["L"], 4, n * batch), dtype)
    out = orc.simulate(st, prop, cfg["h"], steps or cfg["steps"], batch=batch, class_id=cfg["class_id"], ring=ring,
                       rec=cfg["rec_src"], inp=cfg["inp_src"],
                       in_ptr=cfg["in_ptr"] if in_ptr is None else in_ptr,
                       in_events=cfg["in_events"] if in_events is None else in_events, raster=True)
    return out, st, ring


def _gpu_sim(cfg, batch=1, in_ptr=None, in_events=None, resident=False, single_workgroup=True):
    if resident == "many":       # the many-workgroup form of the resident kernel also where one workgroup would do
        resident, single_workgroup = True, False
    sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], batch=batch, class_id=cfg["class_id"], rec=cfg["rec_src"],
                         inp=cfg["inp_src"], ring_slots=cfg["L"], resident=resident, single_workgroup=single_workgroup)
    assert bool(sim.res_span) == bool(resident)
    sim.set_input_events(cfg["in_ptr"] if in_ptr is None else in_ptr,
                         cfg["in_events"] if in_events is None else in_events)
    return sim


@pytest.mark.parametrize("resident", [False, True, "many"])
@pytest.mark.parametrize("classes", [None, 11])
def test_450_neuron_network_raster_and_state(classes, resident):
    """The 450-GLIF3 shape (Erdos-Renyi p=0.1, 1000 Poisson inputs at 10 Hz x 50
    targets, delays 1-4, dt 1 ms, 1000 steps); input weights doubled so the
    network fires at ~5 Hz.  Raster: >= 99.9 % of (neuron, step) entries equal
    to the fp64 oracle's.  State after the first 100 steps (compared only while
    the rasters are still identical): 1e-5 relative against the fp32 oracle,
    2e-4 against the fp64 oracle, values below one unit (mV / pA) held absolutely.  The 1e-5 single-step
    bound against fp64 is checked in test_gpu_state_update.py."""
    cfg = synthetic.small_glif3_network(n=450, n_in=1000, steps=1000, seed=0, in_w_scale=2.0, n_classes=classes)
    want, _, _ = _oracle_run(cfg, np.float64)
    sim = _gpu_sim(cfg, resident=resident)
    out = sim.run(100)
    w100, st100, ring100 = _oracle_run(cfg, np.float64, steps=100)
    f100, sf100, rf100 = _oracle_run(cfg, np.float32, steps=100)
    ras100 = sim.raster(out["bits"]).cpu().numpy()
    got = sim.state.to_numpy()
    if np.array_equal(ras100, f100["raster"]):
        # same fp32 update; only the order of the atomic additions differs
        for k in ("V", "asc", "y1", "y2"):
            assert rel_err(got[k], sf100[k], 1.0) < 1e-5, k
        np.testing.assert_array_equal(got["ref"], sf100["ref"])
        assert rel_err(sim.ring.cpu().numpy(), rf100, 1.0) < 1e-5
    if np.array_equal(ras100, w100["raster"]):
        # against fp64 the fp32 rounding of 100 chained steps has accumulated: 2e-4
        for k in ("V", "asc", "y1", "y2"):
            assert rel_err(got[k], st100[k], 1.0) < 2e-4, k
    assert (ras100 == w100["raster"]).mean() >= 0.999
    out2 = sim.run(900)
    ras = np.concatenate([ras100, sim.raster(out2["bits"]).cpu().numpy()])
    assert want["count"] > 1000
    agree = (ras == want["raster"]).mean()
    assert agree >= 0.999, agree
    # spike list from the compaction kernels == nonzero of the raster
    steps, elems = sim.spikes_from_bits(out2["bits"], step0=100)
    tt, ee = np.nonzero(ras[100:])
    np.testing.assert_array_equal(steps.cpu().numpy(), tt + 100)
    np.testing.assert_array_equal(elems.cpu().numpy(), ee)
    assert sim.synaptic_events(out2["bits"]) == int(np.diff(cfg["rec_src"][0])[ee].sum())


@pytest.mark.parametrize("resident", [False, True])
def test_reference_known_answer_on_gpu(golden_dir, resident):
    """The reference's GLIF3 known-answer protocol run through the GPU path:
    spike time = (step + crossing fraction) * h must hit 14.46548367 ms
    (bmtk/tests/simulator/pointnet/test_glif_utils.py:19) to 1e-3 ms in fp32."""
    kat = json.load(open(os.path.join(golden_dir, "glif_kat.json")))
    for model, exp in kat["expected"].items():
        aibs = json.load(open(os.path.join(golden_dir, exp["file"])))
        _, cell = convert_aibs2nest(model, aibs)
        par, asc_init, u_init = params_table([cell])
        h = 0.1
        pr = kat["protocol"]
        d = int(round(pr["delay_ms"] / h))
        inp = (np.array([0, 1], np.int32), np.array([0], np.int32), np.array([pr["spike_weight_pA"]], np.float32),
               np.array([d], np.uint8), np.array([pr["receptor_type"] - 1], np.uint8))
        n_steps = int(round(pr["tstop_ms"] / h))
        stamps = np.rint(np.array(pr["spike_times_ms"]) / h).astype(np.int64)
        in_ptr = np.zeros(n_steps + 1, np.int64)
        np.add.at(in_ptr, stamps, 1)
        sim = Glif3Simulator(1, par, h, inp=inp, asc_init=asc_init, u_init=u_init, resident=resident)
        sim.set_input_events(np.cumsum(in_ptr), np.zeros(len(stamps), np.int32))
        out = sim.run(n_steps, record_cap=16)
        rec = out["record"]
        c = int(rec["count"].item())
        assert c == len(exp["times"])
        t = (rec["step"][:c].cpu().numpy() + rec["frac"][:c].cpu().numpy().astype(np.float64)) * h
        np.testing.assert_allclose(t, exp["times"], atol=1e-3, rtol=0)


def test_batched_trials_are_independent():
    """Three trials with different input events in one batched run equal three
    single-trial oracle runs."""
    B = 3
    cfg = synthetic.small_glif3_network(n=200, n_in=300, steps=300, seed=3, in_w_scale=3.0, in_fanout=40)
    rng = np.random.default_rng(4)
    per_trial = [synthetic.poisson_events(rng, 300, 10.0, 1.0, 300) for _ in range(B)]
    counts = sum(np.diff(p) for p, _ in per_trial)
    in_ptr = np.concatenate(([0], np.cumsum(counts)))
    ev = []
    for t in range(300):
        step_ev = np.concatenate([e[p[t]:p[t + 1]].astype(np.int64) * B + b for b, (p, e) in enumerate(per_trial)])
        ev.append(np.sort(step_ev))
    in_events = np.concatenate(ev).astype(np.int32)
    sim = _gpu_sim(cfg, batch=B, in_ptr=in_ptr, in_events=in_events)   # batched runs use the per-step launches
    out = sim.run(300)
    ras = sim.raster(out["bits"]).cpu().numpy().reshape(300, cfg["n"], B)
    total = 0
    for b, (p, e) in enumerate(per_trial):
        want, _, _ = _oracle_run(cfg, np.float64, in_ptr=p, in_events=e)
        total += want["count"]
        assert (ras[:, :, b] == want["raster"]).mean() >= 0.999
    assert total > 300
    # and the batched oracle agrees with itself
    wb, _, _ = _oracle_run(cfg, np.float64, batch=B, in_ptr=in_ptr, in_events=in_events)
    assert (ras.reshape(300, -1) == wb["raster"]).mean() >= 0.999


@pytest.mark.parametrize("resident", [False, True])
def test_no_synapses_and_constant_current(resident):
    """Neither table present: the run is the bare state update driven by i_ext."""
    rng = np.random.default_rng(6)
    n, h = 1000, 1.0
    par = synthetic.random_cells(rng, n)
    I = rng.uniform(0, 600, n).astype(np.float32)
    sim = Glif3Simulator(n, par, h, i_ext=I, ring_slots=2, resident=resident)
    out = sim.run(400)
    ras = sim.raster(out["bits"]).cpu().numpy()
    prop = orc.precompute(par, h)
    st = orc.new_state(n, 1, np.float64)
    ring = np.zeros((2, 4, n))
    want = orc.simulate(st, prop, h, 400, ring=ring, i_ext=I.astype(np.float64), raster=True)
    assert want["count"] > 1000
    assert (ras == want["raster"]).mean() >= 0.999


def test_simulate_argument_errors():
    cfg = synthetic.small_glif3_network(n=50, n_in=10, steps=20, seed=1)
    with pytest.raises(ValueError):
        Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], rec=cfg["rec_src"], ring_slots=2)   # delays up to 4 need 5 slots
    sim = _gpu_sim(cfg)
    with pytest.raises(ValueError):
        sim.run(21)                                                                          # beyond the input lists
    with pytest.raises(ValueError):
        sim.set_input_events(np.array([0, 1]), np.array([10 ** 6], np.int32))


def test_resident_mode_multiple_workgroups_and_split_runs():
    """A 3000-neuron network spans dozens of resident workgroups, so spikes
    cross the grid barrier; two runs back to back must continue seamlessly and
    both modes must agree with the oracle."""
    cfg = synthetic.small_glif3_network(n=3000, n_in=500, steps=400, seed=8, in_w_scale=3.0, in_fanout=300,
                                        p_conn=0.03, w_scale=1.5)
    want, _, _ = _oracle_run(cfg, np.float64)
    assert want["count"] > 2000
    for resident in (True, False):
        sim = _gpu_sim(cfg, resident=resident)
        if resident:
            assert sim.res_groups > 8
        a = sim.run(150)
        b = sim.run(250)
        ras = np.concatenate([sim.raster(a["bits"]).cpu().numpy(), sim.raster(b["bits"]).cpu().numpy()])
        assert (ras == want["raster"]).mean() >= 0.999


def _integer_weights(csr):
    """Same table with weights rounded to multiples of 1/4 pA: every partial sum
    is then exact in fp32, whatever the order of the additions."""
    indptr, indices, w, d, r = csr
    return indptr, indices, (np.round(w * 4.0) / 4.0 + np.sign(w) * 0.25).astype(np.float32), d, r


def test_exact_weights_make_every_path_bit_identical():
    """With weights that are exactly representable multiples of 0.25 pA the
    ring sums do not depend on addition order, so the per-step launches, the
    resident kernel and the fp32 oracle must agree to the bit on raster, state
    and ring after 1000 steps.  Any lost, duplicated or late delivery (a
    missed ballot, a race on a ring slot) breaks this."""
    cfg = synthetic.small_glif3_network(n=3000, n_in=500, steps=1000, seed=9, in_w_scale=3.0, in_fanout=300,
                                        p_conn=0.03, w_scale=1.5)
    cfg["rec_src"] = _integer_weights(cfg["rec_src"])
    cfg["inp_src"] = _integer_weights(cfg["inp_src"])
    want, st, ring = _oracle_run(cfg, np.float32)
    assert want["count"] > 5000
    for resident in (False, True):
        sim = _gpu_sim(cfg, resident=resident)
        a = sim.run(400)
        b = sim.run(600)
        ras = np.concatenate([sim.raster(a["bits"]).cpu().numpy(), sim.raster(b["bits"]).cpu().numpy()])
        np.testing.assert_array_equal(ras, want["raster"])
        got = sim.state.to_numpy()
        for k in ("V", "asc", "y1", "y2", "ref"):
            np.testing.assert_array_equal(got[k], st[k], err_msg=k)
        np.testing.assert_array_equal(sim.ring.cpu().numpy(), ring)


def test_v1_scale_resident_equals_per_step_launches():
    """230,924 neurons, ~70 M synapses, exact weights: the resident kernel (242
    workgroups, one grid barrier per step) and the per-step launches must emit
    identical spikes for 2000 steps, the resident run split into two calls."""
    import torch
    rng = np.random.default_rng(3)
    n, n_in, steps = 230924, 17400, 2000
    par = synthetic.random_cells(rng, 111)
    cid = rng.integers(0, 111, n).astype(np.int32)
    _, by_src, _ = synthetic.device_network(n, 300, "lognormal", seed=3)
    by_src = (by_src[0], by_src[1], (torch.round(by_src[2] * 4) / 4 + torch.sign(by_src[2]) * 0.25), by_src[3],
              by_src[4])
    inp = synthetic.device_input_table(n_in, n, 8_000_000, seed=4, w_scale=7.0)
    inp = (inp[0], inp[1], torch.round(inp[2] * 4) / 4 + 0.25, inp[3], inp[4])
    in_ptr, in_ev = synthetic.device_poisson_events(n_in, 5.0, 1.0, steps, seed=5)
    bits = []
    for resident in (False, True):
        sim = Glif3Simulator(n, par, 1.0, class_id=cid, rec=by_src, inp=inp, resident=resident)
        assert bool(sim.res_span) == resident
        sim.set_input_events(in_ptr, in_ev)
        if resident:
            out = {"bits": torch.cat([sim.run(777)["bits"], sim.run(steps - 777)["bits"]])}
        else:
            out = sim.run(steps)
        sim.check()
        bits.append(out["bits"].cpu())
        state = sim.state.to_numpy()
        if resident:
            for k in state:
                np.testing.assert_array_equal(state[k], first_state[k], err_msg=k)
        first_state = state
        del sim
    assert int(ops_popcount(bits[0])) > 1000000
    assert torch.equal(bits[0], bits[1])


def test_resident_with_every_thread_owning_an_element():
    """250,000 neurons on 248 workgroups make the span 1024: the sixteenth wavefront, which otherwise only looks at
    the grid barrier while the others update, has elements of its own here.  Same spikes and state as the
    per-step launches."""
    import torch
    rng = np.random.default_rng(5)
    n, n_in, steps = 250_000, 5000, 200
    par = synthetic.random_cells(rng, 37)
    cid = rng.integers(0, 37, n).astype(np.int32)
    _, by_src, _ = synthetic.device_network(n, 40, "lognormal", seed=6)
    by_src = (by_src[0], by_src[1], (torch.round(by_src[2] * 4) / 4 + torch.sign(by_src[2]) * 0.25) * 4.0, by_src[3],
              by_src[4])
    inp = synthetic.device_input_table(n_in, n, 2_000_000, seed=7, w_scale=9.0)
    inp = (inp[0], inp[1], torch.round(inp[2] * 4) / 4 + 0.25, inp[3], inp[4])
    in_ptr, in_ev = synthetic.device_poisson_events(n_in, 20.0, 1.0, steps, seed=8)
    bits, states = [], []
    for resident in (False, True):
        sim = Glif3Simulator(n, par, 1.0, class_id=cid, rec=by_src, inp=inp, resident=resident)
        assert bool(sim.res_span) == resident and (not resident or sim.res_span == 1024)
        sim.set_input_events(in_ptr, in_ev)
        out = sim.run(steps)
        sim.check()
        bits.append(out["bits"].cpu())
        states.append(sim.state.to_numpy())
        del sim
    assert int(ops_popcount(bits[0])) > 20000
    assert torch.equal(bits[0], bits[1])
    for k in states[0]:
        np.testing.assert_array_equal(states[0][k], states[1][k], err_msg=k)


def ops_popcount(bits):
    import torch
    x = bits.reshape(-1)
    return sum(int(((x >> s) & 1).sum()) for s in range(64))


@pytest.mark.parametrize("batch", [3, 32, 64])
def test_pull_form_of_the_per_step_driver(batch):
    """Batched runs sum the recurrent arrivals of a step in one pass over a target-major copy of the table
    (no global atomics).  With exact weights the run must equal the fp32 oracle bit for bit -- raster and state,
    after 150 + 250 steps as two calls (the history carries the spikes still under way across the calls) -- and
    so must the run that pushes arrivals into the ring."""
    cfg = synthetic.small_glif3_network(n=700, n_in=300, steps=400, seed=12, in_w_scale=3.0, in_fanout=100,
                                        p_conn=0.05, w_scale=1.5, batch=batch)
    cfg["rec_src"] = _integer_weights(cfg["rec_src"])
    cfg["inp_src"] = _integer_weights(cfg["inp_src"])
    want, st, _ = _oracle_run(cfg, np.float32, batch=batch)
    assert want["count"] > 1000 * batch // 4
    for pull, fused in ((True, False), (False, False)) + (((True, True),) if batch in (32, 64) else ()):
        sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], batch=batch, class_id=cfg["class_id"], rec=cfg["rec_src"],
                             inp=cfg["inp_src"], ring_slots=cfg["L"], resident=False, pull=pull, fused=fused)
        assert (sim.pull_table is not None) == (pull and not fused) and (sim.fuse_table is not None) == fused
        sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        a = sim.run(150)
        b = sim.run(250)
        ras = np.concatenate([sim.raster(a["bits"]).cpu().numpy(), sim.raster(b["bits"]).cpu().numpy()])
        np.testing.assert_array_equal(ras, want["raster"])
        got = sim.state.to_numpy()
        for k in ("V", "asc", "y1", "y2", "ref"):
            np.testing.assert_array_equal(got[k], st[k], err_msg=k)
    auto = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], batch=batch, class_id=cfg["class_id"], rec=cfg["rec_src"],
                          resident=False)
    # at the expected 3 Hz and 1 ms steps batches from 20 pull, in the fused form (trials fill whole bytes of bits)
    assert (auto.fuse_table is not None) == (batch in (32, 64)) and auto.pull_table is None
    busy = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], batch=batch, class_id=cfg["class_id"], rec=cfg["rec_src"],
                          resident=False, expected_rate_hz=40.0)
    assert (busy.pull_table is not None) == (batch == 3) and (busy.fuse_table is not None) == (batch != 3)


def test_resident_pull_with_more_fired_rows_than_its_list_holds():
    """20,000 identical neurons driven by the same current fire in the same steps: 20,000 fired rows in one step
    exceed the 8192 entries of the resident kernel's LDS list, so its workgroups fall back to pulling what each
    thread found itself.  Raster and state must still equal the fp32 oracle bit for bit."""
    n, steps = 20000, 60
    rng = np.random.default_rng(21)
    par = synthetic.random_cells(rng, 1)
    class_id = np.zeros(n, np.int32)
    nnz = 10 * n
    src, tgt = rng.integers(0, n, nnz), rng.integers(0, n, nnz)
    w = (rng.integers(1, 20, nnz) * 0.25).astype(np.float32)
    rec = net.coo_to_csr(src, tgt, w, rng.integers(1, 4, nnz), rng.integers(0, 4, nnz).astype(np.uint8), n, "source")
    i_ext = np.full(n, 900.0, np.float32)
    # and 5000 input sources that all fire in steps 5, 6 and 30: several passes of 1024 events per workgroup
    n_in = 5000
    isrc, itgt = np.repeat(np.arange(n_in), 4), rng.integers(0, n, 4 * n_in)
    inp = net.coo_to_csr(isrc, itgt, (rng.integers(1, 40, 4 * n_in) * 0.25).astype(np.float32),
                         rng.integers(1, 4, 4 * n_in), np.zeros(4 * n_in, np.uint8), n_in, "source")
    in_ptr = np.zeros(steps + 1, np.int64)
    for k in (5, 6, 30):
        in_ptr[k + 1:] += n_in
    in_events = np.tile(np.arange(n_in, dtype=np.int32), 3)
    prop = orc.precompute(par, 1.0)
    st = orc.new_state(n, 1, np.float32)
    ring = np.zeros((4, 4, n), np.float32)
    orc.set_threads(1)
    want = orc.simulate(st, prop, 1.0, steps, class_id=class_id, ring=ring, rec=rec, inp=inp, in_ptr=in_ptr,
                        in_events=in_events, i_ext=i_ext, raster=True)
    per_step = want["raster"].sum(1)
    assert per_step.max() > 8192  # the case this test is about
    sim = Glif3Simulator(n, par, 1.0, class_id=class_id, rec=rec, inp=inp, i_ext=i_ext, resident=True)
    sim.set_input_events(in_ptr, in_events)
    out = sim.run(steps)
    sim.check()
    np.testing.assert_array_equal(sim.raster(out["bits"]).cpu().numpy(), want["raster"])
    got = sim.state.to_numpy()
    for k in ("V", "asc", "y1", "y2", "ref"):
        np.testing.assert_array_equal(got[k], st[k], err_msg=k)


def test_resident_barrier_gives_up_cleanly():
    """Failure handling of the grid barrier, forced from the host: with a spin limit of one poll some workgroup
    finds the barrier unfinished, raises the abort word, every workgroup leaves its loop and the kernel ends
    normally; check() then reports the run as invalid.  A following run with the normal limit works."""
    cfg = synthetic.small_glif3_network(n=3000, n_in=500, steps=300, seed=8, in_w_scale=3.0, in_fanout=300,
                                        p_conn=0.03, w_scale=1.5)
    sim = _gpu_sim(cfg, resident=True)
    assert sim.res_groups > 8
    sim.spin_limit = 1
    sim.hist_slots = 3  # no spare history row: the wait closes every step, when the barrier has only begun to fill
    sim.run(200)
    sim.spin_limit = 0
    sim.run(100)            # finds the abort word set and does nothing: the failure cannot be overwritten unseen
    with pytest.raises(RuntimeError, match="barrier"):
        sim.check()
    assert int(sim.res_sync[1].item()) == 0   # cleared by the check that reported it
    want, _, _ = _oracle_run(cfg, np.float64)
    sim = _gpu_sim(cfg, resident=True)
    out = sim.run(300)
    sim.check()
    assert (sim.raster(out["bits"]).cpu().numpy() == want["raster"][:300]).mean() >= 0.999


@pytest.mark.parametrize("every", [1, 3])
def test_membrane_probes_equal_the_per_step_record(every):
    """set_probes on both drivers against the full per-step record of the launch-per-step driver: same potentials,
    bit for bit (exact weights), at the sampled steps, over two calls whose boundary is no multiple of `every`."""
    cfg = synthetic.small_glif3_network(n=3000, n_in=500, steps=200, seed=8, in_w_scale=3.0, in_fanout=300,
                                        p_conn=0.03, w_scale=1.5)
    cfg["rec_src"] = _integer_weights(cfg["rec_src"])
    cfg["inp_src"] = _integer_weights(cfg["inp_src"])
    ref = _gpu_sim(cfg, resident=False)
    full = ref.run(200, save_state=True)["saved"]["v"].view(200, cfg["n"]).cpu().numpy()
    ids = np.array([2999, 0, 17, 1500, 64, 959, 960])
    for resident in (False, True):
        sim = _gpu_sim(cfg, resident=resident)
        sim.set_probes(ids, every=every)
        got_v, got_steps = [], []
        for n in (70, 130):
            out = sim.run(n)["probe"]
            got_v.append(out["v"].cpu().numpy())
            got_steps.append(out["steps"].numpy())
        sim.check()
        steps = np.concatenate(got_steps)
        np.testing.assert_array_equal(steps, np.arange(every - 1, 200, every))
        np.testing.assert_array_equal(np.concatenate(got_v), full[steps][:, ids])
    with pytest.raises(ValueError):
        sim.set_probes([1, 1])
    with pytest.raises(ValueError):
        sim.set_probes([cfg["n"]])


def _with_duplicate_events(cfg, rng, batch):
    """The event lists of `cfg` with every fifth event of a step doubled or tripled (two or three spikes of one
    source inside one step, which NEST delivers one by one), still ascending within each step."""
    ptr, ev = cfg["in_ptr"], cfg["in_events"]
    new_ptr, chunks = [0], []
    for t in range(ptr.size - 1):
        e = ev[ptr[t]:ptr[t + 1]]
        extra = np.repeat(e[::5], rng.integers(1, 3, e[::5].size))
        e = np.sort(np.concatenate([e, extra]))
        chunks.append(e)
        new_ptr.append(new_ptr[-1] + e.size)
    return np.asarray(new_ptr, np.int64), np.concatenate(chunks).astype(np.int32)


@pytest.mark.parametrize("batch,resident", [(1, False), (1, True), (1, "many"), (8, False), (8, "unfused"), (32, False)])
def test_repeated_input_events_within_a_step_are_all_delivered(batch, resident):
    """Two spikes of one generator inside one resolution step are two deliveries.  Every driver must count them:
    the launch-per-step driver, the resident one, and the batched driver, whose pull form of the inputs (bit rows:
    one bit per id and step) delivers the second and later occurrences as events on top.  Exact weights:
    bit-identical to the fp32 oracle."""
    cfg = synthetic.small_glif3_network(n=700, n_in=300, steps=300, seed=14, in_w_scale=3.0, in_fanout=100,
                                        in_rate=30.0, p_conn=0.05, w_scale=1.5, batch=batch)
    cfg["rec_src"] = _integer_weights(cfg["rec_src"])
    cfg["inp_src"] = _integer_weights(cfg["inp_src"])
    in_ptr, in_events = _with_duplicate_events(cfg, np.random.default_rng(3), batch)
    assert in_events.size > 1.2 * cfg["in_events"].size
    want, st, _ = _oracle_run(cfg, np.float32, batch=batch, in_ptr=in_ptr, in_events=in_events)
    plain, _, _ = _oracle_run(cfg, np.float32, batch=batch)
    assert want["count"] > 1.05 * plain["count"] > 500 * batch      # the repeats matter
    if resident == "many":       # 700 neurons on a dozen workgroups instead of one
        kw = dict(resident=True, single_workgroup=False)
    elif resident == "unfused":  # the batched driver with pull and update as separate launches
        kw = dict(resident=False, fused=False, pull=True)
        resident = False
    else:
        kw = dict(resident=resident, pull=True) if batch >= 8 else dict(resident=resident)
    sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], batch=batch, class_id=cfg["class_id"], rec=cfg["rec_src"],
                         inp=cfg["inp_src"], ring_slots=cfg["L"], **kw)
    assert sim.res_groups == (0 if not resident else 1 if resident is True else 11)
    sim.set_input_events(in_ptr, in_events)
    assert sim.in_duplicates
    a, b = sim.run(120), sim.run(180)
    sim.check()
    if batch >= 8:
        if kw.get("fused", True):
            assert sim.fuse_table is not None and sim.pull_table is None
        else:
            assert sim.pull_table is not None and sim.pull_inp_table is not None
        n_rep = in_events.size - sum(np.unique(in_events[in_ptr[t]:in_ptr[t + 1]]).size for t in range(in_ptr.size - 1))
        assert sim.in_repeat_events.numel() == n_rep > 0 and int(sim.in_repeat_ptr[-1]) == n_rep
    ras = np.concatenate([sim.raster(a["bits"]).cpu().numpy(), sim.raster(b["bits"]).cpu().numpy()])
    np.testing.assert_array_equal(ras, want["raster"])
    got = sim.state.to_numpy()
    for k in ("V", "asc", "y1", "y2", "ref"):
        np.testing.assert_array_equal(got[k], st[k], err_msg=k)
    # device tensors take the same checks
    dev = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], batch=batch, class_id=cfg["class_id"], rec=cfg["rec_src"],
                         inp=cfg["inp_src"], ring_slots=cfg["L"], **kw)
    dev.set_input_events(torch.as_tensor(in_ptr, device="cuda"), torch.as_tensor(in_events, device="cuda"))
    assert dev.in_duplicates
    dev.set_input_events(torch.as_tensor(cfg["in_ptr"], device="cuda"), torch.as_tensor(cfg["in_events"], device="cuda"))
    assert not dev.in_duplicates
    bad = in_events.copy()
    k = int(in_ptr[np.flatnonzero(np.diff(in_ptr) >= 2)[0]])
    bad[k] = bad[k + 1] + 1 if bad[k + 1] + 1 < 300 * batch else bad[k]      # descending pair inside a step
    bad[k + 1] = bad[k + 1] if bad[k] > bad[k + 1] else bad[k] - 1
    for form in (lambda x: x, lambda x: torch.as_tensor(x, device="cuda")):
        with pytest.raises(ValueError, match="ascending"):
            dev.set_input_events(form(in_ptr), form(bad))


@pytest.mark.parametrize("resident", [False, True])
def test_spike_record_in_several_lists(resident):
    """A record large enough to be kept as several lists (one counter per group of workgroups instead of one for
    the whole network): joined by collect_record it holds exactly the spikes of the raster, with the fractions of
    the single-list record; a list that runs full is reported."""
    import torch
    from bmtk_amd.simulator import RECORD_WAYS
    cfg = synthetic.small_glif3_network(n=20000, n_in=2000, steps=120, seed=21, in_w_scale=6.0, in_fanout=200,
                                        in_rate=40.0, p_conn=0.002, w_scale=2.0)
    cfg["rec_src"] = _integer_weights(cfg["rec_src"])       # exact sums: the runs below are the same run
    cfg["inp_src"] = _integer_weights(cfg["inp_src"])
    def run(cap, ways=None):
        sim = _gpu_sim(cfg, resident=resident)
        out = sim.run(cfg["steps"], record_cap=cap, record_ways=ways)
        return sim, out
    sim, out = run(RECORD_WAYS * 4096)
    # as many lists as the power of two below the number of workgroups (40 per-step), at most 64; the resident kernel
    # without slack gets 256, a list per workgroup, which appends to it with its count in a register
    assert out["record"]["ways"] == (256 if resident else 32) and bool(sim.res_span) == resident
    assert not resident or sim.res_groups > RECORD_WAYS
    rec = sim.collect_record(out["record"])
    ras = sim.raster(out["bits"]).cpu().numpy()
    assert rec["count"] == int(ras.sum()) > 20000 and not rec["overflow"]
    got = np.zeros_like(ras)
    np.add.at(got, (rec["step"].cpu().numpy(), rec["elem"].cpu().numpy()), 1)
    np.testing.assert_array_equal(got, ras)                       # every spike once, none invented
    # ordered on the device: by time (step + fraction) * resolution, ties by element, as numpy's lexsort orders them
    srt = sim.collect_record(out["record"], sort_scale=0.1)
    st, fr, el = (rec[k].cpu().numpy() for k in ("step", "frac", "elem"))
    t = (st.astype(np.float64) + fr.astype(np.float64)) * 0.1
    order = np.lexsort((el, t))
    np.testing.assert_array_equal(srt["time"].cpu().numpy(), t[order])
    np.testing.assert_array_equal(srt["elem"].cpu().numpy(), el[order])
    sim1, out1 = run(60000, ways=1)                               # one list: the same spikes and fractions
    assert out1["record"]["ways"] == 1
    rec1 = sim1.collect_record(out1["record"])
    def keyed(r):
        key = r["step"].cpu().numpy().astype(np.int64) * cfg["n"] + r["elem"].cpu().numpy()
        order = np.argsort(key)
        return key[order], r["frac"].cpu().numpy()[order]
    k, f = keyed(rec)
    k1, f1 = keyed(rec1)
    np.testing.assert_array_equal(k, k1)
    np.testing.assert_array_equal(f, f1)
    sim64, out64 = run(RECORD_WAYS * 4096, ways=RECORD_WAYS)      # lists shared by workgroups: a counter in memory each
    assert out64["record"]["ways"] == RECORD_WAYS
    k64, f64 = keyed(sim64.collect_record(out64["record"]))
    np.testing.assert_array_equal(k, k64)
    np.testing.assert_array_equal(f, f64)
    frac = f
    assert frac.min() >= 0.0 and frac.max() <= 1.0
    # a record too small for the run: counted in full, reported as incomplete
    sim2 = _gpu_sim(cfg, resident=resident)
    small = sim2.collect_record(sim2.run(cfg["steps"], record_cap=2000)["record"])
    assert small["overflow"] and small["count"] == rec["count"] and small["step"].numel() <= 2000


@pytest.mark.parametrize("n,max_delay,extra", [(1000, 4, 0), (333, 6, 0), (1024, 3, 40), (70, 2, 1)])
def test_single_workgroup_form_equals_the_other_drivers(n, max_delay, extra):
    """A network of up to 1024 neurons runs in ONE workgroup (no grid barrier, ballots handed over in LDS or, with
    a delay offset, through the history).  Exact weights: raster, state, ring, membrane probes and spike record
    equal those of the launch-per-step driver and of the many-workgroup form bit for bit, over three calls."""
    import torch
    cfg = synthetic.small_glif3_network(n=n, n_in=200, steps=400, seed=31 + n, in_w_scale=8.0, in_fanout=min(n, 60),
                                        in_rate=40.0, p_conn=min(0.3, 40.0 / n), w_scale=2.0, max_delay=max_delay)
    for key in ("rec_src", "inp_src"):
        indptr, indices, w, d, r = _integer_weights(cfg[key])
        cfg[key] = (indptr, indices, w, d.astype(np.int32) + extra, r)
    ids = np.unique(np.array([0, n // 2, n - 1]))
    outs = {}
    for name, kw in (("step", dict(resident=False)), ("one", dict(resident=True)),
                     ("many", dict(resident=True, single_workgroup=False))):
        sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], class_id=cfg["class_id"], rec=cfg["rec_src"],
                             inp=cfg["inp_src"], delay_offset=extra, **kw)
        assert sim.delay_offset == extra and sim.res_groups == {"step": 0, "one": 1}.get(name, sim.res_groups)
        if name == "many":
            assert sim.res_groups > 1
        sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        sim.set_probes(ids, every=3)
        bits, probes, recs = [], [], []
        for steps in (1, 149, 250):
            out = sim.run(steps, record_cap=1 << 17)
            bits.append(out["bits"])
            probes.append(out["probe"]["v"])
            rec = sim.collect_record(out["record"], sort_scale=1.0)
            assert not rec["overflow"]
            recs.append(torch.stack([rec["time"], rec["elem"].double()]))
        sim.check()
        outs[name] = dict(bits=torch.cat(bits).cpu().numpy(), probe=torch.cat(probes).cpu().numpy(),
                          rec=torch.cat(recs, dim=1).cpu().numpy(), state=sim.state.to_numpy(),
                          ring=sim.ring.cpu().numpy())
    assert int(ops_popcount(torch.as_tensor(outs["step"]["bits"]))) > 2 * n
    for name in ("one", "many"):
        for k in ("bits", "probe", "rec", "ring"):
            np.testing.assert_array_equal(outs[name][k], outs["step"][k], err_msg="%s %s" % (name, k))
        for k in outs["step"]["state"]:
            np.testing.assert_array_equal(outs[name]["state"][k], outs["step"]["state"][k], err_msg="%s %s" % (name, k))


def test_lists_of_fired_neurons_equal_the_ballots():
    """Beside its ballots a workgroup of the many-workgroup form publishes the neurons that fired as a list of 16
    places, which the other workgroups read instead of expanding the ballots; a step in which some workgroup had more
    spikes than places is read from the ballots.  A network driven into volleys (steps with 40 spikes in one
    workgroup) between quiet stretches (steps with a few) takes both ways: raster, state and ring equal those of a run
    that never uses the lists and those of the launch-per-step driver, bit for bit, over three calls."""
    import torch
    n = 300
    cfg = synthetic.small_glif3_network(n=n, n_in=100, steps=600, seed=77, in_w_scale=8.0, in_fanout=60, in_rate=30.0,
                                        p_conn=0.1, w_scale=2.0, max_delay=4, n_classes=1)
    for key in ("rec_src", "inp_src"):
        cfg[key] = _integer_weights(cfg[key])
    rng = np.random.default_rng(5)
    i_ext = np.where(np.arange(n) % 64 < 40, 3000.0, rng.uniform(0.0, 300.0, n)).astype(np.float32)  # 40 of 64 in step
    outs = {}
    for name, kw in (("step", dict(resident=False)), ("lists", dict(resident=True, single_workgroup=False)),
                     ("ballots", dict(resident=True, single_workgroup=False, fired_lists=False))):
        sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], class_id=cfg["class_id"], rec=cfg["rec_src"],
                             inp=cfg["inp_src"], i_ext=i_ext, **kw)
        if name != "step":
            assert sim.res_groups == 5 and (sim.res_fired is not None) == (name == "lists")
        sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        bits = [sim.run(steps)["bits"] for steps in (1, 249, 350)]
        sim.check()
        outs[name] = dict(raster=sim.raster(torch.cat(bits)).cpu().numpy(), state=sim.state.to_numpy(),
                          ring=sim.ring.cpu().numpy())
    per_group = np.add.reduceat(outs["step"]["raster"].astype(np.int64), np.arange(0, n, 64), axis=1)  # [steps][5]
    busiest = per_group.max(axis=1)
    assert (busiest > 16).sum() >= 50 and ((busiest >= 1) & (busiest <= 16)).sum() >= 50   # both ways are taken
    for name in ("lists", "ballots"):
        for k in ("raster", "ring"):
            np.testing.assert_array_equal(outs[name][k], outs["step"][k], err_msg="%s %s" % (name, k))
        for k in outs["step"]["state"]:
            np.testing.assert_array_equal(outs[name]["state"][k], outs["step"]["state"][k], err_msg="%s %s" % (name, k))


@pytest.mark.parametrize("extra", [0, 2, 6])
def test_single_workgroup_form_with_more_spikes_and_events_than_its_lists_hold(extra):
    """The single-workgroup form hands the rows to walk from step to step as items in LDS: up to 512 fired neurons
    and up to 128 input events; what exceeds them is taken from the ballots and from the event list in place.  800 of
    1024 neurons driven in step (volleys of more than 512 between steps with a few spikes) and 93-148 input events
    per step take every way, without a delay offset (ballots in LDS), with one shorter than the kernel's near rows
    and with a longer one (ballots through the history): raster, state, ring and spike record equal those of the
    launch-per-step driver bit for bit, over three calls."""
    import torch
    n = 1024
    cfg = synthetic.small_glif3_network(n=n, n_in=600, steps=500, seed=91, in_w_scale=4.0, in_fanout=30, in_rate=200.0,
                                        p_conn=0.03, w_scale=1.0, max_delay=3, n_classes=1)
    for key in ("rec_src", "inp_src"):
        indptr, indices, w, d, r = _integer_weights(cfg[key])
        cfg[key] = (indptr, indices, w, d.astype(np.int32) + extra, r)
    rng = np.random.default_rng(5)
    i_ext = np.where(np.arange(n) < 800, 3000.0, rng.uniform(0.0, 300.0, n)).astype(np.float32)
    events = np.diff(cfg["in_ptr"])[:500]
    assert (events > 128).sum() >= 50 and (events <= 128).sum() >= 50
    outs = {}
    for name, kw in (("step", dict(resident=False)), ("one", dict(resident=True))):
        sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], class_id=cfg["class_id"], rec=cfg["rec_src"],
                             inp=cfg["inp_src"], i_ext=i_ext, delay_offset=extra, **kw)
        assert sim.delay_offset == extra and sim.res_groups == (1 if name == "one" else 0)
        sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        bits, recs = [], []
        for steps in (1, 199, 300):
            out = sim.run(steps, record_cap=1 << 19)
            bits.append(out["bits"])
            rec = sim.collect_record(out["record"], sort_scale=1.0)
            assert not rec["overflow"]
            recs.append(torch.stack([rec["time"], rec["elem"].double()]))
        sim.check()
        outs[name] = dict(raster=sim.raster(torch.cat(bits)).cpu().numpy(), rec=torch.cat(recs, dim=1).cpu().numpy(),
                          state=sim.state.to_numpy(), ring=sim.ring.cpu().numpy())
    per_step = outs["step"]["raster"].sum(axis=1)
    assert (per_step > 512).sum() >= 20 and ((per_step >= 1) & (per_step <= 512)).sum() >= 100
    for k in ("raster", "rec", "ring"):
        np.testing.assert_array_equal(outs["one"][k], outs["step"][k], err_msg=k)
    for k in outs["step"]["state"]:
        np.testing.assert_array_equal(outs["one"]["state"][k], outs["step"]["state"][k], err_msg=k)


@pytest.mark.parametrize("n,empty", [(1, ""), (2, ""), (65, "rec"), (65, "inp"), (2049, "rec"), (2049, "rec inp")])
def test_tiny_networks_and_tables_without_a_synapse(n, empty):
    """One neuron (which has nobody to connect to), two, and networks whose recurrent or input table has rows but no
    synapse at all (a population that projects nowhere): every driver runs them, calls of 0 steps included, with
    the raster, state and ring of the launch-per-step driver, bit for bit (exact weights)."""
    import torch
    cfg = synthetic.small_glif3_network(n=n, n_in=20, steps=200, seed=3, in_w_scale=30.0, in_fanout=min(n, 5),
                                        in_rate=100.0, p_conn=min(1.0, 8.0 / max(n, 2)), w_scale=5.0, max_delay=3)
    for key in ("rec_src", "inp_src"):
        indptr, indices, w, d, r = _integer_weights(cfg[key])
        if key[:3] in empty.split():
            indptr, indices, w, d, r = np.zeros_like(indptr), indices[:0], w[:0], d[:0], r[:0]
        cfg[key] = (indptr, indices, w, d, r)
    if n == 1:
        assert cfg["rec_src"][1].size == 0
    outs = {}
    for name, kw in (("step", dict(resident=False)), ("one", dict(resident=True)),
                     ("many", dict(resident=True, single_workgroup=False))):
        sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], class_id=cfg["class_id"], rec=cfg["rec_src"],
                             inp=cfg["inp_src"], i_ext=np.full(n, 400.0, np.float32), **kw)
        sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        bits = []
        for steps in (0, 1, 37, 0, 100):
            out = sim.run(steps, record_cap=1 << 14)
            bits.append(out["bits"])
            rec = sim.collect_record(out["record"], sort_scale=1.0)
            assert rec["count"] == int(sim.raster(out["bits"]).sum()) and not rec["overflow"]
        sim.check()
        outs[name] = dict(raster=sim.raster(torch.cat(bits)).cpu().numpy(), state=sim.state.to_numpy(),
                          ring=sim.ring.cpu().numpy())
    assert outs["step"]["raster"].sum() >= 10 * min(n, 20)
    for name in ("one", "many"):
        for k in ("raster", "ring"):
            np.testing.assert_array_equal(outs[name][k], outs["step"][k], err_msg="%s %s" % (name, k))
        for k in outs["step"]["state"]:
            np.testing.assert_array_equal(outs[name]["state"][k], outs["step"]["state"][k], err_msg="%s %s" % (name, k))


def test_delay_offset_chosen_so_that_a_small_network_fits_one_workgroup():
    """450 cells whose delays are all 20 steps (bmtk's example networks at dt = 0.1 ms: 2 ms everywhere) need 21 ring
    slots, more than one workgroup's LDS holds for them; with the 19 steps all delays have in common taken off, two.
    The automatic choice takes them off and runs the single-workgroup form: same raster, state and spike record as
    the many-workgroup form with the full ring, bit for bit."""
    import torch
    n = 450
    cfg = synthetic.small_glif3_network(n=n, n_in=100, steps=900, seed=5, in_w_scale=8.0, in_fanout=60, in_rate=30.0,
                                        p_conn=0.08, w_scale=2.0, max_delay=1)
    for key in ("rec_src", "inp_src"):
        indptr, indices, w, d, r = _integer_weights(cfg[key])
        cfg[key] = (indptr, indices, w, np.full_like(d, 20), r)
    outs = {}
    for name, kw in (("auto", dict()), ("full ring", dict(delay_offset=0))):
        sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], class_id=cfg["class_id"], rec=cfg["rec_src"],
                             inp=cfg["inp_src"], **kw)
        assert (sim.delay_offset, sim.L, sim.res_groups) == ((19, 2, 1) if name == "auto" else (0, 21, 8))
        sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        bits, recs = [], []
        for steps in (1, 399, 500):
            out = sim.run(steps, record_cap=1 << 17)
            bits.append(out["bits"])
            rec = sim.collect_record(out["record"], sort_scale=1.0)
            assert not rec["overflow"]
            recs.append(torch.stack([rec["time"], rec["elem"].double()]))
        sim.check()
        outs[name] = dict(raster=sim.raster(torch.cat(bits)).cpu().numpy(), rec=torch.cat(recs, dim=1).cpu().numpy(),
                          state=sim.state.to_numpy())
    assert outs["auto"]["raster"].sum() > 2 * n
    np.testing.assert_array_equal(outs["auto"]["raster"], outs["full ring"]["raster"])
    np.testing.assert_array_equal(outs["auto"]["rec"], outs["full ring"]["rec"])
    for k in ("V", "asc", "y1", "y2", "ref"):
        np.testing.assert_array_equal(outs["auto"]["state"][k], outs["full ring"]["state"][k], err_msg=k)
