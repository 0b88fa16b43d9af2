"""Randomly shaped small networks through every forward driver.

Sizes that are not multiples of a wavefront, a single neuron, rows without synapses, no inputs at all, odd
batches, one-step and six-step delays, long delays, parameter classes or per-neuron parameters: with weights that
are multiples of 1/4 pA (sums exact in fp32, whatever their order) every driver must reproduce the fp32 oracle's
raster and state bit for bit.
"""
import numpy as np
import pytest

from oracle import glif3_oracle as orc
from bmtk_amd import synthetic
from bmtk_amd.simulator import Glif3Simulator

pytestmark = pytest.mark.gpu


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.choice([1, 2, 63, 64, 65, 130, 333, 900]))
    n_in = int(rng.choice([0, 1, 7, 40]))
    batch = int(rng.choice([1, 1, 1, 2, 5, 8, 16]))
    max_delay = int(rng.choice([1, 2, 4, 6]))
    extra = int(rng.choice([0, 0, 0, 70]))
    classes = int(rng.choice([0, 0, 3])) or None
    steps = 150
    cfg = synthetic.small_glif3_network(n=n, n_in=n_in, steps=steps, seed=seed, p_conn=float(rng.choice([0.0, 0.05, 0.5])),
                                        in_rate=60.0, in_fanout=max(1, min(n, 20)), max_delay=max_delay,
                                        n_classes=classes, batch=batch, w_scale=6.0, in_w_scale=40.0)
    for key in ("rec_src", "inp_src"):
        indptr, indices, w, d, r = cfg[key]
        cfg[key] = (indptr, indices, (np.round(w * 4.0) / 4.0 + np.sign(w) * 0.25).astype(np.float32),
                    d.astype(np.int32) + extra, r)
    cfg["extra"] = extra
    # a constant current per element, strong enough for a good part of the cells to fire without any input
    cfg["i_ext"] = rng.uniform(0.0, 600.0, n * batch).astype(np.float32)
    return cfg


@pytest.mark.parametrize("seed", range(16))
def test_every_driver_equals_the_oracle(seed):
    cfg = _case(seed)
    n, batch, steps = cfg["n"], cfg["batch"], cfg["steps"]
    has_rec = cfg["rec_src"][1].size > 0
    has_inp = cfg["n_in"] > 0
    rec = cfg["rec_src"] if has_rec else None
    inp = cfg["inp_src"] if has_inp else None
    L = int(max([1] + [int(t[3].max()) for t in (rec, inp) if t is not None])) + 1
    orc.set_threads(1)
    prop = orc.precompute(cfg["par"], cfg["h"])
    st = orc.new_state(n, batch, np.float32)
    ring = np.zeros((L, 4, n * batch), np.float32)
    want = orc.simulate(st, prop, cfg["h"], steps, batch=batch, class_id=cfg["class_id"], ring=ring, rec=rec, inp=inp,
                        in_ptr=cfg["in_ptr"] if has_inp else None, in_events=cfg["in_events"] if has_inp else None,
                        i_ext=cfg["i_ext"], raster=True)
    assert want["count"] > 0
    drivers = [dict(resident=False, pull=False)]
    if has_rec and cfg["extra"] == 0:
        drivers.append(dict(resident=False, pull=True, fused=False))   # pull and update as separate launches
    if (has_rec or has_inp) and cfg["extra"] == 0 and batch in (8, 16):
        drivers.append(dict(resident=False, fused=True))               # ... fused, lane = trial
    if batch == 1:
        drivers.append(dict(resident=True))                           # up to 1024 neurons: the single-workgroup form
        drivers.append(dict(resident=True, single_workgroup=False))   # the many-workgroup form at the same odd sizes
        drivers.append(dict(resident=True, single_workgroup=False, fired_lists=False))   # ... read from the ballots only
    for kw in drivers:
        sim = Glif3Simulator(n, cfg["par"], cfg["h"], batch=batch, class_id=cfg["class_id"], rec=rec, inp=inp,
                             i_ext=cfg["i_ext"], **kw)
        # delays beyond the ring's reach: all that the delays have in common is taken off
        least = min([int(t[3].min()) for t in (rec, inp) if t is not None and t[3].size] or [1])
        assert sim.delay_offset == (least - 1 if cfg["extra"] else 0)
        if kw.get("resident"):
            assert (sim.res_groups == 1) == (kw.get("single_workgroup", True) or n <= 64)
        if has_inp:
            sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        a = sim.run(60)
        b = sim.run(steps - 60)
        sim.check()
        ras = np.concatenate([sim.raster(a["bits"]).cpu().numpy(), sim.raster(b["bits"]).cpu().numpy()])
        np.testing.assert_array_equal(ras, want["raster"], err_msg=str(kw))
        got = sim.state.to_numpy()
        for k in ("V", "asc", "y2", "ref"):
            np.testing.assert_array_equal(got[k], st[k], err_msg="%s %s" % (k, kw))


def _batched_case(seed):
    rng = np.random.default_rng(9000 + seed)
    n = int(rng.choice([1, 15, 16, 17, 65, 333, 900, 2100]))
    n_in = int(rng.choice([0, 1, 7, 40, 300]))
    batch = int(rng.choice([8, 16, 32, 64]))
    max_delay = int(rng.choice([1, 2, 4, 6]))
    classes = int(rng.choice([0, 0, 3])) or None
    cfg = synthetic.small_glif3_network(n=n, n_in=n_in, steps=110, seed=seed, p_conn=float(rng.choice([0.0, 0.05, 0.4])),
                                        in_rate=float(rng.choice([60.0, 400.0])), in_fanout=max(1, min(n, 20)),
                                        max_delay=max_delay, n_classes=classes, batch=batch, w_scale=6.0, in_w_scale=40.0)
    for key in ("rec_src", "inp_src"):
        indptr, indices, w, d, r = cfg[key]
        cfg[key] = (indptr, indices, (np.round(w * 4.0) / 4.0 + np.sign(w) * 0.25).astype(np.float32), d, r)
    cfg["i_ext"] = rng.uniform(0.0, 600.0, n * batch).astype(np.float32)
    return cfg


@pytest.mark.parametrize("seed", range(24))
def test_fused_batched_driver_equals_the_oracle(seed):
    """The batched driver that pulls a neuron's arrivals and advances its trials in one launch (batches of 8, 16,
    32 and 64; a single neuron, neuron counts that are not a multiple of the 16 a workgroup takes at a time, no
    inputs or no recurrent synapses, rows without synapses, one-step delays) against the fp32 oracle: raster and state bit for bit, over two calls, with the activity map at one
    source per bit and at four."""
    cfg = _batched_case(seed)
    n, batch, steps = cfg["n"], cfg["batch"], cfg["steps"]
    has_rec = cfg["rec_src"][1].size > 0
    has_inp = cfg["n_in"] > 0
    if not (has_rec or has_inp):
        pytest.skip("a network without synapses has nothing to pull")
    rec = cfg["rec_src"] if has_rec else None
    inp = cfg["inp_src"] if has_inp else None
    L = int(max([1] + [int(t[3].max()) for t in (rec, inp) if t is not None])) + 1
    orc.set_threads(1)
    prop = orc.precompute(cfg["par"], cfg["h"])
    st = orc.new_state(n, batch, np.float32)
    ring = np.zeros((L, 4, n * batch), np.float32)
    want = orc.simulate(st, prop, cfg["h"], steps, batch=batch, class_id=cfg["class_id"], ring=ring, rec=rec, inp=inp,
                        in_ptr=cfg["in_ptr"] if has_inp else None, in_events=cfg["in_events"] if has_inp else None,
                        i_ext=cfg["i_ext"], raster=True)
    assert want["count"] > 0
    for shift in (None, 2):
        sim = Glif3Simulator(n, cfg["par"], cfg["h"], batch=batch, class_id=cfg["class_id"], rec=rec, inp=inp,
                             i_ext=cfg["i_ext"], resident=False, fused=True)
        assert sim.fuse_table is not None and sim.pull_table is None and sim.fuse_shift == 0
        if shift:
            sim.set_fuse_shift(shift)
        if has_inp:
            sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
        a = sim.run(50)
        b = sim.run(steps - 50)
        ras = np.concatenate([sim.raster(a["bits"]).cpu().numpy(), sim.raster(b["bits"]).cpu().numpy()])
        np.testing.assert_array_equal(ras, want["raster"], err_msg="shift %s" % shift)
        got = sim.state.to_numpy()
        for k in ("V", "asc", "y1", "y2", "ref"):
            np.testing.assert_array_equal(got[k], st[k], err_msg="%s shift %s" % (k, shift))


def _larger_case(seed):
    rng = np.random.default_rng(5000 + seed)
    n = int(rng.choice([1025, 1500, 2000, 3333, 5000, 9000]))
    n_in = int(rng.choice([0, 50, 400]))
    max_delay = int(rng.choice([1, 3, 6]))
    extra = int(rng.choice([0, 0, 2, 5, 70]))
    classes = int(rng.choice([0, 0, 5])) or None
    cfg = synthetic.small_glif3_network(n=n, n_in=n_in, steps=120, seed=seed, p_conn=float(rng.choice([0.0, 10.0 / n, 60.0 / n])),
                                        in_rate=float(rng.choice([20.0, 300.0])), in_fanout=30, max_delay=max_delay,
                                        n_classes=classes, batch=1, w_scale=6.0, in_w_scale=40.0)
    for key in ("rec_src", "inp_src"):
        indptr, indices, w, d, r = cfg[key]
        cfg[key] = (indptr, indices, (np.round(w * 4.0) / 4.0 + np.sign(w) * 0.25).astype(np.float32),
                    d.astype(np.int32) + extra, r)
    cfg["extra"] = extra
    # a constant current: spread out, or the same for most cells, which then fire in volleys
    amp = float(rng.choice([300.0, 600.0, 2500.0]))
    in_step = rng.random() < 0.4
    cfg["i_ext"] = (np.where(rng.random(n) < 0.6, amp, rng.uniform(0.0, 300.0, n)) if in_step
                    else rng.uniform(0.0, amp, n)).astype(np.float32)
    return cfg


@pytest.mark.parametrize("seed", range(16))
def test_many_workgroups_with_volleys_and_delay_offsets(seed):
    """Networks of 1,025 to 9,000 neurons (several resident workgroups, spans of 64 and more), from silent stretches to
    volleys of a thousand spikes in a step, with the part all delays have in common taken off automatically or as asked
    (runs with slack between the workgroups): raster and state of the launch-per-step driver and of the resident
    kernel, reading lists of fired neurons or ballots, equal the fp32 oracle's bit for bit."""
    cfg = _larger_case(seed)
    n, steps = cfg["n"], cfg["steps"]
    rec = cfg["rec_src"] if cfg["rec_src"][1].size else None
    inp = cfg["inp_src"] if cfg["n_in"] > 0 and cfg["inp_src"][1].size else None
    L = int(max([1] + [int(t[3].max()) for t in (rec, inp) if t is not None])) + 1
    orc.set_threads(8)
    prop = orc.precompute(cfg["par"], cfg["h"])
    st = orc.new_state(n, 1, np.float32)
    ring = np.zeros((L, 4, n), np.float32)
    want = orc.simulate(st, prop, cfg["h"], steps, class_id=cfg["class_id"], ring=ring, rec=rec, inp=inp,
                        in_ptr=cfg["in_ptr"] if inp is not None else None,
                        in_events=cfg["in_events"] if inp is not None else None, i_ext=cfg["i_ext"], raster=True)
    assert want["count"] > 0
    offsets = ["auto"] + ([cfg["extra"]] if cfg["extra"] and (rec is not None or inp is not None) else [])
    for off in offsets:
        for kw in (dict(resident=False), dict(resident=True), dict(resident=True, fired_lists=False)):
            sim = Glif3Simulator(n, cfg["par"], cfg["h"], class_id=cfg["class_id"], rec=rec, inp=inp, i_ext=cfg["i_ext"],
                                 delay_offset=off, **kw)
            if kw["resident"]:
                assert sim.res_groups > 1
            if inp is not None:
                sim.set_input_events(cfg["in_ptr"], cfg["in_events"])
            a = sim.run(50)
            b = sim.run(steps - 50)
            sim.check()
            ras = np.concatenate([sim.raster(a["bits"]).cpu().numpy(), sim.raster(b["bits"]).cpu().numpy()])
            tag = "delay offset %s -> %d, %s" % (off, sim.delay_offset, kw)
            np.testing.assert_array_equal(ras, want["raster"], err_msg=tag)
            got = sim.state.to_numpy()
            for k in ("V", "asc", "y2", "ref"):
                np.testing.assert_array_equal(got[k], st[k], err_msg="%s %s" % (k, tag))
