"""The Poisson spike sources generated on the device (``ops.poisson_events``) against what the process fixes and
against the host generator that reproduces the reference's golden vectors
(bmtk/utils/reports/spike_trains/spike_trains.py:166-206).  The device draws from independent counter-based
streams, so the comparison with the host generator is statistical: rate, inter-spike-interval distribution,
independence of sources; structure and binning are checked exactly."""
import numpy as np
import pytest
import torch
from scipy import stats

from oracle import glif3_oracle as orc
from bmtk_amd import network as net, ops, synthetic
from bmtk_amd.simulator import Glif3Simulator
from bmtk_amd.spike_trains import PoissonSpikeGenerator

pytestmark = pytest.mark.gpu


def _host(arrs):
    return [a.cpu().numpy() for a in arrs]


def test_event_lists_are_well_formed_and_binned_like_the_host_side():
    n_src, batch, dt, n_steps = 300, 3, 0.5, 4000
    in_ptr, in_events, (steps, elems, times) = ops.poisson_events(n_src, 35.0, dt, n_steps, batch=batch, seed=7,
                                                                  return_times=True)
    in_ptr, in_events, steps, elems, times = _host([in_ptr, in_events, steps, elems, times])
    assert in_ptr.size == n_steps + 1 and in_ptr[0] == 0 and in_ptr[-1] == in_events.size
    assert in_events.size > 50000
    dup = net.check_input_events(in_ptr, in_events, n_src * batch)     # ascending within every step, ids in range
    np.testing.assert_array_equal(elems, in_events)
    np.testing.assert_array_equal(np.repeat(np.arange(n_steps), np.diff(in_ptr)), steps)
    assert times.min() > 0.0 and times.max() <= n_steps * dt
    # a spike at time t is stamped ceil(t / dt) steps and emitted one step earlier
    np.testing.assert_array_equal(np.maximum(np.ceil(times / dt - 1e-6), 1).astype(np.int64) - 1, steps)
    # per element the times ascend, and every element's train is its own
    order = np.lexsort((times, elems))
    same = elems[order][1:] == elems[order][:-1]
    assert np.all(np.diff(times[order])[same] > 0)
    first = np.array([times[elems == e].min() for e in range(0, n_src * batch, 7)])
    assert np.unique(first).size == first.size
    # the same call again gives the same lists; another seed gives others
    again = _host(ops.poisson_events(n_src, 35.0, dt, n_steps, batch=batch, seed=7))
    np.testing.assert_array_equal(again[0], in_ptr)
    np.testing.assert_array_equal(again[1], in_events)
    other = _host(ops.poisson_events(n_src, 35.0, dt, n_steps, batch=batch, seed=8))
    assert other[1].size != in_events.size or not np.array_equal(other[1], in_events)
    assert isinstance(dup, bool)


def test_rate_interval_distribution_and_independence():
    """2,000 sources at 20 Hz for 5 s: spike counts are Poisson(100) (mean and Fano factor), pooled inter-spike
    intervals are exponential (mean, CV, Kolmogorov-Smirnov against the exponential law and against the host
    generator's intervals), and sources are uncorrelated."""
    n_src, rate, dt, n_steps = 2000, 20.0, 1.0, 5000
    in_ptr, in_events, (steps, elems, times) = ops.poisson_events(n_src, rate, dt, n_steps, seed=3, return_times=True)
    elems, times = _host([elems, times])
    counts = np.bincount(elems, minlength=n_src)
    assert abs(counts.mean() - 100.0) < 5 * np.sqrt(100.0 / n_src)
    assert abs(counts.var() / counts.mean() - 1.0) < 0.12
    order = np.lexsort((times, elems))
    e, t = elems[order], times[order]
    isi = np.diff(t)[e[1:] == e[:-1]]
    assert abs(isi.mean() - 1000.0 / rate) < 0.5
    assert abs(isi.std() / isi.mean() - 1.0) < 0.02
    assert stats.kstest(isi[::7] / (1000.0 / rate), "expon").pvalue > 1e-3
    np.random.seed(12345)
    host = PoissonSpikeGenerator()
    host.add(node_ids=np.arange(300), firing_rate=rate, times=(0.0, 5.0))
    host_isi = np.concatenate([np.diff(np.sort(host.get_times(n))) for n in range(300)])
    assert stats.ks_2samp(isi[::7], host_isi).pvalue > 1e-3
    # independence: counts in 100 ms bins of different sources are uncorrelated
    bins = (times // 100.0).astype(np.int64)
    grid = np.zeros((200, 50))
    keep = elems < 200
    np.add.at(grid, (elems[keep], bins[keep]), 1.0)
    corr = np.corrcoef(grid)
    off = corr[~np.eye(200, dtype=bool)]
    assert abs(off.mean()) < 0.01 and np.abs(off).max() < 0.6


def test_rates_per_source_trials_and_errors():
    rates = np.array([0.0, 5.0, 50.0, 200.0], np.float32)
    in_ptr, in_events = ops.poisson_events(4, rates, 1.0, 20000, batch=8, seed=5)
    counts = np.bincount(in_events.cpu().numpy(), minlength=32).reshape(4, 8)
    assert counts[0].sum() == 0
    for j in (1, 2, 3):
        want = rates[j] * 20.0
        assert np.all(np.abs(counts[j] - want) < 5 * np.sqrt(want))
        assert np.unique(counts[j]).size > 1                        # the trials of a source differ
    # a source at 200 Hz with 1 ms steps fires twice in a step now and then: both events are kept
    assert net.check_input_events(in_ptr.cpu().numpy(), in_events.cpu().numpy(), 32) is True
    with pytest.raises(ValueError, match="negative"):
        ops.poisson_events(4, -1.0, 1.0, 100)
    from bmtk_amd._lib import BmtkAmdError
    with pytest.raises(BmtkAmdError, match="start and stop"):
        ops.poisson_events(4, 1.0, 1.0, 100, t_start_ms=50.0, t_stop_ms=50.0)
    # a window inside the run: no spike outside it
    in_ptr, _ = ops.poisson_events(50, 100.0, 1.0, 1000, t_start_ms=200.0, t_stop_ms=300.0, seed=2)
    p = in_ptr.cpu().numpy()
    assert p[200] == 0 and p[300] == p[-1] and p[300] > 300


def test_device_generated_inputs_drive_the_simulation_like_the_oracle():
    """Event lists made on the device go straight into the resident simulation; the fp32 oracle run on a host copy of
    the same lists gives the same raster bit for bit (quarter-pA weights), including steps in which a source fires
    twice."""
    cfg = synthetic.small_glif3_network(n=600, n_in=200, steps=400, seed=3, in_w_scale=2.0, in_fanout=60, p_conn=0.05,
                                        w_scale=1.5)
    for k in ("rec_src", "inp_src"):
        indptr, indices, w, d, r = cfg[k]
        cfg[k] = (indptr, indices, (np.round(w * 4.0) / 4.0 + np.sign(w) * 0.25).astype(np.float32), d, r)
    in_ptr, in_events = ops.poisson_events(200, 60.0, cfg["h"], 400, seed=9)
    sim = Glif3Simulator(cfg["n"], cfg["par"], cfg["h"], rec=cfg["rec_src"], inp=cfg["inp_src"], ring_slots=cfg["L"],
                         resident=True)
    sim.set_input_events(in_ptr, in_events)
    assert sim.in_duplicates
    out = sim.run(400)
    sim.check()
    prop = orc.precompute(cfg["par"], cfg["h"])
    st = orc.new_state(cfg["n"], 1, np.float32)
    ring = np.zeros((cfg["L"], 4, cfg["n"]), np.float32)
    want = orc.simulate(st, prop, cfg["h"], 400, ring=ring, rec=cfg["rec_src"], inp=cfg["inp_src"],
                        in_ptr=in_ptr.cpu().numpy(), in_events=in_events.cpu().numpy(), raster=True)
    assert want["count"] > 1000
    np.testing.assert_array_equal(sim.raster(out["bits"]).cpu().numpy(), want["raster"])
