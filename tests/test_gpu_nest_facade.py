"""The PyNEST-shaped front end, driven the way bmtk and its tests drive NEST."""
import json
import os

import numpy as np
import pytest

import bmtk_amd.nest as nest
from bmtk_amd.glif_utils import convert_aibs2nest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('model_name,dynamics_params,expected', [
    ('nest:glif_lif_psc', 'glif_models/637930677_lif.json', [14.77547828]),
    ('nest:glif_lif_asc_psc', 'glif_models/637930677_lif_asc.json', [14.46548367]),
])
@pytest.mark.parametrize('resolution', [0.1, 0.05])
def test_converter_psc(golden_dir, model_name, dynamics_params, expected, resolution):
    """The protocol of bmtk/tests/simulator/pointnet/test_glif_utils.py:24-44,
    call for call (the reference sets resolution 0.001, where the 1 ms delay is
    1000 steps -- more than the 62 the fused simulation supports -- so it runs
    at 0.1 and 0.05 ms; the expected times are met far inside the reference's
    atol of 1.0)."""
    nest.ResetKernel()
    nest.SetKernelStatus({"resolution": resolution})

    aibs_params = json.load(open(os.path.join(golden_dir, dynamics_params), 'r'))
    model_name, model_params = convert_aibs2nest(model_name, aibs_params)
    model_name = model_name.split(':')[-1]
    nrn = nest.Create(model_name, 1, model_params)

    sr = nest.Create('spike_recorder')
    espikes = nest.Create(
        'spike_generator',
        params={'spike_times': [5.0, 7.0, 8.0, 9.0, 10.0, 12.0], 'spike_weights': [100.0]*6}
    )
    nest.Connect(espikes, nrn, syn_spec={"receptor_type": 1})
    nest.Connect(nrn, sr)

    nest.Simulate(50.0)
    spikes = nest.GetStatus(sr, 'events')[0]['times']
    assert(len(spikes) == len(expected))
    assert(np.allclose(spikes, expected, atol=1.0, equal_nan=True))
    assert(np.allclose(spikes, expected, atol=2e-3))
    assert nest.GetStatus(sr, 'events')[0]['senders'].tolist() == nrn.tolist()


def _cell(golden_dir):
    return json.load(open(os.path.join(golden_dir, "cell_models", "593618144_glif_lif_asc_psc.json")))


def test_add_nodes_and_edges_counts(golden_dir):
    """bmtk/tests/simulator/pointnet/test_pointnetwork.py:8-43: 100 nodes, 100 one_to_one connections."""
    nest.ResetKernel()
    nest.SetKernelStatus({"resolution": 0.1})
    nodes = nest.Create('glif_psc', 100, _cell(golden_dir))
    assert len(nodes) == 100 and nodes.tolist() == list(range(1, 101))
    src, trg = nodes.tolist(), nodes.tolist()[::-1]
    nest.Connect(src, trg, conn_spec='one_to_one',
                 syn_spec={'synapse_model': 'static_synapse', 'weight': np.full(100, 2.5), 'delay': np.full(100, 2.0),
                           'receptor_type': 1})
    assert len(nest.GetConnections()) == 100
    assert nest.GetKernelStatus('min_delay') == 2.0


def test_bad_delay_raises(golden_dir):
    """bmtk/tests/simulator/pointnet/test_pointnetwork.py:47-57: delay below the resolution."""
    nest.ResetKernel()
    nest.SetKernelStatus({"resolution": 1.0})
    nodes = nest.Create('glif_psc', 2, _cell(golden_dir))
    with pytest.raises(nest.kernel.NESTErrors.BadDelay):
        nest.Connect(nodes[0], nodes[1], conn_spec='one_to_one', syn_spec={'weight': 1.0, 'delay': 0.1})
    with pytest.raises(nest.kernel.NESTError):
        nest.Connect(nodes[0], nodes[1], conn_spec='one_to_one', syn_spec={'weight': 1.0, 'delay': 1.0,
                                                                          'receptor_type': 9})


def test_spike_time_validation():
    """bmtk/tests/simulator/pointnet/test_pointnetwork.py:59-100: empty is fine, zero/negative raise."""
    nest.ResetKernel()
    nest.SetKernelStatus({"resolution": 0.1})
    sg = nest.Create('spike_generator', 3, {'precise_times': True})
    nest.SetStatus(sg[0], {'spike_times': np.array([])})
    nest.SetStatus(sg[1], {'spike_times': np.array([0.5, 1.0, 10.03])})
    with pytest.raises(nest.kernel.NESTError):
        nest.SetStatus(sg[2], {'spike_times': np.array([0.0, 1.0])})
    with pytest.raises(nest.kernel.NESTError):
        nest.SetStatus(sg[2], {'spike_times': np.array([-1.0])})


def test_unsupported_models_raise_instead_of_being_approximated():
    nest.ResetKernel()
    with pytest.raises(nest.kernel.NESTErrors.UnknownModelName):
        nest.Create('iaf_psc_alpha', 3)
    with pytest.raises(nest.kernel.NESTError):
        nest.Create('glif_psc', 1, {'spike_dependent_threshold': True})


def test_small_network_through_the_front_end_matches_the_oracle(golden_dir, tmp_path):
    """Two populations wired like examples/point_450glifs (e2e/e2i/i2e/i2i
    receptor ports, 2 ms delays), driven by generators; recorder output to the
    ascii file bmtk reads back; compared with the fp64 oracle on the same
    arrays."""
    from oracle import glif3_oracle as orc
    from bmtk_amd.glif_utils import params_table
    from bmtk_amd import network as net
    rng = np.random.default_rng(12)
    files = sorted(os.listdir(os.path.join(golden_dir, "cell_models")))
    cells = [json.load(open(os.path.join(golden_dir, "cell_models", f))) for f in files]
    dt, n_e, n_i, n_g, T = 0.5, 60, 20, 30, 400.0
    nest.ResetKernel()
    nest.SetKernelStatus({"resolution": dt, "data_path": str(tmp_path), "overwrite_files": True})
    exc = nest.Create('glif_psc', n_e, cells[0])
    inh = nest.Create('glif_psc', n_i, cells[3])
    gens = nest.Create('spike_generator', n_g, {'precise_times': True})
    trains = []
    for g in gens:
        st = np.sort(np.round(rng.uniform(1.0, T - 1, rng.poisson(40)) / dt) * dt)
        st = np.unique(st[st > 0])
        trains.append(st)
        nest.SetStatus(g, {'spike_times': st})
    edges = []
    def connect(pre, post, p, weight, receptor, delay=2.0):
        s, t = np.nonzero(rng.random((len(pre), len(post))) < p)
        nsyns = rng.integers(1, 5, s.size)
        src, trg = np.array(pre.tolist())[s], np.array(post.tolist())[t]
        nest.Connect(src, trg, conn_spec='one_to_one',
                     syn_spec={'synapse_model': 'static_synapse', 'weight': nsyns * weight,
                               'delay': np.full(s.size, delay), 'receptor_type': receptor})
        edges.append((src, trg, nsyns * weight, delay, receptor))
    connect(exc, exc, 0.2, 8.0, 1); connect(exc, inh, 0.2, 12.0, 3)
    connect(inh, exc, 0.3, -10.0, 2); connect(inh, inh, 0.3, -6.0, 4)
    connect(gens, exc, 0.4, 40.0, 1); connect(gens, inh, 0.4, 45.0, 1)
    sr = nest.Create('spike_recorder', 1, {'label': 'tmp_spike_times', 'record_to': 'ascii'})
    nest.Connect(exc + inh, sr)
    nest.Simulate(T / 2)
    nest.Simulate(T / 2)
    ev = nest.GetStatus(sr, 'events')[0]
    assert len(ev['times']) > 200
    # the same network on the oracle
    n = n_e + n_i
    par, asc_init, u_init = params_table([cells[0]] * n_e + [cells[3]] * n_i)
    prop = orc.precompute(par, dt)
    nid = {gid: k for k, gid in enumerate((exc + inh).tolist())}
    gid_of = {gid: k for k, gid in enumerate(gens.tolist())}
    rec_e = [(np.array([nid[a] for a in s]), np.array([nid[b] for b in t]), w, d, r) for s, t, w, d, r in edges[:4]]
    inp_e = [(np.array([gid_of[a] for a in s]), np.array([nid[b] for b in t]), w, d, r) for s, t, w, d, r in edges[4:]]
    def table(es, rows):
        s = np.concatenate([e[0] for e in es]); t = np.concatenate([e[1] for e in es])
        w = np.concatenate([e[2] for e in es]).astype(np.float32)
        d = np.concatenate([np.full(e[0].size, int(round(e[3] / dt))) for e in es]).astype(np.uint8)
        r = np.concatenate([np.full(e[0].size, e[4] - 1) for e in es]).astype(np.uint8)
        return net.coo_to_csr(s, t, w, d, r, n_rows=rows, major="source")
    from bmtk_amd.spike_trains import bin_spike_times
    steps = int(round(T / dt))
    in_ptr, in_ev = bin_spike_times(trains, dt, steps)
    st = orc.new_state(n, 1, np.float64, asc_init=asc_init, u_init=u_init)
    ring = np.zeros((int(round(2.0 / dt)) + 1, 4, n))
    want = orc.simulate(st, prop, dt, steps, ring=ring, rec=table(rec_e, n), inp=table(inp_e, n_g), in_ptr=in_ptr,
                        in_events=in_ev)
    want_t = (want["step"] + want["frac"]) * dt
    want_s = np.array((exc + inh).tolist())[want["elem"]]
    assert len(ev['times']) == want["count"]
    order = np.lexsort((want_s, want_t))
    # fp32 threshold interpolation against fp64: crossing times agree to a thousandth of a step
    assert np.array_equal(np.sort(ev['senders']), np.sort(want_s))
    np.testing.assert_allclose(np.sort(ev['times']), np.sort(want_t), atol=dt * 2e-2)
    # the ascii file in the form bmtk's SpikesMod reads back
    import pandas as pd
    dat = list(tmp_path.glob('tmp_spike_times*.dat'))
    assert len(dat) == 1
    df = pd.read_csv(dat[0], index_col=False, sep='\t', comment='#')
    assert list(df.columns) == ['sender', 'time_ms'] and len(df) == want["count"]
    np.testing.assert_allclose(np.sort(df['time_ms'].values), np.sort(want_t), atol=dt * 2e-2 + 1e-3)


def test_multimeter_records_membrane_potential(golden_dir, tmp_path):
    """What bmtk's membrane report asks of NEST (bmtk/simulator/pointnet/modules/multimeter_reporter.py:36-46,
    113-115): a multimeter on V_m with an interval, a start and a stop, written as an ascii file with the columns
    sender, time_ms, V_m.  The trace must follow the fp64 oracle stepped one step at a time: the sample stamped t is
    the potential at the end of the step that ends at t."""
    import pandas as pd
    from oracle import glif3_oracle as orc
    from bmtk_amd.glif_utils import params_table
    from bmtk_amd.spike_trains import bin_spike_times
    from bmtk_amd.layout import PAR
    cells = [json.load(open(os.path.join(golden_dir, "cell_models", f)))
             for f in ("318808427_glif_lif_asc_psc.json", "478958894_glif_lif_asc_psc.json")]
    dt, T = 0.1, 40.0
    nest.ResetKernel()
    nest.SetKernelStatus({"resolution": dt, "data_path": str(tmp_path), "overwrite_files": True})
    a = nest.Create('glif_psc', 1, cells[0])
    b = nest.Create('glif_psc', 1, cells[1])
    gen = nest.Create('spike_generator', 1, {'spike_times': [3.0, 5.0, 6.0, 7.5, 9.0, 11.0, 12.0, 20.0]})
    nest.Connect(gen, a + b, syn_spec={'weight': 400.0, 'delay': 1.0, 'receptor_type': 1})
    mm = nest.Create('multimeter', params={'start': 2.0, 'stop': 30.0, 'record_to': 'ascii', 'record_from': ['V_m'],
                                           'label': 'membrane'})
    nest.SetStatus(mm, 'interval', 0.5)
    nest.Connect(mm, a + b)
    with pytest.raises(nest.kernel.NESTErrors.BadProperty):
        nest.Create('multimeter', params={'record_from': ['I_syn']})
    with pytest.raises(nest.kernel.NESTErrors.BadProperty):
        nest.SetStatus(mm, 'interval', 0.25)
    nest.Simulate(T / 2)
    nest.Simulate(T / 2)
    ev = nest.GetStatus(mm, 'events')[0]
    times = np.arange(2.5, 30.0 + 1e-9, 0.5)
    assert ev['times'].size == 2 * times.size
    np.testing.assert_allclose(ev['times'][0::2], times, atol=1e-9)
    assert list(ev['senders'][:2]) == a.tolist() + b.tolist()
    # the oracle, one step at a time
    par, asc_init, u_init = params_table(cells)
    prop = orc.precompute(par, dt)
    steps = int(round(T / dt))
    d = int(round(1.0 / dt))
    inp = (np.array([0, 2], np.int32), np.array([0, 1], np.int32), np.array([400.0, 400.0], np.float32),
           np.array([d, d], np.uint8), np.zeros(2, np.uint8))
    in_ptr, in_ev = bin_spike_times([np.array([3.0, 5.0, 6.0, 7.5, 9.0, 11.0, 12.0, 20.0])], dt, steps)
    st = orc.new_state(2, 1, np.float64, asc_init=asc_init, u_init=u_init)
    ring = np.zeros((d + 1, 4, 2))
    trace = np.zeros((steps, 2))
    for k in range(steps):
        orc.simulate(st, prop, dt, 1, ring=ring, inp=inp, in_ptr=in_ptr, in_events=in_ev, step0=k)
        trace[k] = st["V"] + par[PAR["E_L"]]
    rows = np.rint(times / dt).astype(int) - 1
    want = trace[rows]
    got = ev['V_m'].reshape(-1, 2)
    assert np.abs(want).max() > 50 and np.ptp(want[:, 0]) > 5.0  # the cell is depolarised and fires in the window
    np.testing.assert_allclose(got, want, atol=2e-3)
    df = pd.read_csv(os.path.join(str(tmp_path), "membrane-{}-0.dat".format(mm.tolist()[0])), sep='\t', comment='#')
    assert list(df.columns) == ['sender', 'time_ms', 'V_m'] and len(df) == 2 * times.size
    np.testing.assert_allclose(df['V_m'].to_numpy(), ev['V_m'], atol=1e-6)


def test_constant_input_current_I_e(golden_dir, tmp_path):
    """A neuron's constant input current I_e (pA), given at Create or set between two Simulate calls.  Below threshold
    the potential settles at E_L + I_e / g (closed form: pA / nS = mV), which fixes the scale; above it the spike
    times follow the fp64 oracle driven with the same current, the change taking effect with the call after it."""
    from oracle import glif3_oracle as orc
    from bmtk_amd.glif_utils import params_table
    cell = json.load(open(os.path.join(golden_dir, "cell_models", "318808427_glif_lif_asc_psc.json")))
    g, gap = float(cell["g"]), float(cell["V_th"]) - float(cell["E_L"])     # nS, mV
    low, high, higher = 0.4 * gap * g, 1.6 * gap * g, 2.5 * gap * g
    dt, T = 0.1, 300.0
    nest.ResetKernel()
    nest.SetKernelStatus({"resolution": dt, "data_path": str(tmp_path), "overwrite_files": True})
    quiet = nest.Create('glif_psc', 1, dict(cell, I_e=low))
    driven = nest.Create('glif_psc', 2, dict(cell, I_e=high))
    sr = nest.Create('spike_recorder')
    nest.Connect(quiet + driven, sr)
    mm = nest.Create('multimeter', params={'record_from': ['V_m'], 'interval': 1.0})
    nest.Connect(mm, quiet)
    nest.Connect(np.array([], np.int64), np.array([], np.int64), conn_spec='one_to_one',
                 syn_spec={'weight': np.array([]), 'delay': np.array([]), 'receptor_type': 1})   # no edges: no-op
    nest.Simulate(T)
    nest.SetStatus(driven[1], {'I_e': higher})
    with pytest.raises(nest.NESTError):      # the parameter table is on the device by now
        nest.SetStatus(driven[1], {'V_th': -30.0})
    nest.Simulate(T)
    v = nest.GetStatus(mm, 'events')[0]['V_m']
    np.testing.assert_allclose(v[-1], float(cell["E_L"]) + low / g, atol=2e-3)
    assert abs(v[-1] - v[0]) > 5.0
    ev = nest.GetStatus(sr, 'events')[0]
    # the oracle with the same currents, in the same two pieces
    par, asc_init, u_init = params_table([cell] * 3)
    prop = orc.precompute(par, dt)
    steps = int(round(T / dt))
    st = orc.new_state(3, 1, np.float64, asc_init=asc_init, u_init=u_init)
    ring = np.zeros((2, 4, 3))
    want_t, want_s = [], []
    for piece, cur in enumerate(([low, high, high], [low, high, higher])):
        out = orc.simulate(st, prop, dt, steps, ring=ring, step0=piece * steps, i_ext=np.array(cur, np.float64))
        want_t.append((out["step"] + out["frac"]) * dt)
        want_s.append(np.array((quiet + driven).tolist())[out["elem"]])
    want_t, want_s = np.concatenate(want_t), np.concatenate(want_s)
    assert want_t.size > 20 and not np.any(want_s == quiet.tolist()[0])
    assert (want_s == driven.tolist()[1]).sum() > (want_s == driven.tolist()[0]).sum()
    order_w, order_g = np.lexsort((want_t, want_s)), np.lexsort((ev['times'], ev['senders']))
    assert np.array_equal(ev['senders'][order_g], want_s[order_w])
    # fp32 state against the fp64 oracle over 6000 steps of a regularly firing cell: every crossing inherits the
    # error of the ones before it, a few parts in a million of the elapsed time on top of the interpolation's share
    np.testing.assert_allclose(ev['times'][order_g], want_t[order_w], atol=dt * 2e-2, rtol=2e-5)
