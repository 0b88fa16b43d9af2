"""The reference's example network, from its SONATA files to a spike file, on the GPU.

examples/point_450glifs: 300 GLIF3 cells (5 types) + 150 iaf_psc_alpha cells, 100 LGN spike sources.  The
integrate-and-fire cells are not a GLIF model, so the run silences them (documented in bmtk_amd.sonata); the 300
GLIF cells, their 15,001 recurrent and 24,036 input synapses and the stored LGN spike trains are the example's own.
The reference ships no output for this example, so the expected raster is the fp64 oracle's on the same arrays.
"""
import json
import os

import numpy as np
import pytest

from oracle import glif3_oracle as orc
from bmtk_amd import h5lite, ops, pointnet, sonata
from bmtk_amd.spike_trains import bin_spike_times

pytestmark = pytest.mark.gpu

G = os.path.join(os.path.dirname(__file__), "golden")


def _write_configs(tmp, dt, tstop, extra_inputs=None):
    net_dir = os.path.join(G, "point_450glifs", "network")
    circuit = {"manifest": {"$NETWORK_DIR": net_dir, "$MODELS_DIR": G},
               "components": {"point_neuron_models_dir": "$MODELS_DIR/cell_models",
                              "synaptic_models_dir": "$MODELS_DIR/synaptic_models"},
               "networks": {"nodes": [{"nodes_file": "$NETWORK_DIR/v1_nodes.h5",
                                       "node_types_file": "$NETWORK_DIR/v1_node_types.csv"},
                                      {"nodes_file": "$NETWORK_DIR/lgn_nodes.h5",
                                       "node_types_file": "$NETWORK_DIR/lgn_node_types.csv"}],
                            "edges": [{"edges_file": "$NETWORK_DIR/v1_v1_edges.h5",
                                       "edge_types_file": "$NETWORK_DIR/v1_v1_edge_types.csv"},
                                      {"edges_file": "$NETWORK_DIR/lgn_v1_edges.h5",
                                       "edge_types_file": "$NETWORK_DIR/lgn_v1_edge_types.csv"}]}}
    inputs = {"LGN_spikes": {"input_type": "spikes", "module": "sonata",
                             "input_file": os.path.join(G, "point_450glifs", "inputs", "lgn_spikes.h5"),
                             "node_set": "lgn"}}
    inputs.update(extra_inputs or {})
    sim = {"manifest": {"$BASE_DIR": ".", "$OUTPUT_DIR": "$BASE_DIR/output"}, "target_simulator": "NEST",
           "run": {"tstop": tstop, "dt": dt}, "inputs": inputs,
           "output": {"log_file": "log.txt", "spikes_file": "spikes.h5", "spikes_file_csv": "spikes.csv",
                      "spikes_sort_order": "by_time", "output_dir": "$OUTPUT_DIR"},
           "network": "config.circuit.json"}
    with open(os.path.join(tmp, "config.circuit.json"), "w") as fh:
        json.dump(circuit, fh)
    path = os.path.join(tmp, "config.simulation.json")
    with open(path, "w") as fh:
        json.dump(sim, fh)
    return path


def _oracle_spikes(nw, dt, n_steps, trains, dtype=np.float64):
    rec, inp = nw.tables()
    if dtype == np.float64:
        prop = orc.precompute(nw.par, dt)
    else:  # the fp32 oracle runs on the propagators the device computed
        prop = ops.glif3_precompute(nw.par, dt).cpu().numpy()
        orc.set_threads(1)  # serial delivery: one fixed summation order
    st = orc.new_state(nw.n, 1, dtype, asc_init=nw.asc_init[:, nw.class_id], u_init=nw.u_init[nw.class_id])
    L = int(max(rec[3].max(), inp[3].max())) + 1
    ring = np.zeros((L, 4, nw.n), dtype)
    in_ptr, in_ev = bin_spike_times(trains, dt, n_steps)
    return orc.simulate(st, prop, dtype(dt), n_steps, class_id=nw.class_id, ring=ring, rec=rec, inp=inp,
                        in_ptr=in_ptr, in_events=in_ev)


def _pairs(steps, elems, before=None):
    keep = np.ones(len(steps), bool) if before is None else np.asarray(steps) < before
    return set(zip(np.asarray(steps)[keep].tolist(), np.asarray(elems)[keep].tolist()))


@pytest.mark.parametrize("resident", [True, False])
def test_example_network_end_to_end(tmp_path, resident):
    dt, tstop = 0.1, 1000.0
    cfg_path = _write_configs(str(tmp_path), dt, tstop)
    conf = pointnet.Config.from_json(cfg_path)
    conf.build_env()
    assert conf.dt == dt and conf["output"]["output_dir"] == str(tmp_path / "output")
    graph = pointnet.PointNetwork.from_config(conf, unsupported="silence")
    sim = pointnet.PointSimulator.from_config(conf, graph, resident=resident)
    spikes = sim.run()
    assert bool(sim.simulator.res_span) == resident
    ids, ts = spikes["v1"]
    assert ids.size > 500 and ids.max() < 300  # the silenced cells (node ids 300..449) stay silent
    got_steps = np.floor(ts / dt + 1e-9).astype(int)
    got_pairs = _pairs(got_steps, ids)
    # The example's weights are multiples of 0.5 pA, so arriving sums do not depend on the order of addition and
    # the whole run must equal the fp32 oracle's spike for spike.
    want32 = _oracle_spikes(graph, dt, sim.n_steps, sim._trains, np.float32)
    assert got_pairs == _pairs(want32["step"], want32["elem"])
    # Against fp64 the strongly driven recurrent network (59 Hz) is chaotic: one rounding-induced spike shift
    # spreads, and the fp32 and fp64 ORACLES agree on only 22 % of the spikes after 1 s.  Parity with fp64 is
    # therefore asserted while the trajectories have not separated: the first 100 ms (791 spikes).
    want = _oracle_spikes(graph, dt, sim.n_steps, sim._trains)
    want_pairs = _pairs(want["step"], want["elem"], 1000)
    early = _pairs(got_steps, ids, 1000)
    match = len(early & want_pairs) / max(1, len(early | want_pairs))
    assert len(want_pairs) > 500 and match >= 0.999, match
    # files: what was written is what was returned, sorted by time, in both formats
    back = sonata.read_spikes(str(tmp_path / "output" / "spikes.h5"))
    assert back["v1"][2] == {"sorting": "by_time", "units": "ms"} and np.all(np.diff(back["v1"][1]) >= 0)
    assert sonata.spikes_equal(back, spikes, err=1e-9)
    assert sonata.spikes_equal(sonata.read_spikes_csv(str(tmp_path / "output" / "spikes.csv")), spikes, err=1e-6)
    # and the oracle's spike times (same interpolation rule) agree within the reference's own tolerance for
    # spike-train equality, 1e-5 ms + 1e-5 relative, on the spikes both have
    want_t = {(s, e): (s + f) * dt for s, e, f in zip(want["step"], want["elem"], want["frac"])}
    got_t = {(int(np.floor(t / dt + 1e-9)), int(e)): t for e, t in zip(ids, ts)}
    common = sorted(early & want_pairs)
    err = max(abs(got_t[k] - want_t[k]) for k in common)
    assert err < 0.02 * dt, err  # crossing fraction in fp32 vs fp64


def test_current_clamp_segments(tmp_path):
    """A step current on three cells, no other input: the cells fire only while it is on (plus at most one
    refractory period), and the raster equals the oracle's with the same piecewise-constant current."""
    dt, tstop = 0.1, 300.0
    clamp = {"clamp": {"input_type": "current_clamp", "module": "IClamp", "node_set": {"node_id": [0, 100, 250]},
                       "amp": 400.0, "delay": 50.0, "duration": 150.0}}
    cfg_path = _write_configs(str(tmp_path), dt, tstop, clamp)
    conf = pointnet.Config.from_json(cfg_path)
    del conf["inputs"]["LGN_spikes"]
    graph = pointnet.PointNetwork.from_config(conf, unsupported="silence")
    sim = pointnet.PointSimulator.from_config(conf, graph)
    ids, ts = sim.run()["v1"]
    driven = np.isin(ids, [0, 100, 250])
    assert driven.sum() > 10 and ts[driven].min() > 50.0 and ts[driven].max() < 200.0 + 10.0
    segs = list(sim._segments())
    assert [(a, b) for a, b, _ in segs] == [(0, 501), (501, 2001), (2001, 3000)]
    # oracle, segment by segment
    rec, inp = graph.tables()
    prop = orc.precompute(graph.par, dt)
    st = orc.new_state(graph.n, 1, np.float64, asc_init=graph.asc_init[:, graph.class_id],
                       u_init=graph.u_init[graph.class_id])
    ring = np.zeros((int(rec[3].max()) + 1, 4, graph.n), np.float64)
    want = set()
    for a, b, cur in segs:
        out = orc.simulate(st, prop, dt, b - a, class_id=graph.class_id, ring=ring, rec=rec, i_ext=cur.astype(np.float64),
                           step0=a)
        want |= set(zip(out["step"].tolist(), out["elem"].tolist()))
    got = set(zip(np.floor(ts / dt + 1e-9).astype(int).tolist(), ids.tolist()))
    assert len(got & want) / max(1, len(got | want)) >= 0.999


def test_current_clamp_from_csv_equals_the_list_form(tmp_path):
    """The same stimulus given as a csv file of amplitude changes and as amp/delay/duration lists: same spikes;
    the clamp goes to the whole population (no node ids in the node set)."""
    dt, tstop = 0.1, 200.0
    csv = str(tmp_path / "stim.csv")
    with open(csv, "w") as fh:
        fh.write("timestamps amps\n20.0 300.0\n60.0 0.0\n100.0 450.0\n150.0 0.0\n")
    forms = ({"input_type": "csv", "module": "IClamp", "node_set": {"population": "v1"}, "file": csv},
             {"input_type": "current_clamp", "module": "IClamp", "node_set": {"population": "v1"},
              "amp": [300.0, 450.0], "delay": [20.0, 100.0], "duration": [40.0, 50.0]})
    got = []
    for k, form in enumerate(forms):
        os.makedirs(str(tmp_path / str(k)))
        conf = pointnet.Config.from_json(_write_configs(str(tmp_path / str(k)), dt, tstop, {"clamp": form}))
        del conf["inputs"]["LGN_spikes"]
        graph = pointnet.PointNetwork.from_config(conf, unsupported="silence")
        sim = pointnet.PointSimulator.from_config(conf, graph)
        assert [(a, b) for a, b, _ in sim._segments()] == [(0, 201), (201, 601), (601, 1001), (1001, 1501),
                                                            (1501, 2000)]
        got.append(sim.run()["v1"])
    assert got[0][0].size > 300
    assert np.array_equal(got[0][0], got[1][0]) and np.array_equal(got[0][1], got[1][1])
    assert got[0][1].min() > 20.0


def test_example_at_its_own_resolution(tmp_path):
    """The example's configured resolution, dt = 0.001 ms: its 2 ms delays are 2000 steps, far beyond the ring,
    so the run rests on the delay offset (1999 steps) and a ring of 2 slots.  200 ms = 200,000 steps, resident
    kernel; spike for spike equal to the fp32 oracle run with the true delays and a 2001-slot ring."""
    dt, tstop = 0.001, 200.0
    conf = pointnet.Config.from_json(_write_configs(str(tmp_path), dt, tstop))
    graph = pointnet.PointNetwork.from_config(conf, unsupported="silence")
    assert graph.rec_edges[3].min() == graph.rec_edges[3].max() == 2000
    sim = pointnet.PointSimulator.from_config(conf, graph, resident=True)
    ids, ts = sim.run()["v1"]
    assert sim.simulator.delay_offset == 1999 and sim.simulator.L == 2 and sim.n_steps == 200000
    want = _oracle_spikes(graph, dt, sim.n_steps, sim._trains, np.float32)
    assert want["count"] > 1000
    got = _pairs(np.floor(ts / dt + 1e-9).astype(int), ids)
    assert got == _pairs(want["step"], want["elem"])


def test_membrane_report(tmp_path):
    """A ``reports`` entry as in examples/point_120cells/config.simulation.json: V_m of five cells, here every
    0.5 ms.  The file has bmtk's cell-variable layout and its trace follows the fp64 oracle stepped one step at a
    time, while the trajectories have not separated (first 60 ms)."""
    dt, tstop = 0.1, 100.0
    cfg_path = _write_configs(str(tmp_path), dt, tstop)
    conf = pointnet.Config.from_json(cfg_path)
    cells = [0, 85, 170, 250, 299]
    conf["reports"] = {"membrane_potential": {"cells": {"population": "v1", "node_id": cells}, "variable_name": "V_m",
                                              "module": "multimeter_report", "sections": "soma", "dt": 0.5}}
    graph = pointnet.PointNetwork.from_config(conf, unsupported="silence")
    sim = pointnet.PointSimulator.from_config(conf, graph)
    sim.run()
    ids, times, data, attrs = sonata.read_membrane_report(str(tmp_path / "output" / "membrane_potential.h5"))
    assert list(ids) == cells and attrs == {"variable": "V_m", "units": "mV"}
    np.testing.assert_allclose(times, np.arange(0.5, tstop + 1e-9, 0.5), atol=1e-9)
    assert data.shape == (times.size, len(cells))
    with h5lite.File(str(tmp_path / "output" / "membrane_potential.h5")) as f:
        assert list(f["/report/v1/mapping/time"][()]) == [0.5, tstop + 0.5, 0.5]
        assert list(f["/report/v1/mapping/index_pointer"][()]) == [0, 1, 2, 3, 4, 5]
    # the oracle, stepped
    from bmtk_amd.layout import PAR
    rec, inp = graph.tables()
    prop = orc.precompute(graph.par, dt)
    st = orc.new_state(graph.n, 1, np.float64, asc_init=graph.asc_init[:, graph.class_id],
                       u_init=graph.u_init[graph.class_id])
    ring = np.zeros((21, 4, graph.n))
    n_early = 600
    in_ptr, in_ev = bin_spike_times(sim._trains, dt, n_early)
    e_l = graph.par[PAR["E_L"]][graph.class_id]
    want = np.zeros((n_early // 5, len(cells)))
    for k in range(n_early):
        orc.simulate(st, prop, dt, 1, class_id=graph.class_id, ring=ring, rec=rec, inp=inp, in_ptr=in_ptr,
                     in_events=in_ev, step0=k)
        if (k + 1) % 5 == 0:
            want[(k + 1) // 5 - 1] = (st["V"] + e_l)[cells]
    assert np.ptp(want) > 10.0
    np.testing.assert_allclose(data[:n_early // 5], want, atol=5e-3)
