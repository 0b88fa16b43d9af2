"""SONATA files: the HDF5 subset reader/writer, the node/edge loaders and the spike files (CPU only).

The network files under tests/golden/point_450glifs are the data files of the reference's
examples/point_450glifs (written by h5py).  What pins the reader: facts the example's own tables state
(populations, node counts per type, the edge-type of every edge), the two redundant indices each edge file
carries (a wrong offset or a transposed column breaks them), and, where the HDF5 command line tools exist on
the machine, the HDF5 library's own reading of the same files.  The writer is pinned by that library too
(h5dump / h5repack read what it wrote) and by the reader.
"""
import json
import os
import shutil
import subprocess

import numpy as np
import pytest

from bmtk_amd import h5lite, network as net, sonata

G = os.path.join(os.path.dirname(__file__), "golden")
NETDIR = os.path.join(G, "point_450glifs", "network")


def _tool(name):
    for d in (os.environ.get("HDF5_TOOLS_DIR", ""), "/opt/conda/bin"):
        p = os.path.join(d, name)
        if d and os.path.exists(p):
            return p
    return shutil.which(name)


needs_h5dump = pytest.mark.skipif(_tool("h5dump") is None, reason="HDF5 command line tools not installed")


def _circuit(dt=0.1):
    return {"run": {"dt": dt, "tstop": 3000.0},
            "components": {"point_neuron_models_dir": os.path.join(G, "cell_models"),
                           "synaptic_models_dir": os.path.join(G, "synaptic_models")},
            "networks": {"nodes": [{"nodes_file": os.path.join(NETDIR, "v1_nodes.h5"),
                                    "node_types_file": os.path.join(NETDIR, "v1_node_types.csv")},
                                   {"nodes_file": os.path.join(NETDIR, "lgn_nodes.h5"),
                                    "node_types_file": os.path.join(NETDIR, "lgn_node_types.csv")}],
                         "edges": [{"edges_file": os.path.join(NETDIR, "v1_v1_edges.h5"),
                                    "edge_types_file": os.path.join(NETDIR, "v1_v1_edge_types.csv")},
                                   {"edges_file": os.path.join(NETDIR, "lgn_v1_edges.h5"),
                                    "edge_types_file": os.path.join(NETDIR, "lgn_v1_edge_types.csv")}]}}


def _h5dump_values(path, dataset, dtype):
    out = subprocess.run([_tool("h5dump"), "-d", dataset, "-y", "-w", "65535", path], capture_output=True, text=True,
                         check=True).stdout
    start = out.index("DATA {") + 6
    body = out[start:out.index("}", start)]
    return np.array([t for t in body.replace("\n", " ").replace(",", " ").split() if t], dtype=dtype)


def test_reader_example_structure():
    with h5lite.File(os.path.join(NETDIR, "v1_v1_edges.h5")) as f:
        assert int(f.attrs["magic"]) == 0x0A7A and list(f.attrs["version"]) == [0, 1]
        g = f["/edges/v1_to_v1"]
        assert g.keys() == ["0", "edge_group_id", "edge_group_index", "edge_type_id", "indices", "source_node_id",
                            "target_node_id"]
        assert g["source_node_id"].attrs["node_population"] == "v1"
        assert g["source_node_id"].dtype == np.dtype("<u8") and g["source_node_id"].shape == (28555,)
        assert g["0/nsyns"].dtype == np.dtype("<u4")
        assert "indices/target_to_source/node_id_to_range" in g and "nope" not in g
        with pytest.raises(KeyError):
            g["missing"]
        # edges are written target-major (the builder sorts by target)
        assert np.all(np.diff(g["target_node_id"][()].astype(np.int64)) >= 0)
    with h5lite.File(os.path.join(NETDIR, "v1_nodes.h5")) as f:
        ntid = f["/nodes/v1/node_type_id"][()]
        # 80,80,80 excitatory + 30,30 inhibitory GLIF cells, 2 x 75 integrate-and-fire cells (v1_node_types.csv order)
        assert np.array_equal(np.bincount(ntid.astype(np.int64))[100:], [80, 80, 80, 30, 30, 75, 75])
        assert f["/nodes/v1/0/x"].dtype == np.float64 and f["/nodes/v1/1/x"].shape == (150,)
    with pytest.raises(h5lite.H5Error):
        h5lite.File(os.path.join(NETDIR, "v1_node_types.csv"))


@needs_h5dump
@pytest.mark.parametrize("fname,dataset,dtype", [
    ("v1_v1_edges.h5", "/edges/v1_to_v1/source_node_id", np.uint64),
    ("v1_v1_edges.h5", "/edges/v1_to_v1/0/nsyns", np.uint32),
    ("v1_v1_edges.h5", "/edges/v1_to_v1/indices/source_to_target/range_to_edge_id", np.uint64),
    ("lgn_v1_edges.h5", "/edges/lgn_to_v1/target_node_id", np.uint64),
    ("v1_nodes.h5", "/nodes/v1/0/rotation_angle_yaxis", np.float64),
])
def test_reader_agrees_with_hdf5_library(fname, dataset, dtype):
    path = os.path.join(NETDIR, fname)
    want = _h5dump_values(path, dataset, dtype)
    got = h5lite.File(path)[dataset][()].reshape(-1)
    if dtype == np.float64:
        assert np.allclose(got, want, rtol=1e-5)  # h5dump prints 6 significant digits
    else:
        assert np.array_equal(got, want)


def test_edge_indices_match_edge_lists():
    cfg = _circuit()
    for entry in cfg["networks"]["edges"]:
        for ep in sonata.read_edges(entry["edges_file"], entry["edge_types_file"]).values():
            assert set(ep.indices) == {"source_to_target", "target_to_source"}
            ep.check_indices()
            # and a broken index is noticed
            lookup, ranges = ep.indices["target_to_source"]
            bad = ranges.copy()
            bad[3, 1] += 1
            ep.indices["target_to_source"] = (lookup, bad)
            with pytest.raises(ValueError):
                ep.check_indices()


def test_edge_rules_on_example():
    """weight = nsyns * syn_weight of the edge's type, delay from the type table, receptor from the synaptic-model
    file (bmtk/simulator/pointnet/sonata_adaptors.py:268-357), stated here straight from the csv and json files."""
    entry = _circuit()["networks"]["edges"][0]
    ep = sonata.read_edges(entry["edges_file"], entry["edge_types_file"])["v1_to_v1"]
    assert ep.source_population == "v1" and ep.target_population == "v1"
    src, tgt, w, d, r = ep.to_arrays(os.path.join(G, "synaptic_models"), dt=0.1)
    with h5lite.File(entry["edges_file"]) as f:
        nsyns = f["/edges/v1_to_v1/0/nsyns"][()].astype(np.float64)
        etid = f["/edges/v1_to_v1/edge_type_id"][()]
    table = {}
    with open(entry["edge_types_file"]) as fh:
        head = fh.readline().split()
        for line in fh:
            row = dict(zip(head, line.split()))
            with open(os.path.join(G, "synaptic_models", row["dynamics_params"])) as jf:
                port = json.load(jf).get("receptor_type", 0)
            table[int(row["edge_type_id"])] = (float(row["syn_weight"]), float(row["delay"]), port)
    assert np.array_equal(w, np.array([nsyns[i] * table[t][0] for i, t in enumerate(etid)], np.float32))
    assert np.array_equal(d, np.array([round(table[t][1] / 0.1) for t in etid]))
    assert np.array_equal(r, np.array([table[t][2] for t in etid]))
    assert np.array_equal(src, ep.source_node_id) and np.array_equal(tgt, ep.target_node_id)
    with pytest.raises(net.BadDelay):
        ep.to_arrays(os.path.join(G, "synaptic_models"), dt=2.5)


def test_load_point_network():
    with pytest.raises(NotImplementedError, match="iaf_psc_alpha"):
        sonata.load_point_network(_circuit())
    nw = sonata.load_point_network(_circuit(), unsupported="silence")
    assert nw.population == "v1" and nw.n == 450 and nw.n_inputs == 100 and nw.virtual == {"lgn": 0}
    assert list(nw.supported) == [True] * 5 + [False] * 2
    assert np.array_equal(np.bincount(nw.class_id), [80, 80, 80, 30, 30, 75, 75])
    # the silenced cells neither receive nor send
    silent = ~nw.supported[nw.class_id]
    for e in (nw.rec_edges, nw.inp_edges):
        assert not silent[e[1]].any()
    assert not silent[nw.rec_edges[0]].any()
    rec, inp = nw.tables()
    net.check_csr(rec, 450, 450, 21)
    net.check_csr(inp, 100, 450, 21)
    # class parameters are the converted cell files: E_L of node type 100 (593618144) from its json
    with open(os.path.join(G, "cell_models", "593618144_glif_lif_asc_psc.json")) as fh:
        cell = json.load(fh)
    from bmtk_amd.layout import PAR
    assert nw.par[PAR["E_L"], 0] == cell["E_L"] and nw.par[PAR["C_M"], 0] == cell["C_m"]
    # excitatory sources carry positive weights, inhibitory ones negative (v1_v1_edge_types.csv)
    src_class = nw.class_id[nw.rec_edges[0]]
    assert np.all(nw.rec_edges[2][src_class <= 2] > 0) and np.all(nw.rec_edges[2][src_class >= 3] < 0)


def test_load_config_manifest(tmp_path):
    (tmp_path / "sub").mkdir()
    (tmp_path / "circuit.json").write_text(json.dumps({
        "manifest": {"$BASE_DIR": ".", "$NETWORK_DIR": "$BASE_DIR/network", "$MODELS": "${BASE_DIR}/../models"},
        "components": {"synaptic_models_dir": "$MODELS/syn"},
        "networks": {"nodes": [{"nodes_file": "$NETWORK_DIR/n.h5"}]}}))
    (tmp_path / "sim.json").write_text(json.dumps({
        "manifest": {"$OUT": "$configdir/output"}, "run": {"dt": 0.1}, "output": {"output_dir": "$OUT"},
        "network": "circuit.json"}))
    cfg = sonata.load_config(str(tmp_path / "sim.json"))
    assert cfg["networks"]["nodes"][0]["nodes_file"] == str(tmp_path / "network" / "n.h5")
    assert os.path.normpath(cfg["components"]["synaptic_models_dir"]) == str(tmp_path.parent / "models" / "syn")
    assert cfg["output"]["output_dir"] == str(tmp_path / "output") and cfg["run"]["dt"] == 0.1


def test_input_spike_file():
    sp = sonata.read_spikes(os.path.join(G, "point_450glifs", "inputs", "lgn_spikes.h5"))
    ids, ts, attrs = sp["lgn"]
    assert ids.size == 3044 and set(ids) <= set(range(100)) and attrs == {"sorting": "none", "units": "ms"}
    assert ts.min() > 0 and ts.max() < 3000.0
    # the file was written node by node: times ascend within a node
    for node in (0, 57, 99):
        assert np.all(np.diff(ts[ids == node]) > 0)


def _random_spikes(seed=1, n=5000):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 300, n), rng.random(n) * 3000.0


@pytest.mark.parametrize("order", ["none", "by_time", "by_id", "unknown"])
def test_spike_file_round_trip(tmp_path, order):
    ids, ts = _random_spikes()
    path = str(tmp_path / "out" / "spikes.h5")
    sonata.write_spikes(path, {"v1": (ids, ts), "empty": (np.zeros(0, int), np.zeros(0))}, sort_order=order)
    back = sonata.read_spikes(path)
    assert set(back) == {"v1", "empty"} and back["empty"][0].size == 0
    rid, rts, attrs = back["v1"]
    assert attrs["units"] == "ms" and attrs["sorting"] == order
    if order == "by_time":
        assert np.all(np.diff(rts) >= 0)
    elif order == "by_id":
        assert np.all(np.diff(rid) >= 0) and all(np.all(np.diff(rts[rid == k]) >= 0) for k in (0, 1, 299))
    else:
        assert np.array_equal(rid, ids) and np.array_equal(rts, ts)
    assert sonata.spikes_equal({"v1": (ids, ts)}, {"v1": (rid, rts)})
    with pytest.raises(ValueError, match="already contains"):
        sonata.write_spikes(path, {"v1": (ids, ts)}, mode="a")
    sonata.write_spikes(path, {"lgn": (ids[:10], ts[:10])}, mode="a")
    assert set(sonata.read_spikes(path)) == {"v1", "empty", "lgn"}
    csv = str(tmp_path / "spikes.csv")
    sonata.write_spikes_csv(csv, {"v1": (ids, ts)}, sort_order=order)
    with open(csv) as fh:
        assert fh.readline().strip() == "timestamps population node_ids"
    assert sonata.spikes_equal(sonata.read_spikes_csv(csv), {"v1": (ids, ts)}, err=1e-9)


@needs_h5dump
def test_written_file_is_read_by_hdf5_library(tmp_path):
    ids, ts = _random_spikes(2, 3000)
    path = str(tmp_path / "spikes.h5")
    sonata.write_spikes(path, {"v1": (ids, ts)}, sort_order="by_time")
    text = subprocess.run([_tool("h5dump"), "-A", path], capture_output=True, text=True, check=True).stdout
    for needle in ('ATTRIBUTE "magic"', '(0): 2682', 'ATTRIBUTE "sorting"', '"by_time"', 'ATTRIBUTE "units"', '"ms"',
                   'DATASET "node_ids"', "H5T_STD_U64LE", 'DATASET "timestamps"', "H5T_IEEE_F64LE",
                   "H5T_CSET_UTF8"):
        assert needle in text, needle
    order = np.lexsort((ids, ts))
    assert np.array_equal(_h5dump_values(path, "/spikes/v1/node_ids", np.uint64), ids[order].astype(np.uint64))
    # what bmtk itself writes is chunked and gzip-compressed (spikes_file_writers.py:66-68): let the HDF5 library
    # re-pack our file that way and read it back
    packed = str(tmp_path / "packed.h5")
    subprocess.run([_tool("h5repack"), "-f", "SHUF", "-f", "GZIP=4", "-l", "CHUNK=1000", path, packed], check=True)
    rid, rts, attrs = sonata.read_spikes(packed)["v1"]
    assert np.array_equal(rid, ids[order]) and np.array_equal(rts, ts[order]) and attrs["sorting"] == "by_time"


def test_h5lite_round_trip_types(tmp_path):
    rng = np.random.default_rng(0)
    tree = {"a": {"__attrs__": {"note": "täst", "k": np.int64(-3)},
                  "i8": rng.integers(-100, 100, 17).astype(np.int8), "u16": np.arange(5, dtype=np.uint16),
                  "f32": (rng.random((3, 4)).astype(np.float32), {"scale": 2.5}),
                  "names": np.array(["ab", "cde", ""]), "deep": {"x": np.zeros(0, np.float64)}},
            "flag": np.array([True, False])}
    path = str(tmp_path / "t.h5")
    h5lite.write(path, tree, attrs={"version": np.array([0, 1], np.uint32)})
    with h5lite.File(path) as f:
        assert f.keys() == ["a", "flag"] and f["a"].attrs == {"note": "täst", "k": -3}
        assert np.array_equal(f["a/i8"][()], tree["a"]["i8"]) and f["a/i8"].dtype == np.int8
        assert np.array_equal(f["a/f32"][()], tree["a"]["f32"][0]) and f["a/f32"].attrs["scale"] == 2.5
        assert list(f["a/names"][()]) == [b"ab", b"cde", b""] and f["/a/deep/x"].shape == (0,)
        assert np.array_equal(f["a/u16"][1:3], [1, 2])
    with pytest.raises(h5lite.H5Error):
        h5lite.write(path, {str(i): np.zeros(1) for i in range(100)})  # more members than one group node holds


def test_spike_comparisons():
    a = {"v1": (np.array([0, 0, 1, 2]), np.array([1.0, 5.0, 2.0, 3.0]))}
    same = {"v1": (np.array([2, 1, 0, 0]), np.array([3.0, 2.0, 5.0, 1.001]))}
    # numpy's allclose adds its default relative tolerance of 1e-5 to `err`, in the reference as here
    assert sonata.spikes_equal(a, same, err=1e-2) and not sonata.spikes_equal(a, same)
    fewer = {"v1": (np.array([0, 2]), np.array([5.0, 3.0]))}
    assert not sonata.spikes_equal(a, fewer)
    assert sonata.spikes_is_subset(fewer, a) and not sonata.spikes_is_subset(a, fewer)
    assert sonata.spikes_is_subset(a, same, err=1e-2) and not sonata.spikes_is_subset(a, same, err=1e-2, strict=True)
    moved = {"v1": (np.array([0, 2]), np.array([5.0, 3.5]))}
    assert not sonata.spikes_is_subset(moved, a)
    other_pop = {"lgn": a["v1"]}
    assert not sonata.spikes_equal(a, other_pop) and not sonata.spikes_is_subset(a, other_pop)
    assert sonata.spikes_is_subset({"v1": (np.zeros(0, int), np.zeros(0))}, a)


def test_poisson_generator_files(tmp_path):
    """The calls of examples/point_450glifs/create_inputs.py: ids from a nodes file, trains to SONATA and csv."""
    from bmtk_amd.spike_trains import PoissonSpikeGenerator
    nodes = os.path.join(NETDIR, "lgn_nodes.h5")
    psg = PoissonSpikeGenerator(population="lgn", seed=7)
    psg.add(node_ids=nodes, firing_rate=15.0, times=(0.0, 0.5), population="lgn")
    with h5lite.File(nodes) as h5:
        want_ids = np.asarray(h5["/nodes/lgn/node_id"][()])
    assert psg.node_ids("lgn") == sorted(want_ids.tolist()) or set(psg.node_ids("lgn")) <= set(want_ids.tolist())
    h5p, csvp = str(tmp_path / "in.h5"), str(tmp_path / "in.csv")
    psg.to_sonata(h5p, sort_order="by_id")
    psg.to_csv(csvp)
    ids, ts, attrs = sonata.read_spikes(h5p)["lgn"]
    assert attrs["sorting"] == "by_id" and np.all(np.diff(ids) >= 0)
    assert ids.size == psg.n_spikes("lgn") and ts.min() >= 0 and ts.max() <= 500.0
    for n in (int(ids[0]), int(ids[-1])):
        assert np.array_equal(np.sort(ts[ids == n]), np.sort(psg.get_times(n, "lgn")))
    cid, cts = sonata.read_spikes_csv(csvp)["lgn"][:2]
    assert sonata.spikes_equal({"lgn": (ids, ts)}, {"lgn": (cid, cts)})


def _magic():
    return {"magic": np.uint32(sonata.MAGIC_VAL), "version": np.array(sonata.VERSION, np.uint32)}


def test_write_no_spikes(tmp_path):
    """A run without a single spike still writes a valid file with an empty /spikes group
    (bmtk/tests/utils/reports/spike_trains/test_sonata_adaptor.py:103-116)."""
    path = str(tmp_path / "none.h5")
    sonata.write_spikes(path, {})
    with h5lite.File(path) as h5:
        assert int(h5.attrs["magic"]) == sonata.MAGIC_VAL and len(h5.attrs["version"]) == 2
        assert "/spikes" in h5 and len(h5["/spikes"].keys()) == 0
    assert sonata.read_spikes(path) == {}
    # a population that never fired
    sonata.write_spikes(path, {"V1": (np.zeros(0, np.int64), np.zeros(0))}, sort_order="by_time")
    ids, ts, attrs = sonata.read_spikes(path)["V1"]
    assert ids.size == 0 and ts.size == 0 and attrs["sorting"] == "by_time"


def test_append_keeps_other_populations_and_refuses_an_existing_one(tmp_path):
    """test_sonata_adaptor.py:125-157: mode 'a' adds /spikes/V2 beside an existing (here empty) /spikes/V1 and
    raises ValueError when /spikes/V2 is already there."""
    path = str(tmp_path / "a.h5")
    h5lite.write(path, {"spikes": {"V1": {}}}, attrs=_magic())
    new = {"V2": (np.zeros(100, np.int64), np.linspace(0, 1.0, 100))}
    sonata.write_spikes(path, new, mode="a", sort_order="by_id")
    with h5lite.File(path) as h5:
        assert "/spikes/V1" in h5 and "/spikes/V2" in h5
        assert h5["/spikes/V2/node_ids"].shape == (100,) and h5["/spikes/V2/timestamps"].shape == (100,)
    path2 = str(tmp_path / "b.h5")
    h5lite.write(path2, {"spikes": {"V2": {}}}, attrs=_magic())
    with pytest.raises(ValueError):
        sonata.write_spikes(path2, new, mode="a", sort_order="by_id")
    # appending to a file that holds data keeps that data
    sonata.write_spikes(path, {"V3": (np.array([4, 2]), np.array([1.5, 0.5]))}, mode="a", sort_order="by_time")
    got = sonata.read_spikes(path)
    assert set(got) == {"V2", "V3"} and got["V2"][0].size == 100
    np.testing.assert_array_equal(got["V3"][0], [2, 4])


def test_older_spike_file_layout_and_mixed_file(tmp_path):
    """test_sonata_adaptor.py:242-262 and :268-300: /spikes/gids + /spikes/timestamps without a population group
    is read under the placeholder population; empty population groups are skipped."""
    ids = np.array([0, 0, 0, 0, 2, 1, 2], np.uint64)
    ts = np.array([0.25, 0.5, 0.75, 1.0, 3.0, 0.001, 2.0])
    old = str(tmp_path / "old.h5")
    h5lite.write(old, {"spikes": {"gids": ids, "timestamps": ts}}, attrs=_magic())
    got = sonata.read_spikes(old)
    assert list(got) == ["<sonata:none>"]
    g_ids, g_ts, _ = got["<sonata:none>"]
    assert g_ids.size == 7 and set(g_ids.tolist()) == {0, 1, 2}
    np.testing.assert_allclose(np.sort(g_ts[g_ids == 0]), [0.25, 0.5, 0.75, 1.0])
    new = str(tmp_path / "new.h5")
    h5lite.write(new, {"spikes": {"V1": {"node_ids": ids, "timestamps": ts},
                                  "V2": {"node_ids": np.array([10, 10, 10], np.uint64),
                                         "timestamps": np.array([4.0, 4.0, 4.0])},
                                  "V3": {}}}, attrs=_magic())
    got = sonata.read_spikes(new)
    assert set(got) == {"V1", "V2"} and got["V2"][0].tolist() == [10, 10, 10]
    assert sonata.read_spikes(new, populations=["V2"]).keys() == {"V2"}
    with pytest.raises(ValueError):
        bad = str(tmp_path / "bad.h5")
        h5lite.write(bad, {"other": {}}, attrs=_magic())
        sonata.read_spikes(bad)


def test_csv_without_population_column(tmp_path):
    """bmtk/tests/utils/reports/spike_trains/test_csv_adaptor.py:135-160."""
    path = str(tmp_path / "s.csv")
    with open(path, "w") as fh:
        fh.write("timestamps node_ids\n0.25 0\n0.5 0\n3.0 2\n0.001 1\n")
    got = sonata.read_spikes_csv(path)
    assert list(got) == ["<sonata:none>"]
    assert got["<sonata:none>"][0].tolist() == [0, 0, 2, 1]


def _config(tmp_path, d):
    path = str(tmp_path / "cfg.json")
    with open(path, "w") as fh:
        json.dump(d, fh)
    return sonata.load_config(path)


def test_manifest_rules(tmp_path):
    """bmtk/tests/utils/sonata/test_config.py:156-198: variables may build on each other in both spellings; an
    unknown variable or a circular definition raises."""
    cfg = _config(tmp_path, {"manifest": {"$BASE_DIR": "/base", "$TMP_DIR": "$BASE_DIR/tmp",
                                          "$SHARE_DIR": "${TMP_DIR}_1/share"}, "x": "$SHARE_DIR/y"})
    assert cfg["x"] == "/base/tmp_1/share/y"
    cfg = _config(tmp_path, {"manifest": {"$DIR_DATA": "data", "$DIR_MAT": "mat",
                                          "$APPS": "/${DIR_DATA}/$DIR_MAT/apps"}, "x": "$APPS"})
    assert cfg["x"] == "/data/mat/apps"
    with pytest.raises(ValueError):
        _config(tmp_path, {"manifest": {"$BASE": "/base", "$TMP": "$VAR/Smat"}})
    with pytest.raises(ValueError):
        _config(tmp_path, {"manifest": {"$BASE": "$TMP/share", "$TMP": "$BASE/share"}})


def _bare_simulator(dt=0.1, tstop=3500.0, n=120):
    from types import SimpleNamespace
    from bmtk_amd import pointnet
    net_ = SimpleNamespace(n=n, n_inputs=0, population="cortex", virtual={})
    return pointnet.PointSimulator(net_, dt, tstop)


def test_constant_current_of_the_cell_models_is_the_base_of_every_segment():
    """A cell model's I_e (pA, a constant input current) is not a row of the parameter table: it is the
    external current on which the current clamps are stacked."""
    from types import SimpleNamespace
    from bmtk_amd import pointnet
    net_ = SimpleNamespace(n=6, n_inputs=0, population="cortex", virtual={}, i_e=np.array([0.0, 25.0]),
                           class_id=np.array([0, 1, 1, 0, 1, 0], np.int32))
    sim = pointnet.PointSimulator(net_, 0.5, 100.0)
    sim.add_current_clamp({"input_type": "current_clamp", "module": "IClamp", "node_set": [1, 3], "amp": 100.0,
                           "delay": 20.0, "duration": 30.0})
    segs = [(a, b, cur.tolist()) for a, b, cur in sim._segments()]
    assert segs == [(0, 41, [0.0, 25.0, 25.0, 0.0, 25.0, 0.0]), (41, 101, [0.0, 125.0, 25.0, 100.0, 25.0, 0.0]),
                    (101, 200, [0.0, 25.0, 25.0, 0.0, 25.0, 0.0])]


def test_current_clamp_amplitude_lists():
    """The amplitude times/values bmtk's IClamp module hands to a step_current_generator
    (bmtk/simulator/pointnet/modules/iclamp.py:13-39) for the inputs of examples/point_iclamp."""
    sim = _bare_simulator()
    # config.simulation_iclamp.aslist.json: three steps, each switched off before the next begins
    sim.add_current_clamp({"input_type": "current_clamp", "module": "IClamp", "node_set": {"population": "cortex"},
                           "amp": [0.15, 0.175, 0.2], "delay": [500.0, 1500.0, 2500.0],
                           "duration": [500.0, 500.0, 500.0]})
    ids, times, values = sim._clamps[-1]
    assert ids.tolist() == list(range(120))
    assert times.tolist() == [500.0, 1000.0, 1500.0, 2000.0, 2500.0, 3000.0]
    assert values.tolist() == [0.15, 0.0, 0.175, 0.0, 0.2, 0.0]
    # an amplitude still on when the next begins is replaced, not switched off; an onset at or before dt is skipped
    sim.add_current_clamp({"input_type": "current_clamp", "node_set": {"population": "cortex", "node_ids": [3, 4]},
                           "amp": [9.0, 1.0, 2.0], "delay": [0.1, 10.0, 15.0], "duration": [5.0, 20.0, 5.0]})
    ids, times, values = sim._clamps[-1]
    assert ids.tolist() == [3, 4] and times.tolist() == [10.0, 15.0, 20.0] and values.tolist() == [1.0, 2.0, 0.0]
    # config.simulation_iclamp.csv.json: the file's rows as they are
    sim.add_current_clamp({"input_type": "csv", "module": "IClamp", "node_set": {"population": "cortex"},
                           "file": os.path.join(G, "point_iclamp", "iclamp_inputs_1.csv")})
    _, times, values = sim._clamps[-1]
    assert times.tolist() == [800.0, 1300.0, 1800.0, 2300.0, 2800.0, 3300.0]
    assert values.tolist() == [0.15, 0.0, 0.175, 0.0, 0.2, 0.0]
    with pytest.raises(ValueError):
        sim.add_current_clamp({"input_type": "current_clamp", "node_set": [0], "amp": [1.0, 2.0], "delay": [5.0],
                               "duration": [1.0]})
    with pytest.raises(ValueError):
        sim.add_current_clamp({"input_type": "current_clamp", "node_set": {"population": "thalamus"}, "amp": 1.0,
                               "delay": 5.0, "duration": 1.0})
    with pytest.raises(NotImplementedError):
        sim.add_current_clamp({"input_type": "movie", "node_set": [0]})


def test_current_clamp_from_nwb_sweep(tmp_path):
    """The stimulus of one sweep of an Allen Cell Types NWB file (bmtk/simulator/core/modules/iclamp.py:61-113): a
    file of that layout written here, 20 kHz, a 0.5 nA step from 10 to 20 ms."""
    data = np.zeros(800)
    data[200:400] = 0.5e-9
    path = str(tmp_path / "ephys.nwb")
    h5lite.write(path, {"epochs": {"Sweep_55": {"stimulus": {"timeseries": {
        "data": data, "starting_time": (np.float64(0.0), {"rate": np.float64(20000.0)})}}}}})
    sim = _bare_simulator(dt=0.01, tstop=100.0, n=3)
    sim.add_current_clamp({"input_type": "nwb", "module": "IClamp", "node_set": {"population": "cortex"},
                           "file": path, "sweep_id": 55, "downsample": 0.1})
    ids, times, values = sim._clamps[-1]
    assert ids.tolist() == [0, 1, 2]
    # every second sample (0.1 ms) except the first, whose onset is not after the resolution
    np.testing.assert_allclose(times, np.arange(1, 400) * 0.1)
    on = (times >= 10.0 - 1e-9) & (times < 20.0 - 1e-9)
    np.testing.assert_allclose(values[on], 0.5)
    assert on.sum() == 100 and np.all(values[~on] == 0.0)
    sim.add_current_clamp({"input_type": "nwb", "node_set": [1], "file": path, "sweep_id": "55",
                           "sweep_window": [5.0, 12.0], "delay": 100.0})
    _, times, values = sim._clamps[-1]
    np.testing.assert_allclose(times[[0, -1]], [105.0, 112.0])
    assert values[0] == 0.0 and values[-1] == 0.5
    with pytest.raises(ValueError):
        sim.add_current_clamp({"input_type": "nwb", "node_set": [1], "file": path, "sweep_id": 7})


def test_current_segments_add_up_the_generators():
    """An amplitude set for time t acts from the step that starts at t + dt; the generators on a node add up."""
    sim = _bare_simulator(dt=0.5, tstop=50.0, n=4)
    sim.add_current_clamp({"input_type": "current_clamp", "node_set": [0, 1], "amp": 10.0, "delay": 5.0,
                           "duration": 10.0})
    sim.add_current_clamp({"input_type": "current_clamp", "node_set": [1, 2], "amp": -4.0, "delay": 10.0,
                           "duration": 30.0})
    segs = [(a, b, cur.tolist()) for a, b, cur in sim._segments()]
    assert segs == [(0, 11, [0, 0, 0, 0]), (11, 21, [10, 10, 0, 0]), (21, 31, [10, 6, -4, 0]),
                    (31, 81, [0, -4, -4, 0]), (81, 100, [0, 0, 0, 0])]


def _edges_with_weight_functions(tmp_path):
    """A copy of the example's recurrent edge types in which type 100 names a built-in weight function and type
    101 a user-registered one."""
    entry = _circuit()["networks"]["edges"][0]
    with open(entry["edge_types_file"]) as fh:
        head = fh.readline().split()
        rows = [line.split() for line in fh if line.strip()]
    fn = {"100": "wmax", "101": "by_distance"}
    path = tmp_path / "edge_types.csv"
    with open(path, "w") as fh:
        fh.write(" ".join(head + ["weight_function"]) + "\n")
        for r in rows:
            fh.write(" ".join(r + [fn.get(r[0], "NONE")]) + "\n")
    return entry, str(path)


def test_weight_functions(tmp_path):
    """`weight_function` of an edge type (sonata_adaptors.py:319-335): bmtk's built-in names give nsyns * syn_weight
    (default_setters/synaptic_weights.py), a registered function is called with the type's edges and their source
    and target nodes as dataframes, an unknown name is an error, and types without a function keep the rule."""
    entry, types_file = _edges_with_weight_functions(tmp_path)
    nodes_entry = _circuit()["networks"]["nodes"][0]
    pop = sonata.read_nodes(nodes_entry["nodes_file"], nodes_entry["node_types_file"])["v1"]
    plain = sonata.read_edges(entry["edges_file"], entry["edge_types_file"])["v1_to_v1"]
    _, _, w_plain, d_plain, r_plain = plain.to_arrays(os.path.join(G, "synaptic_models"), dt=0.1)
    ep = sonata.read_edges(entry["edges_file"], types_file)["v1_to_v1"]
    with pytest.raises(Exception, match="by_distance"):
        ep.to_arrays(os.path.join(G, "synaptic_models"), dt=0.1, source_nodes=pop, target_nodes=pop)
    seen = {}

    @sonata.synaptic_weight(name="by_distance")
    def by_distance(edges, source_nodes, target_nodes):
        seen["n"] = len(edges)
        assert len(source_nodes) == len(target_nodes) == len(edges)
        assert np.array_equal(source_nodes.index.values, edges["source_node_id"].values)
        assert np.array_equal(target_nodes["node_id"].values, edges["target_node_id"].values)
        assert set(edges["edge_type_id"]) == {101} and (target_nodes["ei"] == "i").all()
        gap = np.abs(source_nodes["node_id"].values - target_nodes["node_id"].values)
        return edges["syn_weight"].values * edges["nsyns"].values / (1.0 + gap)
    try:
        with pytest.raises(ValueError, match="node populations"):
            ep.to_arrays(os.path.join(G, "synaptic_models"), dt=0.1)
        src, tgt, w, d, r = ep.to_arrays(os.path.join(G, "synaptic_models"), dt=0.1, source_nodes=pop, target_nodes=pop)
    finally:
        sonata._WEIGHT_FUNCTIONS.pop("by_distance", None)
    is101 = ep.edge_type_id == 101
    assert seen["n"] == int(is101.sum()) > 0
    assert np.array_equal(w[~is101], w_plain[~is101])            # wmax and the types without a function: the rule
    want = w_plain[is101].astype(np.float64) / (1.0 + np.abs(src[is101] - tgt[is101]))
    assert np.allclose(w[is101], want, rtol=1e-6) and not np.array_equal(w[is101], w_plain[is101])
    assert np.array_equal(d, d_plain) and np.array_equal(r, r_plain)
    # the dataframes themselves: one row per node / edge, type columns joined in
    ndf = pop.to_dataframe()
    assert len(ndf) == len(pop) and {"node_type_id", "node_id", "model_template", "ei"} <= set(ndf.columns)
    edf = plain.to_dataframe()
    assert len(edf) == len(plain) and {"edge_type_id", "source_node_id", "target_node_id", "nsyns", "syn_weight",
                                       "delay"} <= set(edf.columns)
    assert np.array_equal(edf["nsyns"].values * edf["syn_weight"].values, w_plain.astype(np.float64))
