"""SONATA files <-> the arrays the GPU path works on.

What bmtk's PointNet driver does between opening its files and calling NEST,
restated for GLIF point networks:

* node files + node-type tables -> one parameter class per node type
  (bmtk/simulator/pointnet/sonata_adaptors.py:132-167, bmtk/simulator/core/
  sonata_reader/node_adaptor.py:102-165, bmtk/utils/sonata/population.py);
* edge files + edge-type tables + synaptic-model files -> edge lists with
  ``weight = nsyns * syn_weight``, ``delay`` and ``receptor_type``
  (sonata_adaptors.py:268-357), then synapse tables (bmtk_amd.network);
* spike files: the ``/spikes/<population>/{timestamps,node_ids}`` layout that
  bmtk writes and reads (bmtk/utils/reports/spike_trains/spikes_file_writers.py:35-73,
  spike_train_readers.py:93-292), the space-separated csv twin
  (spikes_file_writers.py:115-126), and the two comparisons its tests use
  (spike_trains_api.py:186-280).

HDF5 access goes through bmtk_amd.h5lite (h5py is not required).
"""
import json
import os
import re

import numpy as np
import pandas as pd

from . import glif_utils, h5lite, network as net
from .layout import NPARAM

MAGIC_VAL = 0x0A7A  # bmtk/utils/sonata/utils.py:30-33
VERSION = (0, 1)
SORT_ORDERS = ("none", "by_id", "by_time", "unknown")  # bmtk/utils/reports/spike_trains/core.py:34-38


# ----------------------------------------------------------------------------------------------------------------
# configuration files
# ----------------------------------------------------------------------------------------------------------------

def _substitute(value, manifest):
    if isinstance(value, str):
        for _ in range(8):
            new = value
            for k, v in manifest.items():
                new = new.replace("${" + k[1:] + "}", v).replace(k, v)
            if new == value:
                break
            value = new
        return value
    if isinstance(value, dict):
        return {k: _substitute(v, manifest) for k, v in value.items()}
    if isinstance(value, list):
        return [_substitute(v, manifest) for v in value]
    return value


def load_config(path):
    """A SONATA/bmtk json configuration with its ``manifest`` variables expanded (``$BASE_DIR`` style, longest
    names first; ``.`` and ``${configdir}`` stand for the directory of the file) and a ``network`` entry that
    names another file merged in, as bmtk/simulator/core/simulation_config.py does."""
    path = os.path.abspath(path)
    with open(path) as fh:
        cfg = json.load(fh)
    base = os.path.dirname(path)
    manifest = {"$configdir": base, "$workingdir": os.getcwd()}
    raw = dict(cfg.get("manifest", {}))
    # a variable is taken into the manifest once nothing in it is left to expand; one that names an unknown
    # variable, or two that name each other, never get there (sonata_config.py:258-330 raises for both)
    pending = dict(raw)
    while pending:
        known = dict(sorted(manifest.items(), key=lambda kv: -len(kv[0])))
        done = {}
        for k, v in pending.items():
            v = _substitute(v, known)
            if not re.search(r"\$\{?[A-Za-z_]\w*\}?", v):
                done[k] = os.path.normpath(os.path.join(base, v)) if v == "." or v.startswith("./") else v
        if not done:
            raise ValueError("{}: manifest variables {} cannot be resolved".format(path, sorted(pending)))
        manifest.update(done)
        pending = {k: v for k, v in pending.items() if k not in done}
    cfg = _substitute(cfg, dict(sorted(manifest.items(), key=lambda kv: -len(kv[0]))))
    for key in ("network", "simulation"):
        if isinstance(cfg.get(key), str):
            sub = cfg[key] if os.path.isabs(cfg[key]) else os.path.join(base, cfg[key])
            merged = load_config(sub)
            merged.update({k: v for k, v in cfg.items() if k != key})
            cfg = merged
    return cfg


def load_csv(path):
    """Type tables are space separated and spell a missing value NONE (bmtk/utils/sonata/utils.py:61-67)."""
    return pd.read_csv(path, sep=" ", na_values="NONE")


def check_magic(h5, path):
    magic = h5.attrs.get("magic")
    if magic is not None and int(np.asarray(magic).reshape(-1)[0]) != MAGIC_VAL:
        raise ValueError("File {} has unexpected magic value (expected {})".format(path, MAGIC_VAL))


# ----------------------------------------------------------------------------------------------------------------
# nodes
# ----------------------------------------------------------------------------------------------------------------

class NodePopulation:
    """One ``/nodes/<name>`` group: ids, type ids, and the type table indexed by ``node_type_id``."""

    def __init__(self, name, node_ids, node_type_ids, group_ids, group_index, groups, types):
        self.name = name
        self.node_ids = node_ids
        self.node_type_ids = node_type_ids
        self.group_ids = group_ids
        self.group_index = group_index
        self.groups = groups  # {group id: {column: array}}
        self.types = types

    def __len__(self):
        return self.node_ids.size

    def type_of(self, node_type_id):
        return self.types.loc[node_type_id]

    def to_dataframe(self):
        """One row per node, indexed by node id: ``node_type_id``, ``node_id``, the per-node group columns and the
        type-table columns (what bmtk's ``get_nodes_df`` hands a weight function)."""
        df = _frame(len(self), self.group_ids, self.group_index, self.groups, self.types, self.node_type_ids,
                    "node_type_id")
        df.insert(0, "node_id", self.node_ids)
        df.insert(0, "node_type_id", self.node_type_ids)
        return df.set_index(self.node_ids)

    def column(self, name):
        """A per-node attribute, from the groups where it is stored per node, else from the type table."""
        out = np.empty(len(self), object)
        have = np.zeros(len(self), bool)
        for gid, cols in self.groups.items():
            if name in cols:
                sel = self.group_ids == gid
                out[sel] = cols[name][self.group_index[sel]]
                have |= sel
        if name in self.types.columns:
            vals = self.types[name].reindex(self.node_type_ids).to_numpy()
            out[~have] = vals[~have]
        elif not have.all():
            raise KeyError(name)
        return out


def _frame(n, group_ids, group_index, groups, types, type_ids, type_key):
    """Per-item table of a population: the group datasets (a column of several components becomes ``name.0``,
    ``name.1`` ...; items whose group lacks a column hold NaN / None) joined with the columns of the type table
    that no group stores, the way bmtk/utils/sonata/group.py:209-243,339-372 builds its dataframes."""
    cols = {}
    for gid, datasets in groups.items():
        sel = group_ids == gid
        for name, values in datasets.items():
            values = np.asarray(values)
            parts = [(name, values)] if values.ndim == 1 else [("{}.{}".format(name, i), values[:, i])
                                                               for i in range(values.shape[1])]
            for cname, v in parts:
                if cname not in cols:
                    numeric = v.dtype.kind in "fiub"
                    cols[cname] = np.full(n, np.nan) if numeric else np.full(n, None, object)
                cols[cname][sel] = v[group_index[sel]]
    df = pd.DataFrame(cols)
    type_cols = [c for c in types.columns if c not in cols and c != type_key]
    for c in type_cols:
        df[c] = types[c].reindex(type_ids).to_numpy()
    return df


def read_nodes(nodes_file, node_types_file):
    """-> {population name: NodePopulation}; node ids must be unique, the type table must cover every type id
    (bmtk/utils/sonata/population.py:150-260)."""
    types = load_csv(node_types_file).set_index("node_type_id", drop=False)
    pops = {}
    with h5lite.File(nodes_file) as h5:
        check_magic(h5, nodes_file)
        for name in h5["/nodes"].keys():
            g = h5["/nodes/" + name]
            ntid = np.asarray(g["node_type_id"][()], np.int64)
            nid = np.asarray(g["node_id"][()], np.int64) if "node_id" in g else np.arange(ntid.size, dtype=np.int64)
            if np.unique(nid).size != nid.size:
                raise ValueError("{}: node ids of population {} are not unique".format(nodes_file, name))
            missing = set(np.unique(ntid)) - set(types.index)
            if missing:
                raise ValueError("{}: node types {} missing from {}".format(nodes_file, sorted(missing),
                                                                            node_types_file))
            groups = {}
            for sub in g.keys():
                if sub.isdigit() and isinstance(g[sub], h5lite.Group):
                    groups[int(sub)] = {k: v[()] for k, v in g[sub].items() if isinstance(v, h5lite.Dataset)}
            gid = np.asarray(g["node_group_id"][()], np.int64) if "node_group_id" in g else np.zeros(nid.size,
                                                                                                     np.int64)
            gix = np.asarray(g["node_group_index"][()], np.int64) if "node_group_index" in g else np.arange(
                nid.size, dtype=np.int64)
            pops[name] = NodePopulation(name, nid, ntid, gid, gix, groups, types)
    return pops


def _load_dynamics(name, directory):
    if isinstance(name, dict):
        return name
    if name is None or (isinstance(name, float) and np.isnan(name)):
        return {}
    with open(os.path.join(directory, name)) as fh:
        return json.load(fh)


def node_parameter_classes(pop, models_dir, unsupported="raise"):
    """One GLIF3 parameter class per node type of a population.

    -> (par fp64 [NPARAM, classes], asc_init [2, classes], u_init [classes], class_id int32 [nodes] ordered by
    node id, supported bool [classes], type ids [classes], i_e fp64 [classes]: a constant input current ``I_e``
    in pA where a cell-model file gives one, which is no row of the parameter table but part of the external
    current).

    ``nest:glif_psc`` with ready NEST-unit parameters is taken as is; ``nest:glif_*`` templates with an Allen
    cell-types file (``"type": "GLIF"``) are converted first (sonata_adaptors.py:155-167).  Any other point model
    raises, or with ``unsupported="silence"`` becomes a class that never fires (threshold out of reach, no
    after-spike currents) so that node ids keep their place; such a network is NOT the one the files describe.
    """
    type_ids = np.unique(pop.node_type_ids)
    cells, supported = [], []
    for t in type_ids:
        row = pop.type_of(t)
        template = str(row.get("model_template", ""))
        model_type = str(row.get("model_type", ""))
        dyn = _load_dynamics(row.get("dynamics_params"), models_dir) if model_type != "virtual" else {}
        ok = False
        if template.startswith("nest:glif"):
            if dyn.get("type") == "GLIF":
                template, dyn = glif_utils.convert_aibs2nest(template, dyn)
            ok = template == "nest:glif_psc"
        if ok:
            cells.append(dyn)
        elif unsupported == "silence":
            cells.append({"C_m": 100.0, "g": 10.0, "E_L": -70.0, "V_th": 1.0e30, "V_reset": -70.0, "t_ref": 1.0,
                          "after_spike_currents": False})
        else:
            raise NotImplementedError("node type {} of population {}: model {!r} ({}) is not a GLIF model the GPU "
                                      "path implements".format(t, pop.name, template, model_type))
        supported.append(ok)
    par, asc_init, u_init = glif_utils.params_table(cells)
    order = np.argsort(pop.node_ids, kind="stable")
    class_of_type = {t: i for i, t in enumerate(type_ids)}
    class_id = np.array([class_of_type[t] for t in pop.node_type_ids[order]], np.int32)
    assert par.shape[0] == NPARAM
    i_e = np.array([float(c.get("I_e", 0.0)) for c in cells], np.float64)
    return par, asc_init, u_init, class_id, np.array(supported), type_ids, i_e


# ----------------------------------------------------------------------------------------------------------------
# edges
# ----------------------------------------------------------------------------------------------------------------

def default_weight_fnc(edge_props, source_nodes, target_nodes):
    """``syn_weight * nsyns`` (bmtk/simulator/pointnet/default_setters/synaptic_weights.py:6-7)."""
    return np.array(edge_props["syn_weight"] * edge_props["nsyns"])


# weight functions by the name an edge type's ``weight_function`` column gives; the three names bmtk registers at
# import (synaptic_weights.py:10-12) all stand for the default rule
_WEIGHT_FUNCTIONS = {"default_weight_fnc": default_weight_fnc, "set_syn_weight": default_weight_fnc,
                     "wmax": default_weight_fnc}


def add_weight_function(func, name=None, overwrite=True):
    """Register ``func(edges_df, source_nodes_df, target_nodes_df) -> weights`` under ``name`` (default: the
    function's own name), as bmtk's ``add_weight_function`` does (bmtk/simulator/core/pyfunction_cache.py)."""
    name = name or func.__name__
    if overwrite or name not in _WEIGHT_FUNCTIONS:
        _WEIGHT_FUNCTIONS[name] = func
    return func


def synaptic_weight(*args, **kwargs):
    """Decorator form: ``@synaptic_weight`` or ``@synaptic_weight(name='...')``."""
    if len(args) == 1 and callable(args[0]) and not kwargs:
        return add_weight_function(args[0])
    name = kwargs.get("name", args[0] if args else None)
    return lambda func: add_weight_function(func, name)


class EdgePopulation:
    def __init__(self, name, source_population, target_population, source_node_id, target_node_id, edge_type_id,
                 group_ids, group_index, groups, indices, types):
        self.name = name
        self.source_population = source_population
        self.target_population = target_population
        self.source_node_id = source_node_id
        self.target_node_id = target_node_id
        self.edge_type_id = edge_type_id
        self.group_ids = group_ids
        self.group_index = group_index
        self.groups = groups
        self.indices = indices  # {"target_to_source" | "source_to_target": (node_id_to_range, range_to_edge_id)}
        self.types = types

    def __len__(self):
        return self.source_node_id.size

    def to_dataframe(self):
        """One row per edge in file order: ``edge_type_id``, ``source_node_id``, ``target_node_id``, the per-edge
        group columns and the type-table columns no group stores (bmtk/utils/sonata/group.py:339-372)."""
        df = _frame(len(self), self.group_ids, self.group_index, self.groups, self.types, self.edge_type_id,
                    "edge_type_id")
        df.insert(0, "target_node_id", self.target_node_id)
        df.insert(0, "source_node_id", self.source_node_id)
        df.insert(0, "edge_type_id", self.edge_type_id)
        return df

    def per_edge(self, name):
        """Per-edge values of a group dataset (``nsyns``, ``syn_weight``, ``delay``) or None when no group has it;
        edges of groups that lack the column hold NaN."""
        if not any(name in cols for cols in self.groups.values()):
            return None
        out = np.full(len(self), np.nan)
        for gid, cols in self.groups.items():
            if name in cols:
                sel = self.group_ids == gid
                out[sel] = cols[name][self.group_index[sel]]
        return out

    def edges_of(self, node_id, index="target_to_source"):
        """Edge ids that the stored index lists for one node (bmtk/utils/sonata/population.py:520-560): the
        node's rows [lo, hi) of ``range_to_edge_id``, each an edge-id range."""
        lookup, ranges = self.indices[index]
        lo, hi = lookup[node_id]
        parts = [np.arange(a, b, dtype=np.int64) for a, b in ranges[int(lo):int(hi)]]
        return np.concatenate(parts) if parts else np.zeros(0, np.int64)

    def check_indices(self):
        """The stored indices must list, for every node, exactly the edges whose target (source) it is."""
        for index, ids in (("target_to_source", self.target_node_id), ("source_to_target", self.source_node_id)):
            if index not in self.indices:
                continue
            lookup, _ = self.indices[index]
            order = np.argsort(ids, kind="stable")
            bounds = np.searchsorted(ids[order], np.arange(lookup.shape[0] + 1))
            for node in range(lookup.shape[0]):
                want = np.sort(order[bounds[node]:bounds[node + 1]])
                got = np.sort(self.edges_of(node, index))
                if not np.array_equal(want, got):
                    raise ValueError("{}: index {} disagrees with the edge list at node {}".format(self.name, index,
                                                                                                   node))

    def to_arrays(self, synaptic_models_dir, dt, source_nodes=None, target_nodes=None):
        """-> (source ids, target ids, weights f32, delay steps, receptor_type), one entry per edge in file
        order, by the rules of sonata_adaptors.py:268-357: per-edge ``delay``/``syn_weight``/``nsyns`` win over
        the type table, ``nsyns`` defaults to 1, a missing ``syn_weight`` is an error, the synaptic-model file
        supplies ``receptor_type`` (NEST's 1-based port; 0 where the file names none, which ``glif_psc`` rejects),
        the template must be a static synapse, and a delay below the resolution is a BadDelay.  An edge type with
        a ``weight_function`` gets its weights from the function registered under that name
        (``add_weight_function``), called with the type's edges and their source and target nodes as dataframes
        (``source_nodes`` / ``target_nodes``: the two ``NodePopulation``s), as sonata_adaptors.py:319-335 does."""
        n = len(self)
        w = np.empty(n, np.float64)
        delay = np.empty(n, np.float64)
        rec = np.empty(n, np.int64)
        nsyns_e, weight_e, delay_e = self.per_edge("nsyns"), self.per_edge("syn_weight"), self.per_edge("delay")
        frames = None  # (edges, source nodes, target nodes) as dataframes, built when a weight function asks
        for et in np.unique(self.edge_type_id):
            row = self.types.loc[et]
            sel = self.edge_type_id == et
            template = str(row.get("model_template", "static_synapse"))
            if template.startswith("nest:"):
                template = template[5:]
            if template != "static_synapse":
                raise NotImplementedError("edge type {}: synapse model {!r} is not implemented".format(et, template))
            weight_function = row.get("weight_function")
            if weight_function is not None and pd.isna(weight_function):
                weight_function = None
            dyn = _load_dynamics(row.get("dynamics_params"), synaptic_models_dir)
            extra = set(dyn) - {"receptor_type", "weight", "delay"}
            if extra:
                raise NotImplementedError("edge type {}: synapse parameters {} are not supported".format(
                    et, sorted(extra)))
            nsyns = nsyns_e[sel] if nsyns_e is not None else row.get("nsyns", 1)
            nsyns = np.where(np.isnan(np.asarray(nsyns, np.float64)), 1, nsyns)
            if weight_e is not None and not np.isnan(weight_e[sel]).any():
                syn_weight = weight_e[sel]
            elif "syn_weight" in row.index and not pd.isna(row["syn_weight"]):
                syn_weight = row["syn_weight"]
            else:
                syn_weight = None
            if weight_function is not None:
                if weight_function not in _WEIGHT_FUNCTIONS:
                    raise Exception('Unable to calculate synaptic weight for "{}" edges, missing "weight_function" '
                                    'attribute value {} function.'.format(self.name, weight_function))
                if source_nodes is None or target_nodes is None:
                    raise ValueError("edge type {}: weight_function {!r} needs the source and target node "
                                     "populations".format(et, weight_function))
                if frames is None:
                    frames = (self.to_dataframe(), source_nodes.to_dataframe(), target_nodes.to_dataframe())
                    if "nsyns" not in frames[0].columns:
                        frames[0]["nsyns"] = 1
                edges = frames[0][sel]
                got = np.asarray(_WEIGHT_FUNCTIONS[weight_function](
                    edges, frames[1].loc[edges["source_node_id"].values], frames[2].loc[edges["target_node_id"].values]),
                    np.float64)
                if got.shape not in ((), (int(sel.sum()),)):
                    raise ValueError("weight_function {!r} returned {} values for {} edges".format(
                        weight_function, got.size, int(sel.sum())))
                w[sel] = got
            else:
                w[sel] = net.edge_weights(nsyns, syn_weight)
            if delay_e is not None and not np.isnan(delay_e[sel]).any():
                delay[sel] = delay_e[sel]
            elif "delay" in row.index and not pd.isna(row["delay"]):
                delay[sel] = row["delay"]
            else:
                delay[sel] = dyn.get("delay", 1.0)  # NEST's default delay
            rec[sel] = int(dyn.get("receptor_type", 0))
        if n and np.any(delay < dt * (1.0 - 1e-12)):
            raise net.BadDelay("synaptic \"delay\" value in edges ({}) is not compatible with simulator "
                               "resolution/\"dt\" ({})".format(delay.min(), dt))
        steps = np.rint(delay / dt).astype(np.int64)
        return (self.source_node_id, self.target_node_id, w.astype(np.float32), steps, rec)


def read_edges(edges_file, edge_types_file):
    """-> {population name: EdgePopulation} (bmtk/utils/sonata/population.py:349-456)."""
    types = load_csv(edge_types_file).set_index("edge_type_id", drop=False)
    pops = {}
    with h5lite.File(edges_file) as h5:
        check_magic(h5, edges_file)
        for name in h5["/edges"].keys():
            g = h5["/edges/" + name]
            src, tgt = g["source_node_id"], g["target_node_id"]
            n = len(src)
            etid = np.asarray(g["edge_type_id"][()], np.int64)
            missing = set(np.unique(etid)) - set(types.index)
            if missing:
                raise ValueError("{}: edge types {} missing from {}".format(edges_file, sorted(missing),
                                                                            edge_types_file))
            groups = {}
            for sub in g.keys():
                if sub.isdigit() and isinstance(g[sub], h5lite.Group):
                    groups[int(sub)] = {k: v[()] for k, v in g[sub].items() if isinstance(v, h5lite.Dataset)}
            indices = {}
            for grp_name in ("indices", "indicies"):  # both spellings exist in the wild (population.py:413-418)
                if grp_name in g:
                    for index_name in g[grp_name].keys():
                        ig = g[grp_name][index_name]
                        if not isinstance(ig, h5lite.Group):
                            continue
                        for col in ("node_id_to_range", "range_to_edge_id"):
                            if col not in ig:
                                raise ValueError("index {} in {} edges is missing column {}.".format(
                                    index_name, name, col))
                        indices[index_name] = (np.asarray(ig["node_id_to_range"][()], np.int64),
                                               np.asarray(ig["range_to_edge_id"][()], np.int64))
                    break
            gid = np.asarray(g["edge_group_id"][()], np.int64) if "edge_group_id" in g else np.zeros(n, np.int64)
            gix = np.asarray(g["edge_group_index"][()], np.int64) if "edge_group_index" in g else np.arange(
                n, dtype=np.int64)
            pops[name] = EdgePopulation(name, src.attrs.get("node_population"), tgt.attrs.get("node_population"),
                                        np.asarray(src[()], np.int64), np.asarray(tgt[()], np.int64), etid, gid, gix,
                                        groups, indices, types)
    return pops


# ----------------------------------------------------------------------------------------------------------------
# spike files
# ----------------------------------------------------------------------------------------------------------------

def _sorted(node_ids, timestamps, sort_order):
    node_ids, timestamps = np.asarray(node_ids), np.asarray(timestamps, np.float64)
    if sort_order == "by_time":
        # a simulation hands its spikes over in this order already; seeing that takes a hundredth of the sort
        if timestamps.size < 2:
            return node_ids, timestamps
        dt = np.diff(timestamps)
        if not (dt < 0).any() and not ((dt == 0) & (np.diff(node_ids) < 0)).any():
            return node_ids, timestamps
        order = np.lexsort((node_ids, timestamps))  # time first, node id breaks ties (spike_trains_api to_dataframe)
    elif sort_order == "by_id":
        order = np.lexsort((timestamps, node_ids))
    elif sort_order in ("none", "unknown"):
        return node_ids, timestamps
    else:
        raise ValueError("sort_order must be one of {}".format(SORT_ORDERS))
    return node_ids[order], timestamps[order]


def write_spikes(path, spikes, sort_order="none", units="ms", mode="w"):
    """Write ``{population: (node_ids, timestamps)}`` the way bmtk's ``write_sonata`` does
    (spikes_file_writers.py:35-73): root attributes ``magic``/``version``, ``/spikes/<pop>`` with attribute
    ``sorting`` (unless the order is "unknown"), ``timestamps`` (float64, attribute ``units``) and ``node_ids``
    (uint64).  Data sets are stored contiguous and uncompressed."""
    if mode not in ("w", "a"):
        raise ValueError("mode must be 'w' or 'a'")
    tree = {}
    if mode == "a" and os.path.exists(path):
        # the file is rewritten with what it held; population groups without data are kept too
        with h5lite.File(path) as h5:
            held = [k for k in h5["/spikes"].keys() if isinstance(h5["/spikes"][k], h5lite.Group)] \
                if "/spikes" in h5 else []
        tree = {pop: {} for pop in held}
        for pop, (ids, ts, attrs) in read_spikes(path).items():
            if pop in tree:
                tree[pop] = {"__attrs__": {k: v for k, v in attrs.items() if k == "sorting" and v != "unknown"},
                             "timestamps": (ts, {"units": "ms"}), "node_ids": np.asarray(ids, np.uint64)}
    for pop, (ids, ts) in spikes.items():
        if pop in tree:
            raise ValueError("sonata file {} already contains a spikes group {}, skiping(use option mode=\"w\" to "
                             "overwrite)".format(path, pop))
        ids, ts = _sorted(ids, ts, sort_order)
        grp = {"timestamps": (np.asarray(ts, np.float64), {"units": units}), "node_ids": np.asarray(ids, np.uint64)}
        if sort_order != "unknown":
            grp["__attrs__"] = {"sorting": sort_order}
        tree[pop] = grp
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    h5lite.write(path, {"spikes": tree}, attrs={"magic": np.uint32(MAGIC_VAL), "version": np.array(VERSION, np.uint32)})


def read_spikes(path, populations=None):
    """-> {population: (node_ids int64, timestamps float64 in ms, {"sorting":…, "units":…})}.  Files of the older
    layout (``/spikes/gids`` + ``/spikes/timestamps`` with no population group) come back under the population
    name ``"<sonata:none>"`` as in spike_train_readers.py:126-133."""
    out = {}
    with h5lite.File(path) as h5:
        if "/spikes" not in h5:
            raise ValueError("Could not find /spikes root")
        root = h5["/spikes"]
        found = {}
        for name in root.keys():
            g = root[name]
            if isinstance(g, h5lite.Group) and "node_ids" in g and "timestamps" in g:
                if populations is None or name in populations:
                    found[name] = (g, "node_ids")
        if not found and "timestamps" in root:
            found["<sonata:none>"] = (root, "gids" if "gids" in root else "node_ids")
        for name, (g, ids_name) in found.items():
            ts = g["timestamps"]
            units = ts.attrs.get("units") or g.attrs.get("units") or "ms"
            scale = {"ms": 1.0, "s": 1000.0, "seconds": 1000.0, "milliseconds": 1.0}.get(str(units).lower())
            if scale is None:
                raise ValueError("unknown time unit {!r}".format(units))
            out[name] = (np.asarray(g[ids_name][()], np.int64), np.asarray(ts[()], np.float64) * scale,
                         {"sorting": g.attrs.get("sorting", "unknown"), "units": units})
    return out


def write_membrane_report(path, population, node_ids, data, tstart, tstop, dt, variable="V_m", units="mV"):
    """A SONATA cell-variable report with one element per node, the layout bmtk's ``CompartmentReport`` writes for
    PointNet membrane reports (bmtk/utils/reports/compartment/compartment_writer.py:175-227,456-516):
    ``/report/<population>/data`` float64 [steps][nodes] with attributes ``variable`` and ``units``, and
    ``/report/<population>/mapping/{node_ids, element_ids, element_pos, index_pointer, time}`` with
    ``time = [tstart, tstop, dt]``, steps = (tstop - tstart) / dt."""
    node_ids = np.asarray(node_ids, np.uint64)
    data = np.asarray(data, np.float64)
    if data.ndim != 2 or data.shape[1] != node_ids.size:
        raise ValueError("data must be [steps, nodes]")
    n = node_ids.size
    tree = {"report": {population: {
        "data": (data, {"variable": variable, "units": units}),
        "mapping": {"node_ids": node_ids, "element_ids": np.zeros(n, np.uint64), "element_pos": np.zeros(n, np.float64),
                    "index_pointer": np.arange(n + 1, dtype=np.uint64),
                    "time": np.array([tstart, tstop, dt], np.float64)}}}}
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    h5lite.write(path, tree, attrs={"magic": np.uint32(MAGIC_VAL), "version": np.array(VERSION, np.uint32)})


def read_membrane_report(path, population=None):
    """-> (node_ids int64 [nodes], times float64 [steps] (the end of each sampled step), data float64 [steps][nodes],
    attributes of the data set)."""
    with h5lite.File(path) as h5:
        root = h5["/report"]
        pop = population or root.keys()[0]
        g = root[pop]
        data = np.asarray(g["data"][()], np.float64)
        t0, t1, dt = (float(x) for x in g["mapping/time"][()])
        ptr = np.asarray(g["mapping/index_pointer"][()], np.int64)
        if not np.array_equal(np.diff(ptr), np.ones(ptr.size - 1, np.int64)):
            raise NotImplementedError("reports with several elements per node are not supported")
        return (np.asarray(g["mapping/node_ids"][()], np.int64), t0 + dt * np.arange(data.shape[0]), data,
                dict(g["data"].attrs))


def write_spikes_csv(path, spikes, sort_order="none"):
    """Space-separated ``timestamps population node_ids`` with a header line (spikes_file_writers.py:115-126)."""
    frames = []
    for pop, (ids, ts) in spikes.items():
        ids, ts = _sorted(ids, ts, sort_order)
        frames.append(pd.DataFrame({"timestamps": np.asarray(ts, np.float64), "population": pop,
                                    "node_ids": np.asarray(ids, np.int64)}))
    df = pd.concat(frames) if frames else pd.DataFrame({"timestamps": [], "population": [], "node_ids": []})
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    df[["timestamps", "population", "node_ids"]].to_csv(path, header=True, index=False, sep=" ")


def read_spikes_csv(path):
    df = pd.read_csv(path, sep=" ")
    if "population" not in df.columns:
        df["population"] = "<sonata:none>"
    return {pop: (g["node_ids"].to_numpy(np.int64), g["timestamps"].to_numpy(np.float64), {"sorting": "unknown",
                                                                                              "units": "ms"})
            for pop, g in df.groupby("population", sort=False)}


def _trains(entry):
    ids, ts = np.asarray(entry[0]), np.asarray(entry[1], np.float64)
    order = np.lexsort((ts, ids))
    ids, ts = ids[order], ts[order]
    uniq, start = np.unique(ids, return_index=True)
    return {int(u): ts[a:b] for u, a, b in zip(uniq, start, list(start[1:]) + [ids.size])}


def spikes_equal(a, b, err=0.00001):
    """bmtk's ``SpikeTrains.__eq__`` (spike_trains_api.py:186-228): same populations, same spiking nodes, and per
    node the sorted times agree within ``err``."""
    if set(a) != set(b):
        return False
    for pop in a:
        ta, tb = _trains(a[pop]), _trains(b[pop])
        if sorted(ta) != sorted(tb):
            return False
        for node in ta:
            if ta[node].size != tb[node].size or not np.allclose(ta[node], tb[node], equal_nan=True, atol=err):
                return False
    return True


def spikes_is_subset(a, b, err=0.00001, strict=False):
    """bmtk's ``SpikeTrains.is_subset`` (spike_trains_api.py:230-280): every (population, node, time) of ``a`` is in
    ``b``; each time of ``a`` is matched to the first time of ``b`` that is not below it."""
    is_equals = set(a) == set(b)
    for pop in a:
        na = np.asarray(a[pop][0]).size
        nb = np.asarray(b[pop][0]).size if pop in b else 0
        is_equals &= na == nb
        if na == 0:
            continue
        if pop not in b or na > nb:
            return False
        ta, tb = _trains(a[pop]), _trains(b[pop])
        if not set(ta) <= set(tb):
            return False
        for node, times in ta.items():
            other = tb[node]
            idx = np.searchsorted(other, times, side="left")
            if np.any(idx >= other.size):
                idx = np.minimum(idx, other.size - 1)
            if not np.allclose(times, other[idx], atol=err):
                return False
    if strict and is_equals:
        return False
    return True


# ----------------------------------------------------------------------------------------------------------------
# a whole network
# ----------------------------------------------------------------------------------------------------------------

class PointNetwork:
    """The arrays a ``Glif3Simulator`` is built from, assembled from a SONATA circuit configuration.

    ``population`` is the simulated (non-virtual) node population; virtual populations that project onto it
    become the rows of the input table, concatenated in the order of ``virtual`` (name -> first row).
    """

    def __init__(self, population, n, par, asc_init, u_init, class_id, supported, rec_edges, inp_edges, virtual,
                 n_inputs, i_e=None):
        self.population, self.n = population, n
        self.i_e = np.zeros(par.shape[1]) if i_e is None else i_e   # constant input current per class, pA
        self.par, self.asc_init, self.u_init, self.class_id, self.supported = par, asc_init, u_init, class_id, supported
        self.rec_edges, self.inp_edges = rec_edges, inp_edges  # (src, tgt, w, delay steps, receptor) or None
        self.virtual, self.n_inputs = virtual, n_inputs

    def tables(self):
        """-> (rec, inp) source-major synapse tables; the delay column is uint8 when every delay fits, int32
        otherwise (a Glif3Simulator takes such tables with a delay offset)."""
        out = []
        for edges, rows in ((self.rec_edges, self.n), (self.inp_edges, self.n_inputs)):
            if edges is None:
                out.append(None)
                continue
            src, tgt, w, d, r = edges
            out.append(net.coo_to_csr(src, tgt, w, d, r, rows, "source"))
        return out


    def device_tables(self, device=None):
        """The same two tables as device tensor tuples, sorted on the device (tens of millions of edges take a
        fraction of a second there against several seconds of host sorting)."""
        from .ops import SynapseTable
        out = []
        for edges, rows in ((self.rec_edges, self.n), (self.inp_edges, self.n_inputs)):
            if edges is None:
                out.append(None)
                continue
            t = SynapseTable.from_edges(*edges, n_rows=rows, n_cols=self.n, device=device)
            out.append((t.indptr, t.indices, t.weights, t.delays, t.receptors))
        return out


def load_point_network(config, dt=None, unsupported="raise"):
    """Read the node and edge files a circuit configuration names (``networks.nodes/edges``, ``components``)."""
    cfg = load_config(config) if isinstance(config, str) else config
    dt = float(dt if dt is not None else cfg.get("run", {}).get("dt", 0.1))
    comp = cfg.get("components", {})
    nodes = {}
    for entry in cfg["networks"]["nodes"]:
        nodes.update(read_nodes(entry["nodes_file"], entry["node_types_file"]))
    real = [p for p in nodes.values() if not (p.column("model_type") == "virtual").all()]
    if len(real) != 1:
        raise NotImplementedError("exactly one non-virtual node population is supported, found {}".format(
            [p.name for p in real]))
    pop = real[0]
    if not np.array_equal(np.sort(pop.node_ids), np.arange(len(pop))):
        raise NotImplementedError("node ids of {} must be 0..n-1".format(pop.name))
    par, asc_init, u_init, class_id, supported, _, i_e = node_parameter_classes(
        pop, comp.get("point_neuron_models_dir", "."), unsupported)
    silent = ~supported[class_id]
    rec, inp, virtual, n_inputs = [], [], {}, 0
    for entry in cfg["networks"].get("edges", []):
        for ep in read_edges(entry["edges_file"], entry["edge_types_file"]).values():
            if ep.target_population != pop.name:
                raise NotImplementedError("edges {} target population {}".format(ep.name, ep.target_population))
            src, tgt, w, d, r = ep.to_arrays(comp.get("synaptic_models_dir", "."), dt,
                                             source_nodes=nodes.get(ep.source_population), target_nodes=pop)
            keep = ~silent[tgt]
            if ep.source_population == pop.name:
                keep &= ~silent[src]
            if np.any(r[keep] < 1) or np.any(r[keep] > 4):
                raise ValueError("edges {}: receptor_type outside 1..4 on a glif_psc target".format(ep.name))
            r = (np.maximum(r, 1) - 1).astype(np.uint8)
            if ep.source_population == pop.name:
                rec.append(tuple(a[keep] for a in (src, tgt, w, d, r)))
            else:
                sp = nodes[ep.source_population]
                if ep.source_population not in virtual:
                    virtual[ep.source_population] = n_inputs
                    n_inputs += int(sp.node_ids.max()) + 1
                inp.append(tuple(a[keep] for a in (src + virtual[ep.source_population], tgt, w, d, r)))

    def cat(parts):
        return tuple(np.concatenate([p[i] for p in parts]) for i in range(5)) if parts else None

    return PointNetwork(pop.name, len(pop), par, asc_init, u_init, class_id, supported, cat(rec), cat(inp), virtual,
                        n_inputs, i_e)
