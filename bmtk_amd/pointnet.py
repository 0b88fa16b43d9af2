"""Run a SONATA/bmtk PointNet configuration on the GPU.

The three calls of a bmtk run script (examples/point_450glifs/run_pointnet.py),

    configure = pointnet.Config.from_json(config_file)
    graph = pointnet.PointNetwork.from_config(configure)
    sim = pointnet.PointSimulator.from_config(configure, graph)
    sim.run()

with the same meaning for GLIF point networks: build the network from the
``networks`` section (bmtk/simulator/pointnet/pointnetwork.py:144-232), attach
the ``inputs`` of type ``spikes`` (modules ``sonata``/``h5`` and ``csv``,
bmtk/simulator/pointnet/pointsimulator.py:229-262; spike-time rules of
pointnetwork.py:39-61) and ``current_clamp``, run ``tstop/dt`` steps
(pointsimulator.py:149-173) and write ``output.spikes_file`` /
``spikes_file_csv`` in ``output.output_dir`` sorted as ``spikes_sort_order``
asks (bmtk/simulator/pointnet/modules/record_spikes.py:53-104).  ``reports``
entries of module ``multimeter_report`` / ``membrane_report`` for ``V_m``
become SONATA cell-variable files
(bmtk/simulator/pointnet/modules/multimeter_reporter.py:64-140).
"""
import math
import os

import numpy as np
import torch

from . import sonata
from .simulator import Glif3Simulator
from .sonata import add_weight_function, synaptic_weight  # noqa: F401  (bmtk.simulator.pointnet's registry calls)
from .spike_trains import bin_spike_times


class Config(dict):
    @classmethod
    def from_json(cls, path):
        return cls(sonata.load_config(path))

    from_dict = classmethod(lambda cls, d: cls(d))

    def build_env(self):
        out = self.get("output", {}).get("output_dir")
        if out:
            os.makedirs(out, exist_ok=True)

    @property
    def dt(self):
        return float(self.get("run", {}).get("dt", 0.001))  # NEST's default resolution is what bmtk falls back to

    @property
    def tstop(self):
        run = self["run"]  # "duration" goes before "tstop" (bmtk/simulator/pointnet/pointsimulator.py:218-221)
        return float(run["duration"] if "duration" in run else run["tstop"])


class PointNetwork(sonata.PointNetwork):
    @classmethod
    def from_config(cls, config, dt=None, unsupported="raise"):
        nw = sonata.load_point_network(config, dt=dt if dt is not None else Config(config).dt,
                                       unsupported=unsupported)
        nw.__class__ = cls
        return nw


def _read_input_spikes(entry):
    module = entry.get("module", "sonata")
    if module in ("sonata", "h5", "hdf5"):
        return sonata.read_spikes(entry["input_file"])
    if module == "csv":
        return sonata.read_spikes_csv(entry["input_file"])
    raise NotImplementedError("spikes input module {!r} is not supported".format(module))


def _read_nwb_stimulus(entry):
    """Times (ms) and amplitudes of one sweep of an Allen Cell Types NWB file, as bmtk's NWBReader takes them
    (bmtk/simulator/core/modules/iclamp.py:61-113): ``/epochs/Sweep_<id>/stimulus/timeseries/data`` times 1e9,
    one value per 1000 / rate ms (attribute ``rate`` of ``starting_time``); ``downsample`` (ms) keeps every n-th
    value, ``sweep_window`` [start, stop] ms cuts, ``delay`` shifts."""
    from . import h5lite
    sweep = entry["sweep_id"]
    try:
        sweep = "Sweep_{}".format(int(sweep))
    except ValueError:
        pass
    with h5lite.File(entry["file"]) as h5:
        if "/epochs" not in h5 or sweep not in h5["/epochs"].keys():
            raise ValueError("{} missing sweep group {}.".format(entry["file"], sweep))
        grp = h5["/epochs/{}/stimulus/timeseries".format(sweep)]
        idt = 1000.0 / float(np.asarray(grp["starting_time"].attrs["rate"]).reshape(-1)[0])
        amps = np.asarray(grp["data"][()], np.float64) * 1.0e9
    delays = np.arange(amps.size) * idt
    down = entry.get("downsample")
    if down is not None and down > idt:
        stride = int(np.round(down / idt))
        amps, delays = amps[::stride], delays[::stride]
    window = entry.get("sweep_window")
    if window is not None:
        if len(window) != 2 or window[0] >= window[1] or window[0] < 0:
            raise ValueError('"sweep_window" parameter must be set to [start_time, stop_time] where '
                             "0 <= start_time < stop_time.")
        first = int(np.argwhere(delays >= window[0]).flatten()[0])
        last = int(np.argwhere(delays <= window[1]).flatten()[-1]) + 1
        amps, delays = amps[first:last], delays[first:last]
    return (delays + float(entry.get("delay", 0.0))).tolist(), amps.tolist()


class PointSimulator:
    def __init__(self, network, dt, tstop, device=None, resident="auto"):
        self.net, self.dt, self.tstop = network, float(dt), float(tstop)
        self.n_steps = int(round(self.tstop / self.dt))
        self.output = {}
        self._trains = [None] * network.n_inputs
        # the cells' own constant current I_e (per parameter class); current clamps add to it
        i_e = getattr(network, "i_e", None)
        self._i_ext = np.zeros(network.n) if i_e is None else np.asarray(i_e, np.float64)[network.class_id]
        self._clamps = []
        self._device, self._resident = device, resident
        self.spikes = None
        self.reports = {}  # name -> dict(node_ids, interval, tstart, tstop, file)

    @classmethod
    def from_config(cls, config, network, dt=None, device=None, resident="auto"):
        config = Config(config)
        sim = cls(network, dt if dt is not None else config.dt, config.tstop, device=device, resident=resident)
        sim.output = dict(config.get("output", {}))
        for name, entry in config.get("inputs", {}).items():
            kind = entry.get("input_type")
            if kind == "spikes":
                sim.add_spike_inputs(_read_input_spikes(entry), entry.get("node_set"))
            elif entry.get("module") == "IClamp" or kind == "current_clamp":
                sim.add_current_clamp(entry)
            else:
                raise NotImplementedError("input {!r}: input_type {!r} is not supported".format(name, kind))
        for name, entry in config.get("reports", {}).items():
            sim.add_report(name, entry)
        return sim

    def add_report(self, name, entry):
        """A membrane potential report: ``cells`` (a node id list, or {"population":…, "node_id": […]}; absent or
        "all" = every node), ``variable_name`` V_m, optional ``file_name``, ``tstart``, ``tstop``, ``dt``
        (sampling interval, a multiple of the resolution)."""
        module = entry.get("module", "multimeter_report")
        if module not in ("multimeter_report", "membrane_report"):
            raise NotImplementedError("report {!r}: module {!r} is not supported".format(name, module))
        var = entry.get("variable_name", "V_m")
        var = var[0] if isinstance(var, (list, tuple)) and len(var) == 1 else var
        if var != "V_m":
            raise NotImplementedError("report {!r}: only V_m is recorded, not {!r}".format(name, var))
        ids = self._node_ids_of(entry.get("cells", "all"))
        interval = float(entry.get("dt") or self.dt)
        every = interval / self.dt
        if every < 1 - 1e-9 or abs(every - round(every)) > 1e-6:
            raise ValueError("report {!r}: the sampling interval must be a multiple of the resolution".format(name))
        self.reports[name] = dict(node_ids=ids, every=int(round(every)), tstart=float(entry.get("tstart") or 0.0),
                                  tstop=float(entry.get("tstop") or self.tstop),
                                  file=entry.get("file_name") or name + ".h5", rows=[])

    def add_spike_inputs(self, spikes, node_set=None):
        """Spike trains of virtual populations; a train is only used by the population it is stored under, and
        ``node_set`` (a population name, or {"population": name}) restricts which populations are taken."""
        if isinstance(node_set, dict):
            node_set = node_set.get("population")
        for pop, entry in spikes.items():
            if pop not in self.net.virtual or (isinstance(node_set, str) and node_set not in (pop, "all")):
                continue
            base = self.net.virtual[pop]
            ids, ts = np.asarray(entry[0]), np.asarray(entry[1], np.float64)
            order = np.lexsort((ts, ids))
            ids, ts = ids[order], ts[order]
            uniq, start = np.unique(ids, return_index=True)
            for u, a, b in zip(uniq, start, list(start[1:]) + [ids.size]):
                row = base + int(u)
                if row < len(self._trains):
                    self._trains[row] = ts[a:b]

    def add_current_clamp(self, entry):
        """One current generator on a set of nodes, as bmtk's IClamp module sets up a NEST
        ``step_current_generator`` (bmtk/simulator/pointnet/modules/iclamp.py:8-54, readers in
        bmtk/simulator/core/modules/iclamp.py:9-58).  ``input_type`` "current_clamp": ``amp`` (pA), ``delay``,
        ``duration`` (ms), scalars or lists of one length; an amplitude is switched off at delay + duration unless
        the next one has begun by then.  "csv": ``file`` with the columns ``timestamps`` and ``amps`` (other names
        through ``timestamps_column`` / ``amplitudes_column``, ``separator`` " "), taken as they are; "nwb": one sweep of an
        Allen Cell Types file (``file``, ``sweep_id``, optional ``downsample``, ``sweep_window``, ``delay``).  Onsets at or
        before the resolution are skipped, as bmtk does.  An amplitude set for time t acts on the update that
        starts at t + dt (NEST)."""
        kind = entry.get("input_type", "current_clamp")
        if kind == "current_clamp":
            amps, delays, durs = (list(v) if isinstance(v, (list, tuple, np.ndarray)) else [v]
                                  for v in (entry["amp"], entry["delay"], entry["duration"]))
            if not len(amps) == len(delays) == len(durs):
                raise ValueError("current clamp parameters amp, delay, duration must be same length when using list.")
        elif kind == "csv":
            import pandas as pd
            table = pd.read_csv(entry["file"], sep=entry.get("separator", " "))
            if len(table) < 2:
                raise ValueError("csv file must be row oriented and contain two or more values.")
            for col in (entry.get("timestamps_column", "timestamps"), entry.get("amplitudes_column", "amps")):
                if col not in table.columns:
                    raise ValueError('csv file missing column "{}".'.format(col))
            delays = table[entry.get("timestamps_column", "timestamps")].to_numpy(np.float64).tolist()
            amps = table[entry.get("amplitudes_column", "amps")].to_numpy(np.float64).tolist()
            durs = None
        elif kind == "nwb":
            delays, amps = _read_nwb_stimulus(entry)
            durs = None
        else:
            raise NotImplementedError("current clamp input_type {!r} is not supported".format(kind))
        times, values = [], []
        for i, (start, amp) in enumerate(zip(delays, amps)):
            if start <= self.dt:
                continue
            times.append(float(start))
            values.append(float(amp))
            if durs is not None:
                stop = start + durs[i]
                if i + 1 == len(delays) or stop <= delays[i + 1]:
                    times.append(float(stop))
                    values.append(0.0)
        if any(b <= a for a, b in zip(times[:-1], times[1:])):
            raise ValueError("current clamp: amplitude times must be strictly increasing")  # NEST's BadProperty
        self._clamps.append((self._node_ids_of(entry.get("node_set")), np.asarray(times), np.asarray(values)))

    def _node_ids_of(self, node_set):
        """Node ids of a ``node_set``: a list, a population name (or "all"), or {"population":…, "node_id"/"node_ids":
        […]} with the ids optional."""
        if isinstance(node_set, dict):
            pop = node_set.get("population", self.net.population)
            if pop != self.net.population:
                raise ValueError("population {!r} is not simulated".format(pop))
            node_set = node_set.get("node_id", node_set.get("node_ids"))
        if node_set is None or (isinstance(node_set, str) and node_set in ("all", self.net.population)):
            return np.arange(self.net.n)
        if isinstance(node_set, str):
            raise NotImplementedError("node set {!r}: only the simulated population or id lists".format(node_set))
        ids = np.asarray(node_set, np.int64)
        if ids.size and (ids.min() < 0 or ids.max() >= self.net.n):
            raise ValueError("node id outside 0..{}".format(self.net.n - 1))
        return ids

    def _segments(self):
        """Step ranges with a constant external current, and that current."""
        def first_step(t):  # the update an amplitude set for time t first acts on
            return min(self.n_steps, max(0, int(round(t / self.dt)) + 1))
        marks = {0, self.n_steps}
        for _, times, _ in self._clamps:
            marks.update(first_step(t) for t in times)
        marks = sorted(marks)
        for a, b in zip(marks[:-1], marks[1:]):
            cur = self._i_ext.astype(np.float32)
            for ids, times, values in self._clamps:
                on = [v for t, v in zip(times, values) if first_step(t) <= a]
                if on:
                    cur[ids] += np.float32(on[-1])
            yield a, b, cur

    def run(self, tstop=None, record_cap=None):
        if tstop is not None:
            self.tstop = float(tstop)
            self.n_steps = int(round(self.tstop / self.dt))
        nw = self.net
        rec, inp = nw.device_tables(self._device)
        sim = Glif3Simulator(nw.n, nw.par, self.dt, class_id=nw.class_id, rec=rec, inp=inp,
                             asc_init=nw.asc_init[:, nw.class_id], u_init=nw.u_init[nw.class_id],
                             i_ext=np.zeros(nw.n, np.float32), device=self._device, resident=self._resident)
        probed = None
        if self.reports:
            # one set of probes serves every report: the union of their cells, at the largest common interval
            probed = np.unique(np.concatenate([rep["node_ids"] for rep in self.reports.values()]))
            every = 0
            for rep in self.reports.values():
                every = math.gcd(every, rep["every"])
            sim.set_probes(probed, every=every)
        if inp is not None:
            sim.set_input_events(*bin_spike_times(self._trains, self.dt, self.n_steps))
        elems, times = [], []
        from .layout import PAR
        e_l = nw.par[PAR["E_L"]][nw.class_id]
        pieces = []
        for a, b, cur in self._segments():
            # a membrane record is taken in pieces of bounded size
            piece = max(1, (1 << 26) * sim.probe_every // probed.size) if self.reports else b - a
            pieces += [(k, min(k + piece, b), cur) for k in range(a, b, piece)]
        for a, b, cur in pieces:
            sim.i_ext.copy_(torch.as_tensor(cur, device=sim.dev))
            cap = record_cap or max(1 << 16, (b - a) * nw.n // 8)
            out = sim.run(b - a, spike_bits=False, record_cap=cap)
            sim.check()
            if self.reports and out["probe"]["steps"].numel():
                # the sample stamped t is the potential at the end of the step that ends at t
                stamps = out["probe"]["steps"].numpy() + 1
                sampled = out["probe"]["v"].cpu().numpy().astype(np.float64)
                for rep in self.reports.values():
                    keep = (stamps % rep["every"] == 0) & (stamps * self.dt > rep["tstart"] + 1e-9) & \
                           (stamps * self.dt <= rep["tstop"] + 1e-9)
                    if keep.any():
                        cols = np.searchsorted(probed, rep["node_ids"])
                        rep["rows"].append((stamps[keep] * self.dt,
                                            sampled[keep][:, cols] + e_l[rep["node_ids"]][None, :]))
            # threshold crossing interpolated inside the step, as glif_psc stamps it; ordered by time (ties by
            # node) on the device.  The pieces follow one another in time, so their order is the run's.
            r = sim.collect_record(out["record"], sort_scale=self.dt)
            if r["overflow"]:
                raise RuntimeError("spike record overflow: " + sim.overflow_message(r))
            r_time, r_elem = sim.to_host(r["time"], r["elem"])
            elems.append(r_elem.astype(np.int64))
            times.append(r_time)
        self.simulator = sim
        self.spikes = {nw.population: (np.concatenate(elems), np.concatenate(times))}
        self._write_outputs()
        return self.spikes

    def _write_outputs(self):
        out = self.output
        base = out.get("output_dir", ".")
        for rep in self.reports.values():
            if rep["rows"]:
                times = np.concatenate([r[0] for r in rep["rows"]])
                data = np.concatenate([r[1] for r in rep["rows"]])
                interval = rep["every"] * self.dt
                path = rep["file"] if os.path.isabs(rep["file"]) else os.path.join(base, rep["file"])
                sonata.write_membrane_report(path, self.net.population, rep["node_ids"], data, float(times[0]),
                                             float(times[-1]) + interval, interval)
                rep["times"], rep["data"], rep["rows"] = times, data, []
        if not out:
            return
        order = out.get("spikes_sort_order", "none")
        if out.get("spikes_file"):
            path = out["spikes_file"] if os.path.isabs(out["spikes_file"]) else os.path.join(base, out["spikes_file"])
            sonata.write_spikes(path, self.spikes, sort_order=order)
        if out.get("spikes_file_csv"):
            path = out["spikes_file_csv"]
            path = path if os.path.isabs(path) else os.path.join(base, path)
            sonata.write_spikes_csv(path, self.spikes, sort_order=order)
