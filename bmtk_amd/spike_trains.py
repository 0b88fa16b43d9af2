"""Input spike sources for the GPU path.

``PoissonSpikeGenerator`` follows the sampling scheme, random stream and units
of bmtk/utils/reports/spike_trains/spike_trains.py:113-251 (exponential
inter-spike intervals on NumPy's global legacy generator, optional refractory
thinning, linear-interpolated rate thinning for time-varying rates), so a
seeded run produces the trains bmtk would write to ``inputs/*.h5``.
``bin_spike_times`` applies the rules NEST's ``spike_generator`` enforces when
bmtk hands it those trains (bmtk/simulator/pointnet/pointnetwork.py:39-61) and
turns them into the per-step event lists the kernels consume.
"""
import os

import numpy as np


def _refractory_rate_correction(abs_ref, tau_ref):
    """Rate lost to refractoriness and the polynomial that inverts it
    (bmtk/utils/reports/spike_trains/spike_trains.py:317-338)."""
    before = np.logspace(0, 3, 40)
    if tau_ref != 0:
        after = (np.exp(-before * abs_ref)
                 - before * np.exp(abs_ref / tau_ref) * tau_ref / (before * tau_ref + 1)
                 * np.exp(-(before + 1 / tau_ref) * abs_ref)) * before
    else:
        after = np.exp(-before * abs_ref) * before
    top = int(np.argmax(after))
    inverse = np.poly1d(np.polyfit(after[:top], before[:top], 10))
    return float(np.max(after)), inverse


class SpikeTrains(object):
    """Spike trains of one or more populations in memory, with the calls of bmtk's ``SpikeTrains``
    (bmtk/utils/reports/spike_trains/spike_trains_api.py:37-309): adding and querying spikes, SONATA/csv files,
    and the comparisons ``==``, ``<=``, ``<`` (equal, subset, strict subset; per node, sorted times within
    ``err``).  Times are kept in ms."""

    def __init__(self, population=None, **kwargs):
        self.default_population = kwargs.get("default_population", population)
        self.units = "ms"
        self._trains = {}  # population -> {node_id: [chunks of times]}

    # -- container ---------------------------------------------------------
    def add_spike(self, node_id, timestamp, population=None, **kwargs):
        self.add_spikes(int(node_id), [timestamp], population)

    def add_spikes(self, node_ids, timestamps, population=None, **kwargs):
        """One node id with its times, or one id per time."""
        pop = population if population is not None else self.default_population
        store = self._trains.setdefault(pop, {})
        timestamps = np.atleast_1d(np.asarray(timestamps, np.float64))
        if np.isscalar(node_ids):
            store.setdefault(int(node_ids), []).append(timestamps)
        else:
            for nid, ts in zip(node_ids, timestamps):
                store.setdefault(int(nid), []).append(np.atleast_1d(ts))

    @property
    def populations(self):
        return list(self._trains.keys())

    def _pop(self, population):
        return population if population is not None else self.default_population

    def node_ids(self, population=None):
        return sorted(self._trains.get(self._pop(population), {}).keys())

    def get_times(self, node_id, population=None, time_window=None):
        chunks = self._trains.get(self._pop(population), {}).get(int(node_id), [])
        ts = np.concatenate(chunks) if chunks else np.zeros(0)
        if time_window is not None:
            ts = ts[(ts >= time_window[0]) & (ts <= time_window[1])]
        return ts

    def n_spikes(self, population=None):
        pops = [population] if population is not None else self.populations
        return int(sum(sum(c.size for c in chunks) for p in pops for chunks in self._trains.get(p, {}).values()))

    def __len__(self):
        return self.n_spikes()

    def time_range(self, population=None):
        pops = [population] if population is not None else self.populations
        ts = np.concatenate([self.get_times(n, p) for p in pops for n in self.node_ids(p)])
        return float(np.min(ts)), float(np.max(ts))

    def to_dataframe(self, populations=None, with_population_col=True):
        import pandas as pd
        pops = self.populations if populations is None else np.atleast_1d(populations).tolist()
        rows_t, rows_p, rows_n = [], [], []
        for p in pops:
            for n in self.node_ids(p):
                t = self.get_times(n, p)
                rows_t.append(t)
                rows_n.append(np.full(t.size, n, np.uint64))
                rows_p.extend([p] * t.size)
        df = pd.DataFrame({"timestamps": np.concatenate(rows_t) if rows_t else [],
                           "population": rows_p, "node_ids": np.concatenate(rows_n) if rows_n else []})
        return df if with_population_col else df.drop(columns="population")

    def spikes(self, populations=None):
        """Iterates (timestamp, population, node id)."""
        for p in (self.populations if populations is None else np.atleast_1d(populations).tolist()):
            for n in self.node_ids(p):
                for t in self.get_times(n, p):
                    yield float(t), p, int(n)

    def _as_spikes(self):
        out = {}
        for p in self.populations:
            ids = self.node_ids(p)
            ts = [self.get_times(n, p) for n in ids]
            out[p] = (np.concatenate([np.full(t.size, n, np.int64) for n, t in zip(ids, ts)]) if ids
                      else np.zeros(0, np.int64), np.concatenate(ts) if ts else np.zeros(0))
        return out

    # -- files ---------------------------------------------------------------
    def to_sonata(self, path, mode="w", sort_order="none", **kwargs):
        """``/spikes/<population>/{node_ids,timestamps}`` as bmtk/utils/reports/spike_trains/spike_trains_api.py:147-158
        writes them; the file is stored uncompressed whatever ``compression`` asks."""
        from . import sonata
        sonata.write_spikes(path, self._as_spikes(), sort_order=getattr(sort_order, "value", sort_order),
                            units=self.units, mode=mode)

    def to_csv(self, path, mode="w", sort_order="none", **kwargs):
        """Space-separated ``timestamps population node_ids`` (spike_trains_api.py:160-169)."""
        from . import sonata
        if mode != "w":
            raise NotImplementedError("to_csv only writes a new file")
        sonata.write_spikes_csv(path, self._as_spikes(), sort_order=getattr(sort_order, "value", sort_order))

    @classmethod
    def _from_spikes(cls, spikes, **kwargs):
        st = cls(**kwargs)
        for pop, entry in spikes.items():
            ids, ts = np.asarray(entry[0]), np.asarray(entry[1], np.float64)
            order = np.argsort(ids, kind="stable")
            ids, ts = ids[order], ts[order]
            uniq, first = np.unique(ids, return_index=True)
            store = st._trains.setdefault(pop, {})
            for u, a, b in zip(uniq, first, list(first[1:]) + [ids.size]):
                store[int(u)] = [ts[a:b]]
        return st

    @classmethod
    def from_sonata(cls, path, population=None, **kwargs):
        from . import sonata
        return cls._from_spikes(sonata.read_spikes(path, None if population is None else np.atleast_1d(population)),
                                **kwargs)

    @classmethod
    def from_csv(cls, path, **kwargs):
        from . import sonata
        return cls._from_spikes(sonata.read_spikes_csv(path), **kwargs)

    @classmethod
    def load(cls, path, file_type=None, **kwargs):
        """By extension (or ``file_type`` "h5"/"sonata"/"csv"), as spike_trains.py:46-73 does."""
        kind = (file_type or os.path.splitext(path)[1].lstrip(".")).lower()
        if kind in ("h5", "hdf5", "sonata"):
            return cls.from_sonata(path, **kwargs)
        if kind in ("csv", "txt"):
            return cls.from_csv(path, **kwargs)
        raise ValueError("cannot tell the type of spikes file {}".format(path))

    # -- comparisons -----------------------------------------------------------
    def is_equal(self, other, err=0.00001):
        from . import sonata
        return sonata.spikes_equal(self._as_spikes(), other._as_spikes(), err=err)

    def is_subset(self, other, err=0.00001, strict=False):
        from . import sonata
        return sonata.spikes_is_subset(self._as_spikes(), other._as_spikes(), err=err, strict=strict)

    def __eq__(self, other):
        return self.is_equal(other)

    def __ne__(self, other):
        return not self == other

    def __lt__(self, other):
        return self.is_subset(other, strict=True)

    def __le__(self, other):
        return self.is_subset(other)

    def __gt__(self, other):
        return other < self

    def __ge__(self, other):
        return other <= self

    __hash__ = None


class PoissonSpikeGenerator(SpikeTrains):
    """Homogeneous / inhomogeneous Poisson spike trains (times stored in ms)."""

    def __init__(self, population=None, seed=None, output_units="ms", **kwargs):
        super().__init__(population=population, **kwargs)
        if seed:  # a seed of 0 / 0.0 / None leaves the global stream where it is, as the reference does
            np.random.seed(seed)
        units = output_units.lower()
        if units in ("ms", "millisecond", "milliseconds"):
            self.units, self.output_conversion = "ms", 1000.0
        elif units in ("s", "second", "seconds"):
            self.units, self.output_conversion = "s", 1.0
        else:
            raise AttributeError("Unknown output_units value {}".format(output_units))

    # -- generators --------------------------------------------------------
    def add(self, node_ids, firing_rate, population=None, times=(0.0, 1.0), abs_ref=0, tau_ref=0):
        """``firing_rate`` in Hz (scalar, or an array paired with ``times``), ``times`` in seconds."""
        if tau_ref < 0:
            raise ValueError("Refractory period time constant (sec) cannot be negative.")
        if abs_ref < 0:
            raise ValueError("Absolute refractory period (sec) cannot be negative.")
        if isinstance(node_ids, str):
            # a nodes file: the ids of ``population`` in it (bmtk/utils/sonata/utils.py:111-115)
            from . import h5lite
            with h5lite.File(node_ids) as h5:
                node_ids = np.asarray(h5["/nodes/{}/node_id".format(population)][()], np.int64)
        if np.isscalar(node_ids):
            node_ids = [node_ids]
        if np.isscalar(firing_rate):
            self._fixed_rate(node_ids, population, firing_rate, times, abs_ref, tau_ref)
        elif isinstance(firing_rate, (list, np.ndarray)):
            self._varying_rate(node_ids, population, np.asarray(firing_rate, np.float64), np.asarray(times),
                               abs_ref, tau_ref)

    def _fixed_rate(self, node_ids, population, fr, times, abs_ref, tau_ref):
        if np.isscalar(times) and times > 0.0:
            tstart, tstop = 0.0, times
        else:
            tstart, tstop = times[0], times[-1]
            if tstart >= tstop:
                raise ValueError("Invalid start and stop times.")
        if fr < 0:
            raise ValueError("Firing rates must not be negative.")
        if abs_ref != 0 or tau_ref != 0:
            limit, inverse = _refractory_rate_correction(abs_ref, tau_ref)
            if fr > limit:
                raise ValueError("Cannot achieve firing rate above {} with these absolute and relative "
                                 "refractory properties.".format(limit))
            fr = inverse(fr)
            self._fixed_rate_refractory(node_ids, population, fr, tstart, tstop, abs_ref, tau_ref)
            return
        # No refractoriness: one uniform draw per candidate spike, the draw that
        # crosses tstop is consumed too.  Draw in blocks for speed, then put the
        # global stream exactly where a draw-by-draw loop would have left it.
        state0 = np.random.get_state()
        block = max(1024, int((tstop - tstart) * fr * 1.2) + 16)
        buf, pos, used = np.zeros(0), 0, 0
        for nid in node_ids:
            c_time, pieces = tstart, []
            while True:
                if pos == buf.size:
                    buf, pos = -np.log(1.0 - np.random.uniform(size=block)) / fr, 0
                acc = np.cumsum(np.concatenate(([c_time], buf[pos:])))[1:]  # sequential adds, as a scalar loop does
                k = int(np.searchsorted(acc, tstop, side="right"))           # first acc > tstop
                pieces.append(acc[:k])
                if k < acc.size:
                    pos += k + 1
                    used += k + 1
                    break
                used += acc.size
                pos = buf.size
                c_time = acc[-1]
            self.add_spikes(nid, np.concatenate(pieces) * self.output_conversion, population)
        np.random.set_state(state0)
        if used:
            np.random.uniform(size=used)

    def _fixed_rate_refractory(self, node_ids, population, fr, tstart, tstop, abs_ref, tau_ref):
        for nid in node_ids:
            c_time, out = tstart, []
            while True:
                interval = -np.log(1.0 - np.random.uniform()) / fr
                c_time += interval
                if c_time > tstop:
                    break
                w = 1 - np.exp(-(interval - abs_ref) / tau_ref) if tau_ref != 0 else 1
                if abs_ref != 0:
                    w = w * (interval > abs_ref)
                if w == 1 or np.random.uniform() < w:
                    out.append(c_time * self.output_conversion)
            self.add_spikes(nid, np.asarray(out), population)

    def _varying_rate(self, node_ids, population, fr, times, abs_ref, tau_ref):
        if np.min(fr) < 0:
            raise ValueError("Firing rates must not be negative")
        if len(fr) != len(times):
            raise ValueError("If using a time series for firing rate, times must be an array of equal length")
        max_fr = np.max(fr)
        limit, inverse = _refractory_rate_correction(abs_ref, tau_ref)
        if max_fr > limit:
            raise ValueError("Cannot achieve firing rate above {} with these absolute and relative "
                             "refractory properties".format(limit))
        fr = inverse(fr)
        tstart, tstop = times[0], times[-1]
        for nid in node_ids:
            c_time, idx, out = tstart, 0, []
            while True:
                interval = -np.log(1.0 - np.random.uniform()) / max_fr
                c_time += interval
                if c_time > tstop:
                    break
                w = 1 - np.exp(-(interval - abs_ref) / tau_ref) if tau_ref != 0 else 1
                if abs_ref != 0:
                    w = w * (interval > abs_ref)
                while times[idx] <= c_time:
                    idx += 1
                t0, t1, f0, f1 = times[idx - 1], times[idx], fr[idx - 1], fr[idx]
                fr_i = f0 + (f1 - f0) * (c_time - t0) / (t1 - t0)
                if not fr_i / max_fr * w < np.random.uniform():
                    out.append(c_time * self.output_conversion)
            self.add_spikes(nid, np.asarray(out), population)


class GammaSpikeGenerator(PoissonSpikeGenerator):
    """Spike trains of a gamma-distributed renewal process with a stationary rate
    (bmtk/utils/reports/spike_trains/spike_trains.py:254-307): per node, ``round(1.5 * rate * duration)`` intervals
    are drawn at once from Gamma(shape ``a``, scale 1/(a*rate)) with SciPy on NumPy's global stream, and spikes are
    kept up to ``tstop``.  ``a`` = 1 gives Poisson statistics."""

    def add(self, node_ids, firing_rate, a, population=None, times=(0.0, 1.0)):
        from scipy.stats import gamma
        if isinstance(node_ids, str):
            from . import h5lite
            with h5lite.File(node_ids) as h5:
                node_ids = np.asarray(h5["/nodes/{}/node_id".format(population)][()], np.int64)
        if np.isscalar(node_ids):
            node_ids = [node_ids]
        if not np.isscalar(firing_rate):
            raise Exception("Firing rate must be stationary for GammaSpikeGenerator")
        if np.isscalar(times) and times > 0.0:
            tstart, tstop = 0.0, times
        else:
            tstart, tstop = times[0], times[-1]
            if tstart >= tstop:
                raise ValueError("Invalid start and stop times.")
        if firing_rate < 0:
            raise Exception("Firing rates must not be negative.")
        if a < 0:
            raise ValueError("Shape parameter `a` cannot be negative.")
        for node_id in node_ids:
            n_draws = int(round((tstop - tstart) * firing_rate * 1.5))
            intervals = gamma.rvs(a, loc=0, scale=1 / (a * firing_rate), size=n_draws)
            # the reference adds the intervals one by one starting from tstart: a running sum in that order
            t = np.cumsum(np.concatenate([[tstart], intervals]))[1:]
            t = t[:np.argmax(t > tstop)] if np.any(t > tstop) else t
            if t.size:
                self.add_spikes([node_id] * t.size, t * self.output_conversion, population=population)


def check_spike_times(st):
    """The rule bmtk applies before ``nest.SetStatus(.., {'spike_times': ..})``
    (bmtk/simulator/pointnet/pointnetwork.py:39-61): empty/None trains are
    skipped, times must be strictly positive, and they are sorted."""
    if st is None or len(st) == 0:
        return None
    st = np.array(st, np.float64)
    if np.any(st <= 0.0):
        raise ValueError("spike train {} contains negative/zero time, unable to run virtual cell".format(st))
    st.sort()
    return st


def bin_spike_times(trains, dt, n_steps, batch=1, trial=0):
    """Per-source spike times (ms) -> (in_ptr int64[n_steps+1], in_events int32[]).

    ``trains`` is a sequence indexed by source id (entries may be None).  A
    spike at time t gets the stamp ``ceil(t/dt)`` steps (on-grid times keep
    their step; an off-grid time is carried to the end of the step that
    contains it, which is what NEST's ``spike_generator`` does with
    ``precise_times`` -- the sub-step offset it also keeps is ignored by
    ``static_synapse`` delivery) and is emitted in step stamp-1.  An event is
    the element id ``source*batch + trial``; events of one step are ascending.
    """
    steps, elems = [], []
    for j, st in enumerate(trains):
        st = check_spike_times(st)
        if st is None:
            continue
        stamp = np.ceil(st / dt - 1e-6).astype(np.int64)
        stamp = np.maximum(stamp, 1)
        emit = stamp - 1
        emit = emit[emit < n_steps]
        steps.append(emit)
        elems.append(np.full(emit.size, j * batch + trial, np.int64))
    if steps:
        steps, elems = np.concatenate(steps), np.concatenate(elems)
    else:
        steps, elems = np.zeros(0, np.int64), np.zeros(0, np.int64)
    order = np.lexsort((elems, steps))
    steps, elems = steps[order], elems[order]
    in_ptr = np.zeros(n_steps + 1, np.int64)
    np.add.at(in_ptr, steps + 1, 1)
    return np.cumsum(in_ptr), elems.astype(np.int32)
