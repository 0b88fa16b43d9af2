"""Forward GLIF3 simulation on one GPU: the work ``nest.Simulate`` does for a
bmtk PointNet network (bmtk/simulator/pointnet/pointsimulator.py:159-166).

``Glif3Simulator`` owns the device state, the ring buffer and the synapse
tables, validates everything a kernel will index with on the host, and drives
``bmtk_glif3_simulate_fwd``.
"""
import ctypes as C
import math

import numpy as np
import torch

from . import _lib, network as net
from .layout import NPARAM, NPROP, NREC
from .ops import Glif3State, SpikeCompactor, SynapseTable, _dev, _p, _stream, glif3_precompute, n_words, unpack_bits


PULL_MAP_BYTES = 40 * 1024      # activity map of bmtk_csr_propagate_pull: what is left of 80 KB beside its accumulators
PULL_MIN_DENSITY = 0.06         # synaptic events per synapse and step from which "auto" pulls instead of pushing
                                # (the unfused pull form: batches other than 8, 16, 32, 64)
# What a step of a batched run costs on one MI355X, in picoseconds, fitted to runs of 51,978 neurons x 60 M synapses at
# batches 8, 16, 32 and 0 - 3.2 Hz and of 230,924 neurons x 77 M synapses at batch 8: the fused pull form streams the
# joint table once per two steps (per synapse, divided by how full a row's blocks of 256 are) and adds a little per
# synaptic event; the event-driven form pays per element for its update (less with a class table) and an atomic per event.
FUSE_PS_PER_SYNAPSE = 1.35
FUSE_PS_PER_EVENT = 6.0
PUSH_PS_PER_ELEMENT = 55.0
PUSH_PS_PER_ELEMENT_CLASS_TABLE = 27.0
PUSH_PS_PER_EVENT = 48.0
FUSE_LDS_BYTES = 150 * 1024     # LDS of one workgroup of the fused batched driver (kFuseLdsMax of csrc/simulate_fused.hip)
FUSE_WAVES = 16                 # wavefronts of one of its workgroups (kFuseWaves)
FUSE_BATCHES = (8, 16, 32, 64)  # lane = trial, whole bytes of spike bits per neuron
RES_LDS_BYTES = 160 * 1024      # LDS of one gfx950 compute unit
RES_ACT_ENTRIES = 8192          # active-row list of the resident kernel (kActCap of csrc/resident.hip), 4 B each
RES_LDS_EXTRA = RES_ACT_ENTRIES * 4 + 256   # the list plus the kernel's static LDS (rounded up)
# the single-workgroup form: per element the spike offsets and probed potentials of two steps (SOLO_LDS_PER_ELEMENT);
# the items (rows to walk) of two steps and its static LDS (SOLO_LDS_EXTRA)
SOLO_LDS_PER_ELEMENT = 4 * 4
SOLO_LDS_EXTRA = 10240 + 2048
RECORD_WAYS = 64                # lists a large spike record is split into (bmtk_glif3_sim.spike_ways)


def resident_span(ne, batch, ring_slots, n_cu, single=True):
    """Elements per workgroup of the resident kernel for a network of ``ne`` elements on ``n_cu`` compute
    units, or 0 when the network does not fit: batch 1, one workgroup per compute unit (rounded down to a
    multiple of 8), at most 1024 elements each, and ring slice + active-row list + static LDS within the
    compute unit's LDS.  ``bmtk_glif3_simulate_fwd`` applies the same bound.  A network of up to 1024 elements
    goes to ONE workgroup when its whole ring fits (``single``): the library then runs the form without a grid
    barrier."""
    cus = n_cu - n_cu % 8
    if batch != 1 or cus <= 0 or ne <= 0:
        return 0
    if single and ne <= 1024:
        whole = -(-ne // 64) * 64
        if (ring_slots * NREC * 4 + SOLO_LDS_PER_ELEMENT) * whole + SOLO_LDS_EXTRA <= RES_LDS_BYTES:
            return whole
    span = -(-(-(-ne // cus)) // 64) * 64
    if span > 1024 or ring_slots * NREC * span * 4 + RES_LDS_EXTRA > RES_LDS_BYTES:
        return 0
    return span


def fused_pays(n_neurons, batch, n_synapses, class_table, rate_hz, h_ms=1.0):
    """Whether the fused pull form of the batched driver is expected to take less time per step than pushing the
    spikes as events, for a network of ``n_neurons`` with ``n_synapses`` recurrent and input synapses at ``batch``
    trials and a mean rate of ``rate_hz``."""
    if n_synapses <= 0:
        return False
    events = n_synapses * batch * float(rate_hz) * 1e-3 * h_ms
    row = n_synapses / float(n_neurons)
    blocks_full = row / (256.0 * math.ceil(row / 256.0))
    fused = FUSE_PS_PER_SYNAPSE * n_synapses / blocks_full + FUSE_PS_PER_EVENT * events
    push = ((PUSH_PS_PER_ELEMENT_CLASS_TABLE if class_table else PUSH_PS_PER_ELEMENT) * n_neurons * batch
            + PUSH_PS_PER_EVENT * events)
    return fused < push


class Glif3Simulator:
    """A population of GLIF3 neurons with recurrent and external synapses.

    par         fp64 [NPARAM, columns] NEST-unit parameters; one column per
                neuron, or per parameter class when ``class_id`` is given
    rec, inp    source-major synapse tables (numpy tuples, see bmtk_amd.network):
                recurrent (rows = neurons) and external (rows = input sources)
    ring_slots  slots of the delay ring buffer; default = largest (residual) delay + 1
    resident    "auto": every ``run`` is one cooperative launch that keeps the state in registers and the ring in
                LDS (the resident kernel) whenever the network fits it -- batch 1, at most 1024 elements per
                compute unit, ring slice within LDS; True: insist on it (ValueError otherwise); False: one launch
                per step, which takes any batch and size
    single_workgroup  resident mode: a network of up to 1024 elements whose whole ring fits LDS runs in ONE
                workgroup, without a grid barrier (about 1 us per step instead of 2.5); False keeps such a network
                on the many-workgroup form
    fired_lists  resident mode with several workgroups: every workgroup publishes the neurons that fired in a step
                as a short list beside its ballots, and the others read the lists instead of expanding the whole
                network's ballots (steps in which a list does not suffice are read from the ballots); False: always
                from the ballots.  Same results either way.
    expected_rate_hz  what "auto" decides ``pull`` / ``fused`` by.  Pushing spikes into the ring costs an atomic per
                synaptic event, pulling a pass over the whole table per step whatever the activity; a synapse
                carries batch * rate * h events per step, and on one MI355X the pass is the cheaper of the two from
                about 0.06 events per synapse and step (measured: 51,978 neurons x 32 trials at 3.2 Hz pull 168 us
                against 340 pushed; 230,924 neurons x 8 and x 16 at 2.8 Hz pushed 132 / 237 us against 321 / 358
                pulled).  Default 3 Hz: batches from 20 at 1 ms steps.  That mark decides the unfused ``pull``;
                ``fused`` is decided by ``fused_pays``, which compares the fitted cost of a step in either form.
    fused       launch-per-step mode, batch 8, 16, 32 or 64, delay_offset 0: one launch per step in which a
                wavefront sums what arrives at a neuron -- over recurrent and input synapses, from a joint
                target-major table and a joint history of spike and input-event bits -- and advances the neuron's
                trials, lane = trial; no arrival sum passes through device memory.  "auto": when ``fused_pays``
                says a step costs less this way than pushed as events (the update's share grows with the batch,
                the table pass does not: 51,978 neurons x 60 M synapses from batch 16 on at any rate, at batch 8
                from about 3.3 Hz); takes any number of sources (above what the activity map in
                LDS holds, one bit of the map stands for 2, 4, ... sources).  False: the pull form as separate
                launches (below).  ``ring`` then holds only the few input ids repeated within a step.
    pull        launch-per-step mode only: sum the recurrent arrivals of a step in one pass over a target-major
                copy of the table from the spike-bit history, instead of pushing them into the ring with global
                atomics as spikes occur -- the faster form for batched runs.  "auto": by ``expected_rate_hz``
                (and delay_offset 0, network small enough for the activity map in LDS).  Recurrent arrivals still ahead at the end
                of a run then live in the history, and ``ring`` holds the input arrivals only.
    delay_offset  B steps taken off every delay before the tables are built; spikes and input events are
                then handed to the tables B steps late from a history of spike bits, which gives the same
                arrivals with a ring B slots shorter.  "auto": 0 while the largest delay is at most 63
                steps (what the ring and the packed tables hold), else the smallest delay minus one --
                the case of NEST networks run at a fine resolution (1-2 ms delays at 0.001-0.1 ms steps).
                Also the smallest delay minus one when that is what lets a network of up to 1024 neurons keep its
                whole ring in ONE workgroup's LDS (the resident form without a grid barrier).
                The delay columns may then be any integer type; residual delays must stay within 63.
    """

    def __init__(self, n_neurons, par, h, batch=1, class_id=None, rec=None, inp=None, ring_slots=None,
                 asc_init=None, u_init=None, i_ext=None, device=None, resident="auto", delay_offset="auto",
                 pull="auto", single_workgroup=True, fired_lists=True, fused="auto", fuse_wg_per_cu=0,
                 expected_rate_hz=3.0):
        self.lib = _lib.load()
        self.dev = device or _dev()
        self.n, self.batch, self.h = int(n_neurons), int(batch), float(h)
        self.ne = self.n * self.batch
        if self.ne >= 2 ** 31:
            raise ValueError("n_neurons*batch must stay below 2^31")
        par = np.ascontiguousarray(par, np.float64)
        if par.shape[0] != NPARAM:
            raise ValueError("par must be [{}, columns]".format(NPARAM))
        if class_id is not None:
            class_id = np.ascontiguousarray(class_id, np.int32)
            if class_id.size != self.n or class_id.min() < 0 or class_id.max() >= par.shape[1]:
                raise ValueError("class_id must map every neuron to a column of par")
        elif par.shape[1] != self.n:
            raise ValueError("par needs one column per neuron when class_id is not given")
        self.prop = glif3_precompute(par, h)
        self.class_id = None if class_id is None else torch.as_tensor(class_id, device=self.dev)
        lo, hi = [], []
        for t in (rec, inp):
            if t is not None and len(t[3]):
                lo.append(int(t[3].min()))
                hi.append(int(t[3].max()))
        min_delay, max_delay = (min(lo), max(hi)) if lo else (1, 1)
        if min_delay < 1:
            raise ValueError("delays must be at least one step")
        if delay_offset == "auto":
            delay_offset = 0 if max_delay <= 63 else min_delay - 1
            if (delay_offset == 0 and min_delay > 1 and resident and single_workgroup and self.batch == 1
                    and self.n <= 1024 and not ring_slots):
                # a small network whose whole ring only fits ONE workgroup's LDS (the form without a grid barrier)
                # once the part all delays have in common is taken off: bmtk's example networks at dt = 0.1 ms
                # (every delay 2 ms: 21 ring slots for 450 cells are 172 KB, 2 slots 16 KB)
                whole = -(-self.n // 64) * 64

                def fits(slots):
                    return (slots * NREC * 4 + SOLO_LDS_PER_ELEMENT) * whole + SOLO_LDS_EXTRA <= RES_LDS_BYTES
                if not fits(max_delay + 1) and fits(max_delay - min_delay + 2):
                    delay_offset = min_delay - 1
        self.delay_offset = int(delay_offset)
        if not 0 <= self.delay_offset < min_delay:
            raise ValueError("delay_offset must lie in 0..smallest delay - 1")
        # residual delays beyond 63 steps: a wider delay field and a longer ring, which only the launch-per-step
        # driver (without the pull form) handles
        residual = max_delay - self.delay_offset
        self.delay_bits = 6 if residual <= 63 else max(7, int(residual).bit_length())
        if self.delay_bits > 6:
            ring_bytes = (residual + 1) * NREC * self.ne * 4
            if (self.delay_bits > 14 or self.n >= 2 ** (30 - self.delay_bits) or ring_bytes > 8 << 30
                    or resident is True or pull is True):
                raise ValueError("delays span {}..{} steps: after taking off {} the largest still exceeds the 63 steps "
                                 "the ring buffer of the resident and pull forms holds, or what the wide form takes "
                                 "({} ring bytes, {} neurons)".format(min_delay, max_delay, self.delay_offset,
                                                                      ring_bytes, self.n))
            resident = pull = False
        wide = self.delay_bits > 6

        def narrow(t):
            return t is None or t[3].dtype == (torch.uint8 if torch.is_tensor(t[3]) else np.uint8)

        if self.delay_offset or wide or not (narrow(rec) and narrow(inp)):
            def shorten(t):
                if t is None:
                    return None
                d = t[3] - self.delay_offset
                if torch.is_tensor(d):
                    d = d.to(torch.int32 if wide else torch.uint8)
                else:
                    d = d.astype(np.int32 if wide else np.uint8)
                return (t[0], t[1], t[2], d, t[4])
            rec, inp = shorten(rec), shorten(inp)
        self.L = int(ring_slots) if ring_slots else max_delay - self.delay_offset + 1
        self.rec = self._table(rec, self.n) if rec is not None else None
        self.inp = self._table(inp, None) if inp is not None else None
        for t in (self.rec, self.inp):
            if t is not None:
                t.delay_bits = self.delay_bits
        self.n_inputs = self.inp.n_rows if self.inp is not None else 0
        # A table without a synapse delivers nothing and its arrays have no address to hand over: the kernels are
        # not given it.  Events of input sources that project nowhere are still accepted (and checked).
        if self.rec is not None and self.rec.nnz == 0:
            self.rec = None
        self.inp_without_synapses = self.inp is not None and self.inp.nnz == 0
        if self.inp_without_synapses:
            self.inp = None
        self.state = Glif3State.zeros(self.n, self.batch, asc_init=asc_init, u_init=u_init, device=self.dev)
        self.ring = torch.zeros(self.L, NREC, self.ne, device=self.dev)
        self.i_ext = None if i_ext is None else torch.as_tensor(np.asarray(i_ext, np.float32), device=self.dev)
        if self.i_ext is not None and self.i_ext.numel() != self.ne:
            raise ValueError("i_ext needs one entry per element")
        self.in_ptr = self.in_events = None
        self.in_steps = 0
        self.in_duplicates = False
        self.in_repeat_ptr = self.in_repeat_events = None   # repeated ids of a step, for the pull form of the inputs
        self.step = 0
        self.words = n_words(self.ne)
        # history of spike bits: 2B+3 rows let resident workgroups drift B steps apart, one more lets them look
        # at the grid barrier only where the spikes behind it are needed; B+3 is the least
        self.hist_slots = 2 * self.delay_offset + 4
        if self.hist_slots * (self.words + 1) * 8 > 2 ** 30:
            self.hist_slots = self.delay_offset + 3
        self.work_bits = torch.zeros(self.hist_slots * (self.words + 1), dtype=torch.int64, device=self.dev)
        if self.n >= 2 ** 24:
            raise ValueError("the packed synapse tables index at most 2^24 neurons")
        self.res_sync = torch.zeros(_lib.RES_SYNC_WORDS, dtype=torch.int32, device=self.dev)
        self.res_span = self.res_groups = 0
        self.rec_seg = self.inp_seg = self.res_unified = self.res_fired = None
        self._pending_check = False
        self.probe_ids = self.probe_col = None
        self.probe_every = 1
        self.spin_limit = 0  # resident mode: polls of the grid barrier before giving up (0 = built-in limit)
        self.single_workgroup = bool(single_workgroup)
        self.fired_lists = bool(fired_lists)
        if resident:
            self._setup_resident(required=(resident is True))
        self.pull_table = self.pull_syn = self.pull_work = None
        self.pull_inp_table = self.pull_inp_syn = self.pull_inp_work = self.in_hist = None
        self.fuse_table = self.fuse_any = None
        self.fuse_wg_per_cu = int(fuse_wg_per_cu)
        can_fuse = ((self.rec is not None or self.inp is not None) and not self.res_span and self.delay_offset == 0
                    and self.delay_bits == 6 and self.batch in FUSE_BATCHES and pull is not False)
        if fused is True and not can_fuse:
            raise ValueError("the fused form needs a synapse table, launch-per-step mode, delay_offset 0, delays "
                             "within 63 steps and a batch of 8, 16, 32 or 64")
        can_pull = (self.rec is not None and not self.res_span and self.delay_offset == 0
                    and self.L * ((self.n + 31) // 32) * 4 <= PULL_MAP_BYTES)
        # the pull form sums in 64-bit fixed point: weights must be finite and below 2^31 in size
        def fixed_point_ok(t):
            w = t.weights
            return not w.numel() or bool(torch.isfinite(w).all() & (w.abs().max() < 2.0 ** 31))
        # events per synapse and step at the expected rate: from PULL_MIN_DENSITY on a pass over the table is cheaper
        dense = self.batch * float(expected_rate_hz) * 1e-3 * self.h >= PULL_MIN_DENSITY
        if can_pull and (pull is True or (pull == "auto" and dense)):
            if not (fixed_point_ok(self.rec) and (self.inp is None or fixed_point_ok(self.inp))):
                if pull is True:
                    raise ValueError("the pull form needs finite weights smaller than 2^31 in size")
                can_pull = False   # the event-driven form propagates IEEE values as they are
        if pull is True and not can_pull:
            raise ValueError("the pull form needs a recurrent table, launch-per-step mode, delay_offset 0 and "
                             "ring_slots * n_neurons / 8 bytes of LDS (at most 40 KB)")
        n_syn = sum(t.nnz for t in (self.rec, self.inp) if t is not None)
        if can_fuse and fused and (fused is True or pull is True or
                                   fused_pays(self.n, self.batch, n_syn, self.class_id is not None, expected_rate_hz, self.h)):
            tables = [t for t in (self.rec, self.inp) if t is not None]
            if all(fixed_point_ok(t) for t in tables):
                self._setup_fused()
            elif fused is True:
                raise ValueError("the fused form needs finite weights smaller than 2^31 in size")
        if self.fuse_table is not None:
            pass
        elif can_pull and (pull is True or (pull == "auto" and dense)):
            self.pull_table = self.rec.transposed(self.n)
            self.pull_syn = torch.zeros(NREC, self.ne, device=self.dev)
            need = self.lib.bmtk_csr_propagate_pull_workspace_bytes(self.L, self.n)
            self.pull_work = torch.zeros(need // 4 + 1, dtype=torch.int32, device=self.dev)
            # the history must hold one row per ring slot, row t % L = spikes of step t
            self.hist_slots = self.L
            self.work_bits = torch.zeros(self.hist_slots * (self.words + 1), dtype=torch.int64, device=self.dev)
            if self.inp is not None and self.L * ((self.n_inputs + 31) // 32) * 4 <= PULL_MAP_BYTES:
                self.pull_inp_table = self.inp.transposed(self.n)
                self.pull_inp_syn = torch.zeros(NREC, self.ne, device=self.dev)
                need = self.lib.bmtk_csr_propagate_pull_workspace_bytes(self.L, self.n_inputs)
                self.pull_inp_work = torch.zeros(need // 4 + 1, dtype=torch.int32, device=self.dev)
                self.in_hist_stride = n_words(self.n_inputs * self.batch) + 1
                self.in_hist = torch.zeros(self.L * self.in_hist_stride, dtype=torch.int64, device=self.dev)

    def _setup_fused(self):
        """Joint target-major table, joint history and activity map of the fused batched driver."""
        n, batch, n_in = self.n, self.batch, self.n_inputs if self.inp is not None else 0
        self.fuse_in_base = -(-n * batch // 64) * 64 // batch
        if self.fuse_in_base + n_in >= 2 ** 24:
            return
        self.fuse_table = SynapseTable.joined_by_target(self.rec, self.inp, n, self.fuse_in_base)
        self.fuse_hist_stride = self.fuse_in_base * batch // 64 + n_words(n_in * batch) + 1
        self.hist_slots = self.L + 4         # two steps per launch: rows read, written and cleared ahead
        self.ring = torch.zeros(self.L + 2, NREC, self.ne, device=self.dev)   # (its ring: two slots more)
        self.work_bits = torch.zeros(self.hist_slots * self.fuse_hist_stride, dtype=torch.int64, device=self.dev)
        # one bit of the activity map per 2^shift sources: the smallest shift whose map fits the LDS beside the
        # accumulators (16 wavefronts x 2 arrival steps x (4 x 64 sums + a stage of 64 synapses) x 8 bytes)
        fixed = FUSE_WAVES * 2 * (NREC * 64 + 64) * 8
        self.fuse_shift = 0
        while fixed + self.L * self._fuse_any_words() * 4 > FUSE_LDS_BYTES:
            self.fuse_shift += 1
        self.fuse_any = self._new_fuse_any()

    def set_fuse_shift(self, shift):
        """Fused form: one bit of the activity map per 2^shift sources (the constructor picks the smallest shift
        whose map fits the LDS).  Before the first run only."""
        if self.fuse_table is None or self.step:
            raise ValueError("set_fuse_shift applies to the fused form before its first run")
        fixed = FUSE_WAVES * 2 * (NREC * 64 + 64) * 8
        old, self.fuse_shift = self.fuse_shift, int(shift)
        if not 0 <= self.fuse_shift <= 16 or fixed + self.L * self._fuse_any_words() * 4 > FUSE_LDS_BYTES:
            self.fuse_shift = old
            raise ValueError("shift must lie in 0..16 and leave the activity map within the LDS")
        self.fuse_any = self._new_fuse_any()

    def _new_fuse_any(self):
        # the activity map (one row per history row) and, behind it, the map of ring cells that hold something
        # (one row per ring slot, a bit per neuron)
        return torch.zeros(self.hist_slots * self._fuse_any_words() + (self.L + 2) * (-(-self.n // 32)), dtype=torch.int32,
                           device=self.dev)

    def _fuse_any_words(self):
        groups = -(-(self.fuse_in_base + (self.n_inputs if self.inp is not None else 0)) // (1 << self.fuse_shift))
        return -(-groups // 32)

    def _setup_resident(self, required):
        """Resident mode keeps state in registers and the ring in LDS for a whole
        run; it needs batch 1, at most 1024 elements per compute unit and a ring
        slice that fits in LDS beside the kernel's active-row list."""
        n_cu = torch.cuda.get_device_properties(self.dev).multi_processor_count
        span = resident_span(self.ne, self.batch, self.L, n_cu, single=self.single_workgroup)
        if not span:
            if required:
                raise ValueError("network does not fit resident mode (batch 1, <= 1024 elements per compute unit, "
                                 "ring slice + {} bytes of lists within the {} bytes of LDS)".format(
                                     RES_LDS_EXTRA, RES_LDS_BYTES))
            return
        groups = -(-self.ne // span)
        if self.rec is not None:
            self.rec = self.rec.sorted_by_index()
            self.rec_seg = self.rec.segment_offsets(span, groups)
        if self.inp is not None:
            self.inp = self.inp.sorted_by_index()
            self.inp_seg = self.inp.segment_offsets(span, groups)
        self.res_unified = None
        if self.rec is not None and self.inp is not None and self.rec.nnz + self.inp.nnz < (1 << 32):
            # One table for both kinds of rows, the input rows behind the recurrent ones: the kernel then needs no
            # choice between two tables per listed row (and fewer of its scarce scalar registers).  The packed
            # records of the two tables become views of the joint array; the input offsets count from its start.
            nr, ni = self.rec.nnz, self.inp.nnz
            packed = torch.empty(max(nr + ni, 1), 2, dtype=torch.int32, device=self.dev)
            packed[:nr] = self.rec.packed()[:nr]
            packed[nr:nr + ni] = self.inp.packed()[:ni]
            self.rec._packed, self.inp._packed = packed[:nr], packed[nr:nr + ni]
            seg = torch.empty(self.n + self.inp.n_rows, groups + 1, dtype=torch.int32, device=self.dev)
            seg[:self.n] = self.rec_seg
            seg[self.n:] = ((self.inp_seg.long() & 0xFFFFFFFF) + nr).to(torch.int32)   # uint32 kept in int32
            self.rec_seg, self.inp_seg = seg[:self.n], seg[self.n:]
            self.res_unified = (packed, seg)
        self.res_span, self.res_groups = span, groups
        # the lists of fired neurons the workgroups publish beside their ballots (bmtk_glif3_sim.res_fired)
        self.res_fired = (torch.zeros(self.hist_slots * groups * _lib.RES_FIRED_SLOTS, dtype=torch.int32, device=self.dev)
                          if groups > 1 and self.fired_lists else None)

    def check(self):
        """Raise if a resident run since the last check gave up on its grid barrier (synchronises).  The abort
        word is sticky on the device: a run that finds it set gives up at once, so a failure cannot be lost
        between two checks; it is cleared here."""
        if self._pending_check:
            self._pending_check = False
            if int(self.res_sync[1].item()) != 0:
                self.res_sync[1] = 0
                raise RuntimeError("resident simulation aborted: grid barrier timed out; results since the last "
                                   "check are invalid")

    def _table(self, csr, n_rows):
        if torch.is_tensor(csr[0]):
            rows = csr[0].numel() - 1 if n_rows is None else n_rows
            return SynapseTable.from_device(csr, rows, self.n, self.L)
        rows = csr[0].size - 1 if n_rows is None else n_rows
        net.check_csr(csr, rows, self.n, self.L)
        return SynapseTable.from_numpy(csr, self.dev)

    def set_input_events(self, in_ptr, in_events):
        """Per-step event lists: events in_events[in_ptr[t]:in_ptr[t+1]] are
        emitted in step t (their spike stamp is t+1).  Within a step the ids
        (source*batch+trial) must be ascending -- the input-weight gradient kernel
        gives every source's run of events one writer and relies on it.  The same id
        may occur more than once in a step (two spikes of one generator inside one
        resolution step, which NEST delivers both): every occurrence is delivered.
        The pull form of the inputs turns a step's events into bits, which hold an id
        once; the second and later occurrences are then listed apart
        (``in_repeat_ptr`` / ``in_repeat_events``) and delivered as events on top."""
        if self.inp is None and not self.inp_without_synapses:
            raise ValueError("no input synapse table")
        if torch.is_tensor(in_ptr):
            ok = bool((in_ptr[0] == 0) & (in_ptr[1:] >= in_ptr[:-1]).all() & (in_ptr[-1] == in_events.numel()))
            if in_events.numel():
                ok = ok and bool((in_events.min() >= 0) & (in_events.max() < self.n_inputs * self.batch))
            if not ok or in_ptr.dtype != torch.int64 or in_events.dtype != torch.int32:
                raise ValueError("device input event lists are inconsistent")
            in_ptr, in_events = in_ptr.contiguous(), in_events.contiguous()
        else:
            in_ptr = np.ascontiguousarray(in_ptr, np.int64)
            in_events = np.ascontiguousarray(in_events, np.int32)
            net.check_input_events(in_ptr, in_events, self.n_inputs * self.batch)
            in_ptr = torch.as_tensor(in_ptr, device=self.dev)
            in_events = torch.as_tensor(in_events, device=self.dev)
        repeat = None
        if in_events.numel() > 1:
            step_start = torch.zeros(in_events.numel() + 1, dtype=torch.bool, device=in_events.device)
            step_start[in_ptr] = True                      # an event that opens a step may be smaller than the last
            d = in_events[1:] - in_events[:-1]
            inside = ~step_start[1:-1]
            if bool(((d < 0) & inside).any()):
                raise ValueError("input events must be ascending within every step")
            repeat = (d == 0) & inside                     # event k+1 repeats event k of the same step
            if not bool(repeat.any()):
                repeat = None
        self.in_ptr = in_ptr
        self.in_events = in_events if in_events.numel() else in_events.new_zeros(1)
        self.in_steps = in_ptr.numel() - 1
        self.in_duplicates = repeat is not None
        self.in_repeat_ptr = self.in_repeat_events = None
        if repeat is not None and (self.pull_inp_table is not None or self.fuse_table is not None):
            where = repeat.nonzero().flatten() + 1         # positions of the second and later occurrences
            self.in_repeat_events = in_events[where].contiguous()
            self.in_repeat_ptr = torch.searchsorted(where, in_ptr).to(torch.int64).contiguous()

    def _struct(self, bits=None, record=None):
        s = _lib.Glif3Sim()
        st = self.state
        s.n_neurons, s.batch, s.ring_slots, s.h = self.n, self.batch, self.L, self.h
        s.V, s.asc, s.y1, s.y2, s.ref = (_p(x) for x in (st.V, st.asc, st.y1, st.y2, st.ref))
        s.prop, s.prop_stride, s.class_id = _p(self.prop), self.prop.shape[1], _p(self.class_id)
        s.ring = _p(self.ring)
        if self.rec is not None:
            s.rec_indptr, s.rec_indices, s.rec_weights, s.rec_delays, s.rec_receptors = self.rec.pointers()
            s.rec_packed = _p(self.rec.packed())
        if self.inp is not None and self.in_ptr is not None:
            s.n_inputs = self.n_inputs
            s.in_ptr, s.in_events = _p(self.in_ptr), _p(self.in_events)
            s.inp_indptr, s.inp_indices, s.inp_weights, s.inp_delays, s.inp_receptors = self.inp.pointers()
            s.inp_packed = _p(self.inp.packed())
        s.i_ext = _p(self.i_ext)
        s.work_bits = _p(self.work_bits)
        s.delay_offset, s.hist_slots, s.delay_bits = self.delay_offset, self.hist_slots, self.delay_bits
        if self.pull_table is not None:
            s.pull_indptr, s.pull_packed = _p(self.pull_table.indptr), _p(self.pull_table.packed())
            s.pull_syn, s.pull_work = _p(self.pull_syn), _p(self.pull_work)
            if self.pull_inp_table is not None and self.in_ptr is not None:
                s.pull_inp_indptr, s.pull_inp_packed = _p(self.pull_inp_table.indptr), _p(self.pull_inp_table.packed())
                s.pull_inp_syn, s.pull_inp_work = _p(self.pull_inp_syn), _p(self.pull_inp_work)
                s.in_hist, s.in_hist_stride = _p(self.in_hist), self.in_hist_stride
                if self.in_repeat_ptr is not None:
                    s.in_repeat_ptr, s.in_repeat_events = _p(self.in_repeat_ptr), _p(self.in_repeat_events)
        if self.fuse_table is not None:
            s.n_inputs = self.n_inputs if self.inp is not None else 0   # the history's layout, events or not
            s.fuse_indptr, s.fuse_packed = _p(self.fuse_table.indptr), _p(self.fuse_table.packed())
            s.fuse_any, s.fuse_hist_stride, s.fuse_in_base = _p(self.fuse_any), self.fuse_hist_stride, self.fuse_in_base
            s.fuse_shift, s.fuse_wg_per_cu = self.fuse_shift, self.fuse_wg_per_cu
            if self.in_repeat_ptr is not None:
                s.in_repeat_ptr, s.in_repeat_events = _p(self.in_repeat_ptr), _p(self.in_repeat_events)
        if self.res_span:
            s.res_span, s.res_groups, s.res_sync = self.res_span, self.res_groups, _p(self.res_sync)
            s.res_spin_limit = int(self.spin_limit)
            s.rec_seg, s.inp_seg = _p(self.rec_seg), _p(self.inp_seg)
            s.res_fired = _p(self.res_fired)
            if self.res_unified is not None and s.inp_packed and self.res_groups > 1:
                s.inp_packed = s.rec_packed      # the input offsets count from the start of the joint table
        if bits is not None:
            s.spike_bits, s.spike_bits_stride = _p(bits), bits.shape[1]
        if record is not None:
            s.spike_step, s.spike_elem, s.spike_frac = _p(record["step"]), _p(record["elem"]), _p(record["frac"])
            s.spike_cap, s.spike_count = record["step"].numel(), _p(record["count"])
            s.spike_ways = record.get("ways", 1)
        return s

    def set_probes(self, element_ids, every=1):
        """Record the membrane potential of some elements (what a multimeter connected to them does): after every
        step t with (t + 1) % every == 0, in both modes.  ``run`` then returns ``probe`` = dict(v=[samples,
        len(element_ids)] fp32 of U = V_m - E_L, steps=int64 [samples], the sampled steps).  None switches it off."""
        if element_ids is None:
            self.probe_ids = self.probe_col = None
            return
        ids = np.asarray(element_ids, np.int64).reshape(-1)
        if ids.size == 0 or ids.min() < 0 or ids.max() >= self.ne or np.unique(ids).size != ids.size:
            raise ValueError("probes need distinct element ids in 0..{}".format(self.ne - 1))
        if int(every) < 1:
            raise ValueError("every must be at least 1")
        col = np.full(self.ne, -1, np.int32)
        col[ids] = np.arange(ids.size, dtype=np.int32)
        self.probe_ids, self.probe_every = ids, int(every)
        self.probe_col = torch.as_tensor(col, device=self.dev)

    def run(self, n_steps, spike_bits=True, record_cap=0, save_state=False, record_ways=None):
        """Advance ``n_steps`` steps.  Returns a dict with ``bits`` (int64
        [n_steps, words], spike bits per step) and, when ``record_cap`` > 0,
        the atomic spike record with crossing fractions (read it with ``collect_record``: a large record is
        kept as several lists); ``save_state`` adds the
        per-step record (potentials and flags) the backward pass reads; ``probe``
        holds the potentials asked for with ``set_probes``.  Does not
        synchronise."""
        if self.in_ptr is not None and self.step + n_steps > self.in_steps:
            raise ValueError("input event lists cover {} steps, run would reach {}".format(
                self.in_steps, self.step + n_steps))
        bits = torch.zeros(n_steps, self.words, dtype=torch.int64, device=self.dev) if spike_bits else None
        record = None
        if record_cap:
            # A large record is kept as RECORD_WAYS lists with a counter each (``collect_record`` joins them): the
            # wavefronts of a whole network bumping ONE counter cost the resident kernel 1.5 of 5.5 us per step.
            # No more lists than workgroups (a list nobody appends to is room lost), each of at least 1024 entries.
            # Workgroups are dealt out to the lists in turn, so a list may serve one workgroup more than another:
            # callers size the record with room to spare, as they had to for one list.
            n_wg = self.res_groups if self.res_span else -(-self.ne // 512)
            ways = 1
            while ways * 2 <= min(RECORD_WAYS, n_wg) and record_cap >= ways * 2 * 1024:
                ways *= 2
            if self.res_groups > RECORD_WAYS and self.delay_offset == 0 and record_cap >= 256 * 1024:
                # the resident kernel without slack: with a list per workgroup (at most 256 are launched) a
                # workgroup keeps its count in a register and no wavefront waits for an atomic on device memory
                ways = 256
            if record_ways is not None:      # the caller's choice: a power of two up to 256
                ways = int(record_ways)
                if ways < 1 or ways > 256 or ways & (ways - 1):
                    raise ValueError("record_ways must be a power of two in 1..256")
            record_cap = -(-int(record_cap) // ways) * ways
            # (only the counted entries are ever read: no need to clear a gigabyte of room first)
            record = dict(step=torch.empty(record_cap, dtype=torch.int32, device=self.dev),
                          elem=torch.empty(record_cap, dtype=torch.int32, device=self.dev),
                          frac=torch.empty(record_cap, dtype=torch.float32, device=self.dev),
                          count=torch.zeros(1 if ways == 1 else ways * _lib.RECORD_COUNT_STRIDE, dtype=torch.int64,
                                            device=self.dev), ways=ways)
        s = self._struct(bits, record)
        saved = None
        if save_state:
            if self.res_span:
                raise ValueError("save_state needs a simulator built with resident=False")
            saved = dict(v=torch.empty(n_steps, self.ne, device=self.dev),
                         flags=torch.empty(n_steps, self.ne, dtype=torch.uint8, device=self.dev), step0=self.step)
            s.save_v, s.save_flags = _p(saved["v"]), _p(saved["flags"])
        probe = None
        if self.probe_col is not None:
            every = self.probe_every
            first = -(-(self.step + 1) // every) * every - 1  # first step t >= self.step with (t + 1) % every == 0
            steps = torch.arange(first, max(first, self.step + n_steps), every, dtype=torch.int64)  # may be none
            room = torch.empty(max(1, steps.numel()), self.probe_ids.size, device=self.dev)  # a call may sample nothing
            probe = dict(v=room[:steps.numel()], steps=steps)
            s.probe_col, s.probe_v = _p(self.probe_col), room.data_ptr()
            s.probe_stride, s.probe_every = self.probe_ids.size, every
        _lib.check(self.lib.bmtk_glif3_simulate_fwd(C.byref(s), self.step, n_steps, _stream()))
        self.step += n_steps
        self._pending_check = bool(self.res_span)
        return dict(bits=bits, record=record, saved=saved, probe=probe)

    def collect_record(self, record, sort_scale=None):
        """The spike record of a ``run(..., record_cap=...)`` as one list: dict(step int32[], elem int32[], frac
        float32[], count int, overflow bool, ways, way_cap, fullest), unordered within a step.  ``count`` is the
        number of spikes the run produced; ``overflow`` says that some of them found no room (then the lists are
        incomplete).  A record kept as ``ways`` lists overflows as soon as ONE list does -- a workgroup appends to
        its own list of ``way_cap`` = cap / ways entries only, so activity concentrated in the neurons of a few
        workgroups can overflow while ``count`` is far below the record's total size; ``fullest`` is the largest
        count of a single list (``overflow_message`` words it).
        With ``sort_scale`` (the resolution in ms) the list comes back ordered by spike time
        (step + frac) * sort_scale, ties by element -- sorted on the device, where two million spikes take
        milliseconds instead of the second a host sort takes -- and ``time`` (float64, ms) is added.
        Synchronises."""
        self.check()
        ways = record.get("ways", 1)
        cap = record["step"].numel()
        way_cap = cap // ways
        counts = record["count"][::_lib.RECORD_COUNT_STRIDE][:ways] if ways > 1 else record["count"][:1]
        counts = counts.cpu()                                  # the one synchronisation
        stored = torch.clamp(counts, max=way_cap).tolist()
        if ways == 1:
            keep = slice(0, stored[0])
        else:                                                  # the filled part of every list, one after the other
            dev = record["step"].device
            filled = torch.tensor(stored, dtype=torch.int64, device=dev)
            first = torch.arange(ways, dtype=torch.int64, device=dev) * way_cap - (torch.cumsum(filled, 0) - filled)
            keep = torch.arange(sum(stored), dtype=torch.int64, device=dev) + torch.repeat_interleave(first, filled)
        out = dict(step=record["step"][keep], elem=record["elem"][keep], frac=record["frac"][keep],
                   count=int(counts.sum()), overflow=bool((counts > way_cap).any()), ways=ways, way_cap=way_cap,
                   fullest=int(counts.max()))
        if sort_scale is not None:
            t = (out["step"].to(torch.float64) + out["frac"].to(torch.float64)) * float(sort_scale)
            by_elem = torch.argsort(out["elem"], stable=True)
            order = by_elem[torch.argsort(t[by_elem], stable=True)]
            out.update(step=out["step"][order], elem=out["elem"][order], frac=out["frac"][order], time=t[order])
        return out

    @staticmethod
    def overflow_message(rec):
        """What a caller reports when ``collect_record`` came back with ``overflow``: the capacity that ran out is
        that of one list, not of the record."""
        if rec["ways"] == 1:
            return "{} spikes, room for {}".format(rec["count"], rec["way_cap"])
        return ("{} spikes in all; the record is kept as {} lists of {} entries (one per group of workgroups) and "
                "the fullest list was asked to hold {}".format(rec["count"], rec["ways"], rec["way_cap"], rec["fullest"]))

    def to_host(self, *tensors):
        """Device tensors -> NumPy arrays through pinned host memory (torch keeps freed pinned blocks for reuse): a
        spike record of two million entries takes a millisecond or two instead of the five a copy into pageable
        memory takes.  The arrays own their memory.  Synchronises."""
        sizes = [t.numel() * t.element_size() for t in tensors]
        offsets = [0]
        for n in sizes:
            offsets.append(-(-(offsets[-1] + n) // 256) * 256)
        stage = torch.empty(max(offsets[-1], 1), dtype=torch.uint8, pin_memory=True)
        views = []
        for t, n, o in zip(tensors, sizes, offsets):
            v = stage[o:o + n].view(t.dtype).view(t.shape) if n else torch.empty(t.shape, dtype=t.dtype)
            if n:
                v.copy_(t.contiguous(), non_blocking=True)
            views.append(v)
        torch.cuda.synchronize(self.dev)
        return tuple(v.numpy() for v in views)   # (an array keeps its block of pinned memory alive)

    def spikes_from_bits(self, bits, step0=0):
        """Spike bits -> (step int64[], element int64[]) ascending, via the
        compaction kernels (exactly ``numpy.nonzero`` of the raster)."""
        self.check()
        n_steps, words = bits.shape
        per = max(1, (2 ** 31 - 64) // (words * 64))
        steps, elems = [], []
        for k0 in range(0, n_steps, per):
            chunk = bits[k0:k0 + per].contiguous()
            n = chunk.numel() * 64
            comp = SpikeCompactor(n, self.dev)
            ids, count = comp(torch.cat([chunk.reshape(-1), chunk.new_zeros(1)]))
            ids = ids[:int(count.item())].to(torch.int64)
            steps.append(ids // (words * 64) + k0 + step0)
            elems.append(ids % (words * 64))
        return torch.cat(steps), torch.cat(elems)

    def raster(self, bits):
        """uint8 [n_steps, ne] from spike bits."""
        self.check()
        return unpack_bits(bits, self.ne)

    def synaptic_events(self, bits):
        """Number of recurrent synaptic events the spikes in ``bits`` caused
        (sum of the out-degree of every spiking neuron)."""
        if self.rec is None:
            return 0
        _, elems = self.spikes_from_bits(bits)
        deg = (self.rec.indptr[1:] - self.rec.indptr[:-1]).to(torch.int64)
        return int(deg[elems // self.batch].sum().item())
