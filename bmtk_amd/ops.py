"""The per-step operations on torch device tensors (torch supplies memory and
streams only; all arithmetic is in ``libbmtk_amd.so``).

Layout: element e = neuron*batch + trial; state tensors are flat ``[ne]`` or
``[k, ne]``; the ring buffer is ``[L, 4, ne]``; spike bits are uint64 words
stored in int64 tensors of ``ceil(ne/64)+1`` entries.
"""
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib
from .layout import NASC, NPARAM, NPROP, NREC


def _dev():
    if not torch.cuda.is_available():
        raise RuntimeError("bmtk_amd needs a ROCm GPU; there is no CPU implementation of these operations")
    return torch.device("cuda", torch.cuda.current_device())


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t, dtype=None, numel=None, name="tensor"):
    """Device pointer of a tensor after checking placement, dtype, contiguity and size."""
    if t is None:
        return None
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError("{} must be a contiguous device tensor".format(name))
    if dtype is not None and t.dtype != dtype:
        raise TypeError("{} must be {}, got {}".format(name, dtype, t.dtype))
    if numel is not None and t.numel() < numel:
        raise ValueError("{} holds {} entries, needs {}".format(name, t.numel(), numel))
    return t.data_ptr()


def n_words(ne):
    return (ne + 63) // 64


@dataclass
class Glif3State:
    """SoA fp32 state of ``ne = n_neurons*batch`` elements."""
    V: torch.Tensor     # [ne]   membrane potential minus E_L (mV)
    asc: torch.Tensor   # [2,ne] after-spike currents (pA)
    y1: torch.Tensor    # [4,ne] alpha-PSC auxiliary state
    y2: torch.Tensor    # [4,ne] post-synaptic currents (pA)
    ref: torch.Tensor   # [ne]   int32 refractory steps left

    @classmethod
    def zeros(cls, n_neurons, batch=1, asc_init=None, u_init=None, device=None):
        dev = device or _dev()
        ne = n_neurons * batch
        st = cls(torch.zeros(ne, device=dev), torch.zeros(NASC, ne, device=dev), torch.zeros(NREC, ne, device=dev),
                 torch.zeros(NREC, ne, device=dev), torch.zeros(ne, dtype=torch.int32, device=dev))
        if asc_init is not None:
            a = torch.as_tensor(np.asarray(asc_init, np.float32).reshape(NASC, n_neurons), device=dev)
            st.asc.copy_(a.repeat_interleave(batch, dim=1))
        if u_init is not None:
            u = torch.as_tensor(np.asarray(u_init, np.float32).reshape(n_neurons), device=dev)
            st.V.copy_(u.repeat_interleave(batch))
        return st

    @classmethod
    def from_numpy(cls, st, device=None):
        dev = device or _dev()
        return cls(*(torch.as_tensor(np.ascontiguousarray(st[k]), device=dev) for k in ("V", "asc", "y1", "y2", "ref")))

    def to_numpy(self):
        return {k: getattr(self, k).cpu().numpy() for k in ("V", "asc", "y1", "y2", "ref")}

    def clone(self):
        return Glif3State(self.V.clone(), self.asc.clone(), self.y1.clone(), self.y2.clone(), self.ref.clone())

    @property
    def ne(self):
        return self.V.numel()


def glif3_precompute(par, h):
    """par: fp64 ``[NPARAM, n]`` NEST-unit parameters (host array or device tensor) ->
    fp32 ``[NPROP, n]`` propagators (NEST ``glif_psc::pre_run_hook``)."""
    lib = _lib.load()
    par = torch.as_tensor(np.ascontiguousarray(par, np.float64) if not torch.is_tensor(par) else par, device=_dev())
    if par.dim() != 2 or par.shape[0] != NPARAM:
        raise ValueError("par must be [{}, n]".format(NPARAM))
    par = par.contiguous()
    n = par.shape[1]
    prop = torch.empty(NPROP, n, dtype=torch.float32, device=par.device)
    _lib.check(lib.bmtk_glif3_precompute(n, _p(par, torch.float64), float(h), _p(prop), _stream()))
    return prop


def glif3_step_fwd(state, prop, h, batch=1, class_id=None, syn=None, clear_syn=False, i_ext=None,
                   z=None, zbits=None, frac=None):
    """One ``glif_psc`` update step in place on ``state``."""
    lib = _lib.load()
    ne = state.ne
    if ne % batch:
        raise ValueError("state size {} is not a multiple of batch {}".format(ne, batch))
    n = ne // batch
    if prop.dim() != 2 or prop.shape[0] != NPROP:
        raise ValueError("prop must be [{}, columns]".format(NPROP))
    if class_id is not None and class_id.numel() != n:
        raise ValueError("class_id must have one entry per neuron")
    _lib.check(lib.bmtk_glif3_step_fwd(
        n, batch, _p(state.V, torch.float32, ne, "V"), _p(state.asc, torch.float32, NASC * ne, "asc"),
        _p(state.y1, torch.float32, NREC * ne, "y1"), _p(state.y2, torch.float32, NREC * ne, "y2"),
        _p(state.ref, torch.int32, ne, "ref"), _p(prop, torch.float32), prop.shape[1],
        _p(class_id, torch.int32, n, "class_id"), float(h), _p(syn, torch.float32, NREC * ne, "syn"),
        1 if clear_syn else 0, _p(i_ext, torch.float32, ne, "i_ext"), _p(z, torch.uint8, ne, "z"),
        _p(zbits, torch.int64, n_words(ne) + 1, "zbits"), _p(frac, torch.float32, ne, "frac"), _stream()))


class SpikeCompactor:
    """Flags or spike bits -> (ascending int32 ids, int32 count on the device).
    Owns the workspace so repeated calls allocate nothing."""

    def __init__(self, n, device=None):
        lib = _lib.load()
        dev = device or _dev()
        self.n = n
        self.workspace = torch.zeros(lib.bmtk_spikes_compact_workspace_bytes(n) // 8 + 1, dtype=torch.int64, device=dev)
        self.ids = torch.empty(n, dtype=torch.int32, device=dev)
        self.count = torch.zeros(1, dtype=torch.int32, device=dev)

    def __call__(self, z):
        lib = _lib.load()
        if z.dtype == torch.uint8:
            _lib.check(lib.bmtk_spikes_compact(_p(z, torch.uint8, self.n, "z"), self.n, _p(self.ids), _p(self.count),
                                               _p(self.workspace), _stream()))
        else:
            _lib.check(lib.bmtk_spikes_compact_bits(_p(z, torch.int64, n_words(self.n), "zbits"), self.n,
                                                    _p(self.ids), _p(self.count), _p(self.workspace), _stream()))
        return self.ids, self.count


def spikes_compact_noalloc(z, ids, count):
    """``bmtk_spikes_compact_noalloc``: byte flags ``z`` -> ascending ids in the caller's ``ids`` (int32, at least
    ``z.numel()`` entries) and their number in ``count`` (int32 [1]); the workspace is inside the library, nothing
    is allocated, ``z.numel()`` is limited to ``_lib.COMPACT_NOALLOC_MAX_N``.  Calls that overlap on one GPU race."""
    lib = _lib.load()
    n = z.numel()
    _lib.check(lib.bmtk_spikes_compact_noalloc(_p(z, torch.uint8, n, "z"), n, _p(ids, torch.int32, n, "ids"),
                                               _p(count, torch.int32, 1, "count"), _stream()))


def spikes_compact(z):
    """Convenience form: returns the id list as a tensor of the exact length (synchronises)."""
    c = SpikeCompactor(z.numel())
    ids, count = c(z)
    return ids[:int(count.item())].clone()


BLOCKED_PAD = 16  # BMTK_BLOCKED_PAD of include/bmtk_amd.h


@dataclass
class SynapseTable:
    """Device copy of a synapse table (see ``bmtk_amd.network``)."""
    indptr: torch.Tensor
    indices: torch.Tensor
    weights: torch.Tensor
    delays: torch.Tensor
    receptors: torch.Tensor
    n_rows: int
    max_row: int

    @classmethod
    def from_numpy(cls, csr, device=None):
        dev = device or _dev()
        indptr, indices, w, d, r = csr
        t = [torch.as_tensor(np.ascontiguousarray(a), device=dev) for a in (indptr, indices, w, d, r)]
        deg = np.diff(indptr)
        return cls(*t, n_rows=indptr.size - 1, max_row=int(deg.max()) if deg.size else 0)

    @classmethod
    def from_edges(cls, src, tgt, w, d, r, n_rows, n_cols, device=None):
        """Edge list (host arrays or device tensors) -> source-major table, rows ordered by (row, column,
        original position), built on the device: what ``bmtk_amd.network.coo_to_csr`` does on the host, without
        its sort of tens of millions of keys on one CPU core."""
        dev = device or _dev()
        src = torch.as_tensor(np.ascontiguousarray(src) if not torch.is_tensor(src) else src, device=dev).long()
        tgt = torch.as_tensor(np.ascontiguousarray(tgt) if not torch.is_tensor(tgt) else tgt, device=dev).long()
        if src.numel() and (int(src.min()) < 0 or int(src.max()) >= n_rows or int(tgt.min()) < 0
                            or int(tgt.max()) >= n_cols):
            raise ValueError("edge endpoints outside 0..{} / 0..{}".format(n_rows - 1, n_cols - 1))
        order = torch.sort(src * n_cols + tgt, stable=True).indices
        counts = torch.bincount(src, minlength=n_rows)
        indptr = torch.zeros(n_rows + 1, dtype=torch.int32, device=dev)
        indptr[1:] = torch.cumsum(counts, 0).to(torch.int32)

        def col(a, dtype):
            a = torch.as_tensor(np.ascontiguousarray(a) if not torch.is_tensor(a) else a, device=dev)
            return a.to(dtype)[order].contiguous()

        d = torch.as_tensor(np.ascontiguousarray(d) if not torch.is_tensor(d) else d, device=dev)
        wide = bool(d.numel()) and int(d.max()) > 255
        return cls(indptr, tgt[order].to(torch.int32).contiguous(), col(w, torch.float32),
                   d.to(torch.int32 if wide else torch.uint8)[order].contiguous(), col(r, torch.uint8),
                   n_rows=n_rows, max_row=int(counts.max().item()) if counts.numel() else 0)

    @classmethod
    def from_device(cls, csr, n_rows, n_cols, ring_slots):
        """Adopt device tensors after the same checks ``network.check_csr`` makes on the host."""
        indptr, indices, w, d, r = (t.contiguous() for t in csr)
        nnz = indices.numel()
        ok = indptr.numel() == n_rows + 1 and int(indptr[0]) == 0 and int(indptr[-1]) == nnz
        ok = ok and bool((indptr[1:] >= indptr[:-1]).all())
        ok = ok and w.numel() == nnz and d.numel() == nnz and r.numel() == nnz
        if ok and nnz:
            ok = bool((indices.min() >= 0) & (indices.max() < n_cols) & (d.min() >= 1) & (d.max() < ring_slots)
                      & (r.max() < NREC))
        if not ok:
            raise ValueError("inconsistent synapse table (indptr, index range, delay range or receptor range)")
        deg = indptr[1:] - indptr[:-1]
        return cls(indptr, indices, w, d, r, n_rows=n_rows, max_row=int(deg.max()) if deg.numel() else 0)

    @property
    def nnz(self):
        return self.indices.numel()

    def max_delay(self):
        """Largest delay in steps (computed once; synchronises the first time)."""
        if getattr(self, "_max_delay", None) is None:
            self._max_delay = int(self.delays.max()) if self.nnz else 0
        return self._max_delay

    def packed(self):
        """The table as 8-byte {index | receptor<<24 | delay<<26, weight} records (built once); with
        ``delay_bits`` above 6 (set by the simulator for delay spreads beyond 63 steps) the delay field is that
        wide and the index field correspondingly narrower."""
        if getattr(self, "_packed", None) is None:
            bits = getattr(self, "delay_bits", 6)
            if self.max_delay() >= (1 << bits):
                raise ValueError("packed tables hold delays below {} steps".format(1 << bits))
            lib = _lib.load()
            out = torch.empty(max(self.nnz, 1), 2, dtype=torch.int32, device=self.indices.device)
            if bits == 6:
                _lib.check(lib.bmtk_csr_pack(self.nnz, *self.pointers()[1:], _p(out), _stream()))
            else:
                _lib.check(lib.bmtk_csr_pack_wide(self.nnz, _p(self.indices), _p(self.weights),
                                                  _p(self.delays.to(torch.int32).contiguous()), _p(self.receptors),
                                                  bits, _p(out), _stream()))
            self._packed = out
        return self._packed

    def sorted_by_index(self):
        """The same table with every row ordered by index (stable), as the segment offsets need."""
        rows = torch.repeat_interleave(torch.arange(self.n_rows, device=self.indices.device),
                                       (self.indptr[1:] - self.indptr[:-1]).long())
        order = torch.sort(rows * (1 << 24) + self.indices.long(), stable=True).indices
        return SynapseTable(self.indptr, self.indices[order].contiguous(), self.weights[order].contiguous(),
                            self.delays[order].contiguous(), self.receptors[order].contiguous(),
                            n_rows=self.n_rows, max_row=self.max_row)

    def transposed(self, n_cols):
        """source-major <-> target-major on the device, keeping the (row, column, position) order
        (what ``bmtk_amd.network.csr_transpose`` does on the host)."""
        dev = self.indices.device
        rows = torch.repeat_interleave(torch.arange(self.n_rows, device=dev, dtype=torch.int32),
                                       (self.indptr[1:] - self.indptr[:-1]).long())
        order = torch.sort(self.indices.long(), stable=True).indices
        counts = torch.bincount(self.indices.long(), minlength=n_cols)
        indptr = torch.zeros(n_cols + 1, dtype=torch.int32, device=dev)
        indptr[1:] = torch.cumsum(counts, 0).to(torch.int32)
        return SynapseTable(indptr, rows[order].contiguous(), self.weights[order].contiguous(),
                            self.delays[order].contiguous(), self.receptors[order].contiguous(), n_rows=n_cols,
                            max_row=int(counts.max().item()) if counts.numel() else 0)

    @staticmethod
    def joined_by_target(rec, inp, n_tgt, in_base):
        """The joint target-major table of the fused batched driver (``bmtk_glif3_sim.fuse_*`` of
        include/bmtk_amd.h) from the source-major recurrent table ``rec`` and input table ``inp`` (either may be
        None): row = target neuron, index field = source in the joint space -- neuron j is j, input source k is
        ``in_base + k``.  Rows keep the recurrent synapses first, each part in (source, position) order."""
        parts = []
        for t, base in ((rec, 0), (inp, in_base)):
            if t is None or t.nnz == 0:
                continue
            dev = t.indices.device
            rows = torch.repeat_interleave(torch.arange(t.n_rows, device=dev, dtype=torch.int64),
                                           (t.indptr[1:] - t.indptr[:-1]).long()) + base
            parts.append((t.indices.long(), rows, t.weights, t.delays, t.receptors))
        if not parts:
            raise ValueError("no synapses to join")
        tgt = torch.cat([p[0] for p in parts])
        order = torch.sort(tgt, stable=True).indices
        counts = torch.bincount(tgt, minlength=n_tgt)
        indptr = torch.zeros(n_tgt + 1, dtype=torch.int32, device=tgt.device)
        indptr[1:] = torch.cumsum(counts, 0).to(torch.int32)

        def col(k, dtype):
            return torch.cat([p[k] for p in parts])[order].to(dtype).contiguous()
        return SynapseTable(indptr, col(1, torch.int32), col(2, torch.float32), col(3, torch.uint8),
                            col(4, torch.uint8), n_rows=n_tgt, max_row=int(counts.max().item()))

    def blocked(self, n_cols, n_blocks):
        """The table regrouped by column range for the transposed propagation of the backward pass
        (``bmtk_glif3_bwd.blk_*`` of include/bmtk_amd.h): columns are cut into ``n_blocks`` equal ranges and the
        records are ordered by (range, row, position in the row).  Returns (indptr int32 [n_blocks*n_rows + 1],
        packed records in the new order followed by ``BLOCKED_PAD`` zero records, order int64 [nnz]: new position ->
        position in this table)."""
        dev = self.indices.device
        span = -(-n_cols // n_blocks)
        rows = torch.repeat_interleave(torch.arange(self.n_rows, device=dev),
                                       (self.indptr[1:] - self.indptr[:-1]).long())
        key = torch.div(self.indices.long(), span, rounding_mode="floor") * self.n_rows + rows
        order = torch.sort(key, stable=True).indices
        counts = torch.bincount(key, minlength=n_blocks * self.n_rows)
        indptr = torch.zeros(n_blocks * self.n_rows + 1, dtype=torch.int32, device=dev)
        indptr[1:] = torch.cumsum(counts, 0).to(torch.int32)
        packed = torch.zeros(self.nnz + BLOCKED_PAD, 2, dtype=torch.int32, device=dev)
        packed[:self.nnz] = self.packed()[:self.nnz][order]
        return indptr, packed, order

    def segment_offsets(self, span, n_groups):
        """uint32 [n_rows, n_groups+1] offsets of the first synapse per row whose index is >= g*span
        (stored in an int32 tensor).  Raises if a row is not sorted by index."""
        lib = _lib.load()
        seg = torch.empty(self.n_rows, n_groups + 1, dtype=torch.int32, device=self.indices.device)
        flag = torch.zeros(1, dtype=torch.int32, device=self.indices.device)
        _lib.check(lib.bmtk_csr_segment_offsets(self.n_rows, _p(self.indptr), _p(self.indices), span, n_groups,
                                                _p(seg), _p(flag), _stream()))
        if int(flag.item()):
            raise ValueError("synapse table rows are not sorted by index")
        return seg

    def pointers(self):
        nnz = self.nnz
        return (_p(self.indptr, torch.int32, self.n_rows + 1, "indptr"), _p(self.indices, torch.int32, nnz, "indices"),
                _p(self.weights, torch.float32, nnz, "weights"),
                _p(self.delays, torch.uint8, nnz, "delays") if self.delays.dtype == torch.uint8 else None,
                _p(self.receptors, torch.uint8, nnz, "receptors"))


def csr_propagate_scatter(active, n_active, table, ring, n_tgt, batch, step, max_active=None):
    """Event-driven delivery of the active element list through a source-major table."""
    lib = _lib.load()
    L = ring.shape[0]
    if ring.numel() != L * NREC * n_tgt * batch:
        raise ValueError("ring must be [L, 4, n_tgt*batch]")
    if max_active is None:
        max_active = active.numel()
    _lib.check(lib.bmtk_csr_propagate_scatter(
        _p(active, torch.int32, None, "active"), _p(n_active, torch.int32, 1, "n_active"), max_active, batch,
        *table.pointers(), _p(ring, torch.float32), L, n_tgt, int(step), _stream()))


def csr_propagate_gather(zbits, n_src, table, ring, n_tgt, batch, step):
    """Deterministic row-wise delivery through a target-major table from spike bits."""
    lib = _lib.load()
    L = ring.shape[0]
    if ring.numel() != L * NREC * n_tgt * batch:
        raise ValueError("ring must be [L, 4, n_tgt*batch]")
    if table.n_rows != n_tgt:
        raise ValueError("target-major table must have one row per target")
    _lib.check(lib.bmtk_csr_propagate_gather(
        _p(zbits, torch.int64, n_words(n_src * batch) + 1, "zbits"), n_src, batch, *table.pointers(),
        _p(ring, torch.float32), L, n_tgt, int(step), _stream()))


def csr_propagate_pull(spike_hist, n_src, table, syn, n_tgt, batch, t_arrive):
    """Everything arriving in step ``t_arrive`` from the spike bits of the last L steps
    (``spike_hist`` int64 [L, words+1], row k mod L = bits of step k) through a target-major table;
    overwrites ``syn`` [4, n_tgt*batch]."""
    lib = _lib.load()
    if table.n_rows != n_tgt or syn.numel() != NREC * n_tgt * batch:
        raise ValueError("target-major table must have one row per target and syn must be [4, n_tgt*batch]")
    L = spike_hist.shape[0]
    if table.max_delay() >= L:
        raise ValueError("spike history of {} steps is shorter than the largest delay".format(L))
    ws = getattr(table, "_pull_ws", None)
    need = lib.bmtk_csr_propagate_pull_workspace_bytes(L, n_src)
    if ws is None or ws.numel() * 4 < need:
        ws = table._pull_ws = torch.zeros(need // 4 + 1, dtype=torch.int32, device=syn.device)
    _lib.check(lib.bmtk_csr_propagate_pull(_p(spike_hist, torch.int64), spike_hist.shape[1], L, n_src, batch,
                                           _p(table.indptr), _p(table.packed()), _p(syn, torch.float32), n_tgt,
                                           int(t_arrive), _p(ws), _stream()))


def csr_propagate_pull2(spike_hist, n_src, table, syn2, n_tgt, batch, t_arrive):
    """Everything arriving in steps ``t_arrive - 1`` and ``t_arrive`` in one pass over a target-major table, from
    the spike bits of steps ``t_arrive - L .. t_arrive - 1`` (``spike_hist`` int64 [L, words+1], row k mod L = bits
    of step k); overwrites ``syn2`` [2, 4, n_tgt*batch]."""
    lib = _lib.load()
    if table.n_rows != n_tgt or syn2.numel() != 2 * NREC * n_tgt * batch:
        raise ValueError("target-major table must have one row per target and syn2 must be [2, 4, n_tgt*batch]")
    L = spike_hist.shape[0]
    if table.max_delay() >= L:
        raise ValueError("spike history of {} steps is shorter than the largest delay".format(L))
    ws = getattr(table, "_pull_ws", None)
    need = lib.bmtk_csr_propagate_pull_workspace_bytes(L, n_src)
    if ws is None or ws.numel() * 4 < need:
        ws = table._pull_ws = torch.zeros(need // 4 + 1, dtype=torch.int32, device=syn2.device)
    _lib.check(lib.bmtk_csr_propagate_pull2(_p(spike_hist, torch.int64), spike_hist.shape[1], L, n_src, batch,
                                            _p(table.indptr), _p(table.packed()), _p(syn2, torch.float32), n_tgt,
                                            int(t_arrive), _p(ws), _stream()))


def csr_propagate_bwd(table, lam_ring, n, batch, step, gz=None, trials_per_lane=0):
    """Transposed propagation (adjoint of the delivery) through a source-major table of ``n`` rows:
    ``gz[j*batch+b] = sum_(j->i,w,d,r) w * lam_ring[(step+d) % L, r, i*batch+b]``.  ``trials_per_lane`` 0 lets the
    library choose its kernel, 1 / 4 pick one (4 needs a batch that is a multiple of 4, at most 64)."""
    lib = _lib.load()
    L = lam_ring.shape[0]
    if table.n_rows != n or lam_ring.numel() != L * NREC * n * batch:
        raise ValueError("source-major table must have one row per neuron and lam_ring must be [L, 4, n*batch]")
    if table.max_delay() >= L:
        raise ValueError("adjoint ring of {} slots is shorter than the largest delay".format(L))
    if gz is None:
        gz = torch.empty(n * batch, device=lam_ring.device)
    _lib.check(lib.bmtk_csr_propagate_bwd(_p(table.indptr, torch.int32), _p(table.packed()), n, batch,
                                          _p(lam_ring, torch.float32), L, int(step),
                                          _p(gz, torch.float32, n * batch, "gz"), int(trials_per_lane), _stream()))
    return gz


def blocked_table_blocks(n, batch, ring_slots, slice_bytes=8 << 20):
    """Number of column ranges (a multiple of 8) that keeps one range's share of an adjoint ring
    [ring_slots, 4, n*batch] fp32 at about ``slice_bytes``.  The default, twice an XCD's 4 MB L2, is where the
    kernel was fastest at 52k neurons x 32 trials (16 to 32 ranges; three quarters of the reads hit the L2):
    fewer, longer row segments outweigh the better hit rate of smaller slices."""
    total = ring_slots * NREC * n * batch * 4
    return 8 * max(1, -(-total // (8 * slice_bytes)))


def csr_propagate_bwd_blocked(blk, n_blocks, lam_ring, n, batch, step, gz_parts=None):
    """Transposed propagation through the blocked form ``blk = table.blocked(n, n_blocks)`` of a source-major
    table: returns the eight partial sums ``gz_parts`` [8, n*batch]; their sum over the first axis is what
    ``csr_propagate_bwd`` returns (up to the order of the additions)."""
    lib = _lib.load()
    L = lam_ring.shape[0]
    indptr, packed = blk[0], blk[1]
    if indptr.numel() != n_blocks * n + 1 or lam_ring.numel() != L * NREC * n * batch:
        raise ValueError("blocked table must have n_blocks*n + 1 offsets and lam_ring must be [L, 4, n*batch]")
    if gz_parts is None:
        gz_parts = torch.empty(8, n * batch, device=lam_ring.device)
    _lib.check(lib.bmtk_csr_propagate_bwd_blocked(_p(indptr, torch.int32), _p(packed), n_blocks, n, batch,
                                                  _p(lam_ring, torch.float32), L, int(step),
                                                  _p(gz_parts, torch.float32, 8 * n * batch, "gz_parts"), _stream()))
    return gz_parts


def blocked_plan(n, batch):
    """Launch geometry of the blocked transposed propagation for ``n`` neurons at ``batch`` on the current device:
    dict(grid, rows_per_workgroup, sweeps, groups_per_wavefront) (``bmtk_csr_propagate_bwd_blocked_plan``)."""
    import ctypes
    lib = _lib.load()
    _dev()
    plan = (ctypes.c_int32 * 4)()
    _lib.check(lib.bmtk_csr_propagate_bwd_blocked_plan(n, batch, ctypes.cast(plan, ctypes.c_void_p)))
    return dict(grid=plan[0], rows_per_workgroup=plan[1], sweeps=plan[2], groups_per_wavefront=plan[3])


class AutoPropagator:
    """Step-by-step delivery with the form chosen on the device (``bmtk_csr_propagate_auto``): few spikes are pushed
    into the ring as events through the source-major table, many are left to the pull over the target-major table
    and the spike history.  Owns the workspace (activity map of the last L steps, record of the pushed steps).

    ``hist`` is the caller's spike history, int64 [L, words+1]: before ``step(k, ...)`` row k % L must hold the
    spike bits of step k.  After the call ring slot (k + 1) % L holds everything that arrives in step k + 1; the
    caller consumes and clears it before the next call.  Default threshold: where pushing costs what a pass costs
    on one MI355X -- an active element's row goes out at 2e10 events/s, a pass streams the packed table at 5 TB/s
    after 20 us of launches and set-up -- i.e. 0.032 n_src + 4e5 n_src / nnz active elements (2,000 at 52 k sources
    with 52 M synapses, where it was measured)."""

    def __init__(self, table_src, table_tgt, hist, ring, n_src, n_tgt, batch, scatter_max_active=None):
        self.lib = _lib.load()
        L = hist.shape[0]
        if ring.numel() != L * NREC * n_tgt * batch or table_tgt.n_rows != n_tgt or table_src.n_rows != n_src:
            raise ValueError("ring must be [L, 4, n_tgt*batch]; tables must have one row per source / per target")
        if table_tgt.max_delay() >= L:
            raise ValueError("spike history of {} steps is shorter than the largest delay".format(L))
        self.src, self.tgt, self.hist, self.ring = table_src, table_tgt, hist, ring
        self.L, self.n_src, self.n_tgt, self.batch = L, n_src, n_tgt, batch
        if scatter_max_active is None:
            scatter_max_active = max(1, int(0.032 * n_src + 4e5 * n_src / max(1, table_tgt.nnz)))
        self.scatter_max_active = int(scatter_max_active)
        need = self.lib.bmtk_csr_propagate_auto_workspace_bytes(L, n_src)
        self.workspace = torch.zeros(need // 4 + 1, dtype=torch.int32, device=ring.device)

    def step(self, k, active, n_active, max_active=None):
        if max_active is None:
            max_active = active.numel()
        _lib.check(self.lib.bmtk_csr_propagate_auto(
            _p(active, torch.int32, None, "active"), _p(n_active, torch.int32, 1, "n_active"), max_active,
            _p(self.hist, torch.int64), self.hist.shape[1], self.L, self.n_src, self.batch, *self.src.pointers(),
            _p(self.tgt.indptr), _p(self.tgt.packed()), _p(self.ring, torch.float32), self.n_tgt, int(k),
            self.scatter_max_active, _p(self.workspace), _stream()))

    def pulled_steps(self):
        """Which of the history rows are left to the pull kernel (bool [L]; synchronises) -- for tests and
        profiles."""
        n_w32 = (self.n_src + 31) // 32
        return self.workspace[self.L * n_w32:self.L * n_w32 + self.L].cpu().numpy() != 0


class AutoPropagator2(AutoPropagator):
    """``AutoPropagator`` for a caller that advances two steps between calls (``bmtk_csr_propagate_auto2``): each of
    the two new steps is pushed or left to the pull by its own count, and the pull sums the arrivals of two steps in
    one pass over the table.  Before ``step2(k, ...)`` rows (k - 1) % L and k % L of ``hist`` must hold the spike
    bits of steps k - 1 and k; after it ring slots k % L and (k + 1) % L hold everything that arrives in steps k
    and k + 1, and the caller consumes and clears both before the next call (k + 2).  Histories of at most 8
    rows.  Default threshold: half the one-step form's, 0.016 n_src + 2.4e5 n_src / nnz active elements per step
    (1,070 at 52 k sources with 52 M synapses)."""

    def __init__(self, table_src, table_tgt, hist, ring, n_src, n_tgt, batch, scatter_max_active=None):
        if scatter_max_active is None:   # a step's share of a pass is half of what the one-step form pays
            scatter_max_active = max(1, int(0.016 * n_src + 2.4e5 * n_src / max(1, table_tgt.nnz)))
        AutoPropagator.__init__(self, table_src, table_tgt, hist, ring, n_src, n_tgt, batch, scatter_max_active)
        if self.L > 8:
            raise ValueError("the two-step form takes histories of at most 8 rows")
        need = self.lib.bmtk_csr_propagate_auto2_workspace_bytes(self.L, n_src)
        self.workspace = torch.zeros(need // 4 + 1, dtype=torch.int32, device=ring.device)

    def step(self, k, active, n_active, max_active=None):
        raise TypeError("the two-step form is advanced with step2")

    def step2(self, k, active_a, n_active_a, active_b, n_active_b, max_active=None):
        if max_active is None:
            max_active = max(active_a.numel(), active_b.numel())
        _lib.check(self.lib.bmtk_csr_propagate_auto2(
            _p(active_a, torch.int32, None, "active_a"), _p(n_active_a, torch.int32, 1, "n_active_a"),
            _p(active_b, torch.int32, None, "active_b"), _p(n_active_b, torch.int32, 1, "n_active_b"), max_active,
            _p(self.hist, torch.int64), self.hist.shape[1], self.L, self.n_src, self.batch, *self.src.pointers(),
            _p(self.tgt.indptr), _p(self.tgt.packed()), _p(self.ring, torch.float32), self.n_tgt, int(k),
            self.scatter_max_active, _p(self.workspace), _stream()))

    def pulled_steps(self):
        return self.workspace[:self.L].cpu().numpy() != 0


def csr_propagate_fwd(mode, table, ring, n_tgt, batch, step, active=None, n_active=None, zbits=None, n_src=None):
    """``mode`` "scatter" (source-major table + active list) or "gather" (target-major table + spike bits); the
    form chosen on the device needs state from step to step, see ``AutoPropagator``."""
    if mode == "scatter":
        return csr_propagate_scatter(active, n_active, table, ring, n_tgt, batch, step)
    if mode == "gather":
        return csr_propagate_gather(zbits, n_src, table, ring, n_tgt, batch, step)
    raise ValueError("mode must be 'scatter' or 'gather'")


def poisson_events(n_sources, rate_hz, dt_ms, n_steps, batch=1, seed=1, t_start_ms=0.0, t_stop_ms=None,
                   return_times=False, device=None):
    """Homogeneous Poisson spike sources generated on the device (exponential inter-spike intervals per source and
    trial, as bmtk's ``PoissonSpikeGenerator`` draws them, bmtk/utils/reports/spike_trains/spike_trains.py:166-206;
    independent streams instead of NumPy's global one) as the per-step event lists a simulation reads:
    ``(in_ptr int64[n_steps+1], in_events int32[])``, ids = source*batch + trial ascending within each step; a
    source that fires twice inside one step appears twice.  ``rate_hz``: scalar or one rate per source.
    ``return_times`` adds ``(step int64[], element int64[], time_ms float64[])`` of every spike, in event order.
    Nothing passes through host memory."""
    lib = _lib.load()
    dev = device or _dev()
    rates = torch.as_tensor(np.broadcast_to(np.asarray(rate_hz, np.float32), (n_sources,)).copy(), device=dev)
    if bool((rates < 0).any()):
        raise ValueError("Firing rates must not be negative.")
    t_stop_ms = n_steps * dt_ms if t_stop_ms is None else t_stop_ms
    n_ids = n_sources * batch
    counts = torch.zeros(n_ids, dtype=torch.int32, device=dev)
    args = (n_sources, batch, _p(rates), float(t_start_ms), float(t_stop_ms), float(dt_ms), int(n_steps),
            int(seed) & (2 ** 64 - 1))
    _lib.check(lib.bmtk_poisson_count(*args, _p(counts), _stream()))
    offsets = torch.zeros(n_ids + 1, dtype=torch.int64, device=dev)
    offsets[1:] = torch.cumsum(counts, 0)
    total = int(offsets[-1].item())
    keys = torch.empty(max(total, 1), dtype=torch.int64, device=dev)
    times = torch.empty(max(total, 1), dtype=torch.float64, device=dev) if return_times else None
    _lib.check(lib.bmtk_poisson_fill(*args, _p(offsets), _p(keys), _p(times), _stream()))
    keys = keys[:total]
    order = torch.sort(keys, stable=True).indices if return_times else None
    keys = keys[order] if return_times else torch.sort(keys).values
    steps = keys // n_ids
    in_ptr = torch.searchsorted(steps, torch.arange(n_steps + 1, device=dev, dtype=torch.int64)).to(torch.int64)
    in_events = (keys - steps * n_ids).to(torch.int32)
    if return_times:
        return in_ptr, in_events, (steps, in_events.to(torch.int64), times[:total][order])
    return in_ptr, in_events


def unpack_bits(bits, ne):
    """int64 spike-bit words ``[..., words]`` -> uint8 flags ``[..., ne]`` (host or device)."""
    shifts = torch.arange(64, device=bits.device, dtype=torch.int64)
    flags = ((bits.unsqueeze(-1) >> shifts) & 1).to(torch.uint8)
    return flags.reshape(*bits.shape[:-1], bits.shape[-1] * 64)[..., :ne]
