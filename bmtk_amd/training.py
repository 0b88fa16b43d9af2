"""Backward pass (BPTT) through the GLIF3 simulation on the GPU.

bmtk has no gradient code; the definition of the differentiable model is this
package's own and is stated in ``include/bmtk_amd.h`` (``bmtk_glif3_bwd``):
triangular surrogate spike derivative, refractory bookkeeping not
differentiated, everything else the exact transpose of the forward update.
"""
import ctypes as C

import numpy as np
import torch

from . import _lib
from .layout import NASC, NREC
from .ops import _p, _stream


def spike_counts(bits, ne):
    """int32 [ne] spikes per element over all rows of ``bits`` (int64 [n_steps, words])."""
    lib = _lib.load()
    counts = torch.empty(ne, dtype=torch.int32, device=bits.device)
    _lib.check(lib.bmtk_spike_counts(_p(bits, torch.int64), bits.shape[1], bits.shape[0], ne, _p(counts), _stream()))
    return counts


def rate_mse(counts, n_steps, batch, pop_id, targets):
    """MSE between population rates and targets, and its derivative per spike.

    counts  int32 [n*batch] spikes per element; pop_id int64 [n] population of
    every neuron; targets float [batch, n_pops] in spikes per neuron per step.
    The rate of population p in trial b is mean over its neurons and steps of z.
    Returns (loss, dl_dz_const float32 [n*batch])."""
    dev = counts.device
    n = pop_id.numel()
    n_pops = targets.shape[1]
    size = torch.bincount(pop_id, minlength=n_pops).to(torch.float32)
    c = counts.view(n, batch).to(torch.float32)
    rate = torch.zeros(n_pops, batch, device=dev).index_add_(0, pop_id, c) / (size.view(-1, 1) * n_steps)
    err = rate.t() - targets
    loss = (err * err).mean()
    # d loss / d z[b, i, t] = 2 err[b, p(i)] / (batch * n_pops) / (size[p(i)] * n_steps)
    g = 2.0 * err / (batch * n_pops) / (size.view(1, -1) * n_steps)
    return loss, g.t()[pop_id].contiguous().view(-1)


class Glif3Bptt:
    """Reverse-time adjoint over a recorded forward run of a ``Glif3Simulator``
    built with ``resident=False``."""

    # adjoint rings above this size use the table regrouped by target range (the ring no longer fits the L2s)
    BLOCKED_MIN_RING_BYTES = 32 << 20

    def __init__(self, sim, dampening=0.3, blocked=None, n_blocks=None, two_steps=True):
        """``blocked``: use the recurrent table regrouped by target range for the transposed propagation (None:
        when the adjoint ring exceeds ``BLOCKED_MIN_RING_BYTES`` and the batch allows it); ``n_blocks``: number of
        target ranges, a multiple of 8 (None: ``ops.blocked_table_blocks``); ``two_steps``: let the blocked form take
        two steps per pass over its table (batches above 16; ``gz`` then holds the partial sums of both)."""
        if sim.res_span or sim.delay_offset:
            raise ValueError("the backward pass needs a simulator built with resident=False and delay_offset 0")
        self.sim, self.dampening = sim, float(dampening)
        self.lib = _lib.load()
        dev, ne = sim.dev, sim.ne
        self.lam_V = torch.zeros(ne, device=dev)
        self.lam_asc = torch.zeros(NASC, ne, device=dev)
        self.lam_y1 = torch.zeros(NREC, ne, device=dev)
        self.lam_y2 = torch.zeros(NREC, ne, device=dev)
        self.lam_ring = torch.zeros(sim.L, NREC, ne, device=dev)
        self.d_rec_w = torch.zeros(sim.rec.nnz, device=dev) if sim.rec is not None else None
        can_block = sim.rec is not None and sim.batch % 4 == 0 and sim.batch <= 64 and sim.L * NREC * ne < (1 << 30)
        if blocked is None:
            blocked = can_block and sim.L * NREC * ne * 4 > self.BLOCKED_MIN_RING_BYTES
        elif blocked and not can_block:
            raise ValueError("the blocked table needs a recurrent table and a batch that is a multiple of 4 up to 64")
        self.blk = None
        if blocked:
            from . import ops
            self.n_blocks = int(n_blocks or ops.blocked_table_blocks(sim.n, sim.batch, sim.L))
            if self.n_blocks % 8:
                raise ValueError("n_blocks must be a multiple of 8")
            self.blk = sim.rec.blocked(sim.n, self.n_blocks)
            self.d_blk_w = torch.zeros(sim.rec.nnz, device=dev)
        # the blocked form takes two steps per pass over its table when gz has room for both steps' partial sums
        self.gz_planes = (16 if two_steps else 8) if blocked else 1
        self.gz = torch.zeros(self.gz_planes * ne, device=dev)
        self.d_inp_w = torch.zeros(sim.inp.nnz, device=dev) if sim.inp is not None and sim.in_ptr is not None else None

    def zero(self):
        for t in (self.lam_V, self.lam_asc, self.lam_y1, self.lam_y2, self.lam_ring, self.gz, self.d_rec_w, self.d_inp_w):
            if t is not None:
                t.zero_()

    def _struct(self, fwd, dl_dz_const, dl_dz, blocked):
        sim, saved, bits = self.sim, fwd["saved"], fwd["bits"]
        if saved is None or bits is None:
            raise ValueError("forward run was made without save_state=True or without spike bits")
        n_steps = bits.shape[0]
        a = _lib.Glif3Bwd()
        a.n_neurons, a.batch, a.ring_slots, a.h, a.dampening = sim.n, sim.batch, sim.L, sim.h, self.dampening
        a.prop, a.prop_stride, a.class_id = _p(sim.prop), sim.prop.shape[1], _p(sim.class_id)
        a.save_v, a.save_flags = _p(saved["v"], torch.float32, n_steps * sim.ne), _p(saved["flags"], torch.uint8)
        a.spike_bits, a.spike_bits_stride = _p(bits, torch.int64), bits.shape[1]
        if sim.rec is not None:
            a.rec_indptr, a.rec_packed = _p(sim.rec.indptr), _p(sim.rec.packed())
            if not blocked:
                a.d_rec_w = _p(self.d_rec_w)
            else:
                a.blk_count, a.blk_indptr, a.blk_packed = self.n_blocks, _p(self.blk[0]), _p(self.blk[1])
                a.gz_planes = self.gz_planes
                a.d_blk_w = _p(self.d_blk_w)
        if self.d_inp_w is not None:
            a.in_ptr, a.in_events = _p(sim.in_ptr), _p(sim.in_events)
            a.inp_indptr, a.inp_packed = _p(sim.inp.indptr), _p(sim.inp.packed())
            a.d_inp_w = _p(self.d_inp_w)
        a.dl_dz = _p(dl_dz, torch.float32, n_steps * sim.ne, "dl_dz")
        a.dl_dz_const = _p(dl_dz_const, torch.float32, sim.ne, "dl_dz_const")
        a.lam_V, a.lam_asc, a.lam_y1, a.lam_y2 = (_p(x) for x in (self.lam_V, self.lam_asc, self.lam_y1, self.lam_y2))
        a.lam_ring, a.gz = _p(self.lam_ring), _p(self.gz)
        return a, saved["step0"], n_steps

    def backward(self, fwd, dl_dz_const=None, dl_dz=None):
        """``fwd`` is what ``sim.run(n, save_state=True)`` returned.  Accumulates
        into ``d_rec_w`` / ``d_inp_w`` (same order as ``sim.rec`` / ``sim.inp``).
        Calls for consecutive chunks must come in reverse time order."""
        a, step0, n_steps = self._struct(fwd, dl_dz_const, dl_dz, self.blk is not None)
        _lib.check(self.lib.bmtk_glif3_simulate_bwd(C.byref(a), step0, n_steps, _stream()))
        if self.blk is not None:  # the blocked kernel accumulates in its table's order: back to the order of sim.rec
            self.d_rec_w.index_add_(0, self.blk[2], self.d_blk_w)
            self.d_blk_w.zero_()

    def backward_stepwise(self, fwd, dl_dz_const=None, dl_dz=None, between=None):
        """The same pass as a loop over the three per-step entry points (transposed propagation through the
        source-major table, state adjoint, weight gradients), calling ``between(k)`` after the state adjoint of
        record row ``k`` -- the place for work of the caller's own on the adjoint state (clipping, a loss that
        depends on it).  Several launches per step where ``backward`` has two: for training loops use ``backward``."""
        from . import ops
        sim = self.sim
        a, step0, n_steps = self._struct(fwd, dl_dz_const, dl_dz, False)
        gz = self.gz[:sim.ne]
        for k in range(n_steps - 1, -1, -1):
            if sim.rec is not None:
                ops.csr_propagate_bwd(sim.rec, self.lam_ring, sim.n, sim.batch, step0 + k, gz=gz)
            else:
                gz.zero_()
            _lib.check(self.lib.bmtk_glif3_step_bwd(C.byref(a), step0, k, 1, _stream()))
            if self.d_rec_w is not None or self.d_inp_w is not None:
                _lib.check(self.lib.bmtk_csr_weight_grad(C.byref(a), step0, k, _stream()))
            if between is not None:
                between(k)
