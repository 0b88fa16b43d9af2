"""Host-side assembly of the synapse tables the kernels read.

A synapse table is the tuple ``(indptr int32[n_rows+1], indices int32[nnz],
weights float32[nnz], delays uint8[nnz] (steps, >= 1), receptors uint8[nnz]
(0-based))``.  "source-major" rows are presynaptic neurons and ``indices``
holds targets (the form event-driven delivery walks); "target-major" rows are
postsynaptic neurons and ``indices`` holds sources (the order SONATA edge
files are written in, bmtk/builder/network_adaptors/dm_network.py:257-258).

``syn_spec_to_arrays`` applies the rules bmtk and NEST apply when an edge
batch is connected (bmtk/simulator/pointnet/sonata_adaptors.py:268-357,
bmtk/simulator/pointnet/pointnetwork.py:161-173,229-248).
"""
import numpy as np

from .layout import NREC


class BadDelay(ValueError):
    """Delay shorter than the resolution (NEST's ``BadDelay``, which bmtk
    special-cases in bmtk/simulator/pointnet/pointnetwork.py:234-243)."""


def edge_weights(nsyns, syn_weight):
    """``weight = nsyns * syn_weight`` (bmtk/simulator/pointnet/sonata_adaptors.py:338-354);
    a missing ``syn_weight`` is an error there too."""
    if syn_weight is None:
        raise Exception("Could not find syn_weight value")
    return np.asarray(nsyns if nsyns is not None else 1) * np.asarray(syn_weight)


def syn_spec_to_arrays(n_edges, syn_spec, dt):
    """NEST ``syn_spec`` dict -> (weights f32, delay steps u8 (int32 beyond 255), receptor u8 0-based).

    Scalars are broadcast over the batch; ``receptor_type`` is 1-based as in
    NEST; a delay below the resolution raises ``BadDelay``; delays are rounded
    to the nearest step as NEST does."""
    w = np.broadcast_to(np.asarray(syn_spec["weight"], np.float64), (n_edges,))
    delay_ms = np.broadcast_to(np.asarray(syn_spec.get("delay", 1.0), np.float64), (n_edges,))
    if np.any(delay_ms < dt * (1.0 - 1e-12)):
        raise BadDelay("synaptic \"delay\" value in edges ({}) is not compatible with simulator "
                       "resolution/\"dt\" ({})".format(np.min(delay_ms), dt))
    steps = np.rint(delay_ms / dt).astype(np.int64)
    rec = int(syn_spec.get("receptor_type", 1))
    if rec < 1 or rec > NREC:
        raise ValueError("receptor_type {} outside 1..{}".format(rec, NREC))
    steps = steps.astype(np.uint8 if (steps.size == 0 or steps.max() <= 255) else np.int32)
    return (w.astype(np.float32), steps, np.full(n_edges, rec - 1, np.uint8))


def coo_to_csr(src, tgt, w, d, r, n_rows, major="source"):
    """Edge list -> synapse table, rows ordered by (row, column, original position)."""
    src = np.asarray(src, np.int64)
    tgt = np.asarray(tgt, np.int64)
    row, col = (src, tgt) if major == "source" else (tgt, src)
    if row.size and (row.min() < 0 or row.max() >= n_rows):
        raise ValueError("row id outside 0..{}".format(n_rows - 1))
    order = np.lexsort((np.arange(row.size), col, row))
    indptr = np.zeros(n_rows + 1, np.int64)
    np.add.at(indptr, row + 1, 1)
    indptr = np.cumsum(indptr)
    if indptr[-1] >= 2 ** 31:
        raise ValueError("more than 2^31-1 synapses in one table")
    d = np.asarray(d)
    d = d.astype(np.uint8 if (d.size == 0 or d.max() <= 255) else np.int32)  # long delays keep a wide column
    return (indptr.astype(np.int32), col[order].astype(np.int32), np.asarray(w, np.float32)[order],
            d[order], np.asarray(r, np.uint8)[order])


def csr_rows(indptr):
    """Row id of every stored synapse."""
    return np.repeat(np.arange(indptr.size - 1, dtype=np.int32), np.diff(indptr))


def csr_transpose(csr, n_cols):
    """source-major <-> target-major, keeping the (row, column, position) order."""
    indptr, indices, w, d, r = csr
    rows = csr_rows(indptr)
    order = np.argsort(indices, kind="stable")
    new_ptr = np.zeros(n_cols + 1, np.int64)
    np.add.at(new_ptr, indices.astype(np.int64) + 1, 1)
    return (np.cumsum(new_ptr).astype(np.int32), rows[order], w[order], d[order], r[order])


def check_csr(csr, n_rows, n_cols, ring_slots):
    """Host-side validation run before any kernel sees a table: shapes,
    monotone indptr, index range, delay range.  Kernels index with these
    values unchecked, so a table that fails here must never be launched on."""
    indptr, indices, w, d, r = csr
    nnz = int(indptr[-1])
    if indptr.size != n_rows + 1 or indptr[0] != 0 or np.any(np.diff(indptr) < 0):
        raise ValueError("indptr must be non-decreasing, start at 0 and have n_rows+1 entries")
    for name, a in (("indices", indices), ("weights", w), ("delays", d), ("receptors", r)):
        if a.size != nnz:
            raise ValueError("{} has {} entries, indptr says {}".format(name, a.size, nnz))
    if nnz:
        if indices.min() < 0 or indices.max() >= n_cols:
            raise ValueError("index outside 0..{}".format(n_cols - 1))
        if d.min() < 1 or d.max() >= ring_slots:
            raise ValueError("delays must lie in 1..{} steps for a ring of {} slots".format(ring_slots - 1, ring_slots))
        if r.max() >= NREC:
            raise ValueError("receptor outside 0..{}".format(NREC - 1))


def check_input_events(in_ptr, in_events, n_ids):
    """Host-side validation of per-step input event lists (``in_events[in_ptr[t]:in_ptr[t+1]]`` are the
    element ids source*batch+trial emitted in step t): ``in_ptr`` non-decreasing from 0 to the number of
    events, ids within 0..n_ids-1 and ascending within every step (the input-weight gradient kernel gives a
    source's run of events one writer and relies on the order).  Returns True when some id occurs more than
    once within a step -- two spikes of one generator inside one resolution step, which NEST delivers both;
    the pull form of the inputs then needs the repeats listed apart (Glif3Simulator.set_input_events)."""
    in_ptr = np.asarray(in_ptr)
    in_events = np.asarray(in_events)
    if in_ptr.size < 1 or in_ptr[0] != 0 or np.any(np.diff(in_ptr) < 0) or in_ptr[-1] != in_events.size:
        raise ValueError("in_ptr must be non-decreasing from 0 to len(in_events)")
    if in_events.size and (in_events.min() < 0 or in_events.max() >= n_ids):
        raise ValueError("input event id outside 0..n_inputs*batch-1")
    if in_events.size < 2:
        return False
    step_start = np.zeros(in_events.size + 1, bool)
    step_start[in_ptr] = True                 # an event that opens a step may be smaller than the one before it
    d = np.diff(in_events.astype(np.int64))
    inside = ~step_start[1:-1]
    if np.any((d < 0) & inside):
        raise ValueError("input events must be ascending within every step")
    return bool(np.any((d == 0) & inside))
