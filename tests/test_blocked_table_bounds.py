"""How far past a row's end the blocked transposed propagation reads its table (host model, no GPU).

``bwd_gather_blocked_kernel`` (bmtk_amd/csrc/backward.hip) lets the lane groups of a wavefront walk their rows'
segments side by side, ``kBlkInFlight`` records at a time with the next ``kBlkInFlight`` fetched ahead, until the
longest segment of the visit is done; lane groups whose segment has ended stay at its end (``p = min(p + kF, p1)``).
The contract of ``include/bmtk_amd.h`` gives the table ``BMTK_BLOCKED_PAD`` readable records after its last one.
This walks the same index sequence on the host for tables whose last rows are much shorter than their neighbours
(the case in which lanes that have finished keep fetching while others work) and checks the largest index read."""
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _constants():
    src = open(os.path.join(ROOT, "bmtk_amd", "csrc", "backward.hip")).read()
    hdr = open(os.path.join(ROOT, "include", "bmtk_amd.h")).read()
    k_f = int(re.search(r"constexpr int kBlkInFlight = (\d+);", src).group(1))
    pad = int(re.search(r"#define BMTK_BLOCKED_PAD (\d+)", hdr).group(1))
    assert "p = min(p + kF, p1);" in src          # the rule this model follows
    return k_f, pad


def _largest_index_read(seg_lo, seg_hi, k_f, clamp=True):
    """One visit: lane groups with segments [seg_lo[g], seg_hi[g]) side by side.  Every turn reads records
    [p, p + kF) and fetches [p + kF, p + 2 kF) ahead, for every lane group, while any group has records left."""
    p = np.array(seg_lo, np.int64)
    p1 = np.array(seg_hi, np.int64)
    largest = -1
    while np.any(p < p1):
        largest = max(largest, int((p + 2 * k_f - 1).max()))
        p = np.minimum(p + k_f, p1) if clamp else p + k_f
    return largest


@pytest.mark.parametrize("lengths", [[400, 380, 1, 390, 2, 0, 0, 3], [64, 64, 64, 64, 64, 64, 64, 1], [1] * 8,
                                     [1000, 0, 0, 0, 0, 0, 0, 1], [17, 9, 8, 7, 16, 15, 1, 2]])
def test_reads_stay_within_the_pad_when_the_last_rows_are_short(lengths):
    k_f, pad = _constants()
    # the visit's rows are the LAST rows of the table: the segments end at nnz, the short ones last
    order = np.argsort(-np.array(lengths), kind="stable")
    lo = np.zeros(len(lengths), np.int64)
    hi = np.zeros(len(lengths), np.int64)
    at = 0
    for g in order:                       # long rows first in memory, so that the short last row ends the table
        lo[g], hi[g] = at, at + lengths[g]
        at += lengths[g]
    nnz = at
    assert _largest_index_read(lo, hi, k_f) < nnz + pad
    # without the clamp a finished lane group keeps advancing with the longest one and leaves the pad
    if max(lengths) > min(lengths) + 3 * k_f and lengths[int(order[-1])] < max(lengths) - 3 * k_f:
        assert _largest_index_read(lo, hi, k_f, clamp=False) >= nnz + pad


def test_pad_covers_two_fetches_past_any_row_end():
    k_f, pad = _constants()
    assert pad >= 2 * k_f
    rng = np.random.default_rng(0)
    for _ in range(200):
        lengths = rng.integers(0, 300, 8)
        lo = np.concatenate([[0], np.cumsum(lengths)[:-1]])
        hi = np.cumsum(lengths)
        if hi[-1] == 0:
            continue
        assert _largest_index_read(lo, hi, k_f) <= hi.max() + 2 * k_f - 1
