"""The compaction entry point that allocates nothing (``bmtk_spikes_compact_noalloc``: workspace inside the
library) against ``bmtk_spikes_compact`` with a caller's workspace: bit-exact ids and count, on calls in a row that
share the built-in workspace, the later ones smaller than the first."""
import numpy as np
import pytest
import torch

from bmtk_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _both(z):
    n = z.numel()
    ids = torch.full((n,), -7, dtype=torch.int32, device=z.device)
    count = torch.full((1,), -7, dtype=torch.int32, device=z.device)
    ops.spikes_compact_noalloc(z, ids, count)
    want_ids, want_count = ops.SpikeCompactor(n)(z)
    c = int(count.item())
    assert c == int(want_count.item())
    assert torch.equal(ids[:c], want_ids[:c])
    assert bool((ids[c:] == -7).all())          # nothing written past the count
    return c


def test_noalloc_compaction_equals_the_workspace_form_on_calls_in_a_row():
    g = torch.Generator(device="cuda").manual_seed(11)
    sizes = [(3_326_592, 5e-3), (1_000_003, 0.3), (65, 1.0), (64, 0.0), (1, 1.0), (2_000_000, 1e-4)]
    total = 0
    for n, p in sizes:                           # the second and later calls are smaller than the first
        z = (torch.rand(n, device="cuda", generator=g) < p).to(torch.uint8) if p < 1.0 else \
            torch.ones(n, dtype=torch.uint8, device="cuda")
        total += _both(z)
        np.testing.assert_array_equal(np.flatnonzero(z.cpu().numpy()).size, int(z.sum().item()))
    assert total > 300_000
    # the same large input again after the small ones: what they left in the workspace must not matter
    z = (torch.rand(sizes[0][0], device="cuda", generator=g) < 0.02).to(torch.uint8)
    c = _both(z)
    assert c == int(z.sum().item())
    # non-zero flags other than 1 and flags off a 16-byte boundary take the other packing kernel
    z = (torch.rand(100_001, device="cuda", generator=g) < 0.05).to(torch.uint8) * 200
    _both(z[3:])


def test_noalloc_compaction_at_its_limit_and_beyond():
    n = _lib.COMPACT_NOALLOC_MAX_N
    z = torch.zeros(n, dtype=torch.uint8, device="cuda")
    hot = torch.tensor([0, 63, 64, n // 2 + 1, n - 1], device="cuda")
    z[hot] = 1
    ids = torch.empty(n, dtype=torch.int32, device="cuda")
    count = torch.zeros(1, dtype=torch.int32, device="cuda")
    ops.spikes_compact_noalloc(z, ids, count)
    assert int(count.item()) == 5 and torch.equal(ids[:5].long(), hot)
    big = torch.zeros(n + 1, dtype=torch.uint8, device="cuda")
    with pytest.raises(_lib.BmtkAmdError, match="exceeds"):
        ops.spikes_compact_noalloc(big, torch.empty(n + 1, dtype=torch.int32, device="cuda"), count)


def test_noalloc_compaction_allocates_no_device_memory():
    """torch's allocator statistics do not move across the call (the library itself calls no allocator: its
    workspace is a device array of the code object)."""
    z = (torch.rand(500_000, device="cuda") < 0.01).to(torch.uint8)
    ids = torch.empty(500_000, dtype=torch.int32, device="cuda")
    count = torch.zeros(1, dtype=torch.int32, device="cuda")
    ops.spikes_compact_noalloc(z, ids, count)    # first call on the device: looks up the workspace address
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    for _ in range(3):
        ops.spikes_compact_noalloc(z, ids, count)
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    assert torch.cuda.mem_get_info()[0] == free0
    assert int(count.item()) == int(z.sum().item())
