"""GPU parity of spike compaction and of the two delivery kernels."""
import numpy as np
import pytest
import torch

from oracle import glif3_oracle as orc
from bmtk_amd import network as net, ops
from gpu_util import bits_of, rel_err, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n", [1, 63, 64, 65, 1000, 16384, 16385, (1 << 20) + 3])
@pytest.mark.parametrize("p", [0.0, 0.003, 0.3, 1.0])
def test_compaction_is_flatnonzero(n, p):
    rng = np.random.default_rng(n % 1000 + int(p * 1000))
    z = (rng.random(n) < p).astype(np.uint8) if p < 1.0 else np.ones(n, np.uint8)
    want = np.flatnonzero(z).astype(np.int32)
    comp = ops.SpikeCompactor(n)
    for src in (to_dev(z), to_dev(bits_of(z))):
        ids, count = comp(src)
        c = int(count.item())
        assert c == want.size
        np.testing.assert_array_equal(ids[:c].cpu().numpy(), want)


def test_compaction_other_paths():
    """Flags that do not start on a 16-byte boundary (the packing then goes through the one-flag-per-thread kernel),
    non-zero flags other than 1, and an input beyond the size the fused two-launch form takes."""
    rng = np.random.default_rng(77)
    z = (rng.random(100_001) < 0.01).astype(np.uint8) * rng.integers(1, 256, 100_001).astype(np.uint8)
    dev = to_dev(z)
    for off in (1, 5, 16):
        comp = ops.SpikeCompactor(z.size - off)
        ids, count = comp(dev[off:])
        want = np.flatnonzero(z[off:]).astype(np.int32)
        assert int(count.item()) == want.size
        np.testing.assert_array_equal(ids[:want.size].cpu().numpy(), want)
    n = (1 << 26) + 5
    big = torch.zeros(n, dtype=torch.uint8, device=dev.device)
    hot = torch.as_tensor(np.sort(rng.choice(n, 50_000, replace=False)), device=dev.device)
    big[hot] = 1
    ids, count = ops.SpikeCompactor(n)(big)
    assert int(count.item()) == 50_000 and torch.equal(ids[:50_000].long(), hot)


def test_compaction_ignores_bits_beyond_n():
    z = np.zeros(100, np.uint8)
    z[[3, 99]] = 1
    bits = bits_of(z).copy()
    bits[1] |= np.int64(-1) << 40          # garbage above element 100 in the last word
    comp = ops.SpikeCompactor(100)
    ids, count = comp(to_dev(bits))
    assert ids[:int(count.item())].cpu().tolist() == [3, 99]


def _edges(rng, n_src, n_tgt, nnz, max_delay=5):
    src = rng.integers(0, n_src, nnz).astype(np.int32)
    tgt = rng.integers(0, n_tgt, nnz).astype(np.int32)
    w = (rng.lognormal(0, 1, nnz) * rng.choice([-1, 1], nnz)).astype(np.float32)
    d = rng.integers(1, max_delay + 1, nnz).astype(np.uint8)
    r = rng.integers(0, 4, nnz).astype(np.uint8)
    return src, tgt, w, d, r


@pytest.mark.parametrize("batch,p", [(1, 0.05), (1, 1.0), (5, 0.2), (64, 0.02), (100, 0.1)])
def test_scatter_matches_oracle(batch, p):
    """fp32 atomics add in an arbitrary order, so the comparison is against the
    fp64 oracle: |diff| <= 1e-5 * max(|want|, sum of |w| into the cell * 1e-2)
    -- the floor is the magnitude rounding errors scale with when signed
    weights cancel."""
    rng = np.random.default_rng(30)
    n_src, n_tgt, L = 300, 257, 6
    src, tgt, w, d, r = _edges(rng, n_src, n_tgt, 20000)
    csr = net.coo_to_csr(src, tgt, w, d, r, n_rows=n_src, major="source")
    table = ops.SynapseTable.from_numpy(csr)
    ring_d = torch.zeros(L, 4, n_tgt * batch, device="cuda")
    ring_c = np.zeros((L, 4, n_tgt * batch))
    mag_c = np.zeros((L, 4, n_tgt * batch))
    csr_abs = (csr[0], csr[1], np.abs(csr[2]), csr[3], csr[4])
    comp = ops.SpikeCompactor(n_src * batch)
    for step in (0, 4, 11):
        z = (rng.random(n_src * batch) < p).astype(np.uint8)
        ids, count = comp(to_dev(z))
        ops.csr_propagate_scatter(ids, count, table, ring_d, n_tgt, batch, step)
        orc.deliver_events(np.flatnonzero(z), batch, csr, ring_c, n_tgt, step)
        orc.deliver_events(np.flatnonzero(z), batch, csr_abs, mag_c, n_tgt, step)
    got = ring_d.cpu().numpy()
    assert np.abs(ring_c).max() > 0
    assert np.max(np.abs(got - ring_c) / np.maximum(np.abs(ring_c), 1e-2 * mag_c + 1e-30)) < 1e-5
    assert np.all(got[mag_c == 0] == 0)


@pytest.mark.parametrize("batch,p", [(1, 0.1), (5, 0.2), (32, 0.05), (64, 0.02), (64, 0.6), (100, 0.1), (130, 0.05)])
def test_gather_bit_exact_vs_fp32_oracle(batch, p):
    """Each ring cell is updated by one wavefront in stored synapse order
    starting from the value already there: identical to the scalar fp32 loop,
    including on a ring that already holds values."""
    rng = np.random.default_rng(31)
    n_src, n_tgt, L = 211, 190, 6
    src, tgt, w, d, r = _edges(rng, n_src, n_tgt, 15000)
    csr = net.coo_to_csr(src, tgt, w, d, r, n_rows=n_tgt, major="target")
    table = ops.SynapseTable.from_numpy(csr)
    ring_c = rng.normal(0, 1, (L, 4, n_tgt * batch)).astype(np.float32)
    ring_d = to_dev(ring_c)
    for step in (0, 5, 9):
        z = (rng.random(n_src * batch) < p).astype(np.uint8)
        ops.csr_propagate_gather(to_dev(bits_of(z)), n_src, table, ring_d, n_tgt, batch, step)
        orc.gather_rows(z, batch, csr, ring_c, n_tgt, step)
        np.testing.assert_array_equal(ring_d.cpu().numpy(), ring_c)


def test_gather_equals_scatter_and_dense_bruteforce():
    rng = np.random.default_rng(32)
    n, L, batch = 150, 6, 64
    src, tgt, w, d, r = _edges(rng, n, n, 9000)
    by_src = net.coo_to_csr(src, tgt, w, d, r, n_rows=n, major="source")
    by_tgt = net.csr_transpose(by_src, n)
    z = (rng.random(n * batch) < 0.05).astype(np.uint8)
    want = orc.dense_deliver_bruteforce(z, batch, src, tgt, w, d, r, L, n, 7)
    ring_g = torch.zeros(L, 4, n * batch, device="cuda")
    ring_s = torch.zeros(L, 4, n * batch, device="cuda")
    ops.csr_propagate_fwd("gather", ops.SynapseTable.from_numpy(by_tgt), ring_g, n, batch, 7,
                          zbits=to_dev(bits_of(z)), n_src=n)
    ids, count = ops.SpikeCompactor(n * batch)(to_dev(z))
    ops.csr_propagate_fwd("scatter", ops.SynapseTable.from_numpy(by_src), ring_s, n, batch, 7,
                          active=ids, n_active=count)
    # floor 1e-2: a hundredth of the unit weight scale (lognormal(0,1) pA), sums of a few signed terms
    assert rel_err(ring_g.cpu().numpy(), want, 1e-2) < 1e-5
    assert rel_err(ring_s.cpu().numpy(), want, 1e-2) < 1e-5


def test_empty_rows_and_no_spikes():
    n, L = 70, 4
    csr = net.coo_to_csr(np.array([5], np.int32), np.array([9], np.int32), np.array([2.0], np.float32),
                         np.array([3], np.uint8), np.array([1], np.uint8), n_rows=n, major="source")
    ring = torch.zeros(L, 4, n, device="cuda")
    comp = ops.SpikeCompactor(n)
    z = np.zeros(n, np.uint8)
    ids, count = comp(to_dev(z))
    ops.csr_propagate_scatter(ids, count, ops.SynapseTable.from_numpy(csr), ring, n, 1, 2)
    assert not ring.any()
    z[[5, 6]] = 1
    ids, count = comp(to_dev(z))
    ops.csr_propagate_scatter(ids, count, ops.SynapseTable.from_numpy(csr), ring, n, 1, 2)
    assert ring[(2 + 3) % L, 1, 9].item() == 2.0 and ring.sum().item() == 2.0


def test_propagate_argument_errors():
    from bmtk_amd._lib import BmtkAmdError
    n = 10
    csr = net.coo_to_csr(np.array([1], np.int32), np.array([2], np.int32), np.array([1.0], np.float32),
                         np.array([1], np.uint8), np.array([0], np.uint8), n_rows=n, major="target")
    t = ops.SynapseTable.from_numpy(csr)
    zb = torch.zeros(2, dtype=torch.int64, device="cuda")
    with pytest.raises(BmtkAmdError):
        ops.csr_propagate_gather(zb, n, t, torch.zeros(17, 4, n, device="cuda"), n, 1, 0)   # L > 16
    with pytest.raises(ValueError):
        ops.csr_propagate_gather(zb, n, t, torch.zeros(4, 4, n + 1, device="cuda"), n, 1, 0)
    with pytest.raises(ValueError):
        net.check_csr(csr, n, n, 1)         # delay 1 needs at least 2 slots


@pytest.mark.parametrize("batch,p", [(1, 0.3), (5, 0.2), (32, 0.05), (64, 0.01), (64, 0.3), (100, 0.1), (130, 0.05)])
def test_pull_matches_oracle(batch, p):
    """Pull form: what arrives in step tau computed from the spike bits of the
    last L steps.  LDS atomics add in arbitrary order, so the comparison is with
    the fp64 oracle at 1e-5 of max(|want|, 1e-2 * sum of |w| into the cell)."""
    rng = np.random.default_rng(40 + batch)
    n_src, n_tgt, L = 211, 190, 6
    src, tgt, w, d, r = _edges(rng, n_src, n_tgt, 15000)
    by_src = net.coo_to_csr(src, tgt, w, d, r, n_rows=n_src, major="source")
    by_tgt = net.coo_to_csr(src, tgt, w, d, r, n_rows=n_tgt, major="target")
    table = ops.SynapseTable.from_numpy(by_tgt)
    words = ops.n_words(n_src * batch)
    hist = torch.zeros(L, words + 1, dtype=torch.int64, device="cuda")
    abs_src = (by_src[0], by_src[1], np.abs(by_src[2]), by_src[3], by_src[4])
    z_of = {}
    syn = torch.full((4, n_tgt * batch), 7.0, device="cuda")      # must be overwritten, not accumulated
    for tau in range(1, 14):
        k = tau - 1                                                  # the newest emitting step
        z_of[k] = (rng.random(n_src * batch) < p).astype(np.uint8)
        hist[k % L] = to_dev(bits_of(z_of[k]))
        ring = np.zeros((L, 4, n_tgt * batch))
        mag = np.zeros((L, 4, n_tgt * batch))
        for kk in range(max(0, tau - (L - 1)), tau):
            orc.deliver_events(np.flatnonzero(z_of[kk]), batch, by_src, ring, n_tgt, kk)
            orc.deliver_events(np.flatnonzero(z_of[kk]), batch, abs_src, mag, n_tgt, kk)
        ops.csr_propagate_pull(hist, n_src, table, syn, n_tgt, batch, tau)
        got = syn.cpu().numpy()
        want, m = ring[tau % L], mag[tau % L]
        assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-2 * m + 1e-30)) < 1e-5
        assert np.all(got[m == 0] == 0)
    assert np.abs(want).max() > 0


@pytest.mark.parametrize("batch,p,n_src,L", [(1, 0.3, 211, 6), (5, 0.2, 211, 6), (32, 0.05, 1500, 6), (64, 0.01, 211, 6),
                                              (64, 0.3, 211, 6), (100, 0.1, 97, 6), (130, 0.05, 211, 6),
                                              (64, 0.05, 211, 2), (32, 0.05, 400, 8), (64, 0.05, 211, 9), (5, 0.2, 300, 14)])
def test_two_step_pull_equals_two_pulls(batch, p, n_src, L):
    """``csr_propagate_pull2`` (the arrivals of steps tau-1 and tau in one pass over the table) == two calls of
    ``csr_propagate_pull`` over the same spike history, bit for bit: both add the same Q31.32 weights, whose sum
    does not depend on the order.  (The one-step form is pinned against the oracle above.)  Histories of up to 8
    rows take the form with one byte of activity per source, longer ones the form with one bit per row and
    source; delays run up to L - 1 steps, the longest a history of L rows serves."""
    rng = np.random.default_rng(70 + batch + L)
    n_tgt = 190
    src, tgt, w, d, r = _edges(rng, n_src, n_tgt, 15000, max_delay=L - 1)
    table = ops.SynapseTable.from_numpy(net.coo_to_csr(src, tgt, w, d, r, n_rows=n_tgt, major="target"))
    words = ops.n_words(n_src * batch)
    hist = torch.zeros(L, words + 1, dtype=torch.int64, device="cuda")
    one = torch.full((2, 4, n_tgt * batch), 7.0, device="cuda")
    two = torch.full((2, 4, n_tgt * batch), -3.0, device="cuda")      # must be overwritten, not accumulated
    for tau in range(1, 2 * L + 4):
        hist[(tau - 1) % L] = to_dev(bits_of((rng.random(n_src * batch) < p).astype(np.uint8)))
        if tau <= L:                                                   # both steps need their L-1 steps of history
            continue
        # the row of step tau-1 is never read by the pull of step tau-1: delays are at least one step
        ops.csr_propagate_pull(hist, n_src, table, one[0], n_tgt, batch, tau - 1)
        ops.csr_propagate_pull(hist, n_src, table, one[1], n_tgt, batch, tau)
        ops.csr_propagate_pull2(hist, n_src, table, two, n_tgt, batch, tau)
        assert torch.equal(one, two), tau
        assert float(one[0].abs().max()) > 0 and not torch.equal(one[0], one[1])


@pytest.mark.parametrize("batch,L", [(64, 6), (5, 6), (32, 8), (64, 2), (1, 3)])
def test_two_step_auto_delivery_equals_the_oracle(batch, L):
    """``ops.AutoPropagator2`` (bmtk_csr_propagate_auto2): called every second step, each of the two new steps goes
    out as events or is left to a pull that sums two arrival steps in one pass.  The same run as for the one-step
    switch -- activity from nothing to 20 % and back, so that pushed and pulled steps mix within and across calls
    and arrival slots hold pushed weights when the pull adds its sums -- with quarter-pA weights: after every call
    both arrival slots must equal the fp32 oracle's bit for bit, also with thresholds that force one form."""
    rng = np.random.default_rng(34 + batch + L)
    n, T = 500, 40
    src, tgt, w, d, r = _edges(rng, n, n, 30000, max_delay=L - 1)
    w = (np.round(w * 4) / 4 + np.sign(w) * 0.25).astype(np.float32)
    by_src = net.coo_to_csr(src, tgt, w, d, r, n_rows=n, major="source")
    by_tgt = net.csr_transpose(by_src, n)
    t_src, t_tgt = ops.SynapseTable.from_numpy(by_src), ops.SynapseTable.from_numpy(by_tgt)
    ne = n * batch
    comp_a, comp_b = ops.SpikeCompactor(ne), ops.SpikeCompactor(ne)
    rates = [0.0, 0.0, 0.002, 0.2, 0.002, 0.0, 0.2, 0.2, 0.01, 0.002, 0.2, 0.0, 0.002] * 4
    zs = [(rng.random(ne) < rates[k]).astype(np.uint8) for k in range(T)]
    counts = sorted(int(z.sum()) for z in zs)
    mid = counts[len(counts) // 2]
    for thr in (mid, 0, ne, counts[-1] - 1):
        want = np.zeros((L, 4, ne), np.float32)
        hist = torch.zeros(L, ops.n_words(ne) + 1, dtype=torch.int64, device="cuda")
        ring = torch.zeros(L, 4, ne, device="cuda")
        auto = ops.AutoPropagator2(t_src, t_tgt, hist, ring, n, n, batch, scatter_max_active=thr)
        seen = set()
        for k in range(1, T, 2):
            lists = []
            for step, comp in ((k - 1, comp_a), (k, comp_b)):
                orc.gather_rows(zs[step], batch, by_tgt, want, n, step)
                hist[step % L] = to_dev(bits_of(zs[step]))
                lists += list(comp(to_dev(zs[step])))
            auto.step2(k, *lists)
            pulled = auto.pulled_steps()
            seen |= {bool(pulled[(k - 1) % L]), bool(pulled[k % L])}
            for slot in (k % L, (k + 1) % L):
                np.testing.assert_array_equal(ring[slot].cpu().numpy(), want[slot],
                                              err_msg="call %d slot %d threshold %d" % (k, slot, thr))
                ring[slot].zero_()    # the consumer's part: both slots are read and cleared before the next call
                want[slot] = 0.0
        if thr == mid:
            assert seen == {True, False}      # both forms ran
        elif thr == ne:
            assert seen == {False}


def test_table_from_edges_on_the_device_equals_the_host_build():
    from bmtk_amd import network as net
    rng = np.random.default_rng(5)
    n_rows, n_cols, nnz = 300, 450, 20000
    src, tgt = rng.integers(0, n_rows, nnz), rng.integers(0, n_cols, nnz)
    w = rng.normal(size=nnz).astype(np.float32)
    r = rng.integers(0, 4, nnz).astype(np.uint8)
    for d in (rng.integers(1, 6, nnz), rng.integers(100, 1000, nnz)):
        want = net.coo_to_csr(src, tgt, w, d, r, n_rows, "source")
        got = ops.SynapseTable.from_edges(src, tgt, w, d, r, n_rows, n_cols)
        for a, b in zip(want, (got.indptr, got.indices, got.weights, got.delays, got.receptors)):
            np.testing.assert_array_equal(a, b.cpu().numpy())
            assert a.dtype == b.cpu().numpy().dtype
    with pytest.raises(ValueError):
        ops.SynapseTable.from_edges(src, tgt + n_cols, w, d, r, n_rows, n_cols)


@pytest.mark.parametrize("batch", [1, 24, 64])
def test_auto_delivery_picks_a_form_on_the_device_and_the_ring_is_the_oracles(batch):
    """``ops.AutoPropagator`` (bmtk_csr_propagate_auto): step by step the active count decides on the device whether
    a step's spikes are pushed into the ring as events or left to the pull over the spike history.  A run whose
    activity goes from nothing to 20 % and back mixes the two forms in every way -- pushed steps between pulled
    ones, arrival slots that hold pushed weights when the pull adds its sums, stretches with nothing to pull.
    Quarter-pA weights: after every call the arrival slot must equal the fp32 oracle's bit for bit, whatever the
    mix, also with thresholds that force one form throughout."""
    rng = np.random.default_rng(33)
    n, L, T = 500, 6, 40
    src, tgt, w, d, r = _edges(rng, n, n, 30000)
    w = (np.round(w * 4) / 4 + np.sign(w) * 0.25).astype(np.float32)
    by_src = net.coo_to_csr(src, tgt, w, d, r, n_rows=n, major="source")
    by_tgt = net.csr_transpose(by_src, n)
    t_src, t_tgt = ops.SynapseTable.from_numpy(by_src), ops.SynapseTable.from_numpy(by_tgt)
    ne = n * batch
    comp = ops.SpikeCompactor(ne)
    rates = [0.0, 0.0, 0.002, 0.2, 0.002, 0.0, 0.2, 0.2, 0.01, 0.002] * 4
    zs = [(rng.random(ne) < rates[k]).astype(np.uint8) for k in range(T)]
    counts = sorted(int(z.sum()) for z in zs)
    mid = counts[len(counts) // 2]
    for thr in (mid, 0, ne, counts[-1] - 1):
        want = np.zeros((L, 4, ne), np.float32)
        hist = torch.zeros(L, ops.n_words(ne) + 1, dtype=torch.int64, device="cuda")
        ring = torch.zeros(L, 4, ne, device="cuda")
        auto = ops.AutoPropagator(t_src, t_tgt, hist, ring, n, n, batch, scatter_max_active=thr)
        seen = set()
        for k in range(T):
            orc.gather_rows(zs[k], batch, by_tgt, want, n, k)
            hist[k % L] = to_dev(bits_of(zs[k]))
            ids, cnt = comp(to_dev(zs[k]))
            auto.step(k, ids, cnt)
            seen.add(bool(auto.pulled_steps()[k % L]))
            slot = (k + 1) % L
            np.testing.assert_array_equal(ring[slot].cpu().numpy(), want[slot], err_msg="step %d threshold %d" % (k, thr))
            ring[slot].zero_()        # the consumer's part: the slot is read and cleared before the next call
            want[slot] = 0.0
        assert np.abs(want).max() > 0 or thr == mid
        if thr == mid:
            assert seen == {True, False}      # both forms ran
        elif thr == 0:
            assert seen == {True} or 0 in counts
        elif thr == ne:
            assert seen == {False}
