"""The backward pass at the launch geometry the training configuration runs at: 51,978 neurons x batch 32, the
52 M-synapse table regrouped into 24 target ranges.  There a workgroup of ``bwd_gather_blocked_kernel`` holds 1,632
source rows, more than the 1,024 one sweep keeps in LDS: two sweeps, seven row groups per wavefront, the partial
sums in LDS zeroed again for the second sweep, the recurrent weight gradient riding along.  Smaller networks never
reach that path (one sweep, at most three groups).

Operands are exact in fp32 (weights in quarters, adjoints in eighths, sums far below 2^24 of their unit), so every
form of the same sum must agree BIT FOR BIT whatever the order of its additions.  The checkers are the row-by-row
kernel (pinned against W^T lambda on the host at 12,000 neurons, tests/test_gpu_fullsize.py), W^T lambda on the
host again here for a network with two sweeps, and plain torch gathers for the weight gradient.  Gradients have no
counterpart in the reference (parity unpinned)."""
import numpy as np
import pytest
import torch

from bmtk_amd import ops, synthetic, training
from bmtk_amd.layout import NREC, PROP
from bmtk_amd.simulator import Glif3Simulator
from gpu_util import to_dev
from test_gpu_fullsize import N52K, _adjoint_ring, _network, _quarter

pytestmark = pytest.mark.gpu

F_SPIKE, F_INTEGRATING, F_RESET = 1, 2, 4


def test_blocked_transposed_propagation_at_the_training_size_equals_row_by_row():
    """51,978 rows of ~1000 synapses, batch 32, 24 target ranges (what ``Glif3Bptt`` picks at this size): the eight
    partial sums of the blocked form added up == the row-by-row kernel (four trials per lane), bit for bit."""
    n, batch, L, step = N52K, 32, 6, 4
    n_blocks = ops.blocked_table_blocks(n, batch, L)
    assert n_blocks == 24
    plan = ops.blocked_plan(n, batch)
    assert plan["sweeps"] >= 2 and plan["groups_per_wavefront"] >= 7, plan
    _, t_src, _ = _network(n, 1000, seed=2)
    assert t_src.nnz > 51_000_000
    lam = to_dev(_adjoint_ring(np.random.default_rng(5), L, n * batch))
    want = ops.csr_propagate_bwd(t_src, lam, n, batch, step, trials_per_lane=4)
    assert float(want.abs().max()) > 100.0
    parts = ops.csr_propagate_bwd_blocked(t_src.blocked(n, n_blocks), n_blocks, lam, n, batch, step)
    assert torch.equal(parts.sum(0), want)
    # and once more into the same buffer: the second sweep's zeroed partial sums leave nothing behind
    again = ops.csr_propagate_bwd_blocked(t_src.blocked(n, n_blocks), n_blocks, lam, n, batch, step, gz_parts=parts)
    assert torch.equal(again.sum(0), want)


@pytest.mark.parametrize("n,batch,n_blocks", [(34000, 32, 8), (34000, 32, 24), (17500, 64, 16)])
def test_blocked_transposed_propagation_with_two_sweeps_equals_the_host_sum(n, batch, n_blocks):
    """A network small enough for the host (in-degree ~50) whose rows per workgroup still exceed one sweep:
    blocked form == row by row == W^T lambda computed on the host from the target-major copy, bit for bit."""
    L, step = 6, 2
    plan = ops.blocked_plan(n, batch)
    assert plan["sweeps"] >= 2, plan
    t_tgt, t_src, host_tgt = _network(n, 50, seed=41)
    rng = np.random.default_rng(n_blocks)
    lam = _adjoint_ring(rng, L, n * batch)
    lam_d = to_dev(lam)
    g4 = ops.csr_propagate_bwd(t_src, lam_d, n, batch, step, trials_per_lane=4)
    parts = ops.csr_propagate_bwd_blocked(t_src.blocked(n, n_blocks), n_blocks, lam_d, n, batch, step)
    assert torch.equal(parts.sum(0), g4)
    indptr, src, w, d, r = host_tgt
    tgt = np.repeat(np.arange(n), np.diff(indptr))
    cells = lam.reshape(L, 4, n, batch)[(step + d.astype(np.int64)) % L, r, tgt]         # [nnz, batch]
    want = np.zeros((n, batch), np.float64)
    np.add.at(want, src, w[:, None].astype(np.float64) * cells)
    np.testing.assert_array_equal(g4.cpu().numpy().reshape(n, batch), want.astype(np.float32))


def _one_crafted_step(sim, blocked, n_blocks, step, rec, lam, fired_bits):
    """One backward step over a made-up forward record: returns the ``Glif3Bptt`` after it."""
    bptt = training.Glif3Bptt(sim, dampening=0.3, blocked=blocked, n_blocks=n_blocks if blocked else None)
    bptt.lam_ring.copy_(lam)
    fwd = dict(saved=dict(v=rec["v"], flags=rec["flags"], step0=step), bits=fired_bits)
    bptt.backward(fwd, dl_dz_const=rec["dl"])
    return bptt


def _host_free_gradient(t_src, lam, fired, n, batch, L, step, chunk=1 << 22):
    """d w[p] = sum over the trials b in which the source of synapse p fired of lam[(step + d) % L, r, i*batch + b],
    with plain torch gathers, a few million synapses at a time."""
    lam4 = lam.view(L, NREC, n, batch)
    rows = torch.repeat_interleave(torch.arange(n, device="cuda"), (t_src.indptr[1:] - t_src.indptr[:-1]).long())
    out = torch.empty(t_src.nnz, device="cuda")
    for p0 in range(0, t_src.nnz, chunk):
        p1 = min(t_src.nnz, p0 + chunk)
        slot = (step + t_src.delays[p0:p1].long()) % L
        cells = lam4[slot, t_src.receptors[p0:p1].long(), t_src.indices[p0:p1].long()]    # [chunk, batch]
        out[p0:p1] = (cells * fired[rows[p0:p1]]).sum(1)
    return out


@pytest.mark.parametrize("n,mean_in,n_blocks", [(N52K, 1000, 24), (34000, 50, 8)])
def test_fused_weight_gradient_of_the_blocked_form_at_two_sweeps(n, mean_in, n_blocks):
    """One backward step at the training size over a made-up record (potentials around threshold, a third of the
    elements refractory, 3 % of the elements spiking, adjoint ring in eighths): the blocked form with the gradient
    riding along (``d_blk_w``, brought back through the sort permutation) == the row-by-row kernel with its own
    fused gradient == the sums taken with torch gathers, bit for bit; and since the transposed sums are exact, the
    adjoint state the step leaves behind is the same bit for bit in both forms."""
    batch, L, step = 32, 6, 9
    plan = ops.blocked_plan(n, batch)
    assert plan["sweeps"] >= 2, plan
    ne = n * batch
    rng = np.random.default_rng(n_blocks)
    par = synthetic.random_cells(rng, n)
    by_tgt, by_src, _ = synthetic.device_network(n, mean_in, "poisson", seed=2, max_delay=L - 1)
    by_src = (by_src[0], by_src[1], _quarter(by_src[2]), by_src[3], by_src[4])
    del by_tgt
    sim = Glif3Simulator(n, par, 1.0, batch=batch, rec=by_src, resident=False, pull=False, ring_slots=L)
    th = sim.prop[PROP["TH"]].repeat_interleave(batch)
    g = torch.Generator(device="cuda").manual_seed(3)
    # potentials between 0 and 2.2 th: |v/th - 1| < 1 for most, beyond it for some (their rows may be skipped)
    v = (th * (torch.rand(ne, device="cuda", generator=g) * 2.2)).view(1, ne).contiguous()
    kind = torch.rand(ne, device="cuda", generator=g)
    flags = torch.zeros(ne, dtype=torch.uint8, device="cuda")
    flags[kind < 0.65] = F_INTEGRATING
    flags[(kind >= 0.65) & (kind < 0.7)] = F_RESET
    fired = torch.rand(n, batch, device="cuda", generator=g) < 0.03
    flags = (flags | (fired.view(-1) & (flags == F_INTEGRATING)).to(torch.uint8) * F_SPIKE).view(1, ne).contiguous()
    words = ops.n_words(ne)
    bits = torch.zeros(1, words, dtype=torch.int64, device="cuda")
    f64 = torch.zeros(words * 64, dtype=torch.int64, device="cuda")
    f64[:ne] = fired.view(-1).long()
    bits[0] = (f64.view(words, 64) << torch.arange(64, device="cuda")).sum(1)
    lam = to_dev(_adjoint_ring(np.random.default_rng(1), L, ne))
    dl = (torch.randint(-8, 9, (ne,), device="cuda", generator=g) / 8.0).float()
    rec = dict(v=v, flags=flags, dl=dl)
    a = _one_crafted_step(sim, True, n_blocks, step, rec, lam, bits)
    b = _one_crafted_step(sim, False, None, step, rec, lam, bits)
    assert a.blk is not None and b.blk is None
    want = _host_free_gradient(sim.rec, lam, fired.float(), n, batch, L, step)
    assert float(want.abs().max()) > 1.0 and float((want != 0).float().mean()) > 0.3
    assert torch.equal(b.d_rec_w, want)
    assert torch.equal(a.d_rec_w, want)
    for name in ("lam_V", "lam_asc", "lam_y1", "lam_y2", "lam_ring"):
        assert torch.equal(getattr(a, name), getattr(b, name)), name
    assert float(a.lam_V.abs().max()) > 0


def test_pull_equals_gather_at_in_degree_1000_batch_64():
    """The isolated-propagation configuration as the benchmark times it -- 51,978 rows of ~1000 synapses (rows of
    sixteen 64-synapse chunks), batch 64, 5 Hz -- pull == the ring slot the gathers filled, bit for bit (quarter-pA
    weights).  A property between two device forms: the gather kernel equals the oracle at in-degree 120
    (tests/test_gpu_fullsize.py)."""
    n, batch, L = N52K, 64, 6
    t_tgt, _, _ = _network(n, 1000, seed=2)
    assert t_tgt.nnz > 51_000_000
    ne = n * batch
    g = torch.Generator(device="cuda").manual_seed(9)
    words = ops.n_words(ne)
    hist = torch.zeros(L, words + 1, dtype=torch.int64, device="cuda")
    ring = torch.zeros(L, 4, ne, device="cuda")
    for k in range(L):
        z = (torch.rand(ne, device="cuda", generator=g) < 5e-3).view(words, 64).long()
        hist[k, :words] = (z << torch.arange(64, device="cuda")).sum(1)
        ops.csr_propagate_gather(hist[k], n, t_tgt, ring, n, batch, k)
    syn = torch.full((4, ne), 3.0, device="cuda")
    ops.csr_propagate_pull(hist, n, t_tgt, syn, n, batch, L)
    assert float(ring[0].abs().max()) > 10.0
    assert torch.equal(syn, ring[0])
    # the two-step pull over the same history: arrivals of step L == the above, of step L-1 == the one-step pull's
    before = torch.empty_like(syn)
    ops.csr_propagate_pull(hist, n, t_tgt, before, n, batch, L - 1)
    both = torch.full((2, 4, ne), -1.0, device="cuda")
    ops.csr_propagate_pull2(hist, n, t_tgt, both, n, batch, L)
    assert torch.equal(both[1], syn) and torch.equal(both[0], before)
    assert not torch.equal(before, syn)


def test_two_steps_per_pass_at_the_training_size_equal_one():
    """51,978 x batch 32, 24 ranges: five and then four steps of a real forward run differentiated through the
    two-step form of the blocked kernel (four sweeps of four row groups) and through the one-step form: adjoint
    state and ring bit for bit, gradients to 1e-6 of the largest."""
    n, batch, L = N52K, 32, 6
    rng = np.random.default_rng(6)
    par = synthetic.random_cells(rng, n)
    _, by_src, _ = synthetic.device_network(n, 1000, "poisson", seed=2, max_delay=L - 1, w_scale=0.2)
    inp = synthetic.device_input_table(17400, n, 8_000_000, seed=4, w_scale=2.0)
    in_ptr, in_ev = ops.poisson_events(17400, 5.0, 1.0, 64, batch=batch, seed=5)
    sim = Glif3Simulator(n, par, 1.0, batch=batch, rec=by_src, inp=inp, resident=False, ring_slots=L)
    sim.set_input_events(in_ptr, in_ev)
    sim.run(40)
    chunks = [sim.run(4, save_state=True), sim.run(5, save_state=True)]
    g = torch.Generator(device="cuda").manual_seed(2)
    dl = torch.randn(n * batch, device="cuda", generator=g) * 1e-3
    one = training.Glif3Bptt(sim, dampening=0.3, blocked=True, n_blocks=24, two_steps=False)
    two = training.Glif3Bptt(sim, dampening=0.3, blocked=True, n_blocks=24, two_steps=True)
    for b in (one, two):
        for c in reversed(chunks):
            b.backward(c, dl_dz_const=dl)
    for name in ("lam_V", "lam_asc", "lam_y1", "lam_y2", "lam_ring"):
        assert torch.equal(getattr(one, name), getattr(two, name)), name
    assert float(one.lam_V.abs().max()) > 0 and float(one.d_rec_w.abs().max()) > 0
    for name in ("d_rec_w", "d_inp_w"):
        got, want = getattr(two, name), getattr(one, name)
        assert float((got - want).abs().max()) <= 1e-6 * float(want.abs().max()), name
