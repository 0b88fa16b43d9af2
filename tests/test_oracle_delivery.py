"""Pins the oracle's spike delivery (NEST static_synapse -> ring buffer) with a
dense-matrix brute force, invariants, and the timing rule; pins compaction and
CSR transposition host helpers."""
import numpy as np
import pytest

from oracle import glif3_oracle as orc
from bmtk_amd import network as net


def _random_edges(rng, n_src, n_tgt, nnz, max_delay=5):
    src = rng.integers(0, n_src, nnz).astype(np.int32)
    tgt = rng.integers(0, n_tgt, nnz).astype(np.int32)
    w = (rng.lognormal(0, 1, nnz) * rng.choice([-1, 1], nnz)).astype(np.float32)
    d = rng.integers(1, max_delay + 1, nnz).astype(np.uint8)
    r = rng.integers(0, 4, nnz).astype(np.uint8)
    return src, tgt, w, d, r


@pytest.mark.parametrize("batch", [1, 3])
def test_delivery_equals_dense_matrix_product(batch):
    rng = np.random.default_rng(10)
    n_src, n_tgt, L = 48, 64, 6
    src, tgt, w, d, r = _random_edges(rng, n_src, n_tgt, 900)
    by_src = net.coo_to_csr(src, tgt, w, d, r, n_rows=n_src, major="source")
    by_tgt = net.coo_to_csr(src, tgt, w, d, r, n_rows=n_tgt, major="target")
    for step in (0, 7, 123):
        z = (rng.random(n_src * batch) < 0.3).astype(np.uint8)
        want = orc.dense_deliver_bruteforce(z, batch, src, tgt, w, d, r, L, n_tgt, step)
        ring = np.zeros((L, 4, n_tgt * batch))
        orc.deliver_events(np.flatnonzero(z), batch, by_src, ring, n_tgt, step)
        np.testing.assert_allclose(ring, want, rtol=1e-12, atol=1e-12)
        ring2 = np.zeros((L, 4, n_tgt * batch))
        orc.gather_rows(z, batch, by_tgt, ring2, n_tgt, step)
        np.testing.assert_allclose(ring2, want, rtol=1e-12, atol=1e-12)
        # nothing lands in the slot of the emitting step itself (delays >= 1, L > max delay)
        assert not ring[step % L].any()


def test_delivery_is_linear_and_permutation_invariant():
    rng = np.random.default_rng(11)
    n, L = 40, 6
    src, tgt, w, d, r = _random_edges(rng, n, n, 600)
    csr = net.coo_to_csr(src, tgt, w, d, r, n_rows=n, major="source")
    perm = rng.permutation(src.size)
    csr_p = net.coo_to_csr(src[perm], tgt[perm], w[perm], d[perm], r[perm], n_rows=n, major="source")
    za = (rng.random(n) < 0.2).astype(np.uint8)
    zb = ((rng.random(n) < 0.2) & (za == 0)).astype(np.uint8)
    ra, rb, rab, rp = (np.zeros((L, 4, n)) for _ in range(4))
    orc.deliver_events(np.flatnonzero(za), 1, csr, ra, n, 3)
    orc.deliver_events(np.flatnonzero(zb), 1, csr, rb, n, 3)
    orc.deliver_events(np.flatnonzero(za | zb), 1, csr, rab, n, 3)
    orc.deliver_events(np.flatnonzero(za | zb), 1, csr_p, rp, n, 3)
    np.testing.assert_allclose(ra + rb, rab, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(rp, rab, rtol=1e-12, atol=1e-12)


def test_spike_in_step_t_with_delay_d_first_moves_U_in_step_t_plus_d_plus_1():
    """Neuron 0 is driven over threshold by a current; its only synapse (delay
    d) targets neuron 1.  U of neuron 1 must stay 0 through step t+d and move
    in step t+d+1; y1 of neuron 1 must jump at the end of step t+d."""
    from bmtk_amd.glif_utils import params_table
    cell = dict(C_m=100.0, g=5.0, E_L=-70.0, V_th=-50.0, V_reset=-70.0, t_ref=3.0, asc_decay=(0.05, 0.3),
                asc_amps=(0.0, 0.0), tau_syn=(5.5, 8.5, 2.8, 5.8))
    par, _, _ = params_table([cell, cell])
    h = 1.0
    prop = orc.precompute(par, h)
    for d in (1, 2, 4):
        L = 5
        csr = net.coo_to_csr(np.array([0], np.int32), np.array([1], np.int32), np.array([50.0], np.float32),
                             np.array([d], np.uint8), np.array([2], np.uint8), n_rows=2, major="source")
        st = orc.new_state(2, 1, np.float64)
        ring = np.zeros((L, 4, 2))
        i_ext = np.array([400.0, 0.0])
        U1, y1, t_spk = [], [], None
        for t in range(30):
            syn = ring[t % L].copy(); ring[t % L] = 0
            z, _ = orc.step(st, prop, h, syn=syn, i_ext=i_ext)
            if z[0] and t_spk is None:
                t_spk = t
            orc.deliver_events(np.flatnonzero(z), 1, csr, ring, 2, t)
            U1.append(st["V"][1]); y1.append(st["y1"][2, 1])
        assert t_spk is not None
        assert all(u == 0 for u in U1[:t_spk + d + 1]) and U1[t_spk + d + 1] != 0
        assert all(v == 0 for v in y1[:t_spk + d]) and y1[t_spk + d] == pytest.approx(50.0 * np.e / 2.8)


def test_simulate_equals_stepwise_loop():
    """The whole-run driver is the per-step functions chained in NEST's order."""
    from bmtk_amd import synthetic
    cfg = synthetic.small_glif3_network(n=60, n_in=40, steps=120, seed=5, in_rate=30.0, in_w_scale=12.0, w_scale=3.0)
    prop = orc.precompute(cfg["par"], cfg["h"])
    n, L = cfg["n"], cfg["L"]
    st_a = orc.new_state(n, 1, np.float64)
    ring_a = np.zeros((L, 4, n))
    out = orc.simulate(st_a, prop, cfg["h"], cfg["steps"], ring=ring_a, rec=cfg["rec_src"], inp=cfg["inp_src"],
                       in_ptr=cfg["in_ptr"], in_events=cfg["in_events"], raster=True)
    st_b = orc.new_state(n, 1, np.float64)
    ring_b = np.zeros((L, 4, n))
    ras = np.zeros((cfg["steps"], n), np.uint8)
    for t in range(cfg["steps"]):
        syn = ring_b[t % L].copy(); ring_b[t % L] = 0
        z, _ = orc.step(st_b, prop, cfg["h"], syn=syn)
        ras[t] = z
        orc.deliver_events(np.flatnonzero(z), 1, cfg["rec_src"], ring_b, n, t)
        ev = cfg["in_events"][cfg["in_ptr"][t]:cfg["in_ptr"][t + 1]]
        orc.deliver_events(ev, 1, cfg["inp_src"], ring_b, n, t)
    assert out["count"] == ras.sum() and out["count"] > 20
    np.testing.assert_array_equal(out["raster"], ras)
    np.testing.assert_array_equal(st_a["V"], st_b["V"])
    np.testing.assert_array_equal(ring_a, ring_b)
    tt, ee = np.nonzero(ras)
    np.testing.assert_array_equal(out["step"], tt)
    np.testing.assert_array_equal(out["elem"], ee)


def test_csr_transpose_round_trip():
    rng = np.random.default_rng(12)
    src, tgt, w, d, r = _random_edges(rng, 30, 50, 400)
    a = net.coo_to_csr(src, tgt, w, d, r, n_rows=30, major="source")
    b = net.csr_transpose(a, n_cols=50)
    c = net.coo_to_csr(src, tgt, w, d, r, n_rows=50, major="target")
    for x, y in zip(b, c):
        np.testing.assert_array_equal(x, y)
    a2 = net.csr_transpose(b, n_cols=30)
    for x, y in zip(a, a2):
        np.testing.assert_array_equal(x, y)
