"""GPU parity of the propagator precompute and the fused GLIF3 state update
against the CPU oracle, called through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import glif3_oracle as orc
from bmtk_amd import ops, synthetic
from bmtk_amd.layout import PROP
from gpu_util import prop_pair, rel_err, to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("h", [0.1, 1.0])
def test_precompute_matches_oracle(h):
    rng = np.random.default_rng(20)
    par = synthetic.random_cells(rng, 3001)
    par[12, 5] = par[0, 5] / par[1, 5]          # tau_syn == tau_m: the singular branch
    p64, p32 = prop_pair(par, h)
    got = p32.cpu().numpy()
    want32 = p64.astype(np.float32)
    # device exp/expm1 may differ from the host libm in the last fp64 bit, which can move the
    # rounded fp32 value by one ulp: allow 1 ulp (2^-23 relative), require most entries identical
    assert rel_err(got, want32, 1e-30) <= 1.2e-7
    assert np.mean(got == want32) > 0.99
    np.testing.assert_array_equal(got[PROP["NREF"]], want32[PROP["NREF"]])


@pytest.mark.parametrize("n,batch,classes", [(1, 1, None), (1000, 1, None), (777, 3, None), (130, 64, None),
                                             (5000, 1, 111), (300, 32, 7)])
def test_step_bit_exact_vs_fp32_oracle_and_close_to_fp64(n, batch, classes):
    """200 steps with random arriving weights and currents.  The kernel uses
    the oracle's operation order without fused multiply-add, so against the
    fp32 oracle every state word and every spike flag must be identical.
    Against the fp64 oracle a single step from identical fp32 states must
    agree to 1e-5 relative; values below one unit (1 mV, 1 pA) are held to 1e-5
    of a unit instead, since a membrane potential near zero is a sum of cancelling
    terms of the order of 10 mV."""
    rng = np.random.default_rng(21)
    h = 1.0
    par = synthetic.random_cells(rng, classes or n)
    class_id = rng.integers(0, classes, n).astype(np.int32) if classes else None
    p64 = orc.precompute(par, h)
    p32 = p64.astype(np.float32)
    ne = n * batch
    st0 = synthetic.random_state(rng, par, n, batch, class_id)
    cpu = {k: v.copy() for k, v in st0.items()}
    gpu = ops.Glif3State.from_numpy(st0)
    prop_d = to_dev(p32)
    cid_d = None if class_id is None else to_dev(class_id)
    z_d = torch.zeros(ne, dtype=torch.uint8, device="cuda")
    zb_d = torch.zeros(ops.n_words(ne) + 1, dtype=torch.int64, device="cuda")
    fr_d = torch.zeros(ne, device="cuda")
    n_spk = 0
    for t in range(200):
        syn = (rng.lognormal(0, 1, (4, ne)) * (rng.random((4, ne)) < 0.05) * 30).astype(np.float32)
        I = rng.normal(100, 50, ne).astype(np.float32)
        if t == 0:
            # one step against fp64 from identical states
            c64 = {k: (v.astype(np.float64) if v.dtype == np.float32 else v.copy()) for k, v in cpu.items()}
            z64, _ = orc.step(c64, p64, h, batch=batch, class_id=class_id, syn=syn.astype(np.float64),
                              i_ext=I.astype(np.float64))
        z_c, fr_c = orc.step(cpu, p32, h, batch=batch, class_id=class_id, syn=syn, i_ext=I, want_frac=True)
        syn_d = to_dev(syn)
        ops.glif3_step_fwd(gpu, prop_d, h, batch=batch, class_id=cid_d, syn=syn_d, clear_syn=True, i_ext=to_dev(I),
                           z=z_d, zbits=zb_d, frac=fr_d)
        got = gpu.to_numpy()
        for k in ("V", "asc", "y1", "y2", "ref"):
            np.testing.assert_array_equal(got[k], cpu[k], err_msg="{} at step {}".format(k, t))
        z_g = z_d.cpu().numpy()
        np.testing.assert_array_equal(z_g, z_c)
        np.testing.assert_array_equal(ops.unpack_bits(zb_d[:-1], ne).cpu().numpy(), z_c)
        np.testing.assert_array_equal(fr_d.cpu().numpy()[z_c == 1], fr_c[z_c == 1])
        assert not syn_d.any()                      # slot cleared after reading
        if t == 0:
            keep = z64 == z_c                        # a flipped threshold decision is a raster matter, not a state one
            assert keep.mean() > 0.999
            for k in ("V", "asc", "y1", "y2"):
                g = got[k].reshape(-1, ne)[:, keep]
                w = c64[k].reshape(-1, ne)[:, keep]
                assert rel_err(g, w, 1.0) < 1e-5, k
        n_spk += int(z_c.sum())
    assert n_spk > 0


def test_step_without_inputs_and_outputs():
    """syn, i_ext, z, zbits, frac are all optional."""
    rng = np.random.default_rng(22)
    n, h = 500, 1.0
    par = synthetic.random_cells(rng, n)
    p32 = orc.precompute(par, h).astype(np.float32)
    st0 = synthetic.random_state(rng, par, n, 1)
    cpu = {k: v.copy() for k, v in st0.items()}
    gpu = ops.Glif3State.from_numpy(st0)
    for _ in range(20):
        orc.step(cpu, p32, h)
        ops.glif3_step_fwd(gpu, to_dev(p32), h)
    got = gpu.to_numpy()
    for k in cpu:
        np.testing.assert_array_equal(got[k], cpu[k])


@pytest.mark.parametrize("classes", [1, 3, 7, 111, 423, 500])
def test_class_table_in_any_size_and_alignment_equals_one_column_per_neuron(classes):
    """The class table is copied into LDS sixteen bytes at a time when it is 16-byte aligned and at most 48 KB
    (423 classes), and read through the caches otherwise: word counts that are no multiple of four (3 x 29, 7 x 29),
    the largest staged table, a larger one and a table that starts 4 bytes past an aligned address must all give,
    bit for bit, what one parameter column per neuron gives (the form the oracle test above covers)."""
    rng = np.random.default_rng(23 + classes)
    n, batch, h = 3000, 2, 1.0
    par = synthetic.random_cells(rng, classes)
    class_id = rng.integers(0, classes, n).astype(np.int32)
    class_id[:min(classes, n)] = np.arange(min(classes, n))   # every class occurs
    p32 = orc.precompute(par, h).astype(np.float32)
    st0 = synthetic.random_state(rng, par, n, batch, class_id)
    table = to_dev(p32)
    shifted = torch.empty(p32.size + 1, device="cuda")[1:].view(p32.shape)
    shifted.copy_(table)
    assert table.data_ptr() % 16 == 0 and shifted.data_ptr() % 16 == 4
    forms = {"per neuron": (to_dev(np.ascontiguousarray(p32[:, class_id])), None),
             "table": (table, to_dev(class_id)), "table off alignment": (shifted, to_dev(class_id))}
    got = {}
    for name, (prop, cid) in forms.items():
        st = ops.Glif3State.from_numpy(st0)
        zb = torch.zeros(ops.n_words(n * batch) + 1, dtype=torch.int64, device="cuda")
        spikes = 0
        r = np.random.default_rng(5)
        for t in range(60):
            syn = to_dev((r.lognormal(0, 1, (4, n * batch)) * (r.random((4, n * batch)) < 0.05) * 30).astype(np.float32))
            cur = to_dev(r.normal(100, 50, n * batch).astype(np.float32))
            ops.glif3_step_fwd(st, prop, h, batch=batch, class_id=cid, syn=syn, i_ext=cur, zbits=zb)
            spikes += int(ops.unpack_bits(zb, n * batch).sum())
        got[name] = (st.to_numpy(), spikes)
    assert got["per neuron"][1] > 0
    for name in ("table", "table off alignment"):
        assert got[name][1] == got["per neuron"][1]
        for k, v in got["per neuron"][0].items():
            np.testing.assert_array_equal(got[name][0][k], v, err_msg="%s %s" % (name, k))


def test_step_argument_errors():
    from bmtk_amd._lib import BmtkAmdError
    st = ops.Glif3State.zeros(10)
    prop = torch.zeros(len(PROP), 10, device="cuda")
    with pytest.raises(BmtkAmdError):
        ops.glif3_step_fwd(st, prop, -1.0)
    with pytest.raises(BmtkAmdError):
        ops.glif3_step_fwd(st, prop[:, :5].contiguous(), 1.0)   # fewer columns than neurons, no class table
    with pytest.raises(ValueError):
        ops.glif3_step_fwd(st, prop, 1.0, batch=3)
    with pytest.raises(TypeError):
        ops.glif3_step_fwd(st, prop.double(), 1.0)
