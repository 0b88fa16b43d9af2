"""Host-side edge assembly rules (bmtk/simulator/pointnet/sonata_adaptors.py:268-357,
bmtk/simulator/pointnet/pointnetwork.py:229-248)."""
import numpy as np
import pytest

from bmtk_amd import network as net


def test_weight_is_nsyns_times_syn_weight():
    np.testing.assert_array_equal(net.edge_weights(np.array([1, 2, 3]), 2.5), [2.5, 5.0, 7.5])
    assert net.edge_weights(None, -6.5) == -6.5
    with pytest.raises(Exception, match="syn_weight"):
        net.edge_weights(np.array([1]), None)


def test_syn_spec_conversion():
    w, d, r = net.syn_spec_to_arrays(3, {"weight": np.array([1.0, 2.0, 3.0]), "delay": 2.0, "receptor_type": 3}, dt=0.5)
    assert w.dtype == np.float32 and d.tolist() == [4, 4, 4] and r.tolist() == [2, 2, 2]
    w, d, r = net.syn_spec_to_arrays(2, {"weight": 5.0, "delay": np.array([1.0, 1.6])}, dt=1.0)
    assert w.tolist() == [5.0, 5.0] and d.tolist() == [1, 2] and r.tolist() == [0, 0]


def test_bad_delay_and_receptor():
    with pytest.raises(net.BadDelay):
        net.syn_spec_to_arrays(1, {"weight": 1.0, "delay": 0.05}, dt=0.1)
    with pytest.raises(ValueError):
        net.syn_spec_to_arrays(1, {"weight": 1.0, "delay": 1.0, "receptor_type": 5}, dt=0.1)
    with pytest.raises(ValueError):
        net.syn_spec_to_arrays(1, {"weight": 1.0, "delay": 1.0, "receptor_type": 0}, dt=0.1)
    # delays beyond 255 steps keep a wide column (the simulator takes them with a delay offset)
    w, d, r = net.syn_spec_to_arrays(2, {"weight": 1.0, "delay": 300.0}, dt=1.0)
    assert d.dtype == np.int32 and list(d) == [300, 300]
    w, d, r = net.syn_spec_to_arrays(2, {"weight": 1.0, "delay": 3.0}, dt=1.0)
    assert d.dtype == np.uint8 and list(d) == [3, 3]


def test_check_csr_rejects_what_a_kernel_would_trip_over():
    good = net.coo_to_csr([0, 1], [1, 0], [1.0, 2.0], [1, 2], [0, 3], n_rows=2, major="source")
    net.check_csr(good, 2, 2, 3)
    indptr, indices, w, d, r = good
    with pytest.raises(ValueError):
        net.check_csr((indptr, indices + 5, w, d, r), 2, 2, 3)
    with pytest.raises(ValueError):
        net.check_csr((indptr, indices, w, d, r), 2, 2, 2)           # delay 2 needs 3 slots
    with pytest.raises(ValueError):
        net.check_csr((indptr[::-1].copy(), indices, w, d, r), 2, 2, 3)
    with pytest.raises(ValueError):
        net.check_csr((indptr, indices, w[:1], d, r), 2, 2, 3)
    with pytest.raises(ValueError):
        net.coo_to_csr([5], [0], [1.0], [1], [0], n_rows=2, major="source")


@pytest.mark.parametrize("dt", [0.001, 1.0, 5.0, 10.0])
def test_multimeter_at_any_resolution(dt, tmp_path):
    """bmtk/tests/simulator/pointnet/test_multimeter_report.py:10-28: the calls MultimeterMod.initialize makes
    (bmtk/simulator/pointnet/modules/multimeter_reporter.py:103-115) go through at small and large steps."""
    from bmtk_amd import nest
    nest.ResetKernel()
    nest.SetKernelStatus({"resolution": dt, "overwrite_files": True, "print_time": False})
    cells = nest.Create("glif_psc", 4, {})
    mm = nest.Create("multimeter", params={"start": 0.0, "stop": 100.0, "record_to": "ascii",
                                            "record_from": ["V_m"], "label": str(tmp_path / "__bmtk_nest_test")})
    nest.SetStatus(mm, "interval", dt)
    nest.Connect(mm, cells)
    assert nest.GetStatus(mm, "interval")[0] == dt
    assert nest.GetKernelStatus("min_delay") == dt
    with pytest.raises(nest.kernel.NESTError):
        nest.SetStatus(mm, "interval", dt * 0.5)  # not a multiple of the resolution
    nest.ResetKernel()


def test_input_event_lists_are_validated():
    """Ascending ids within a step are required (the input-weight gradient relies on it); a repeated id within a
    step is legal (NEST delivers both spikes) and is reported so that the bit-row form of the delivery is not used."""
    ptr = np.array([0, 2, 2, 5], np.int64)
    assert net.check_input_events(ptr, np.array([3, 7, 0, 4, 9], np.int32), 10) is False
    assert net.check_input_events(ptr, np.array([3, 7, 0, 4, 4], np.int32), 10) is True
    assert net.check_input_events(np.array([0, 0], np.int64), np.zeros(0, np.int32), 10) is False
    # the first event of a step may be smaller than the last of the step before
    assert net.check_input_events(np.array([0, 1, 2], np.int64), np.array([9, 0], np.int32), 10) is False
    with pytest.raises(ValueError, match="ascending"):
        net.check_input_events(ptr, np.array([7, 3, 0, 4, 9], np.int32), 10)
    with pytest.raises(ValueError, match="outside"):
        net.check_input_events(ptr, np.array([3, 7, 0, 4, 10], np.int32), 10)
    with pytest.raises(ValueError, match="in_ptr"):
        net.check_input_events(np.array([0, 3, 2, 5], np.int64), np.array([3, 7, 0, 4, 9], np.int32), 10)


def test_resident_fit_bound_counts_the_active_row_list():
    """The resident kernel keeps its ring slice AND an 8192-entry active-row list (plus a few static words) in
    the 160 KB of LDS: ring slices between 128 KB and 150 KB used to pass the host check and then fail at launch."""
    from bmtk_amd.simulator import RES_LDS_BYTES, RES_LDS_EXTRA, resident_span
    assert resident_span(230924, 1, 6, 256) == 960                 # the 230k-neuron network: 92 KB ring slice
    assert resident_span(230924, 2, 6, 256) == 0                   # batch 1 only
    assert resident_span(256 * 1024 + 1, 1, 2, 256) == 0           # more than 1024 elements per compute unit
    assert resident_span(256 * 960, 1, 8, 256) == 960              # 122,880 B + 33,024 B = 155,904 B fits
    assert resident_span(256 * 960, 1, 9, 256) == 0                # 138,240 B ring slice: over with the list
    assert resident_span(256 * 1024, 1, 8, 256) == 0               # 131,072 B ring slice: over with the list
    assert resident_span(256 * 1024, 1, 7, 256) == 1024
    for L in range(2, 40):
        for ne in (1000, 100_000, 245_760, 262_144):
            span = resident_span(ne, 1, L, 256, single=False)
            if span:
                assert span % 64 == 0 and span <= 1024 and span * 256 >= ne
                assert L * 4 * span * 4 + RES_LDS_EXTRA <= RES_LDS_BYTES
    assert resident_span(1000, 1, 6, 250, single=False) == 64      # 248 usable compute units
    assert resident_span(1000, 1, 6, 250) == 1024                  # a small network: one workgroup holds all of it
    assert resident_span(300, 1, 6, 256) == 320 and resident_span(1024, 1, 8, 256) == 1024
    assert resident_span(1024, 1, 9, 256) == 64                    # its whole ring does not fit: many workgroups
    assert resident_span(1025, 1, 6, 256) == 64
