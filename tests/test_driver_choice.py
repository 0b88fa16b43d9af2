"""Which form of the batched forward driver ``Glif3Simulator`` picks when left to choose: the cost model behind
``fused="auto"`` against the step times measured on one MI355X (microseconds per step, recorded here as data)."""
import pytest

from bmtk_amd.simulator import fused_pays

# (neurons, batch, synapses, class table, rate in Hz, pushed us per step, fused us per step)
MEASURED = [
    (51978, 8, 60_000_000, False, 0.0, 24.9, 81.8),
    (51978, 8, 60_000_000, False, 0.3, 31.1, 85.6),
    (51978, 8, 60_000_000, False, 3.2, 104.6, 99.6),
    (51978, 16, 60_000_000, False, 0.0, 41.6, 76.1),
    (51978, 16, 60_000_000, False, 0.3, 51.9, 79.6),
    (51978, 16, 60_000_000, False, 3.2, 193.4, 93.3),
    (51978, 32, 60_000_000, False, 0.0, 99.2, 79.9),
    (51978, 32, 60_000_000, False, 0.3, 116.6, 85.2),
    (51978, 32, 60_000_000, False, 3.2, 374.3, 104.2),
    (230924, 8, 77_271_647, True, 2.8, 132.0, 165.0),
    (230924, 16, 77_271_647, True, 2.74, 237.6, 197.3),
    (230924, 32, 77_271_647, True, 2.72, 486.7, 289.6),
]


@pytest.mark.parametrize("n, batch, nnz, classes, rate, pushed, fused", MEASURED)
def test_choice_follows_the_measured_step_times(n, batch, nnz, classes, rate, pushed, fused):
    # where the two forms are within 10 % of each other either choice is right
    if abs(pushed - fused) <= 0.1 * max(pushed, fused):
        return
    assert fused_pays(n, batch, nnz, classes, rate) == (fused < pushed)


def test_a_wrong_choice_costs_little_where_the_model_errs():
    # the model may only err where the measured times are close: never by more than 40 % of the better time
    for n, batch, nnz, classes, rate, pushed, fused in MEASURED:
        got = fused if fused_pays(n, batch, nnz, classes, rate) else pushed
        assert got <= 1.4 * min(pushed, fused), (n, batch, rate, got)


def test_more_activity_and_more_trials_only_move_the_choice_toward_the_fused_form():
    for batch in (8, 16, 32, 64):
        seen = False
        for rate in (0.0, 0.5, 1.0, 2.0, 4.0, 8.0, 16.0, 40.0):
            now = fused_pays(51978, batch, 60_000_000, False, rate)
            assert now or not seen
            seen = now
    for rate in (0.0, 1.0, 3.0, 10.0):
        seen = False
        for batch in (8, 16, 32, 64):
            now = fused_pays(51978, batch, 60_000_000, False, rate)
            assert now or not seen
            seen = now


def test_no_table_no_fused_form():
    assert not fused_pays(100, 32, 0, False, 50.0)
