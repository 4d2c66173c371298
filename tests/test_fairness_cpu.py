"""Jain's fairness index tool (reference tools/calculate_jains_fairness_index.py) on hand-made stats rows."""
import numpy as np
import pytest

from paella_amd import fairness


def _row(x, n, elapsed, blocks):
    """A stats row as llis_app_client writes it: blocks = [(mean, p50, p90, p95, p99, max, sd), ...], all-requests first."""
    return [x, n, elapsed] + [v for b in blocks for v in b]


def test_index_closed_forms():
    assert fairness.jain_index([3.0, 3.0, 3.0, 3.0]) == pytest.approx(1.0)
    assert fairness.jain_index([0.0, 0.0, 5.0, 0.0]) == pytest.approx(0.25)        # one of n served: 1/n
    assert fairness.jain_index([1.0, 2.0, 3.0]) == pytest.approx(36.0 / 42.0)
    assert fairness.jain_index([10.0, 20.0, 30.0]) == pytest.approx(36.0 / 42.0)   # scale-free
    rows = fairness.jain_index([[1.0, 1.0], [1.0, 3.0]])
    np.testing.assert_allclose(rows, [1.0, 16.0 / 20.0])


def test_slowdowns_use_the_per_type_statistic_and_the_baseline_of_the_model_alone():
    alone0 = _row(0, 100, 1e6, [(200, 190, 250, 260, 300, 400, 20), (200, 190, 250, 260, 300, 400, 20)])
    alone1 = _row(0, 100, 1e6, [(1000, 900, 1500, 1600, 2000, 2500, 100), (1000, 900, 1500, 1600, 2000, 2500, 100)])
    sweep = [_row(0.1, 3000, 5e6, [(700, 0, 0, 0, 0, 0, 0), (400, 380, 0, 0, 900, 0, 0), (3000, 2700, 0, 0, 4000, 0, 0)]),
             _row(100.0, 3000, 5e6, [(650, 0, 0, 0, 0, 0, 0), (220, 200, 0, 0, 330, 0, 0), (9000, 9000, 0, 0, 20000, 0, 0)])]
    t = fairness.slowdown_table(sweep, [alone0, alone1])
    np.testing.assert_allclose(t[:, 0], [0.1, 100.0])
    np.testing.assert_allclose(t[:, 2:], [[2.0, 3.0], [1.1, 9.0]])
    np.testing.assert_allclose(t[:, 1], [25.0 / (2 * 13.0), 10.1 ** 2 / (2 * (1.21 + 81.0))])
    t99 = fairness.slowdown_table(sweep, [alone0, alone1], stat="p99")
    np.testing.assert_allclose(t99[:, 2:], [[3.0, 2.0], [1.1, 10.0]])
    with pytest.raises(ValueError):
        fairness.slowdown_table(sweep, [alone0])


def test_reference_indexing_is_reproduced_on_request(tmp_path):
    # the reference script: data[:, 9::7] / [baseline[2] ...]  -- columns 9, 16, 23 against three baselines
    sweep = [_row(1.0, 10, 77.0, [(1, 2, 3, 4, 5, 6, 8.0), (1, 2, 3, 4, 5, 6, 9.0), (1, 2, 3, 4, 5, 6, 12.0)])]
    bases = [[0, 0, 2.0, 0], [0, 0, 3.0, 0], [0, 0, 4.0, 0]]
    t = fairness.slowdown_table(sweep, bases, reference_columns=True)
    np.testing.assert_allclose(t[0, 2:], [4.0, 3.0, 3.0])
    np.testing.assert_allclose(t[0, 1], 100.0 / (3 * 34.0))
    # and through the command line, files in, file out
    np.savetxt(tmp_path / "sweep.txt", np.array(sweep), delimiter=",")
    for i, b in enumerate(bases):
        np.savetxt(tmp_path / ("b%d.txt" % i), np.array([b]), delimiter=",")
    out = tmp_path / "out.txt"
    fairness.main(["-i", str(tmp_path / "sweep.txt"), "-o", str(out), "--reference-columns"] + sum([["-b", str(tmp_path / ("b%d.txt" % i))] for i in range(3)], []))
    np.testing.assert_allclose(np.atleast_2d(np.genfromtxt(out, delimiter=",")), t)
