"""Larger systems with a direction that is not periodic: a list that has arrays from earlier calls picks its grid
from the extent of the points of the call before, finds the extent of its own points on the way, and starts over with
a pass over the points when the points turn out to be somewhere else altogether. The rows are the oracle's on every
call."""

import re

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from vesin_amd import NeighborList

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}


def _compute(calculator, points, box, periodic, quantities="PSdD"):
    import torch

    outputs = calculator.compute(
        torch.tensor(np.ascontiguousarray(points), device="cuda:0"),
        torch.tensor(np.ascontiguousarray(box), device="cuda:0"),
        periodic,
        quantities,
    )
    return {NAMES[q]: out.cpu().numpy() for q, out in zip(quantities, outputs)}


def _far_outside(err):
    """One number per call that started from the extent of the call before: the points it found far outside."""
    return [int(n) for n in re.findall(r"grid from the extent of the call before: (\d+) points far outside", err)]


def _blobs(rng, n_points, n_blobs, spread, sigma):
    centres = rng.uniform(0.0, spread, size=(n_blobs, 3))
    return centres[rng.integers(0, n_blobs, size=n_points)] + rng.normal(scale=sigma, size=(n_points, 3))


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
@pytest.mark.parametrize(
    "periodic,box",
    [
        ((False, False, False), np.zeros((3, 3))),
        ((True, True, False), np.array([[60.0, 0.0, 0.0], [9.0, 58.0, 0.0], [0.0, 0.0, 1.0]])),
        ((False, True, False), np.array([[1.0, 0.0, 0.0], [3.0, 55.0, -4.0], [0.0, 0.0, 1.0]])),
    ],
    ids=["free", "slab", "wire"],
)
def test_points_that_drift_grow_jump_and_collapse(periodic, box, full, capfd, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(51)
    points = _blobs(rng, 6000, 12, 60.0, 4.0)
    calculator = NeighborList(cutoff=3.0, full_list=full, sorted=False)
    guessed = []
    for step in range(22):
        if step == 5:
            points = (points - points.mean(axis=0)) * 1.05 + points.mean(axis=0)  # grows past the outermost cells
        elif step == 8:
            points = points + np.array([900.0, -700.0, 400.0])  # jumps
        elif step == 19:
            points = (points - points.mean(axis=0)) * 0.6 + points.mean(axis=0)  # collapses
        else:
            points = points + rng.normal(scale=0.1, size=points.shape)
        expected = oracle.neighbors(points, box, list(periodic), 3.0, full, False, "ijSdD")
        capfd.readouterr()
        result = _compute(calculator, points, box, list(periodic))
        guessed.append(_far_outside(capfd.readouterr().err))
        assert_same_list(result, expected, what=f"step {step}")
    # the first call has no arrays, the second no extent, the third may still be learning that the box stays
    assert all(g == [0] for g in guessed[4:8]), guessed
    # the jump: every point is far outside of what the call before left (a direction that is periodic brings them
    # back, so only the directions that are not count); the list then finds the extent first for a few calls
    assert len(guessed[8]) == 1 and guessed[8][0] > 0, guessed
    assert all(g == [] for g in guessed[9:15]), guessed
    assert all(g == [0] for g in guessed[17:]), guessed


def test_points_a_cell_or_less_outside_stay_in_the_outermost_cells(capfd, monkeypatch):
    """Every call moves a few points out of the extent of the call before by less than a cell: no call starts over,
    and the points that left are found all the same."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(52)
    points = rng.random((9000, 3)) * np.array([50.0, 40.0, 30.0])
    box = np.zeros((3, 3))
    calculator = NeighborList(cutoff=3.0, full_list=True, sorted=False)
    far = []
    for step in range(8):
        # the outermost points of every direction step outwards by up to two thirds of a cell
        for axis in range(3):
            order = np.argsort(points[:, axis])
            points[order[:40], axis] -= rng.random(40) * 2.0
            points[order[-40:], axis] += rng.random(40) * 2.0
        expected = oracle.neighbors(points, box, [False] * 3, 3.0, True, False, "ijSdD")
        capfd.readouterr()
        result = _compute(calculator, points, box, [False] * 3)
        far += _far_outside(capfd.readouterr().err)
        assert_same_list(result, expected, what=f"step {step}")
    assert len(far) >= 5 and all(n == 0 for n in far), far


def test_a_fresh_extent_on_request(capfd, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    monkeypatch.setenv("VESIN_HIP_EXTENT", "fresh")
    rng = np.random.default_rng(53)
    points = _blobs(rng, 5000, 8, 50.0, 4.0)
    box = np.zeros((3, 3))
    calculator = NeighborList(cutoff=3.0, full_list=True, sorted=False)
    expected = oracle.neighbors(points, box, [False] * 3, 3.0, True, False, "ijSdD")
    for step in range(5):
        capfd.readouterr()
        result = _compute(calculator, points, box, [False] * 3)
        assert _far_outside(capfd.readouterr().err) == []
        assert_same_list(result, expected, what=f"step {step}")


def test_a_coordinate_that_is_not_finite_is_still_reported(monkeypatch):
    rng = np.random.default_rng(54)
    points = _blobs(rng, 5000, 8, 50.0, 4.0)
    box = np.zeros((3, 3))
    calculator = NeighborList(cutoff=3.0, full_list=True, sorted=False)
    for step in range(5):
        _compute(calculator, points, box, [False] * 3)
    points[1234, 1] = np.inf
    with pytest.raises(RuntimeError, match="point 1234"):
        _compute(calculator, points, box, [False] * 3)
    points[1234, 1] = 3.0
    expected = oracle.neighbors(points, box, [False] * 3, 3.0, True, False, "ijSdD")
    assert_same_list(_compute(calculator, points, box, [False] * 3), expected, what="after the error")


def test_a_dense_cluster_on_the_one_pass_cell_build_jumps(capfd, monkeypatch):
    """Cells of ordinary occupation: the one-pass cell build leaves out the points it finds far outside of the
    remembered extent, as the packed build does; the call starts over and the rows are the oracle's."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(55)
    points = rng.random((9000, 3)) * np.array([50.0, 40.0, 30.0])
    box = np.zeros((3, 3))
    calculator = NeighborList(cutoff=3.0, full_list=False, sorted=False)
    far = []
    builds = []
    for step in range(9):
        if step == 5:
            points = points + np.array([-400.0, 250.0, 90.0])
        else:
            points = points + rng.normal(scale=0.05, size=points.shape)
        expected = oracle.neighbors(points, box, [False] * 3, 3.0, False, False, "ijSdD")
        capfd.readouterr()
        result = _compute(calculator, points, box, [False] * 3)
        err = capfd.readouterr().err
        far.append(_far_outside(err))
        builds += [line for line in err.splitlines() if line.startswith("single pass:") and "one-pass cell build" in line]
        assert_same_list(result, expected, what=f"step {step}")
    assert builds, "these cells are what the one-pass build takes"
    assert all(f == [0] for f in far[3:5]), far
    assert len(far[5]) == 1 and far[5][0] > 0, far
