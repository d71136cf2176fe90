"""Batches of free molecules (no periodic direction, at most 64 points per system, 256 for sorted lists) have kernels of
their own: no cell lists, every system's rows in (i, j) order. Per system the rows are those of a call on that system
alone (``-m gpu``)."""

import numpy as np
import pytest

import oracle
from vesin_amd import NeighborList

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}


def batch(calculator, molecules, letters="PSdD", flags=None, boxes=None):
    import torch

    first_point = np.cumsum([0] + [len(m) for m in molecules])
    points = torch.as_tensor(np.concatenate(molecules).astype(np.float64).reshape(-1, 3), device="cuda:0")
    if boxes is None:
        boxes = np.zeros((len(molecules), 3, 3))
    if flags is None:
        flags = np.zeros((len(molecules), 3), dtype=bool)
    outputs, first_pair = calculator.compute_batch(
        points, first_point, torch.as_tensor(np.asarray(boxes, dtype=np.float64), device="cuda:0"),
        torch.as_tensor(np.asarray(flags, dtype=bool), device="cuda:0"), letters,
    )
    whole = {NAMES[q]: out.cpu().numpy() for q, out in zip(letters, outputs)}
    assert first_pair[0] == 0 and first_pair[-1] == len(whole["pairs"])
    return [
        {key: value[int(first_pair[s]) : int(first_pair[s + 1])] for key, value in whole.items()}
        for s in range(len(molecules))
    ]


def check_in_order(lists, molecules, cutoff, full, what, flags=None, boxes=None):
    """The rows of these kernels are in the order of sorted lists whether asked for or not."""
    for s, points in enumerate(molecules):
        periodic = [False] * 3 if flags is None else [bool(f) for f in flags[s]]
        box = np.zeros((3, 3)) if boxes is None else boxes[s]
        expected = oracle.canonicalize(oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD"))
        for key, value in lists[s].items():
            assert np.array_equal(value, expected[key]), f"{what}, system {s}: {key} differ or are out of order"


def random_molecules(rng, n_systems, most):
    return [
        rng.normal(scale=1.0 + 0.25 * n ** (1 / 3), size=(n, 3)) + rng.uniform(-30, 30, size=3)
        for n in rng.integers(0, most + 1, size=n_systems)
    ]


@pytest.mark.parametrize("is_sorted", [False, True], ids=["unsorted", "sorted"])
@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
@pytest.mark.parametrize("most", [8, 16, 32, 64, 100, 256], ids=lambda m: f"up to {m} points")
def test_molecules_of_every_size(most, full, is_sorted, capfd, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(100 + most)
    molecules = random_molecules(rng, 700 if most <= 64 else 150, most)
    molecules[5] = np.zeros((0, 3))
    molecules[-1] = rng.normal(size=(most, 3))
    calculator = NeighborList(cutoff=2.4, full_list=full, sorted=is_sorted)
    for call in range(3):
        capfd.readouterr()
        lists = batch(calculator, molecules)
        report = capfd.readouterr().err
        # (with systems of more than 64 points, only sorted lists come from these kernels)
        expected_here = most <= 64 or is_sorted
        assert ("batch of free molecules" in report) == expected_here, report
        if expected_here:
            assert f"{most if most <= 64 else 256} lanes per system" in report
            check_in_order(lists, molecules, 2.4, full, f"call {call}")
        else:
            for s, rows in enumerate(lists):
                expected = oracle.canonicalize(oracle.neighbors(molecules[s], np.zeros((3, 3)), [False] * 3, 2.4, full, False, "ijSdD"))
                got = oracle.canonicalize(rows)
                for key in got:
                    assert np.array_equal(got[key], expected[key]), (s, key)
        molecules = [m + 0.05 * rng.normal(size=m.shape) for m in molecules]


def test_rows_that_outgrow_the_arrays_and_outputs_on_request():
    rng = np.random.default_rng(7)
    molecules = random_molecules(rng, 300, 40)
    calculator = NeighborList(cutoff=1.5, full_list=True)
    few = sum(len(rows["pairs"]) for rows in batch(calculator, molecules))
    for scale in (1.0, 0.5, 0.25):
        shrunk = [m.mean(axis=0) + (m - m.mean(axis=0)) * scale if len(m) else m for m in molecules]
        for letters in ("PSdD", "P", "Pd"):
            lists = batch(calculator, shrunk, letters)
            check_in_order(lists, shrunk, 1.5, True, f"scale {scale}, {letters}")
    assert sum(len(rows["pairs"]) for rows in lists) > 3 * few


def test_what_sends_a_batch_back_to_the_general_path(capfd, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(11)
    molecules = random_molecules(rng, 120, 30)
    cutoff = 2.2
    calculator = NeighborList(cutoff=cutoff, full_list=True, sorted=True)
    for _ in range(2):
        lists = batch(calculator, molecules)
    check_in_order(lists, molecules, cutoff, True, "free molecules")

    # one system becomes periodic: the kernels notice, the general path takes over and stays
    flags = np.zeros((120, 3), dtype=bool)
    flags[17] = (True, False, True)
    boxes = np.zeros((120, 3, 3))
    boxes[17] = 6.0 * np.eye(3)
    for call in range(2):
        capfd.readouterr()
        lists = batch(calculator, molecules, flags=flags, boxes=boxes)
        report = capfd.readouterr().err
        assert ("free molecules no more" in report) == (call == 0)
        assert "batch of free molecules" not in report
        for s, rows in enumerate(lists):
            expected = oracle.canonicalize(oracle.neighbors(molecules[s], boxes[s], list(flags[s]), cutoff, True, False, "ijSdD"))
            got = oracle.canonicalize(rows)
            for key in got:
                assert np.array_equal(got[key], expected[key]), (call, s, key)
    # free again: the general path once, then the kernels for molecules
    for call in range(2):
        capfd.readouterr()
        lists = batch(calculator, molecules)
        assert ("batch of free molecules" in capfd.readouterr().err) == (call == 1)
    check_in_order(lists, molecules, cutoff, True, "free again")

    # another division into systems: these kernels at once; one molecule of 257 atoms, a forced cell list: the general path
    other = random_molecules(rng, 90, 30)
    big = other[:40] + [rng.normal(scale=3.0, size=(257, 3))] + other[40:]
    for molecules_now, options in ((other, {}), (big, {}), (other, {"algorithm": "cell_list"})):
        calc = NeighborList(cutoff=cutoff, full_list=True, sorted=True, **options) if options else calculator
        for call in range(2):
            capfd.readouterr()
            lists = batch(calc, molecules_now)
            report = capfd.readouterr().err
            expected_fast = molecules_now is other and not options
            assert ("batch of free molecules" in report) == expected_fast, (len(molecules_now), options, call)
            for s, rows in enumerate(lists):
                expected = oracle.canonicalize(oracle.neighbors(molecules_now[s], np.zeros((3, 3)), [False] * 3, cutoff, True, False, "ijSdD"))
                got = oracle.canonicalize(rows)
                for key in got:
                    assert np.array_equal(got[key], expected[key]), (s, key)


def test_errors_and_negative_zero():
    rng = np.random.default_rng(13)
    molecules = random_molecules(rng, 50, 20)
    molecules[3] = np.array([[0.0, 1.0, -0.0], [0.0, 1.0, 0.0], [-0.0, 1.0, 0.5]])  # components of -0 - 0 and 0 - (-0)
    calculator = NeighborList(cutoff=2.0, full_list=True)
    for _ in range(2):
        lists = batch(calculator, molecules)
    check_in_order(lists, molecules, 2.0, True, "with zeros of both signs")
    expected = oracle.canonicalize(oracle.neighbors(molecules[3], np.zeros((3, 3)), [False] * 3, 2.0, True, False, "ijSdD"))
    assert np.array_equal(np.signbit(lists[3]["vectors"]), np.signbit(expected["vectors"]))

    broken = [m.copy() for m in molecules]
    broken[20][1, 2] = np.inf
    where = sum(len(m) for m in molecules[:20]) + 1
    with pytest.raises(RuntimeError, match=f"point {where} has non-finite coordinate along axis 2"):
        batch(calculator, broken)
    lists = batch(calculator, molecules)
    check_in_order(lists, molecules, 2.0, True, "after the error")


def test_a_hundred_thousand_tiny_molecules():
    rng = np.random.default_rng(17)
    sizes = rng.integers(3, 9, size=100_000)
    molecules = [rng.random((n, 3)) * (n ** (1 / 3)) * 1.6 for n in sizes]
    calculator = NeighborList(cutoff=5.0, full_list=True, sorted=True)
    for _ in range(2):
        lists = batch(calculator, molecules, "PSd")
    # (almost every pair of every molecule is within the cutoff)
    wanted = [int((np.linalg.norm(m[:, None, :] - m[None, :, :], axis=2) < 5.0).sum()) - len(m) for m in molecules]
    assert [len(rows["pairs"]) for rows in lists] == wanted
    for s in rng.choice(100_000, size=40, replace=False):
        expected = oracle.canonicalize(oracle.neighbors(molecules[s], np.zeros((3, 3)), [False] * 3, 5.0, True, False, "ijSd"))
        for key, value in lists[s].items():
            assert np.array_equal(value, expected[key]), (s, key)


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_molecules_of_very_different_sizes_in_one_batch(full):
    """A few large molecules among many small ones in a sorted batch: every system gets a workgroup, most of whose
    waves have no points."""
    rng = np.random.default_rng(19)
    molecules = random_molecules(rng, 400, 12)
    for at, n in ((3, 256), (77, 65), (200, 129), (399, 193), (10, 64), (11, 1), (12, 0)):
        molecules[at] = rng.normal(scale=1.0 + 0.25 * max(n, 1) ** (1 / 3), size=(n, 3))
    calculator = NeighborList(cutoff=3.0, full_list=full, sorted=True)
    for call in range(3):
        lists = batch(calculator, molecules)
        check_in_order(lists, molecules, 3.0, full, f"call {call}")
        molecules = [m + 0.02 * rng.normal(size=m.shape) for m in molecules]


def test_other_molecules_with_every_call_and_a_list_that_starts_with_crystals(capfd, monkeypatch):
    """A loader hands over other molecules with every call: every call goes through the kernels for molecules, the
    first one of a new list included. A new list given crystals guesses wrong once and not again."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(23)
    calculator = NeighborList(cutoff=2.5, full_list=False, sorted=True)
    for call in range(6):
        molecules = random_molecules(rng, int(rng.integers(1, 300)), int(rng.choice([6, 20, 64, 200])))
        capfd.readouterr()
        lists = batch(calculator, molecules)
        assert "batch of free molecules" in capfd.readouterr().err, call
        check_in_order(lists, molecules, 2.5, False, f"call {call}")

    crystals = [rng.random((n, 3)) * 5.0 for n in (8, 20, 33)]
    boxes = np.array([np.eye(3) * 5.0] * 3)
    flags = np.ones((3, 3), dtype=bool)
    another = NeighborList(cutoff=2.5, full_list=True, sorted=True)
    for call in range(3):
        capfd.readouterr()
        lists = batch(another, crystals, flags=flags, boxes=boxes)
        assert ("free molecules no more" in capfd.readouterr().err) == (call == 0)
        check_in_order(lists, crystals, 2.5, True, f"crystals, call {call}", flags=flags, boxes=boxes)
