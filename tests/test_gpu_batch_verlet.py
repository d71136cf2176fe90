"""``vesin_hip_neighbors_batch`` with ``options.skin > 0``: one candidate list for the whole batch, filtered per call.
Whatever the cache does, every system has the rows of a direct calculation on it alone (``-m gpu``); the cases
follow the reference's for single systems (python/vesin/tests/test_numpy.py:405-551)."""

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from vesin_amd import NeighborList, configs

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}


def batch(calculator, all_points, all_boxes, flags, letters="PSdD"):
    import torch

    first_point = np.cumsum([0] + [len(p) for p in all_points])
    points = torch.as_tensor(np.concatenate(all_points).astype(np.float64).reshape(-1, 3), device="cuda:0")
    boxes = torch.as_tensor(np.stack(all_boxes).astype(np.float64), device="cuda:0")
    periodic = torch.as_tensor(np.array(flags, dtype=bool).reshape(len(all_points), 3), device="cuda:0")
    outputs, first_pair = calculator.compute_batch(points, first_point, boxes, periodic, letters)
    whole = {NAMES[q]: out.cpu().numpy() for q, out in zip(letters, outputs)}
    assert first_pair[0] == 0 and first_pair[-1] == len(whole["pairs"])
    assert np.all(np.diff(first_pair.astype(np.int64)) >= 0)
    return [
        {key: value[int(first_pair[s]) : int(first_pair[s + 1])] for key, value in whole.items()}
        for s in range(len(all_points))
    ]


def check(lists, all_points, all_boxes, flags, cutoff, full, ordered, what):
    for s, (points, box, periodic) in enumerate(zip(all_points, all_boxes, flags)):
        expected = oracle.neighbors(points, box, [bool(p) for p in periodic], cutoff, full, False, "ijSdD")
        assert_same_list(lists[s], expected, ordered=ordered, what=f"{what}, system {s}")


def mixed_systems(rng):
    all_points, all_boxes, all_flags = [], [], []
    for n, flags in (
        (5, (False, False, False)),
        (120, (False, False, False)),
        (64, (True, True, True)),
        (0, (True, True, True)),
        (300, (True, True, False)),
        (1, (True, True, True)),
        (90, (False, True, False)),
        (700, (True, True, True)),
        (2, (False, False, False)),
    ):
        edge = 7.0 + 3.0 * rng.random()
        box = np.eye(3) * edge + 0.4 * rng.normal(size=(3, 3))
        all_points.append(rng.random((n, 3)) @ box)
        all_boxes.append(box if any(flags) else np.zeros((3, 3)))
        all_flags.append(flags)
    return all_points, all_boxes, all_flags


@pytest.mark.parametrize("is_sorted", [False, True], ids=["unsorted", "sorted"])
@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_a_trajectory_of_a_mixed_batch(full, is_sorted, capfd, monkeypatch):
    """Small steps are filtered from the kept candidates, a box that breathes eats into the skin, and a jump of one
    point of one system computes all candidates again: always the rows of a direct calculation, in order when asked."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(7)
    all_points, all_boxes, flags = mixed_systems(rng)
    cutoff, skin = 3.0, 0.6
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=is_sorted, skin=skin)
    rebuilt = []
    for step in range(12):
        if step in (5, 9):
            # one point of one system jumps
            s = 2 if step == 5 else 6
            all_points[s][3] += np.array([0.0, 1.1, 0.0])
        elif step > 0:
            all_points = [p + 0.02 * rng.normal(size=p.shape) for p in all_points]
            all_boxes = [b * (1.0 + 0.001 * rng.normal()) for b in all_boxes]
        capfd.readouterr()
        lists = batch(calculator, all_points, all_boxes, flags)
        report = capfd.readouterr().err
        rebuilt.append("the candidates are computed again" in report)
        assert step == 0 or "rows filtered from" in report, "the call did not go through the kept candidates"
        check(lists, all_points, all_boxes, flags, cutoff, full, is_sorted, f"step {step}")
    assert rebuilt[5] and rebuilt[9], "the jumps went unnoticed"
    assert not rebuilt[1] and not rebuilt[2], "steps of a fraction of the skin computed the candidates again"


def test_pairs_enter_and_leave_the_cutoff_between_calls():
    calculator = NeighborList(cutoff=1.0, full_list=False, skin=0.5)
    boxes = [10.0 * np.eye(3)] * 3
    flags = [(False,) * 3, (True,) * 3, (False,) * 3]
    far = [np.array([[0.0, 0.0, 0.0], [1.10, 0.0, 0.0]]) for _ in range(3)]
    near = [np.array([[0.0, 0.0, 0.0], [0.95, 0.0, 0.0]]) for _ in range(3)]
    lists = batch(calculator, far, boxes, flags, "Pd")
    assert [len(rows["pairs"]) for rows in lists] == [0, 0, 0]
    # the second system only: the rows of the others stay empty, and first_pair says so
    lists = batch(calculator, [far[0], near[1], far[2]], boxes, flags, "Pd")
    assert [rows["pairs"].tolist() for rows in lists] == [[], [[0, 1]], []]
    assert lists[1]["distances"].tolist() == [0.95]
    lists = batch(calculator, near, boxes, flags, "Pd")
    assert [rows["pairs"].tolist() for rows in lists] == [[[0, 1]]] * 3
    lists = batch(calculator, far, boxes, flags, "Pd")
    assert [len(rows["pairs"]) for rows in lists] == [0, 0, 0]


def test_no_candidates_at_all():
    calculator = NeighborList(cutoff=1.0, full_list=True, skin=0.3)
    boxes = [20.0 * np.eye(3)] * 2
    flags = [(True,) * 3, (False,) * 3]
    apart = [np.array([[0.0, 0.0, 0.0], [5.0, 0.0, 0.0]]), np.array([[1.0, 1.0, 1.0]])]
    for _ in range(3):
        lists = batch(calculator, apart, boxes, flags)
        assert [len(rows["pairs"]) for rows in lists] == [0, 0]
    # ... until two points meet: far beyond the skin, so the candidates are computed again
    together = [np.array([[0.0, 0.0, 0.0], [0.5, 0.0, 0.0]]), apart[1]]
    lists = batch(calculator, together, boxes, flags)
    check(lists, together, boxes, flags, 1.0, True, False, "after the points met")


def test_the_division_into_systems_and_the_options_are_part_of_the_cache():
    rng = np.random.default_rng(11)
    all_points, all_boxes, flags = mixed_systems(rng)
    calculator = NeighborList(cutoff=2.5, full_list=True, skin=0.5)
    for _ in range(2):
        check(batch(calculator, all_points, all_boxes, flags), all_points, all_boxes, flags, 2.5, True, False, "all systems")
    # fewer systems, then the same number of points divided differently
    fewer = (all_points[:5], all_boxes[:5], flags[:5])
    for _ in range(2):
        check(batch(calculator, *fewer), *fewer, 2.5, True, False, "five systems")
    merged_points = [np.concatenate([all_points[1], all_points[0]])] + all_points[2:5]
    merged = (merged_points, all_boxes[1:5], flags[1:5])
    for _ in range(2):
        check(batch(calculator, *merged), *merged, 2.5, True, False, "other division")
    # another cutoff on the same list, then no skin, then a skin again
    calculator.cutoff = 3.0
    for _ in range(2):
        check(batch(calculator, *merged), *merged, 3.0, True, False, "other cutoff")
    calculator.skin = 0.0
    check(batch(calculator, *merged), *merged, 3.0, True, False, "without a skin")
    calculator.skin = 0.3
    for _ in range(2):
        check(batch(calculator, *merged), *merged, 3.0, True, False, "with a skin again")


def test_the_periodic_flags_of_one_system_change():
    rng = np.random.default_rng(13)
    all_points, all_boxes, flags = mixed_systems(rng)
    all_boxes = [b if b.any() else 9.0 * np.eye(3) for b in all_boxes]
    calculator = NeighborList(cutoff=2.8, full_list=False, skin=0.4)
    for _ in range(2):
        check(batch(calculator, all_points, all_boxes, flags), all_points, all_boxes, flags, 2.8, False, False, "before")
    flags = list(flags)
    flags[4] = (True, True, True)
    flags[0] = (False, False, True)
    for _ in range(2):
        check(batch(calculator, all_points, all_boxes, flags), all_points, all_boxes, flags, 2.8, False, False, "after")


def test_rows_beyond_what_the_arrays_hold():
    """A gas that is compressed: every call has more rows than the one before, from the same candidates while the
    points move little between calls (here they do not: only the box scales, which is a jump, so both ways happen)."""
    rng = np.random.default_rng(17)
    calculator = NeighborList(cutoff=2.0, full_list=True, skin=0.5)
    fractional = [rng.random((n, 3)) for n in (400, 30, 900)]
    flags = [(True,) * 3] * 3
    rows = []
    for edge in (14.0, 13.9, 12.0, 11.95, 9.0, 8.97, 8.95):
        all_boxes = [edge * np.eye(3)] * 3
        all_points = [f * edge for f in fractional]
        lists = batch(calculator, all_points, all_boxes, flags)
        check(lists, all_points, all_boxes, flags, 2.0, True, False, f"edge {edge}")
        rows.append(sum(len(l["pairs"]) for l in lists))
    assert rows[-1] > 3 * rows[0]


def test_points_given_several_boxes_outside_of_boxes_that_change():
    """Candidates with shifts of several boxes move further than a box corner when the box changes: the limit on the
    change of the box follows the largest shift of every system's candidates."""
    rng = np.random.default_rng(19)
    calculator = NeighborList(cutoff=2.0, full_list=True, skin=0.3)
    edge = 6.0
    base = [rng.random((n, 3)) * edge for n in (150, 40)]
    flags = [(True,) * 3, (True, True, False)]
    reach = [rng.integers(-4, 5, size=p.shape).astype(np.float64) for p in base]
    reach[1][:, 2] = 0.0
    for step in range(8):
        scale = 1.0 + 0.004 * step
        all_boxes = [edge * scale * np.eye(3), edge * (2.0 - scale) * np.eye(3)]
        all_points = [p + r @ b for p, r, b in zip(base, reach, all_boxes)]
        lists = batch(calculator, all_points, all_boxes, flags)
        check(lists, all_points, all_boxes, flags, 2.0, True, False, f"step {step}")


def test_many_replicas_that_vibrate():
    """512 replicas of the 64-atom small-cell case: candidates with 5^3 images per system, filtered over thousands of
    chunks; sorted, so the rows of every system must come out in order from the sorted candidates."""
    rng = np.random.default_rng(23)
    replicas = [configs.config3(r)[:2] for r in range(8)]
    all_points = [replicas[r % 8][0].copy() for r in range(512)]
    all_boxes = [replicas[r % 8][1] for r in range(512)]
    flags = [(True,) * 3] * 512
    calculator = NeighborList(cutoff=3.2, full_list=True, sorted=True, skin=0.3)
    for step in range(3):
        all_points = [p + 0.01 * rng.normal(size=p.shape) for p in all_points]
        lists = batch(calculator, all_points, all_boxes, flags, "PSd")
        for s in rng.choice(512, size=24, replace=False):
            expected = oracle.neighbors(all_points[s], all_boxes[s], True, 3.2, True, False, "ijSd")
            assert_same_list(lists[s], expected, ordered=True, what=f"step {step}, replica {s}")
        # all replicas of one structure moved differently, but every list must be consistent with its own points
        lengths = np.array([len(l["pairs"]) for l in lists])
        assert lengths.min() > 0


def test_a_single_call_between_batches_with_a_skin():
    import torch

    rng = np.random.default_rng(29)
    all_points, all_boxes, flags = mixed_systems(rng)
    calculator = NeighborList(cutoff=2.5, full_list=True, skin=0.4)
    for _ in range(2):
        check(batch(calculator, all_points, all_boxes, flags), all_points, all_boxes, flags, 2.5, True, False, "batch")
    points, box = all_points[7], all_boxes[7]
    for _ in range(2):
        P, S, d, D = calculator.compute(torch.tensor(points, device="cuda:0"), torch.tensor(box, device="cuda:0"), True, "PSdD")
        got = {"pairs": P.cpu().numpy(), "shifts": S.cpu().numpy(), "distances": d.cpu().numpy(), "vectors": D.cpu().numpy()}
        assert_same_list(got, oracle.neighbors(points, box, True, 2.5, True, False, "ijSdD"), what="single call")
    for _ in range(2):
        check(batch(calculator, all_points, all_boxes, flags), all_points, all_boxes, flags, 2.5, True, False, "batch again")


def test_shifts_beyond_what_the_kept_candidates_can_hold(capfd, monkeypatch):
    """The filter keeps a shift in 21 bits per direction. A point given more than a million boxes away from its
    neighbours has larger ones: such a batch is searched directly on every call, with the same rows."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(31)
    edge = 4.0
    all_boxes = [edge * np.eye(3), edge * np.eye(3)]
    flags = [(True,) * 3] * 2
    base = [rng.random((20, 3)) * edge, rng.random((30, 3)) * edge]
    reach = [np.zeros((20, 3)), np.zeros((30, 3))]
    reach[1][7, 0] = float(2**20 + 5)
    reach[1][9, 1] = -float(2**20 - 1)  # this one still fits
    calculator = NeighborList(cutoff=2.0, full_list=True, skin=0.4)
    for step in range(4):
        all_points = [p + 0.01 * step + r * edge for p, r in zip(base, reach)]
        capfd.readouterr()
        lists = batch(calculator, all_points, all_boxes, flags)
        assert "rows filtered from" not in capfd.readouterr().err
        check(lists, all_points, all_boxes, flags, 2.0, True, False, f"step {step}")
        assert np.abs(lists[1]["shifts"]).max() >= 2**20 + 4
    # without that point the candidates are kept again, after a while
    reach[1][7, 0] = 3.0
    for step in range(24):
        all_points = [p + 0.01 * step + r * edge for p, r in zip(base, reach)]
        capfd.readouterr()
        lists = batch(calculator, all_points, all_boxes, flags)
        report = capfd.readouterr().err
        check(lists, all_points, all_boxes, flags, 2.0, True, False, f"step {step} with all shifts in range")
    assert "rows filtered from" in report


@pytest.mark.parametrize("seed", range(24))
def test_random_sequences_of_batches_with_a_skin(seed):
    """Random batches (sizes, shapes, flags, points given boxes away) through random sequences of small moves, box
    changes, unchanged calls and new batches on one list: every call has the rows of a direct calculation."""
    rng = np.random.default_rng(770_000 + seed)
    cutoff = float(rng.choice([1.5, 2.5, 3.5]))
    skin = float(rng.choice([0.1, 0.4, 1.0]))
    full = bool(rng.integers(0, 2))
    is_sorted = bool(rng.integers(0, 2))
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=is_sorted, skin=skin)

    def new_batch():
        n_systems = int(rng.choice([1, 2, 5, 30, 120]))
        all_points, all_boxes, all_flags, all_reach = [], [], [], []
        for _ in range(n_systems):
            n = int(rng.choice([0, 1, 2, 7, 40, 150, 400], p=[0.05, 0.05, 0.1, 0.3, 0.3, 0.15, 0.05]))
            if rng.random() < 0.5:
                flags = tuple(bool(x) for x in rng.integers(0, 2, size=3))
            else:
                flags = (True,) * 3 if rng.random() < 0.6 else (False,) * 3
            edge = float(rng.choice([2.0, 5.0, 9.0])) * (1 + rng.random())
            box = np.eye(3) * edge + 0.2 * edge * rng.normal(size=(3, 3)) * (rng.random() < 0.5)
            reach = np.zeros((n, 3))
            if rng.random() < 0.2:
                reach = rng.integers(-3, 4, size=(n, 3)).astype(np.float64) * np.array(flags, dtype=np.float64)
            all_points.append(rng.random((n, 3)) @ box)
            all_boxes.append(box)
            all_flags.append(flags)
            all_reach.append(reach)
        return all_points, all_boxes, all_flags, all_reach

    all_points, all_boxes, flags, reach = new_batch()
    for step in range(6):
        kind = rng.random()
        if step > 0 and kind < 0.6:
            amplitude = skin * float(rng.choice([0.02, 0.1, 0.3]))
            all_points = [p + amplitude * rng.normal(size=p.shape) for p in all_points]
        elif step > 0 and kind < 0.8:
            all_boxes = [b * (1 + 0.01 * skin * rng.normal()) for b in all_boxes]
        elif step > 0 and kind < 0.9:
            all_points, all_boxes, flags, reach = new_batch()
        given = [p + r @ b for p, r, b in zip(all_points, reach, all_boxes)]
        lists = batch(calculator, given, all_boxes, flags)
        check(lists, given, all_boxes, flags, cutoff, full, is_sorted, f"seed {seed}, step {step}")


def test_errors_on_a_list_with_kept_candidates(monkeypatch):
    """What a direct batch refuses, a batch with a skin refuses with the same message, also on a call that would
    only have filtered; the list works again afterwards."""
    rng = np.random.default_rng(37)
    all_points, all_boxes, flags = mixed_systems(rng)
    calculator = NeighborList(cutoff=2.5, full_list=True, skin=0.4)
    for _ in range(2):
        check(batch(calculator, all_points, all_boxes, flags), all_points, all_boxes, flags, 2.5, True, False, "before")

    broken = [p.copy() for p in all_points]
    broken[4][17, 2] = np.nan
    with pytest.raises(RuntimeError, match="non-finite coordinate along axis 2"):
        batch(calculator, broken, all_boxes, flags)
    singular = [b.copy() for b in all_boxes]
    singular[7][2] = singular[7][1]
    with pytest.raises(RuntimeError, match="the box matrix is not invertible"):
        batch(calculator, all_points, singular, flags)
    for _ in range(2):
        check(batch(calculator, all_points, all_boxes, flags), all_points, all_boxes, flags, 2.5, True, False, "after")

    # the reference's limit on pairs per point applies to the filtered rows as to a direct search
    total = sum(len(oracle.neighbors(p, b, list(f), 2.5, True, False, "ij")["pairs"]) for p, b, f in zip(all_points, all_boxes, flags))
    n_points = sum(len(p) for p in all_points)
    monkeypatch.setenv("VESIN_CUDA_MAX_PAIRS_PER_POINT", str(max(1, total // n_points - 1)))
    with pytest.raises(RuntimeError, match="exceeds the maximum capacity"):
        batch(calculator, all_points, all_boxes, flags)
    monkeypatch.setenv("VESIN_CUDA_MAX_PAIRS_PER_POINT", str(total // n_points + 1))
    check(batch(calculator, all_points, all_boxes, flags), all_points, all_boxes, flags, 2.5, True, False, "within the limit")


def test_candidates_that_keep_getting_outdated_are_given_up_for_a_while(capfd, monkeypatch):
    """One system of the batch jumps at every call: after three sets of candidates that served a call each, the list
    searches directly for 64 calls, keeping nothing, then tries candidates again. Always the same rows."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(41)
    all_points, all_boxes, flags = mixed_systems(rng)
    calculator = NeighborList(cutoff=2.0, full_list=True, skin=0.4)
    reports = []
    for call in range(72):
        if call < 4:
            all_points[7][call] += np.array([0.9, 0.0, 0.0])
        capfd.readouterr()
        lists = batch(calculator, all_points, all_boxes, flags, "PSd")
        reports.append(capfd.readouterr().err)
        if call < 6 or call > 66 or call % 16 == 0:
            check(lists, all_points, all_boxes, flags, 2.0, True, False, f"call {call}")
    assert "candidates are computed again" in reports[1] and "candidates are computed again" in reports[2]
    assert "direct searches for a while" in reports[3]
    assert not any("rows filtered from" in report for report in reports[3:69])
    assert all("rows filtered from" in report for report in reports[69:])
