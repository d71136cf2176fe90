"""Small systems on a reused list: cell list, counting, scan and writing happen in ONE launch whose workgroups wait
for each other (small_system_kernel). Sorted lists are checked in place against the canonicalised oracle, unsorted
ones as sets of rows: the shapes of the launch, half and full lists, several work items per point, boxes with images,
mixed periodicity, the cases the launch leaves to the other paths (too many rows per point, too many candidates,
wraps beyond the key's range, rows that do not fit, workgroups that give up waiting, which the host forces through
the spin limit), and VESIN_HIP_LAUNCHES=separate."""

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from vesin_amd import NeighborList, configs

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


def _expected(points, box, periodic, cutoff, full):
    flags = [bool(periodic)] * 3 if isinstance(periodic, (bool, np.bool_)) else [bool(p) for p in periodic]
    return oracle.canonicalize(oracle.neighbors(points, box, flags, cutoff, full, False, "ijSdD"))


def _same(result, expected, what):
    for key in result:
        assert result[key].shape == expected[key].shape, (what, key, result[key].shape, expected[key].shape)
        assert np.array_equal(result[key], expected[key]), (what, key)


def _one_launch_lines(err):
    return [line for line in err.splitlines() if line.startswith("one launch:")]


def _liquid(n, density, seed, triclinic=False):
    rng = np.random.default_rng(seed)
    edge = (n / density) ** (1.0 / 3.0)
    box = np.eye(3) * edge
    if triclinic:
        box = box + 0.15 * edge * rng.normal(size=(3, 3)) * (np.arange(3)[:, None] > np.arange(3)[None, :])
    return rng.random((n, 3)) @ box, box


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
@pytest.mark.parametrize("n", [1, 3, 64, 216, 960, 961, 1920, 1921, 2048])
def test_every_shape_of_the_launch(n, full, capfd, monkeypatch):
    """4, 8 and 16 waves per workgroup, at the sizes where one shape hands over to the next; the second and third call
    of a list go through the one launch and say so."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    points, box = _liquid(n, 0.05, seed=n, triclinic=n % 2 == 1)
    expected = _expected(points, box, True, 4.0, full)
    calculator = NeighborList(cutoff=4.0, full_list=full, sorted=True)
    for call in range(3):
        capfd.readouterr()
        result = _compute(calculator, points, box, True)
        lines = _one_launch_lines(capfd.readouterr().err)
        _same(result, expected, f"n={n} call {call}")
        if call == 0:
            assert not lines  # a list without arrays sizes them with the counting pass first
        elif n >= 64:  # (the boxes of the smallest ones need more images than the in-order search takes)
            assert len(lines) == 1 and "gave up 0" in lines[0], lines


def test_config0_on_a_reused_list(capfd, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    points, box, periodic, options = configs.config0()
    expected = _expected(points, box, True, options["cutoff"], True)
    calculator = NeighborList(cutoff=options["cutoff"], full_list=True, sorted=True)
    for call in range(4):
        capfd.readouterr()
        for letters in ("PSdD", "P", "Sd"):
            result = _compute(calculator, points, box, True, letters)
            _same(result, {key: expected[key] for key in result}, f"call {call} {letters}")
    assert _one_launch_lines(capfd.readouterr().err)


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_images_of_a_small_box_and_mixed_periodicity(full, capfd, monkeypatch):
    """One cell whose stencil is the images of the box (every point pairs with its own images), slabs and free
    clusters, points outside of the box: all on one reused list."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(23)
    calculator = NeighborList(cutoff=3.0, full_list=full, sorted=True)
    small = np.array([[3.2, 0.0, 0.0], [0.4, 3.1, 0.0], [-0.3, 0.2, 3.3]])
    wide = np.array([[11.0, 0.0, 0.0], [1.5, 10.0, 0.0], [-2.0, 0.7, 12.0]])
    used = 0
    for step in range(12):
        box = small if step % 3 == 0 else wide
        n = int(rng.choice([5, 7])) if box is small else int(rng.choice([40, 150, 400]))
        points = rng.random((n, 3)) @ box
        if step % 2 == 1:
            points = points + rng.integers(-2, 3, size=(n, 3)) @ box  # wraps within the key's range
        periodic = [(True, True, True), (True, True, False), (False, False, False), (True, False, True)][step % 4]
        if box is small:
            periodic = (True, True, True)
        expected = _expected(points, box, periodic, 3.0, full)
        capfd.readouterr()
        result = _compute(calculator, points, box, list(periodic))
        used += len(_one_launch_lines(capfd.readouterr().err))
        _same(result, expected, f"step {step} n={n} periodic={periodic}")
    assert used >= 8


def test_what_the_launch_leaves_to_the_other_paths(capfd, monkeypatch):
    """Too many rows per point (more than 256), too many candidates per point (more than 1024), wraps beyond +-255,
    more rows than the arrays hold: the call's result is the oracle's all the same, and the list then stays away
    from the one launch for a while."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    calculator = NeighborList(cutoff=4.0, full_list=True, sorted=True)
    ordinary, box = _liquid(300, 0.05, seed=1)
    _same(_compute(calculator, ordinary, box, True), _expected(ordinary, box, True, 4.0, True), "first call")
    capfd.readouterr()
    _same(_compute(calculator, ordinary, box, True), _expected(ordinary, box, True, 4.0, True), "second call")
    assert _one_launch_lines(capfd.readouterr().err)

    # dense: 1.2 points per cubic A, 320 rows per point
    dense, dense_box = _liquid(500, 1.2, seed=2)
    expected = _expected(dense, dense_box, True, 4.0, True)
    assert len(expected["pairs"]) / 500 > 256
    capfd.readouterr()
    _same(_compute(calculator, dense, dense_box, True), expected, "dense")
    lines = _one_launch_lines(capfd.readouterr().err)
    assert len(lines) == 1 and "gave up 0" in lines[0]
    # ... and the next calls do not ask again
    capfd.readouterr()
    _same(_compute(calculator, ordinary, box, True), _expected(ordinary, box, True, 4.0, True), "after dense")
    assert not _one_launch_lines(capfd.readouterr().err)

    # a fresh list for each of the other cases, warmed up with the ordinary system
    def warmed():
        fresh = NeighborList(cutoff=4.0, full_list=True, sorted=True)
        _compute(fresh, ordinary, box, True)
        return fresh

    # points hundreds of boxes away
    far = ordinary + np.array([300, -400, 260]) @ box
    fresh = warmed()
    capfd.readouterr()
    _same(_compute(fresh, far, box, True), _expected(far, box, True, 4.0, True), "far away")
    lines = _one_launch_lines(capfd.readouterr().err)
    assert len(lines) == 1 and "unsuitable 0" not in lines[0]

    # more rows than the arrays of the list hold: the ordinary system, then one four times as dense
    denser, denser_box = _liquid(1200, 0.2, seed=3)
    fresh = warmed()
    capfd.readouterr()
    _same(_compute(fresh, denser, denser_box, True), _expected(denser, denser_box, True, 4.0, True), "grown")
    assert len(_one_launch_lines(capfd.readouterr().err)) == 1


def test_a_coordinate_that_is_not_finite(monkeypatch):
    import torch

    calculator = NeighborList(cutoff=4.0, full_list=True, sorted=True)
    points, box = _liquid(100, 0.05, seed=4)
    _compute(calculator, points, box, True)
    _compute(calculator, points, box, True)
    broken = points.copy()
    broken[37, 1] = np.inf
    with pytest.raises(RuntimeError, match="point 37"):
        calculator.compute(torch.tensor(broken, device="cuda:0"), torch.tensor(box, device="cuda:0"), True, "P")
    # the list is as good as before
    _same(_compute(calculator, points, box, True), _expected(points, box, True, 4.0, True), "after the error")


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_workgroups_that_give_up_waiting(full, capfd, monkeypatch):
    """A spin limit of zero makes every workgroup that is not the last to arrive give up at once: nothing is written
    by that launch, the host goes on with the separate passes, the rows are the oracle's."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    points, box = _liquid(700, 0.05, seed=5, triclinic=True)
    expected = _expected(points, box, True, 4.0, full)
    calculator = NeighborList(cutoff=4.0, full_list=full, sorted=True)
    _same(_compute(calculator, points, box, True), expected, "first call")
    monkeypatch.setenv("VESIN_HIP_CHAIN_SPINS", "0")
    capfd.readouterr()
    _same(_compute(calculator, points, box, True), expected, "gave up")
    lines = _one_launch_lines(capfd.readouterr().err)
    assert len(lines) == 1 and "gave up 1" in lines[0], lines
    monkeypatch.delenv("VESIN_HIP_CHAIN_SPINS")
    # the list leaves the one launch alone for 64 calls, then comes back to it
    for call in range(64):
        capfd.readouterr()
        result = _compute(calculator, points, box, True, "P")
        assert not _one_launch_lines(capfd.readouterr().err), call
    _same(result, {"pairs": expected["pairs"]}, "while resting")
    capfd.readouterr()
    _same(_compute(calculator, points, box, True), expected, "back")
    lines = _one_launch_lines(capfd.readouterr().err)
    assert len(lines) == 1 and "gave up 0" in lines[0], lines


def test_separate_launches_on_request(capfd, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    monkeypatch.setenv("VESIN_HIP_LAUNCHES", "separate")
    points, box, periodic, options = configs.config0()
    expected = _expected(points, box, True, options["cutoff"], True)
    calculator = NeighborList(cutoff=options["cutoff"], full_list=True, sorted=True)
    for call in range(3):
        _same(_compute(calculator, points, box, True), expected, f"call {call}")
    assert not _one_launch_lines(capfd.readouterr().err)


# ---------------------------------------------------------------------------------------------------------------------
# unsorted lists: one work item per point and slice of its candidates, the upper half of the stencil


def _unsorted_expected(points, box, periodic, cutoff, full):
    flags = [bool(periodic)] * 3 if isinstance(periodic, (bool, np.bool_)) else [bool(p) for p in periodic]
    return oracle.neighbors(points, box, flags, cutoff, full, False, "ijSdD")


def _items_per_point(lines):
    return [int(line.split(" items per point")[0].split()[-1]) for line in lines]


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
@pytest.mark.parametrize("n,density", [(30, 0.05), (64, 0.3), (216, 0.05), (216, 0.4), (300, 0.2), (700, 0.05), (960, 0.05)])
def test_unsorted_lists_with_one_or_several_items_per_point(n, density, full, capfd, monkeypatch):
    """From one item per point to as many as the launch takes; with three items per point and four waves per
    workgroup the slices of most points are counted by different workgroups, whose copies of the points are in
    different orders inside the cells."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    points, box = _liquid(n, density, seed=n + int(100 * density), triclinic=True)
    points = points + np.random.default_rng(n).integers(-1, 2, size=(n, 3)) @ box
    expected = _unsorted_expected(points, box, True, 4.0, full)
    calculator = NeighborList(cutoff=4.0, full_list=full)
    seen = []
    for call in range(4):
        capfd.readouterr()
        result = _compute(calculator, points, box, True)
        lines = _one_launch_lines(capfd.readouterr().err)
        assert_same_list(result, expected, what=f"n={n} density={density} call {call}")
        if call > 0:
            assert len(lines) == 1 and "gave up 0" in lines[0], lines
            seen += _items_per_point(lines)
    assert len(set(seen)) == 1
    if density >= 0.2 and n <= 300:
        assert seen[0] > 1


def test_unsorted_single_replica_of_the_small_cell_case(capfd, monkeypatch):
    """64 atoms in a box of 7.134 A with a cutoff of 10 A: 63 stencil entries of images, 726 rows per point."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    for replica in (0, 5):
        points, box, periodic, options = configs.config3(replica)
        expected = _unsorted_expected(points, box, True, options["cutoff"], True)
        calculator = NeighborList(cutoff=options["cutoff"], full_list=True)
        for call in range(3):
            capfd.readouterr()
            result = _compute(calculator, points, box, True)
            lines = _one_launch_lines(capfd.readouterr().err)
            assert_same_list(result, expected, what=f"replica {replica} call {call}")
            assert len(lines) == (0 if call == 0 else 1)
        assert _items_per_point(lines)[0] > 4


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_unsorted_mixed_periodicity_images_and_changing_systems(full, capfd, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(31)
    calculator = NeighborList(cutoff=3.0, full_list=full)
    small = np.array([[3.2, 0.0, 0.0], [0.4, 3.1, 0.0], [-0.3, 0.2, 3.3]])
    wide = np.array([[11.0, 0.0, 0.0], [1.5, 10.0, 0.0], [-2.0, 0.7, 12.0]])
    used = 0
    for step in range(16):
        box = small if step % 3 == 0 else wide
        n = int(rng.choice([5, 7, 12])) if box is small else int(rng.choice([40, 150, 400, 900]))
        points = rng.random((n, 3)) @ box
        if step % 2 == 1:
            points = points + rng.integers(-2, 3, size=(n, 3)) @ box
        periodic = [(True, True, True), (True, True, False), (False, False, False), (True, False, True)][step % 4]
        if box is small:
            periodic = (True, True, True)
        expected = _unsorted_expected(points, box, periodic, 3.0, full)
        capfd.readouterr()
        result = _compute(calculator, points, box, list(periodic))
        used += len(_one_launch_lines(capfd.readouterr().err))
        assert_same_list(result, expected, what=f"step {step} n={n} periodic={periodic}")
    assert used >= 10


def test_what_the_unsorted_launch_leaves_to_the_other_paths(capfd, monkeypatch):
    """More rows than the arrays hold, wraps beyond +-255, workgroups that give up: the rows are the oracle's."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    ordinary, box = _liquid(300, 0.05, seed=1)

    def warmed():
        fresh = NeighborList(cutoff=4.0, full_list=True)
        _compute(fresh, ordinary, box, True)
        capfd.readouterr()
        assert_same_list(_compute(fresh, ordinary, box, True), _unsorted_expected(ordinary, box, True, 4.0, True))
        assert _one_launch_lines(capfd.readouterr().err)
        return fresh

    # 260 of the 300 points within 1 A of one place: 67,000 rows where the list's arrays hold 4,000. The launch counts
    # them, writes nothing, the call goes on with the other passes and grown arrays, and the next call fits
    clump = ordinary.copy()
    clump[:260] = clump[0] + np.random.default_rng(2).normal(scale=0.5, size=(260, 3))
    calculator = warmed()
    for call in range(2):
        capfd.readouterr()
        assert_same_list(_compute(calculator, clump, box, True), _unsorted_expected(clump, box, True, 4.0, True), what="clump")
        lines = _one_launch_lines(capfd.readouterr().err)
        assert len(lines) == 1 and "gave up 0" in lines[0] and "unsuitable 0" in lines[0]

    far = ordinary + np.array([300, -400, 260]) @ box
    calculator = warmed()
    capfd.readouterr()
    assert_same_list(_compute(calculator, far, box, True), _unsorted_expected(far, box, True, 4.0, True), what="far away")
    lines = _one_launch_lines(capfd.readouterr().err)
    assert len(lines) == 1 and "unsuitable 0" not in lines[0]

    calculator = warmed()
    monkeypatch.setenv("VESIN_HIP_CHAIN_SPINS", "0")
    capfd.readouterr()
    assert_same_list(_compute(calculator, ordinary, box, True), _unsorted_expected(ordinary, box, True, 4.0, True), what="gave up")
    lines = _one_launch_lines(capfd.readouterr().err)
    assert len(lines) == 1 and "gave up 1" in lines[0], lines


# ---------------------------------------------------------------------------------------------------------------------
# directions that are not periodic: the extent of the points is remembered from call to call


@pytest.mark.parametrize("is_sorted", [True, False], ids=["sorted", "unsorted"])
@pytest.mark.parametrize("periodic", [(False, False, False), (True, False, True)], ids=["free", "slab"])
def test_a_cluster_that_moves_grows_and_jumps(periodic, is_sorted, capfd, monkeypatch):
    """The same number of points on every call, so that every call after the second starts from the box and the
    extent the call before left: points that drift, a cluster that doubles its size, one that is suddenly somewhere
    else entirely (every point outside of the remembered extent), one that collapses. The rows are the oracle's
    every time."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(41)
    box = np.array([[14.0, 0.0, 0.0], [2.0, 13.0, 0.0], [0.0, -1.0, 15.0]])
    points = rng.random((180, 3)) * 12.0
    calculator = NeighborList(cutoff=3.5, full_list=True, sorted=is_sorted)
    used = 0
    for step in range(24):
        if step in (6, 7):
            points = points * 1.4  # grows
        elif step == 12:
            points = points + np.array([500.0, -300.0, 120.0])  # jumps
        elif step == 16:
            points = (points - points.mean(axis=0)) * 0.3 + points.mean(axis=0)  # collapses
        else:
            points = points + rng.normal(scale=0.15, size=points.shape)
        expected = oracle.neighbors(points, box, list(periodic), 3.5, True, False, "ijSdD")
        capfd.readouterr()
        result = _compute(calculator, points, box, list(periodic))
        used += len(_one_launch_lines(capfd.readouterr().err))
        if is_sorted:
            _same(result, oracle.canonicalize(expected), f"step {step}")
        else:
            assert_same_list(result, expected, what=f"step {step}")
    assert used >= 18
