"""sorted=True: the search that produces the rows in order, the cases it leaves to the radix sort, and the radix
sort itself (VESIN_HIP_SORT=radix) give the same list, in the order (i, j, S) of the canonicalised oracle."""

import numpy as np
import pytest

import oracle
from vesin_amd import NeighborList, configs

pytestmark = pytest.mark.gpu


def _sorted_list(points, box, periodic, cutoff, full, quantities="PSdD"):
    import torch

    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
    outputs = calculator.compute(
        torch.tensor(np.ascontiguousarray(points), device="cuda:0"),
        torch.tensor(np.ascontiguousarray(box), device="cuda:0"),
        periodic,
        quantities,
    )
    names = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}
    return {names[q]: out.cpu().numpy() for q, out in zip(quantities, outputs)}


def _check(points, box, periodic, cutoff, full, capfd, monkeypatch, expect):
    """`expect`: "used" / "left to the radix sort" for what the in-order search must report, None when it must
    not even be tried."""
    flags = [bool(periodic)] * 3 if isinstance(periodic, (bool, np.bool_)) else [bool(p) for p in periodic]
    expected = oracle.canonicalize(oracle.neighbors(points, box, flags, cutoff, full, False, "ijSdD"))
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    for mode in ("default", "radix"):
        if mode == "radix":
            monkeypatch.setenv("VESIN_HIP_SORT", "radix")
        else:
            monkeypatch.delenv("VESIN_HIP_SORT", raising=False)
        capfd.readouterr()
        result = _sorted_list(points, box, periodic, cutoff, full)
        err = capfd.readouterr().err
        lines = [line for line in err.splitlines() if line.startswith("in-order search:")]
        if mode == "radix" or expect is None:
            assert not lines, err
        else:
            assert lines and all(line.endswith(expect) for line in lines), err
        assert result["pairs"].shape == expected["pairs"].shape, mode
        for key in result:
            assert np.array_equal(result[key], expected[key]), (mode, key)


@pytest.mark.parametrize("full", [True, False])
@pytest.mark.parametrize(
    "replicas,expect",
    [
        # one conventional cell with cutoff 5 needs two images per direction: 125 cells, more than that search holds
        (1, None),
        (3, "used"),
        # 4 cells of 6.2 A per direction: 43 atoms per cell, 1175 candidates per tile
        (7, "left to the radix sort"),
        (8, "used"),
    ],
)
def test_crystal(full, replicas, expect, capfd, monkeypatch):
    points, box, periodic = configs.diamond(replicas, seed=replicas)
    _check(points, box, True, 5.0, full, capfd, monkeypatch, expect)


@pytest.mark.parametrize("full", [True, False])
def test_small_box_with_self_images(full, capfd, monkeypatch):
    """Box barely wider than the cutoff: a single cell whose stencil is the 27 images; every point pairs with its
    own images, which the half list keeps under the reference's rule."""
    rng = np.random.default_rng(17)
    box = np.array([[3.2, 0.0, 0.0], [0.4, 3.1, 0.0], [-0.3, 0.2, 3.3]])
    points = rng.random((7, 3)) @ box
    _check(points, box, True, 3.0, full, capfd, monkeypatch, "used")


@pytest.mark.parametrize("periodic", [(True, True, False), (False, False, False), (True, False, True)])
@pytest.mark.parametrize("full", [True, False])
def test_mixed_periodicity_and_points_outside_of_the_box(periodic, full, capfd, monkeypatch):
    rng = np.random.default_rng(23)
    box = np.diag([11.0, 12.0, 13.0])
    points = rng.uniform(-6.0, 18.0, size=(900, 3))  # many are wrapped by a box vector or two
    _check(points, box, periodic, 3.0, full, capfd, monkeypatch, "used")


def test_rows_of_one_point_beyond_the_ranking(capfd, monkeypatch):
    """400 points within a ball of radius 1.2: every point has 399 rows, more than are ranked in one go."""
    rng = np.random.default_rng(29)
    directions = rng.normal(size=(400, 3))
    points = 1.2 * directions / np.linalg.norm(directions, axis=1)[:, None] * rng.random((400, 1)) ** (1 / 3) + 10.0
    _check(points, np.diag([20.0, 20.0, 20.0]), True, 3.0, True, capfd, monkeypatch, "left to the radix sort")


def test_candidates_of_one_tile_beyond_the_registers(capfd, monkeypatch):
    """A dense liquid: 148 points per cell, 4000 candidates around every tile."""
    rng = np.random.default_rng(31)
    points = rng.random((4000, 3)) * np.array([9.0, 9.0, 9.0])
    _check(points, np.diag([9.0, 9.0, 9.0]), True, 3.0, False, capfd, monkeypatch, "left to the radix sort")


def test_points_many_boxes_away(capfd, monkeypatch):
    """Wraps of several hundred box vectors do not fit the packed shifts of that search."""
    rng = np.random.default_rng(37)
    box = np.diag([4.0, 4.0, 4.0])
    points = rng.random((60, 3)) * 4.0
    points[::2] += np.array([1600.0, -1200.0, 0.0])
    _check(points, box, True, 2.0, True, capfd, monkeypatch, "left to the radix sort")


@pytest.mark.parametrize("n_points", [1, 2, 5, 33, 70])
def test_few_points(n_points, capfd, monkeypatch):
    rng = np.random.default_rng(n_points)
    box = np.diag([6.0, 7.0, 8.0])
    points = rng.random((n_points, 3)) @ box
    _check(points, box, True, 2.9, True, capfd, monkeypatch, "used")
    _check(points, box, False, 2.9, False, capfd, monkeypatch, "used")


def test_a_system_that_search_does_not_cover_is_not_asked_again(capfd, monkeypatch):
    import torch

    rng = np.random.default_rng(31)
    points = rng.random((4000, 3)) * 9.0
    box = np.diag([9.0, 9.0, 9.0])
    expected = oracle.canonicalize(oracle.neighbors(points, box, [True] * 3, 3.0, False, False, "ijSdD"))
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    calculator = NeighborList(cutoff=3.0, full_list=False, sorted=True)
    device_points = torch.tensor(points, device="cuda:0")
    device_box = torch.tensor(box, device="cuda:0")
    tried = []
    for _ in range(3):
        capfd.readouterr()
        P, S, d = calculator.compute(device_points, device_box, True, "PSd")
        tried.append(any(line.startswith("in-order search:") for line in capfd.readouterr().err.splitlines()))
        assert np.array_equal(P.cpu().numpy(), expected["pairs"])
        assert np.array_equal(S.cpu().numpy(), expected["shifts"])
        assert np.array_equal(d.cpu().numpy(), expected["distances"])
    assert tried == [True, False, False]


# ---------------------------------------------------------------------------------------------------------------
# Systems with enough tiles for the candidates of every tile to be put in order once (ordered_sort_kernel): the
# order of the input decides how (a window of original indices counted through a bit set, or buckets).


def _lattice(nx, ny, nz, seed, a=3.567):
    """Jittered diamond, atoms numbered cell by cell with x changing slowest: what a crystal builder hands over."""
    basis = np.array([[0, 0, 0], [0, 2, 2], [2, 0, 2], [2, 2, 0], [1, 1, 1], [1, 3, 3], [3, 1, 3], [3, 3, 1]]) / 4.0
    cells = np.stack(np.meshgrid(np.arange(nx), np.arange(ny), np.arange(nz), indexing="ij"), axis=-1).reshape(-1, 3)
    points = (cells[:, None, :] + basis[None, :, :]).reshape(-1, 3) * a
    points += np.random.default_rng(seed).normal(scale=0.05, size=points.shape)
    return points, np.diag([nx * a, ny * a, nz * a])


def _modes(err):
    import re

    found = re.findall(r"of (\d+) tiles ordered by window and of (\d+) by buckets", err)
    assert found, err
    return int(found[-1][0]), int(found[-1][1])


def _check_order_once(points, box, periodic, cutoff, full, capfd, monkeypatch, report=_modes):
    expected = oracle.canonicalize(oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD"))
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    capfd.readouterr()
    result = _sorted_list(points, box, periodic, cutoff, full)
    err = capfd.readouterr().err
    assert any(line.startswith("in-order search:") and line.endswith("used") for line in err.splitlines()), err
    assert result["pairs"].shape == expected["pairs"].shape
    for key in result:
        assert np.array_equal(result[key], expected[key]), key
    return report(err)


@pytest.mark.parametrize("full", [True, False])
def test_lattice_order_in_one_round_of_the_window(full, capfd, monkeypatch):
    # 110,592 atoms: any tile sees a range of original indices well below 65,536
    points, box = _lattice(24, 24, 24, seed=1)
    windowed, bucketed = _check_order_once(points, box, [True] * 3, 5.0, full, capfd, monkeypatch)
    assert windowed > 2048 and bucketed == 0


def test_lattice_order_in_several_rounds_and_around_the_end(capfd, monkeypatch):
    # 12 x 48 x 48 cells, 221,184 atoms: three search cells of x are 5 or 6 of the 12 lattice cells, about 100,000
    # indices; at the two ends of x the neighbourhood continues at the other end of the numbering
    points, box = _lattice(12, 48, 48, seed=2)
    windowed, bucketed = _check_order_once(points, box, [True] * 3, 5.0, True, capfd, monkeypatch)
    assert windowed > 2048 and bucketed == 0


def test_lattice_order_too_wide_for_the_window(capfd, monkeypatch):
    # 6 x 96 x 96 cells, 442,368 atoms: four search cells along x, three of them in every stencil, so a tile sees
    # dense runs of indices spread over two thirds of the numbering or more, whichever way around: beyond 262,144
    points, box = _lattice(6, 96, 96, seed=3)
    windowed, bucketed = _check_order_once(points, box, [True] * 3, 5.0, True, capfd, monkeypatch)
    assert bucketed > 2048


@pytest.mark.parametrize("full", [True, False])
def test_no_order_in_the_input(full, capfd, monkeypatch):
    # 373,248 atoms: more than the window holds, and every tile sees indices from all over
    points, box = _lattice(36, 36, 36, seed=4)
    points = points[np.random.default_rng(5).permutation(len(points))]
    windowed, bucketed = _check_order_once(points, box, [True] * 3, 5.0, full, capfd, monkeypatch)
    assert bucketed > 2048 and windowed == 0


def test_no_order_in_an_input_the_window_holds(capfd, monkeypatch):
    points, box = _lattice(30, 30, 30, seed=9)
    points = points[np.random.default_rng(10).permutation(len(points))]
    windowed, bucketed = _check_order_once(points, box, [True] * 3, 5.0, True, capfd, monkeypatch)
    assert windowed > 2048 and bucketed == 0


@pytest.mark.parametrize("shuffle", [False, True])
def test_two_images_of_a_point_among_the_candidates(shuffle, capfd, monkeypatch):
    # two search cells along x: the stencil reaches the same cell from both sides, a tile sees points twice, with
    # different shifts; only the buckets tell such candidates apart
    points, box = _lattice(3, 70, 70, seed=6)
    if shuffle:
        points = points[np.random.default_rng(7).permutation(len(points))]
    windowed, bucketed = _check_order_once(points, box, [True] * 3, 5.0, True, capfd, monkeypatch)
    assert bucketed > 2048 and windowed == 0


def test_slab_with_free_directions(capfd, monkeypatch):
    points, box = _lattice(40, 40, 6, seed=8)
    windowed, bucketed = _check_order_once(points, box, [True, True, False], 5.0, False, capfd, monkeypatch)
    assert windowed + bucketed > 2048


# ---------------------------------------------------------------------------------------------------------------
# The points of a tile dealt to several waves of the writing pass


def _waves_per_tile(err):
    import re

    found = re.findall(r"(\d+) tiles written by (\d+) waves each", err)
    assert found, err
    return int(found[-1][0]), int(found[-1][1])


@pytest.mark.parametrize("waves", [2, 3, 4])
@pytest.mark.parametrize("full", [True, False])
def test_any_number_of_waves_per_tile_writes_the_same_rows(waves, full, capfd, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_WRITE_SPLIT", str(waves))
    # candidates in the order found once per tile (more than 2048 tiles) ...
    points, box = _lattice(20, 20, 20, seed=11)
    tiles, each = _check_order_once(points, box, [True] * 3, 5.0, full, capfd, monkeypatch, report=_waves_per_tile)
    assert tiles > 2048 and each == waves
    # ... ranked per point (few tiles), with tiles of fewer points than waves, outside points and a free direction
    rng = np.random.default_rng(waves)
    box = np.diag([11.0, 12.0, 13.0])
    points = rng.uniform(-6.0, 18.0, size=(900, 3))
    _check(points, box, (True, False, True), 3.0, full, capfd, monkeypatch, "used")


def test_well_filled_tiles_that_barely_exceed_the_resident_waves_get_four_waves_each(capfd, monkeypatch):
    """110,592 atoms in 4,913 cells: the list's first call learns the number of tiles, the calls after it deal
    every tile's points to four waves; both give the oracle's list."""
    import torch

    points, box = _lattice(24, 24, 24, seed=12)
    expected = oracle.canonicalize(oracle.neighbors(points, box, [True] * 3, 5.0, False, False, "ijSdD"))
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    calculator = NeighborList(cutoff=5.0, full_list=False, sorted=True)
    device_points = torch.tensor(points, device="cuda:0")
    device_box = torch.tensor(box, device="cuda:0")
    waves = []
    for _ in range(3):
        capfd.readouterr()
        P, S, d, D = calculator.compute(device_points, device_box, True, "PSdD")
        tiles, each = _waves_per_tile(capfd.readouterr().err)
        assert 4096 < tiles < 6144
        waves.append(each)
        assert np.array_equal(P.cpu().numpy(), expected["pairs"])
        assert np.array_equal(S.cpu().numpy(), expected["shifts"])
        assert np.array_equal(d.cpu().numpy(), expected["distances"])
        assert np.array_equal(D.cpu().numpy(), expected["vectors"])
    assert waves == [1, 4, 4]


@pytest.mark.parametrize("waves", [2, 3, 4])
@pytest.mark.parametrize("full", [True, False])
def test_any_number_of_waves_per_tile_counts_the_same_rows(waves, full, capfd, monkeypatch):
    """The candidates of a tile dealt to several waves of the counting pass, which add up their rows per point."""
    monkeypatch.setenv("VESIN_HIP_COUNT_SPLIT", str(waves))
    points, box = _lattice(20, 20, 20, seed=13)
    _check_order_once(points, box, [True] * 3, 5.0, full, capfd, monkeypatch)
    # a tile with fewer pairs of units than waves, points outside of the box, a free direction
    rng = np.random.default_rng(waves)
    box = np.diag([31.0, 32.0, 33.0])
    points = rng.uniform(-6.0, 38.0, size=(9000, 3))
    _check(points, box, (True, False, True), 3.0, full, capfd, monkeypatch, "used")


def test_rows_of_one_point_beyond_the_ranking_counted_by_several_waves(capfd, monkeypatch):
    """The most rows of a point are known to the wave of the tile that adds its share last."""
    monkeypatch.setenv("VESIN_HIP_COUNT_SPLIT", "2")
    rng = np.random.default_rng(29)
    directions = rng.normal(size=(400, 3))
    ball = 1.2 * directions / np.linalg.norm(directions, axis=1)[:, None] * rng.random((400, 1)) ** (1 / 3) + 10.0
    points = np.concatenate([ball, rng.random((5000, 3)) * 40.0])
    _check(points, np.diag([40.0, 40.0, 40.0]), True, 3.0, True, capfd, monkeypatch, "left to the radix sort")


@pytest.mark.parametrize("share", [1, 2, 4, 8, 16, 32])
def test_any_share_of_a_tile_per_wave_gives_the_same_list(share, capfd, monkeypatch):
    """The points of a tile that one wave takes: chosen by the size of the system, forced here."""
    monkeypatch.setenv("VESIN_HIP_ORDERED_SHARE", str(share))
    rng = np.random.default_rng(share)
    box = np.array([[44.0, 0.0, 0.0], [5.0, 41.0, 0.0], [-3.0, 2.0, 46.0]])
    points = rng.uniform(-0.2, 1.2, size=(7000, 3)) @ box
    _check(points, box, (True, True, False), 4.0, share % 3 != 0, capfd, monkeypatch, "used")


def _pairs_at_the_cutoff(n_pairs, cutoff, box, seed):
    """Points in pairs whose distance is the cutoff to within a few units in the last place, some below, some at,
    some above: `n_pairs` pairs spread over the box, far enough from each other to stay pairs."""
    rng = np.random.default_rng(seed)
    per_edge = int(np.ceil(n_pairs ** (1.0 / 3.0)))
    grid = np.stack(np.meshgrid(*[np.arange(per_edge)] * 3, indexing="ij"), axis=-1).reshape(-1, 3)[:n_pairs]
    first = (grid + 0.5 + rng.uniform(-0.05, 0.05, size=grid.shape)) / per_edge @ box
    direction = rng.normal(size=first.shape)
    direction /= np.linalg.norm(direction, axis=1)[:, None]
    # distances cutoff * (1 + m 2^-52), m from -6 to 6: squared distances a few units in the last place around cutoff^2
    steps = rng.integers(-6, 7, size=len(first)).astype(np.float64)
    second = first + direction * (cutoff * (1.0 + steps * 2.0**-52))[:, None]
    return np.concatenate([first, second])


@pytest.mark.parametrize("full", [True, False])
@pytest.mark.parametrize(
    "name",
    ["cube", "triclinic", "points moved by box vectors", "slab"],
)
def test_pairs_next_to_the_cutoff(name, full, capfd, monkeypatch):
    """The counting pass decides most pairs in single precision; what that cannot decide, pairs within rounding of the
    cutoff above all, must come out as the reference's own arithmetic has it: thousands of pairs whose squared
    distance is within a few units in the last place of the squared cutoff, on either side."""
    cutoff = 3.0
    periodic = True
    if name == "triclinic":
        box = np.array([[64.0, 0.0, 0.0], [11.0, 61.0, 0.0], [-9.0, 13.0, 66.0]])
    else:
        box = np.eye(3) * 64.0
    points = _pairs_at_the_cutoff(4096, cutoff, box, seed=len(name))
    if name == "points moved by box vectors":
        moves = np.random.default_rng(3).integers(-3, 4, size=points.shape)
        points = points + moves @ box
    if name == "slab":
        periodic = (True, True, False)
    flags = [bool(periodic)] * 3 if isinstance(periodic, bool) else list(periodic)
    expected = oracle.neighbors(points, box, flags, cutoff, True, False, "ijd")
    # the system is what it is meant to be: about half of the pairs are in, and their distances crowd the cutoff
    near = np.abs(expected["distances"] - cutoff) < 1e-12
    assert 1000 < near.sum() // 2 < 3500
    _check(points, box, periodic, cutoff, full, capfd, monkeypatch, "used")
