"""``sorted=True`` on ``vesin_hip_neighbors_batch`` (``-m gpu``): the rows come out of the search in (i, j, shift)
order, system after system, with nothing sorted afterwards: systems of a single cell through the search over their
images, the others through the search over the tiles of their whole stencil. Every call is compared row by row,
in place, with the oracle's rows put in that order (vesin/include/vesin.h:55-57, vesin/src/cpu_cell_list.cpp:634-730),
and what the library says about the way it took (VESIN_HIP_DEBUG) is checked too."""

import numpy as np
import pytest

import oracle
from vesin_amd import NeighborList, configs

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}
KEYS = {"P": "ij", "S": "S", "d": "d", "D": "D"}


def _in_order_lines(capfd):
    return [line for line in capfd.readouterr().err.splitlines() if line.startswith("in-order search (batch)")]


def _call_and_check(calculator, systems, cutoff, full, letters, what):
    """One batched call; every system's rows must be the oracle's, in order."""
    import torch

    all_points = [s[0] for s in systems]
    first_point = np.cumsum([0] + [len(p) for p in all_points])
    points = torch.as_tensor(np.concatenate(all_points).astype(np.float64).reshape(-1, 3), device="cuda:0")
    boxes = torch.as_tensor(np.stack([s[1] for s in systems]).astype(np.float64), device="cuda:0")
    flags = np.array([s[2] for s in systems], dtype=bool)
    outputs, first_pair = calculator.compute_batch(points, first_point, boxes, flags, letters)
    whole = {NAMES[q]: out.cpu().numpy() for q, out in zip(letters, outputs)}
    assert first_pair[0] == 0 and first_pair[-1] == len(whole["pairs"])
    for s, (system_points, box, periodic) in enumerate(systems):
        expected = oracle.canonicalize(oracle.neighbors(system_points, box, list(periodic), cutoff, full, False, "ijSdD"))
        rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
        for key, value in whole.items():
            assert np.array_equal(value[rows], expected[key]), f"{what}, system {s}: {key} differ or are out of order"


def _small_cell_systems(rng):
    systems = []
    for replica in range(5):
        points, box, periodic, _ = configs.config3(replica)  # 64 atoms, 5^3 images less the corners
        systems.append((points, box, tuple(bool(p) for p in np.broadcast_to(periodic, 3))))
    # boxes of one cell in every shape, points up to a box vector outside of them (wraps of -1, 0, 1 and more)
    for n, flags, reach in (
        (0, (True, True, True), 1), (1, (True, True, True), 1), (2, (True, True, True), 3), (31, (True, True, True), 1),
        (64, (True, True, True), 2), (65, (True, True, True), 1), (130, (True, False, True), 1), (200, (True, True, False), 1),
        (256, (True, True, True), 1), (20, (False, False, False), 1), (7, (False, True, False), 2), (90, (True, True, True), 0),
    ):
        # (edges below twice the cutoff: one cell per direction; along a direction that is not periodic the points stay
        # within the box, or their extent would make several cells)
        edge = 4.5 + 2.5 * rng.random()
        box = np.eye(3) * edge + 0.3 * rng.normal(size=(3, 3))
        inside = rng.random((n, 3)) @ box
        moved = (rng.integers(-reach, reach + 1, size=(n, 3)) * np.array(flags)) @ box if reach > 0 else 0.0
        systems.append((inside + moved, box, flags))
    return systems


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_systems_of_one_cell_come_out_in_order(full, capfd, monkeypatch):
    """First call of a list (count, the host sizes the arrays, write), second call (written into the arrays the list
    has, checked on the device), a call for other quantities, and one with the systems in another order."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(571)
    systems = _small_cell_systems(rng)
    cutoff = 4.2
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
    capfd.readouterr()
    for call, letters in (("first call", "PSdD"), ("second call", "PSdD"), ("third call", "Pd"), ("fourth call", "PSD")):
        _call_and_check(calculator, systems, cutoff, full, letters, call)
        lines = _in_order_lines(capfd)
        assert len(lines) == 1 and lines[0].endswith(": used"), (call, lines)
    _call_and_check(calculator, systems[::-1], cutoff, full, "PSdD", "systems in reverse")
    assert _in_order_lines(capfd)[-1].endswith(": used")


def test_small_cell_case_with_many_images(capfd, monkeypatch):
    """The 64-atom configuration whose cutoff exceeds the box: about 727 rows per point over 81 images."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    systems = []
    for replica in range(100, 124):
        points, box, periodic, options = configs.config3(replica)
        systems.append((points, box, tuple(bool(p) for p in np.broadcast_to(periodic, 3))))
    cutoff = options["cutoff"]
    for full in (True, False):
        calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
        capfd.readouterr()
        for call in ("first call", "second call"):
            _call_and_check(calculator, systems, cutoff, full, "PSdD", call)
            lines = _in_order_lines(capfd)
            assert len(lines) == 1 and lines[0].endswith(": used"), (call, lines)


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_thousands_of_rows_per_point(full, capfd, monkeypatch):
    """Boxes of half the cutoff: a point has several thousand neighbours, more than a wave lines up at a time. One
    system's box is large enough for the 27 nearest images, so that its pairs use one of the batch's two words; a box
    of less than half the cutoff needs more images than this search keeps, and the batch is then left to the sort."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(574)
    cutoff = 7.9
    systems = []
    for n, edge in ((200, 4.5), (33, 4.8), (256, 9.5), (3, 4.6)):
        box = np.eye(3) * edge + 0.2 * rng.normal(size=(3, 3))
        systems.append((rng.random((n, 3)) @ box + rng.integers(-1, 2, size=(n, 3)) @ box, box, (True, True, True)))
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
    capfd.readouterr()
    for call in ("first call", "second call"):
        _call_and_check(calculator, systems, cutoff, full, "PSdD", call)
        lines = _in_order_lines(capfd)
        assert len(lines) == 1 and lines[0].endswith(": used"), (call, lines)
    box = np.eye(3) * 3.0
    _call_and_check(calculator, systems + [(rng.random((20, 3)) @ box, box, (True, True, True))], cutoff, full, "PSd", "343 images")
    assert not _in_order_lines(capfd)


def test_a_list_that_grows_and_brute_force(capfd, monkeypatch):
    """More rows than the arrays of the list hold: the launch that would write them writes nothing and is repeated
    after the host made room. algorithm="brute_force" makes every system one cell; beyond 256 points the batch is
    left to the sort."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(572)
    cutoff = 3.0
    calculator = NeighborList(cutoff=cutoff, full_list=True, sorted=True, algorithm="brute_force")

    def systems_of(sizes, edge):
        return [(rng.random((n, 3)) * edge, np.eye(3) * edge, (True, True, True)) for n in sizes]

    capfd.readouterr()
    _call_and_check(calculator, systems_of([40, 50, 60], 9.0), cutoff, True, "PSdD", "sparse")
    _call_and_check(calculator, systems_of([40, 50, 60], 9.0), cutoff, True, "PSdD", "sparse again")
    _call_and_check(calculator, systems_of([250, 256, 200, 3], 9.0), cutoff, True, "PSdD", "dense")
    lines = _in_order_lines(capfd)
    assert len(lines) == 3 and all(line.endswith(": used") for line in lines), lines
    # a system of 300 points in one cell is left to the search over tiles, whose counting pass finds more candidates
    # around a tile than it holds: the rows come from the two passes and the sort, and the next call does not ask again
    _call_and_check(calculator, systems_of([300, 20], 9.0), cutoff, True, "PSdD", "too many points in one cell")
    lines = _in_order_lines(capfd)
    assert len(lines) == 1 and lines[0].endswith(": left to the radix sort"), lines
    _call_and_check(calculator, systems_of([30, 20], 9.0), cutoff, True, "PSdD", "small again")
    assert not _in_order_lines(capfd)
    another = NeighborList(cutoff=cutoff, full_list=True, sorted=True, algorithm="brute_force")
    _call_and_check(another, systems_of([30, 20], 9.0), cutoff, True, "PSdD", "small, another list")
    assert _in_order_lines(capfd)[-1].endswith(": used")


def test_molecules_whose_grids_are_picked_on_the_device(capfd, monkeypatch):
    """Systems without periodic directions get their grids on the device from the second call on: the host does not
    know their shapes then. In a sorted batch a molecule of up to 256 atoms is one cell however far it spreads (the
    search over images is at its best there), so such batches stay with that search; a larger molecule is not its
    to search: the kernels say so, the rows come from the two passes and the sort, and the next calls do not ask
    again for a while. (Batches of free molecules of up to 256 atoms have kernels of their own, which are switched
    off here: the general path is meant.)"""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    monkeypatch.setenv("VESIN_HIP_MOLECULES", "off")
    rng = np.random.default_rng(573)
    cutoff = 2.5
    sizes = [1, 2, 5, 17, 40, 31, 12, 3, 200]
    # (the molecules of 40 and of 200 atoms spread over several cutoffs: a cell list would give them many cells)
    molecules = [rng.normal(scale=3.0 if n >= 40 else 1.2, size=(n, 3)) + rng.uniform(-30, 30, size=3) for n in sizes]
    zero = np.zeros((3, 3))

    def systems():
        return [(m, zero, (False, False, False)) for m in molecules]

    calculator = NeighborList(cutoff=cutoff, full_list=True, sorted=True)
    capfd.readouterr()
    for call in range(4):
        _call_and_check(calculator, systems(), cutoff, True, "PSdD", f"call {call}")
        lines = _in_order_lines(capfd)
        assert len(lines) == 1 and lines[0].endswith(": used") and " 0 by tiles" in lines[0], (call, lines)
        assert ("grids picked on the device" in lines[0]) == (call >= 1), (call, lines)
        molecules = [m + rng.normal(scale=0.02, size=m.shape) for m in molecules]
    # with a molecule of 300 atoms: the host gives it to the search over tiles; the device's grids are only for the
    # search over images
    molecules.append(rng.normal(scale=3.0, size=(300, 3)))
    calculator = NeighborList(cutoff=cutoff, full_list=True, sorted=True)
    _call_and_check(calculator, systems(), cutoff, True, "PSdD", "with a large molecule, first call")
    lines = _in_order_lines(capfd)
    assert len(lines) == 1 and lines[0].endswith(": used") and " 1 by tiles" in lines[0], lines
    _call_and_check(calculator, systems(), cutoff, True, "PSdD", "second call")
    lines = _in_order_lines(capfd)
    assert len(lines) == 1 and lines[0].endswith(": left to the radix sort") and "grids picked on the device" in lines[0], lines
    _call_and_check(calculator, systems(), cutoff, True, "PSdD", "the call after")
    assert not _in_order_lines(capfd)


def _systems_of_several_cells(rng, sizes_and_flags):
    systems = []
    for n, flags in sizes_and_flags:
        edge = (n / 0.06) ** (1.0 / 3.0)
        box = np.eye(3) * edge + 0.05 * edge * rng.normal(size=(3, 3))
        moved = (rng.integers(-1, 2, size=(n, 3)) * np.array(flags)) @ box
        systems.append((rng.random((n, 3)) @ box + moved, box, flags))
    return systems


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_systems_of_several_cells_come_out_in_order(full, capfd, monkeypatch):
    """Systems of a few hundred to a few thousand points with several cells each (periodic, slabs, wires, clusters;
    points up to a box vector outside of the box), and the same together with systems of one cell: both searches in
    one call, one scan over the points of all systems."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(575)
    cutoff = 4.0
    several = _systems_of_several_cells(rng, [
        (700, (True, True, True)), (300, (True, True, False)), (1500, (True, False, False)), (450, (False, False, False)),
        (3000, (True, True, True)), (100, (True, True, True)),
    ])
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
    capfd.readouterr()
    for call, letters in (("first call", "PSdD"), ("second call", "PSdD"), ("third call", "Pd")):
        _call_and_check(calculator, several, cutoff, full, letters, call)
        lines = _in_order_lines(capfd)
        assert len(lines) == 1 and lines[0].endswith(": used") and " 0 systems by images" in lines[0], (call, lines)
    mixed = several[:3] + _small_cell_systems(rng) + several[3:]
    for call in ("mixed, first call", "mixed, second call"):
        _call_and_check(calculator, mixed, cutoff, full, "PSdD", call)
        lines = _in_order_lines(capfd)
        assert len(lines) == 1 and lines[0].endswith(": used") and " 0 systems by" not in lines[0], (call, lines)


def test_a_dense_system_among_the_others(capfd, monkeypatch):
    """One system with more candidates around a tile than the search over tiles holds (1024): its counting pass says
    so, nothing is written in order, and the rows of the whole batch come from the two passes and the sort."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(576)
    cutoff = 4.0
    systems = _systems_of_several_cells(rng, [(600, (True, True, True)), (900, (True, True, True))])
    edge = 20.3
    systems.append((rng.random((2500, 3)) * edge, np.eye(3) * edge, (True, True, True)))  # 0.3 per cubic A: 80 rows per point
    edge = 12.0
    systems.append((rng.random((2500, 3)) * edge, np.eye(3) * edge, (True, True, True)))  # 1.45 per cubic A: every point a candidate
    calculator = NeighborList(cutoff=cutoff, full_list=True, sorted=True)
    capfd.readouterr()
    _call_and_check(calculator, systems[:3], cutoff, True, "PSd", "up to 1024 candidates per tile")
    _call_and_check(calculator, systems[:3], cutoff, True, "PSd", "again")
    lines = _in_order_lines(capfd)
    assert len(lines) == 2 and all(line.endswith(": used") for line in lines), lines
    _call_and_check(calculator, systems, cutoff, True, "PSd", "more than 1024 candidates around a tile")
    lines = _in_order_lines(capfd)
    assert len(lines) == 1 and lines[0].endswith(": left to the radix sort"), lines
    _call_and_check(calculator, systems, cutoff, True, "PSd", "the call after")
    assert not _in_order_lines(capfd)


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_pairs_next_to_the_cutoff_in_systems_of_one_cell(full, capfd, monkeypatch):
    """The counting pass over images decides most pairs in single precision, from where the points are once they are
    moved into the box; pairs within rounding of the cutoff must come out as the reference's own arithmetic has them.
    Every system holds 60 pairs whose distance is the cutoff to within a few units in the last place, across the box's
    faces and with points up to three boxes outside; the same with every pair tested in double precision."""
    rng = np.random.default_rng(577)
    cutoff = 4.0
    systems = []
    n_close = 0
    for s in range(24):
        edge = rng.uniform(4.4, 7.5)
        box = np.eye(3) * edge + (0.3 * rng.normal(size=(3, 3)) if s % 2 else 0.0)
        first = rng.random((60, 3)) @ box
        direction = rng.normal(size=first.shape)
        direction /= np.linalg.norm(direction, axis=1)[:, None]
        steps = rng.integers(-6, 7, size=len(first)).astype(np.float64)
        second = first + direction * (cutoff * (1.0 + steps * 2.0**-52))[:, None]
        points = np.concatenate([first, second])
        if s % 3 == 0:
            points = points + rng.integers(-3, 4, size=points.shape) @ box
        systems.append((points, box, (True, True, True)))
        expected = oracle.neighbors(points, box, [True] * 3, cutoff, True, False, "ijd")
        n_close += int((np.abs(expected["distances"] - cutoff) < 1e-12).sum()) // 2
    assert 300 < n_close < 24 * 60  # about half of the pairs made for it are in, and crowd the cutoff
    for tests in ("single precision first", "double"):
        if tests == "double":
            monkeypatch.setenv("VESIN_HIP_TESTS", "double")
        monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
        calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
        capfd.readouterr()
        for call in ("first call", "second call"):
            _call_and_check(calculator, systems, cutoff, full, "PSdD", f"{tests}, {call}")
            lines = _in_order_lines(capfd)
            assert len(lines) == 1 and lines[0].endswith(": used"), (tests, call, lines)


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_batches_whose_systems_all_have_few_points(full, capfd, monkeypatch):
    """No system with more than 32 points: every system is searched by one wave instead of one workgroup. Crystals of
    1 to 32 atoms in boxes of every shape (up to 125 images, wraps), slabs, and free molecules, whose grids are picked
    on the device from the second call on; several hundred systems, so that workgroups hold four of them, some none."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(578)
    cutoff = 4.2
    crystals = []
    for k in range(301):
        n = int(rng.integers(0, 33))
        edge = rng.uniform(2.2, 7.5) if k % 3 else rng.uniform(4.5, 7.5)
        box = np.eye(3) * edge + 0.2 * rng.normal(size=(3, 3))
        flags = (True, True, True) if k % 5 else (True, False, True)
        moved = (rng.integers(-2, 3, size=(n, 3)) * np.array(flags)) @ box
        crystals.append((rng.random((n, 3)) @ box + moved, box, flags))
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
    capfd.readouterr()
    for call in ("first call", "second call"):
        _call_and_check(calculator, crystals, cutoff, full, "PSdD", f"crystals, {call}")
        lines = _in_order_lines(capfd)
        assert len(lines) == 1 and lines[0].endswith(": used"), (call, lines)
    molecules = [(rng.normal(scale=1.5, size=(int(rng.integers(1, 33)), 3)) + rng.uniform(-40, 40, size=3), np.zeros((3, 3)),
                  (False, False, False)) for _ in range(203)]
    # (batches of free molecules have kernels of their own from their second call on: here the general path is meant)
    monkeypatch.setenv("VESIN_HIP_MOLECULES", "off")
    for call in range(3):
        _call_and_check(calculator, molecules, cutoff, full, "PSd", f"molecules, call {call}")
        lines = _in_order_lines(capfd)
        assert len(lines) == 1 and lines[0].endswith(": used"), (call, lines)
        assert ("grids picked on the device" in lines[0]) == (call >= 1), (call, lines)
        molecules = [(m[0] + rng.normal(scale=0.03, size=m[0].shape), m[1], m[2]) for m in molecules]
    monkeypatch.delenv("VESIN_HIP_MOLECULES")
    for call in range(2):
        capfd.readouterr()
        _call_and_check(calculator, molecules, cutoff, full, "PSd", f"molecules with their own kernels, call {call}")
        assert "batch of free molecules" in capfd.readouterr().err
