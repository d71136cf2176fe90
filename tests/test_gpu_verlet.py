"""options.skin > 0 (Verlet caching): whatever the cache does, the rows are those of a direct calculation.

The cases are the reference's own (python/vesin/tests/test_numpy.py:405-551), checked against the CPU oracle at
the cutoff instead of against a second calculator, plus larger systems where the filter runs over many chunks.
"""

import ctypes

import numpy as np
import pytest

import oracle
from vesin_amd import NeighborList, configs
from vesin_amd._c_api import VesinCUDA, VesinDevice, VesinNeighborList, VesinOptions, get_library

pytestmark = pytest.mark.gpu


def _compute(calculator, points, box, periodic, quantities="PSdD"):
    import torch

    outputs = calculator.compute(
        torch.tensor(np.ascontiguousarray(points), device="cuda:0"),
        torch.tensor(np.ascontiguousarray(box), device="cuda:0"),
        periodic,
        quantities,
    )
    names = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}
    return {names[q]: out.cpu().numpy() for q, out in zip(quantities, outputs)}


def _assert_direct(result, points, box, periodic, cutoff, full, ordered=False):
    flags = [bool(periodic)] * 3 if isinstance(periodic, (bool, np.bool_)) else list(periodic)
    expected = oracle.canonicalize(oracle.neighbors(points, box, flags, cutoff, full, False, "ijSdD"))
    got = result if ordered else oracle.canonicalize(result)
    assert got["pairs"].shape == expected["pairs"].shape
    for key in got:
        assert np.array_equal(got[key], expected[key]), key


@pytest.mark.parametrize("cutoff,full_list", [(3.0, True), (3.0, False), (1.5, True)])
def test_verlet_matches_direct(cutoff, full_list):
    points = np.array([[0.0, 0.0, 0.0], [1.0, 0.0, 0.0], [0.0, 1.0, 0.0]])
    box = 10 * np.eye(3)
    calculator = NeighborList(cutoff=cutoff, full_list=full_list, skin=1.5)
    for _ in range(3):
        _assert_direct(_compute(calculator, points, box, True), points, box, True, cutoff, full_list)


def test_verlet_pair_gets_inside_cutoff():
    """A pair outside the cutoff but inside the skin appears on the second call, which only filters."""
    calculator = NeighborList(cutoff=1.0, full_list=False, skin=0.5)
    box = 10.0 * np.eye(3)

    points = np.array([[0.0, 0.0, 0.0], [1.10, 0.0, 0.0]])
    result = _compute(calculator, points, box, False, "Pd")
    assert len(result["pairs"]) == 0

    points = np.array([[0.0, 0.0, 0.0], [0.95, 0.0, 0.0]])
    result = _compute(calculator, points, box, False, "Pd")
    assert result["pairs"].tolist() == [[0, 1]]
    assert result["distances"].tolist() == [0.95]


def test_verlet_non_periodic():
    points = np.array(
        [
            [0.134, 1.282, 1.701],
            [-0.273, 1.026, -1.471],
            [1.922, -0.124, 1.900],
            [1.400, -0.464, 0.480],
            [0.149, 1.865, 0.635],
        ]
    )
    box = np.zeros((3, 3))
    calculator = NeighborList(cutoff=3.42, full_list=False, skin=0.5)
    for _ in range(2):
        _assert_direct(_compute(calculator, points, box, False), points, box, False, 3.42, False)


def test_verlet_trajectory():
    rng = np.random.default_rng(7)
    points = np.array([[0.0, 0.0, 0.0], [1.5, 0.0, 0.0], [0.0, 1.5, 0.0], [0.0, 0.0, 1.5]])
    box = 5.0 * np.eye(3)
    skin = 0.5
    calculator = NeighborList(cutoff=3.0, full_list=False, skin=skin)
    initial = points.copy()
    for _ in range(100):
        points = points + 0.1 * rng.normal(size=points.shape)
        _assert_direct(_compute(calculator, points, box, True), points, box, True, 3.0, False)
    assert np.any(np.linalg.norm(points - initial, axis=1) > skin)


def test_verlet_trajectory_changing_box():
    """Anisotropic scaling and shear of the box, sometimes large enough to use up the skin."""
    rng = np.random.default_rng(0)
    points = np.array(
        [[0.0, 0.0, 0.0], [1.5, 0.0, 0.0], [0.0, 1.5, 0.0], [0.0, 0.0, 1.5], [1.5, 1.5, 1.5]]
    )
    base = 5.0 * np.eye(3)
    calculator = NeighborList(cutoff=3.0, full_list=False, skin=0.5)
    for _ in range(100):
        points = points + 0.05 * rng.normal(size=points.shape)
        box = base + 0.3 * rng.normal(size=(3, 3))
        _assert_direct(_compute(calculator, points, box, True), points, box, True, 3.0, False)


def test_verlet_trajectory_small_box_changes():
    """Deformations well inside the skin: most calls filter candidates made for another box."""
    rng = np.random.default_rng(1)
    points, box0, periodic = configs.diamond(3, seed=4)
    calculator = NeighborList(cutoff=4.0, full_list=True, skin=1.0)
    for _ in range(30):
        points = points + 0.01 * rng.normal(size=points.shape)
        box = box0 + 0.02 * rng.normal(size=(3, 3))
        _assert_direct(_compute(calculator, points, box, True), points, box, True, 4.0, True)


def test_verlet_trajectory_changing_box_mixed_pbc():
    rng = np.random.default_rng(0)
    points = rng.uniform(-2.0, 2.0, size=(8, 3))
    periodic = [True, True, False]
    calculator = NeighborList(cutoff=3.0, full_list=False, skin=0.5)
    for _ in range(100):
        points = points + 0.05 * rng.normal(size=points.shape)
        box = np.diag([5.0, 5.0, 20.0])
        box[:2, :2] += 0.3 * rng.normal(size=(2, 2))
        _assert_direct(_compute(calculator, points, box, periodic), points, box, periodic, 3.0, False)


@pytest.mark.parametrize("full_list", [True, False])
@pytest.mark.parametrize("sorted_rows", [True, False])
def test_verlet_crystal_trajectory(full_list, sorted_rows):
    """1728 atoms: thousands of candidate chunks per call; small steps that the filter absorbs, then a jump."""
    rng = np.random.default_rng(12)
    points, box, periodic = configs.diamond(6, seed=9)
    calculator = NeighborList(cutoff=5.0, full_list=full_list, sorted=sorted_rows, skin=0.8)
    for step in range(12):
        scale = 0.5 if step == 7 else 0.02
        points = points + scale * rng.normal(size=points.shape)
        result = _compute(calculator, points, box, True)
        _assert_direct(result, points, box, True, 5.0, full_list, ordered=sorted_rows)


@pytest.mark.parametrize("quantities", ["P", "PS", "Pd", "PD", "PdD"])
def test_verlet_quantities(quantities):
    points, box, periodic = configs.diamond(3, seed=2)
    calculator = NeighborList(cutoff=4.5, full_list=True, sorted=True, skin=0.6)
    expected = oracle.canonicalize(oracle.neighbors(points, box, [True] * 3, 4.5, True, False, "ijSdD"))
    names = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}
    for _ in range(2):
        result = _compute(calculator, points, box, True, quantities)
        for letter in quantities:
            assert np.array_equal(result[names[letter]], expected[names[letter]]), letter


@pytest.mark.parametrize("mode", ["cache", "direct", None])
def test_verlet_million_candidates(mode, monkeypatch):
    """125,000 atoms (11 M rows, 19 M candidates). Left alone, the library searches lists of this length directly
    on every call instead of filtering; VESIN_HIP_VERLET=cache keeps it on the filter (grid-stride loop over the
    candidates, growth of the arrays)."""
    from golden import systems

    if mode is None:
        monkeypatch.delenv("VESIN_HIP_VERLET", raising=False)
    else:
        monkeypatch.setenv("VESIN_HIP_VERLET", mode)

    rng = np.random.default_rng(3)
    points, box, periodic = configs.diamond(25, seed=6)
    calculator = NeighborList(cutoff=5.0, full_list=True, skin=1.0)
    direct = NeighborList(cutoff=5.0, full_list=True)
    for _ in range(3):
        points = points + 0.03 * rng.normal(size=points.shape)
        result = _compute(calculator, points, box, True, "PSd")
        reference = _compute(direct, points, box, True, "PSd")
        assert len(result["pairs"]) == len(reference["pairs"])
        assert systems.fingerprints(result) == systems.fingerprints(reference)


@pytest.mark.parametrize("mode", ["cache", "direct"])
def test_verlet_forced_modes_on_a_small_system(mode, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_VERLET", mode)
    rng = np.random.default_rng(5)
    points, box, periodic = configs.diamond(3, seed=3)
    calculator = NeighborList(cutoff=4.0, full_list=False, skin=0.7)
    for _ in range(6):
        points = points + 0.05 * rng.normal(size=points.shape)
        _assert_direct(_compute(calculator, points, box, True), points, box, True, 4.0, False)


def test_verlet_system_that_grows_past_the_filter():
    """One list, first with few points (cached candidates), then with many (direct search), then few again."""
    rng = np.random.default_rng(8)
    small = configs.diamond(3, seed=1)
    large = configs.diamond(14, seed=2)
    calculator = NeighborList(cutoff=5.0, full_list=True, skin=0.5)
    for points, box, periodic in (small, small, large, large, small, small):
        points = points + 0.01 * rng.normal(size=points.shape)
        _assert_direct(_compute(calculator, points, box, True), points, box, True, 5.0, True)


def _raw_call(lib, neighbors, points, box, periodic, cutoff, skin, full=True):
    options = VesinOptions()
    options.cutoff = cutoff
    options.full = full
    options.sorted = True
    options.return_shifts = True
    options.return_distances = True
    options.return_vectors = True
    options.skin = skin
    message = ctypes.c_char_p()
    status = lib.vesin_neighbors(
        points.data_ptr(), points.shape[0], box.data_ptr(), periodic.data_ptr(), VesinDevice(VesinCUDA, 0), options,
        ctypes.byref(neighbors), ctypes.byref(message),
    )
    assert status == 0, message.value


def test_verlet_options_and_sizes_change_on_one_list():
    """One VesinNeighborList through changes that invalidate the cache: cutoff, skin, full, number of points, and
    back to no skin at all (vesin/src/verlet.cpp:48-54, :65-71; vesin/src/cpu_cell_list.cpp:235-238)."""
    import torch

    from test_gpu_stream import _to_host

    lib = get_library()
    points, box, periodic = configs.diamond(3, seed=8)
    device_box = torch.tensor(box, device="cuda:0")
    device_periodic = torch.tensor(periodic, device="cuda:0")
    neighbors = VesinNeighborList()
    steps = [
        (4.0, 0.5, True, 216), (4.0, 0.5, True, 216), (4.5, 0.5, True, 216), (4.5, 0.9, True, 216),
        (4.5, 0.9, False, 216), (4.5, 0.9, False, 150), (4.5, 0.9, False, 216), (4.5, 0.0, False, 216),
        (4.5, 0.3, True, 216),
    ]
    try:
        for cutoff, skin, full, n in steps:
            device_points = torch.tensor(points[:n], device="cuda:0")
            _raw_call(lib, neighbors, device_points, device_box, device_periodic, cutoff, skin, full)
            result = _to_host(neighbors)
            expected = oracle.canonicalize(oracle.neighbors(points[:n], box, [True] * 3, cutoff, full, False, "ijSdD"))
            for key in ("pairs", "shifts", "distances", "vectors"):
                assert np.array_equal(result[key], expected[key]), (cutoff, skin, full, n, key)
    finally:
        lib.vesin_free(ctypes.byref(neighbors))


def test_verlet_no_points_and_no_pairs():
    calculator = NeighborList(cutoff=1.0, full_list=True, skin=0.3)
    box = 10.0 * np.eye(3)
    result = _compute(calculator, np.zeros((0, 3)), box, True)
    assert result["pairs"].shape == (0, 2) and result["vectors"].shape == (0, 3)
    result = _compute(calculator, np.array([[0.0, 0.0, 0.0], [5.0, 5.0, 5.0]]), box, True)
    assert result["pairs"].shape == (0, 2)
    result = _compute(calculator, np.array([[0.0, 0.0, 0.0], [0.5, 0.0, 0.0]]), box, True)
    assert sorted(result["pairs"].tolist()) == [[0, 1], [1, 0]]


@pytest.mark.parametrize("full_list", [True, False])
def test_verlet_points_given_several_boxes_outside_of_a_box_that_changes(full_list):
    """Points given up to three boxes outside of the box make pairs with shifts of up to seven boxes, and the image
    of such a pair moves seven times as far as a corner of the box when the box changes: the reference's bound on the
    change of the box (vesin/src/verlet.cpp:10-34, :80-84) covers the images one box away. The rows must be those of
    a direct calculation all the same: the cache knows the largest shift among its candidates and rebuilds earlier."""
    rng = np.random.default_rng(2158)
    cutoff, skin = 1.1, 0.3
    box = np.array([[3.735, 0.0, 0.0], [-0.261, 3.735, 0.0], [-0.43, 0.357, 3.735]])
    points = rng.random((600, 3)) @ box + rng.integers(-3, 4, size=(600, 3)) @ box
    calculator = NeighborList(cutoff=cutoff, full_list=full_list, skin=skin)
    checked = 0
    for step in range(12):
        result = _compute(calculator, points, box, True)
        _assert_direct(result, points, box, True, cutoff, full_list)
        checked += len(result["pairs"])
        # small moves, which alone would let the cache live on, and a box that changes by up to 0.03 per element
        points = points + rng.normal(scale=0.01, size=points.shape)
        if step % 2 == 0:
            box = box + rng.normal(scale=0.015, size=(3, 3)) * (np.abs(box) > 0)
    assert checked > 100000 and np.abs(result["shifts"]).max() >= 5
