"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real MI355X (``-m gpu``).

The bar: identical (i, j, S) sets; ``sorted=True`` output identical, row by row, to the lexicographically ordered
CPU list; distances and vectors bit-identical (the acceptance bar is 1e-12 relative; pairs whose distance lies
within 1e-12 * cutoff of the cutoff would be reported separately -- with identical arithmetic there are none to
excuse, and the count is asserted to be what the oracle has).
"""

import json
import os

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list, gpu_neighbors, near_cutoff_count
from golden import systems
from vesin_amd import configs

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.realpath(__file__))
with open(os.path.join(HERE, "golden", "reference_checksums.json")) as fd:
    GOLDEN = json.load(fd)

SMALL = systems.small_systems()


@pytest.mark.parametrize("name", list(SMALL))
@pytest.mark.parametrize("cutoff", [3.0, 5.0, 7.0, 10.0])
@pytest.mark.parametrize("full", [True, False])
@pytest.mark.parametrize("algorithm", ["cell_list", "brute_force", "auto"])
def test_small_systems(name, cutoff, full, algorithm):
    # the design of python/vesin/tests/test_gpu_consistency.py:43-106; unlike the reference's brute force, this one
    # also serves cutoffs above half the box
    points, box, periodic = SMALL[name]
    expected = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
    actual = gpu_neighbors(points, box, periodic, cutoff, full, False, "ijSdD", algorithm)
    assert_same_list(actual, expected, what=f"{name} rc={cutoff} full={full} {algorithm}")
    ordered = gpu_neighbors(points, box, periodic, cutoff, full, True, "ijSdD", algorithm)
    assert_same_list(ordered, expected, ordered=True, what=f"{name} rc={cutoff} full={full} {algorithm} sorted")


@pytest.mark.parametrize("name", list(SMALL))
@pytest.mark.parametrize("seed,translate", [(11, False), (12, True), (13, True)])
def test_rotated_and_translated(name, seed, translate):
    points, box, periodic = systems.transformed(SMALL[name], seed, translate)
    for algorithm in ("cell_list", "brute_force"):
        expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
        actual = gpu_neighbors(points, box, periodic, 5.0, True, False, "ijSdD", algorithm)
        assert_same_list(actual, expected, what=f"{name} seed={seed} {algorithm}")


@pytest.mark.parametrize("mask", range(8))
@pytest.mark.parametrize("full", [True, False])
def test_mixed_periodicity(mask, full):
    # python/vesin/tests/test_numpy.py:231-269
    periodic = [(mask >> d) & 1 == 1 for d in range(3)]
    points, box, periodic = systems.mixed_periodic(periodic)
    expected = oracle.neighbors(points, box, periodic, 0.35, full, False, "ijSdD")
    for algorithm in ("cell_list", "brute_force"):
        actual = gpu_neighbors(points, box, periodic, 0.35, full, True, "ijSdD", algorithm)
        assert_same_list(actual, expected, ordered=True, what=f"mixed {periodic} {algorithm}")


@pytest.mark.parametrize("quantities", ["ij", "ijS", "ijd", "ijD", "ijSd", "ijdD"])
@pytest.mark.parametrize("sorted_", [False, True])
def test_every_combination_of_outputs(quantities, sorted_):
    points, box, periodic = systems.diamond_crystal()
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    actual = gpu_neighbors(points, box, periodic, 5.0, True, sorted_, quantities)
    assert set(actual) == {"pairs"} | {{"S": "shifts", "d": "distances", "D": "vectors"}[q] for q in quantities if q in "SdD"}
    if sorted_:
        # canonical order even when the shifts were not asked for
        trimmed = {k: v for k, v in oracle.canonicalize(expected).items() if k in actual}
        for key in actual:
            assert np.array_equal(actual[key], trimmed[key]), key
    elif "S" in quantities:
        assert_same_list(actual, {k: v for k, v in expected.items() if k in actual})
    else:
        assert sorted(map(tuple, actual["pairs"].tolist())) == sorted(map(tuple, expected["pairs"].tolist()))


def test_points_far_outside_the_box():
    # wrap shifts of hundreds of box lengths, different per point: exercises the per-point shift path
    rng = np.random.default_rng(5)
    points, box, periodic = systems.read_xyz("carbon")
    points = points + rng.integers(-300, 300, size=(len(points), 3)).astype(float) @ box
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    for algorithm in ("cell_list", "brute_force"):
        actual = gpu_neighbors(points, box, periodic, 5.0, True, True, "ijSdD", algorithm)
        assert_same_list(actual, expected, ordered=True, what=algorithm)


@pytest.mark.parametrize("shape", ["orthorhombic", "rotated", "sheared", "slab", "flat-cells"])
@pytest.mark.parametrize("full", [True, False])
def test_stencils_of_several_cells_per_direction(shape, full):
    # Boxes much narrower than the cutoff: stencils of radius 2 to 5, different per direction. In a box of
    # orthogonal vectors the entries at the corners of the stencil cannot hold a neighbour and are dropped; a pair
    # dropped with them would be missing here. "sheared" has no such shortcut, "rotated" has it although no
    # component of its matrix is zero, "slab" mixes it with an open direction, "flat-cells" has several cells along
    # the long direction and images along the short ones. Points lie in and around the box.
    rng = np.random.default_rng(77)
    box = np.diag([3.1, 4.3, 5.7])
    periodic = [True, True, True]
    n_points = 40
    if shape == "rotated":
        q, _ = np.linalg.qr(rng.normal(size=(3, 3)))
        box = box @ q
    elif shape == "sheared":
        box[1, 0] = 0.9
        box[2, 1] = -1.3
    elif shape == "slab":
        periodic = [True, False, True]
    elif shape == "flat-cells":
        box = np.diag([3.1, 4.3, 61.0])
        n_points = 300
    points = (rng.random((n_points, 3)) * 1.6 - 0.3) @ box
    for cutoff in (6.0, 9.5):
        expected = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
        for algorithm in ("cell_list", "brute_force"):
            actual = gpu_neighbors(points, box, periodic, cutoff, full, False, "ijSdD", algorithm)
            assert_same_list(actual, expected, what=f"{shape} rc={cutoff} {algorithm}")
            ordered = gpu_neighbors(points, box, periodic, cutoff, full, True, "ijSdD", algorithm)
            assert_same_list(ordered, expected, ordered=True, what=f"{shape} rc={cutoff} {algorithm} sorted")


def test_coincident_points_are_neighbours():
    # the CPU engine keeps distinct points at zero distance (the reference's CUDA kernel drops them,
    # vesin/src/cuda/cell_list.cu:631); this path follows the CPU
    points = np.array([[1.0, 1.0, 1.0], [1.0, 1.0, 1.0], [2.0, 1.0, 1.0]])
    expected = oracle.neighbors(points, np.eye(3) * 10, True, 1.5, True, False, "ijSdD")
    actual = gpu_neighbors(points, np.eye(3) * 10, True, 1.5, True, False, "ijSdD")
    assert_same_list(actual, expected)
    assert len(actual["pairs"]) == 6 and np.sum(actual["distances"] == 0.0) == 2


def test_heavy_cell_and_many_tiles():
    # 3000 points inside one cutoff-sized cell: many tiles, canonical ordering of a crowded cell
    rng = np.random.default_rng(8)
    points = rng.random((3000, 3)) * 2.0 + 20.0
    box = np.eye(3) * 60.0
    expected = oracle.neighbors(points, box, True, 0.4, True, False, "ijSd")
    for algorithm in ("cell_list", "brute_force"):
        actual = gpu_neighbors(points, box, True, 0.4, True, False, "ijSd", algorithm)
        assert_same_list(actual, expected, what=algorithm)


REDUCED = [
    ("config0", lambda: configs.config0()),
    ("config1-8cubed", lambda: configs.config1(8)),
    ("config2-5k", lambda: configs.config2(5000)),
    ("config3-replica0", lambda: configs.config3(0)),
    ("config3-replica4095", lambda: configs.config3(4095)),
    ("config4a-20k", lambda: configs.config4(20000, (False, False, False))),
    ("config4b-20k", lambda: configs.config4(20000, (True, True, False))),
]


@pytest.mark.parametrize("name,make", REDUCED, ids=[r[0] for r in REDUCED])
def test_reduced_configs_against_oracle_and_golden(name, make):
    points, box, periodic, options = make()
    full = options["full_list"]
    expected = oracle.neighbors(points, box, periodic, options["cutoff"], full, False, "ijSdD")
    actual = gpu_neighbors(points, box, periodic, options["cutoff"], full, options["sorted"], "ijSdD")
    assert_same_list(actual, expected, ordered=options["sorted"], what=name)
    assert near_cutoff_count(actual, options["cutoff"]) == near_cutoff_count(expected, options["cutoff"])
    prints = systems.fingerprints(actual)
    for key in ("n_pairs", "ijS", "d", "D"):
        assert prints[key] == GOLDEN[name][key], f"{name}: {key} differs from the compiled reference's fingerprint"


def check_properties(result, points, box, periodic, cutoff, full, is_sorted):
    """Size-independent checks for lists too large to compare row by row on the host in seconds."""
    pairs = result["pairs"]
    i = pairs[:, 0].astype(np.int64)
    j = pairs[:, 1].astype(np.int64)
    n = len(points)
    assert i.min() >= 0 and i.max() < n and j.min() >= 0 and j.max() < n
    H = np.asarray(box, dtype=np.float64).copy()
    H[~np.asarray(periodic, dtype=bool)] = 0.0
    S = result["shifts"] if "shifts" in result else np.zeros((len(i), 3), dtype=np.int32)
    if "distances" in result:
        assert np.all(result["distances"] < cutoff)
        # sample: the definition r_j - r_i + S.H, recomputed
        pick = np.random.default_rng(0).integers(0, len(i), size=min(len(i), 2_000_000))
        vectors = points[j[pick]] - points[i[pick]] + S[pick].astype(np.float64) @ H
        # (numpy's own rounding of the shifted difference bounds this check, not the kernel: the bitwise comparison
        # is the fingerprint test)
        assert np.allclose(np.linalg.norm(vectors, axis=1), result["distances"][pick], rtol=1e-12, atol=1e-11)
        if "vectors" in result:
            assert np.allclose(vectors, result["vectors"][pick], rtol=1e-12, atol=1e-11)
    if is_sorted:
        assert np.all(np.diff(i) >= 0)
    if not full:
        assert np.all(i <= j)
    return i, j, S


def test_config1_full_size():
    """1,000,000 atoms, 89 M pairs: order-independent fingerprints against the compiled reference, plus the
    symmetry of a full list (every (i, j, S) has its (j, i, -S))."""
    points, box, periodic, options = configs.config1()
    result = gpu_neighbors(points, box, periodic, options["cutoff"], True, False, "ijSd")
    golden = GOLDEN["config1"]
    prints = systems.fingerprints(result)
    assert prints["n_pairs"] == golden["n_pairs"] == 89117880
    assert prints["ijS"] == golden["ijS"]
    assert prints["d"] == golden["d"]
    i, j, S = check_properties(result, points, box, periodic, options["cutoff"], True, False)
    mirrored = systems.fingerprints({"pairs": np.stack([j, i], axis=1).astype(np.uint64), "shifts": -S})
    assert mirrored["ijS"] == prints["ijS"]
    # per-point degree is what a diamond lattice with 0.05 A jitter gives: 86 within 5 A plus the tail of the next shell
    degree = np.bincount(i, minlength=len(points))
    assert degree.min() >= 86 and degree.max() <= 100


def test_config2_full_size_sorted_half():
    points, box, periodic, options = configs.config2()
    result = gpu_neighbors(points, box, periodic, options["cutoff"], False, True, "ijSdD")
    golden = GOLDEN["config2"]
    prints = systems.fingerprints(result)
    for key in ("n_pairs", "ijS", "d", "D"):
        assert prints[key] == golden[key], key
    check_properties(result, points, box, periodic, options["cutoff"], False, True)
    # full lexicographic order, without re-sorting the GPU side
    order = oracle.canonical_order(result["pairs"], result["shifts"])
    assert np.array_equal(order, np.arange(len(order)))


@pytest.mark.parametrize("which", ["config4a", "config4b"])
def test_config4_full_size(which):
    periodic = (False, False, False) if which == "config4a" else (True, True, False)
    points, box, periodic, options = configs.config4(periodic=periodic)
    result = gpu_neighbors(points, box, periodic, options["cutoff"], True, False, "ijd")
    golden = GOLDEN[which]
    assert len(result["pairs"]) == golden["n_pairs"]
    # the golden fingerprints include the shifts: compare on the pair-and-distance level by recomputing them without
    full = gpu_neighbors(points, box, periodic, options["cutoff"], True, False, "ijSd")
    prints = systems.fingerprints(full)
    assert prints["ijS"] == golden["ijS"] and prints["d"] == golden["d"]
    check_properties(full, points, box, periodic, options["cutoff"], True, False)
    # independent of the requested outputs (rows of an unsorted list come in order of arrival: compare as sets)
    without_shifts = {"pairs": full["pairs"], "distances": full["distances"]}
    assert systems.fingerprints(result) == systems.fingerprints(without_shifts)


def test_config3_batch_of_replicas():
    """The small-cell, many-image case: 64 atoms, cutoff above the box. Replicas go through the stock entry point
    one call each; a few are compared row by row, a larger sample by fingerprint of the oracle."""
    for replica in (0, 1, 2, 3, 4095):
        points, box, periodic, options = configs.config3(replica)
        expected = oracle.neighbors(points, box, periodic, options["cutoff"], True, False, "ijSd")
        actual = gpu_neighbors(points, box, periodic, options["cutoff"], True, False, "ijSd")
        assert_same_list(actual, expected, what=f"replica {replica}")
        assert np.abs(actual["shifts"]).max() == 2
    for name in ("config3-replica0", "config3-replica1", "config3-replica4095"):
        replica = int(name.split("replica")[1])
        points, box, periodic, options = configs.config3(replica)
        actual = gpu_neighbors(points, box, periodic, options["cutoff"], True, False, "ijSdD")
        prints = systems.fingerprints(actual)
        for key in ("n_pairs", "ijS", "d", "D"):
            assert prints[key] == GOLDEN[name][key]


def test_same_output_twice(monkeypatch):
    # a sorted list is the same array on every run; an unsorted one is when the rows are asked to be ordered
    points, box, periodic, options = configs.config1(12)
    first = gpu_neighbors(points, box, periodic, 5.0, True, True, "ijSdD")
    second = gpu_neighbors(points, box, periodic, 5.0, True, True, "ijSdD")
    for key in first:
        assert np.array_equal(first[key], second[key]), key
    monkeypatch.setenv("VESIN_HIP_ROWS", "ordered")
    first = gpu_neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    second = gpu_neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    for key in first:
        assert np.array_equal(first[key], second[key]), key


@pytest.mark.parametrize("n_points", [300, 6000], ids=["one launch", "searches of the large systems"])
@pytest.mark.parametrize("periodic", [True, False], ids=["periodic", "open"])
def test_zeros_of_both_signs_keep_their_sign_in_the_vectors(n_points, periodic):
    """Coordinates that are +0.0 and -0.0: a component of r_j - r_i is then -0.0 or +0.0 depending on which zero is
    whose, and the reference adds the shift vector to it, whose components for a zero shift are zeros of a sign that
    follows the signs of the box (vesin/src/cpu_cell_list.cpp:135-138, vesin/src/types.hpp:232-243): the vectors of
    the rows must have the reference's bits, signs of zero included, on every path (first call of a list and
    reused list, sorted and not, full and half)."""
    rng = np.random.default_rng(202)
    edge = 9.0 if n_points == 300 else 24.0
    # (a column of the box with negative entries only makes that component of the zero shift's vector -0.0, and only
    # then does a difference of -0.0 keep its sign)
    box = np.diag([edge, -edge, edge]) + np.array([[0.0, -0.3, 0.0], [0.5, 0.0, 0.0], [0.0, -0.4, 0.0]])
    points = rng.random((n_points, 3)) @ np.abs(box)
    # a cluster of points on the planes through the origin, zeros of both signs among their coordinates
    for k in range(60):
        axis = k % 3
        points[k] = rng.random(3) * 1.5
        points[k, axis] = 0.0 if k % 2 == 0 else -0.0
        if k % 5 == 0:
            points[k, (axis + 1) % 3] = -0.0
    cutoff = 2.5
    for full in (True, False):
        for is_sorted in (False, True):
            expected = oracle.canonicalize(oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD"))
            actual = gpu_neighbors(points, box, periodic, cutoff, full=full, sorted=is_sorted)
            what = f"full={full} sorted={is_sorted}"
            assert_same_list(actual, expected, ordered=is_sorted, what=what)
            actual = oracle.canonicalize(actual)
            negative_zeros = np.signbit(expected["vectors"]) & (expected["vectors"] == 0.0)
            positive_zeros = ~np.signbit(expected["vectors"]) & (expected["vectors"] == 0.0)
            assert np.any(positive_zeros) and (np.any(negative_zeros) or not periodic), "the case lost its point"
            assert np.array_equal(
                actual["vectors"].view(np.uint64), expected["vectors"].view(np.uint64)
            ), f"{what}: vectors differ in the sign of a zero"
