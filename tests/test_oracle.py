"""Pins the CPU oracle (oracle/vesin_oracle.c), on the CPU:

* against fingerprints of the compiled reference for every golden case (tests/golden/reference_checksums.json,
  written by tests/golden/make_golden.py) -- counts, (i, j, S) sets, bits of distances and vectors;
* against the compiled reference itself, raw output order included, when oracle/_ref is present;
* against an independent numpy brute force over all periodic images (catches a dropped term, a wrong sign, a
  transposed box);
* against what the mathematics fixes: orthorhombic closed forms for the grid, symmetry of the full list, the half-list
  rule keeping exactly one of {S, -S}.
"""

import itertools
import json
import os

import numpy as np
import pytest

import oracle
from golden import systems

HERE = os.path.dirname(os.path.realpath(__file__))
with open(os.path.join(HERE, "golden", "reference_checksums.json")) as fd:
    GOLDEN = json.load(fd)

SMALL_CASES = list(systems.golden_cases(full_size=False))


@pytest.mark.parametrize("case", SMALL_CASES, ids=[c[0] for c in SMALL_CASES])
def test_oracle_matches_reference_fingerprints(case):
    name, points, box, periodic, cutoff, full = case
    result = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
    actual = systems.fingerprints(result)
    expected = GOLDEN[name]
    for key in ("n_pairs", "ijS", "d", "D"):
        assert actual[key] == expected[key], f"{name}: {key}"


@pytest.mark.skipif(not oracle.have_ref(), reason="compiled reference (oracle/_ref) not present")
@pytest.mark.parametrize("case", SMALL_CASES[::7], ids=[c[0] for c in SMALL_CASES[::7]])
def test_oracle_equals_compiled_reference_row_by_row(case):
    name, points, box, periodic, cutoff, full = case
    ours = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
    theirs = oracle.ref_neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
    for key in ("pairs", "shifts", "distances", "vectors"):
        # same rows in the same order: the oracle keeps the reference's cell-major enumeration
        assert np.array_equal(ours[key], theirs[key]), f"{name}: {key}"


@pytest.mark.skipif(not oracle.have_ref(), reason="compiled reference (oracle/_ref) not present")
def test_thread_count_does_not_change_the_output():
    points, box, periodic = systems.diamond_crystal()
    base = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD", n_threads=1)
    for threads in (2, 3, 8):
        other = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD", n_threads=threads)
        for key in base:
            assert np.array_equal(base[key], other[key])


def brute_force(points, box, periodic, cutoff, full):
    """All (i, j, S) with |r_j - r_i + S.H| < cutoff by direct enumeration in numpy, S over a range that provably
    covers the cutoff sphere. Independent of any cell list."""
    points = np.asarray(points, dtype=np.float64)
    box = np.asarray(box, dtype=np.float64).copy()
    periodic = np.asarray(periodic, dtype=bool)
    n = len(points)
    ranges = []
    spread = np.ptp(points, axis=0).max() if n else 0.0
    for d in range(3):
        if not periodic[d]:
            ranges.append([0])
            box[d] = 0.0
            continue
        others = [box[e] for e in range(3) if e != d and periodic[e]]
        # height of the cell along d, ignoring non-periodic directions
        if len(others) == 2:
            normal = np.cross(others[0], others[1])
        elif len(others) == 1:
            normal = np.cross(np.cross(others[0], box[d]), others[0])
        else:
            normal = box[d]
        height = abs(np.dot(normal / np.linalg.norm(normal), box[d]))
        m = int(np.ceil((cutoff + spread * np.sqrt(3)) / height)) + 1
        ranges.append(list(range(-m, m + 1)))
    rows = []
    for S in itertools.product(*ranges):
        T = np.array(S, dtype=np.float64) @ box
        delta = points[None, :, :] - points[:, None, :] + T
        d2 = np.sum(delta * delta, axis=-1)
        ii, jj = np.nonzero(d2 < cutoff * cutoff)
        for i, j in zip(ii, jj):
            if i == j and S == (0, 0, 0):
                continue
            if not full and not oracle.half_list_keeps(i, j, S):
                continue
            rows.append((i, j, *S))
    return sorted(rows)


BRUTE_CASES = [
    ("diamond", 3.0), ("diamond", 5.0), ("carbon", 5.0), ("carbon", 7.0), ("slab", 5.0), ("polymer_chain", 5.0),
    ("graphene_sheet", 5.0), ("issue_153", 5.0), ("rotated_box", 7.0), ("Cd2I4O12", 7.0), ("diamond_crystal", 5.0),
]


@pytest.mark.parametrize("name,cutoff", BRUTE_CASES)
@pytest.mark.parametrize("full", [True, False])
def test_oracle_against_numpy_brute_force(name, cutoff, full):
    points, box, periodic = systems.small_systems()[name]
    result = oracle.canonicalize(oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD"))
    rows = [(int(p[0]), int(p[1]), *map(int, s)) for p, s in zip(result["pairs"], result["shifts"])]
    assert rows == brute_force(points, box, periodic, cutoff, full)
    # vectors and distances recomputed from the definition r_j - r_i + S.H
    H = np.asarray(box, dtype=np.float64).copy()
    H[~np.asarray(periodic, dtype=bool)] = 0.0
    i, j = result["pairs"][:, 0].astype(int), result["pairs"][:, 1].astype(int)
    vectors = points[j] - points[i] + result["shifts"].astype(np.float64) @ H
    assert np.allclose(result["vectors"], vectors, rtol=1e-13, atol=1e-13)
    assert np.allclose(result["distances"], np.linalg.norm(vectors, axis=1), rtol=1e-13, atol=0)


@pytest.mark.parametrize("mask", range(8))
def test_oracle_mixed_periodicity_against_brute_force(mask):
    periodic = [(mask >> d) & 1 == 1 for d in range(3)]
    points, box, periodic = systems.mixed_periodic(periodic)
    result = oracle.canonicalize(oracle.neighbors(points, box, periodic, 0.35, True, False, "ijS"))
    rows = [(int(p[0]), int(p[1]), *map(int, s)) for p, s in zip(result["pairs"], result["shifts"])]
    assert rows == brute_force(points, box, periodic, 0.35, True)


def test_half_list_rule_keeps_exactly_one_of_each_mirror_pair():
    for S in itertools.product(range(-2, 3), repeat=3):
        mirrored = tuple(-s for s in S)
        if S == (0, 0, 0):
            continue
        assert oracle.half_list_keeps(3, 3, S) != oracle.half_list_keeps(3, 3, mirrored), S
    assert oracle.half_list_keeps(1, 2, (0, 0, 0)) and not oracle.half_list_keeps(2, 1, (5, 5, 5))


def test_full_list_is_the_half_list_and_its_mirror():
    points, box, periodic = systems.read_xyz("carbon")
    full = oracle.canonicalize(oracle.neighbors(points, box, periodic, 6.0, True, False, "ijSdD"))
    half = oracle.neighbors(points, box, periodic, 6.0, False, False, "ijSdD")
    mirrored = {
        "pairs": np.concatenate([half["pairs"], half["pairs"][:, ::-1]]),
        "shifts": np.concatenate([half["shifts"], -half["shifts"]]),
        "distances": np.concatenate([half["distances"], half["distances"]]),
        "vectors": np.concatenate([half["vectors"], -half["vectors"]]),
    }
    mirrored = oracle.canonicalize(mirrored)
    for key in full:
        assert np.array_equal(full[key], mirrored[key] + 0 if key == "vectors" else mirrored[key]), key


def test_grid_closed_forms_for_an_orthorhombic_box():
    # face distances = edge lengths, inverse = diag(1/L), n_cells = trunc(L / cutoff), n_search = 1
    lengths = np.array([10.7, 23.1, 37.9])
    points = np.random.default_rng(3).random((50, 3)) * lengths
    grid = oracle.neighbors(points, np.diag(lengths), True, 5.0, return_grid=True)["grid"]
    assert np.allclose(grid["face_distances"], lengths, rtol=1e-15)
    assert np.allclose(grid["inverse"], np.diag(1.0 / lengths), rtol=1e-15)
    assert grid["n_cells"].tolist() == [2, 4, 7]
    assert grid["n_search"].tolist() == [1, 1, 1]
    # cutoff above the box: one cell, ceil(cutoff / L) images on each side
    grid = oracle.neighbors(points, np.diag(lengths), True, 25.0, return_grid=True)["grid"]
    assert grid["n_cells"].tolist() == [1, 1, 1]
    assert grid["n_search"].tolist() == [3, 2, 1]


def test_errors():
    points = np.zeros((2, 3))
    with pytest.raises(RuntimeError, match="the box matrix is not invertible"):
        oracle.neighbors(points, np.zeros((3, 3)), True, 1.0)
    with pytest.raises(RuntimeError, match="cutoff must be a finite, positive number"):
        oracle.neighbors(points, np.eye(3), True, -1.0)
    with pytest.raises(RuntimeError, match="cutoff is too small"):
        oracle.neighbors(points, np.eye(3), True, 1e-7)
    bad = np.array([[0.0, 0.0, 0.0], [0.0, np.nan, 0.0]])
    with pytest.raises(RuntimeError, match="point 1 has non-finite coordinate along axis 1: nan"):
        oracle.neighbors(bad, np.eye(3), True, 1.0)
    if oracle.have_ref():
        with pytest.raises(RuntimeError, match="point 1 has non-finite coordinate along axis 1: nan"):
            oracle.ref_neighbors(bad, np.eye(3), True, 1.0)


def test_sorted_is_monotone_in_i():
    points, box, periodic = systems.diamond_crystal()
    result = oracle.neighbors(points, box, periodic, 5.0, True, True, "ijS")
    first = result["pairs"][:, 0].astype(np.int64)
    assert np.all(np.diff(first) >= 0)
