"""Known-answer tests: the literal vectors the reference's own tests hold for this path, re-expressed here and run
against both the CPU oracle (pins the oracle, runs anywhere) and the HIP path (``-m gpu``).

Sources: vesin/tests/neighbors.cpp:86-328, vesin/tests/memory.cpp:5-87, vesin/tests/cuda.cpp:22-126,
fortran/tests/tests.f90:19-82, python/vesin/tests/test_numpy.py:115-128,328-370, test_cupy.py:25-125.
"""

import numpy as np
import pytest

import oracle
from _helpers import ENGINES, run_engine, ulp_close
from golden import systems


def canonical(result):
    return oracle.canonicalize(result)


@pytest.mark.parametrize("engine", ENGINES)
def test_non_periodic(engine):
    # vesin/tests/neighbors.cpp:86-135 (expected values computed with ASE, 4 ULP)
    points = [
        [0.134, 1.282, 1.701],
        [-0.273, 1.026, -1.471],
        [1.922, -0.124, 1.900],
        [1.400, -0.464, 0.480],
        [0.149, 1.865, 0.635],
    ]
    result = canonical(run_engine(engine, points, np.zeros((3, 3)), False, 3.42, full=False, quantities="ijSd"))
    assert result["pairs"].tolist() == [[0, 1], [0, 2], [0, 3], [0, 4], [1, 3], [1, 4], [2, 3], [2, 4], [3, 4]]
    expected = [
        3.2082345612501593, 2.283282943482914, 2.4783286706972505, 1.215100818862369, 2.9707625283755013,
        2.3059143522689647, 1.550639867925496, 2.9495550511899244, 2.6482573515427084,
    ]
    assert ulp_close(result["distances"], expected)
    assert np.all(result["shifts"] == 0)


@pytest.mark.parametrize("engine", ENGINES)
def test_fcc_unit_cell(engine):
    # vesin/tests/neighbors.cpp:137-182: one atom, 6 half-list pairs with its own images
    box = [[0.0, 1.5, 1.5], [1.5, 0.0, 1.5], [1.5, 1.5, 0.0]]
    result = canonical(run_engine(engine, [[0.0, 0.0, 0.0]], box, True, 3.0, full=False))
    assert result["pairs"].tolist() == [[0, 0]] * 6
    assert result["shifts"].tolist() == [[-1, 0, 1], [-1, 1, 0], [0, -1, 1], [0, 0, 1], [0, 1, 0], [1, 0, 0]]
    assert result["vectors"].tolist() == [
        [1.5, 0.0, -1.5], [1.5, -1.5, 0.0], [0.0, 1.5, -1.5], [1.5, 1.5, 0.0], [1.5, 0.0, 1.5], [0.0, 1.5, 1.5],
    ]
    assert ulp_close(result["distances"], [2.1213203435596424] * 6)


@pytest.mark.parametrize("engine", ENGINES)
@pytest.mark.parametrize("full", [False, True])
def test_large_box_small_cutoff(engine, full):
    # vesin/tests/neighbors.cpp:184-223 and python/vesin/tests/test_cupy.py:25-125: points outside the box
    points = [[0.0, 0.0, 0.0], [0.0, 2.0, 0.0], [0.0, 0.0, 2.0], [-6.0, 0.0, 0.0], [-6.0, -2.0, 0.0], [-6.0, 0.0, -2.0]]
    result = canonical(run_engine(engine, points, np.eye(3) * 54.0, True, 2.1, full=full))
    if full:
        assert result["pairs"].tolist() == [[0, 1], [0, 2], [1, 0], [2, 0], [3, 4], [3, 5], [4, 3], [5, 3]]
        vectors = [[0, 2, 0], [0, 0, 2], [0, -2, 0], [0, 0, -2], [0, -2, 0], [0, 0, -2], [0, 2, 0], [0, 0, 2]]
    else:
        assert result["pairs"].tolist() == [[0, 1], [0, 2], [3, 4], [3, 5]]
        vectors = [[0, 2, 0], [0, 0, 2], [0, -2, 0], [0, 0, -2]]
    assert np.all(result["shifts"] == 0)
    assert np.all(result["distances"] == 2.0)
    assert np.array_equal(result["vectors"], np.array(vectors, dtype=float))


@pytest.mark.parametrize("engine", ENGINES)
def test_cutoff_larger_than_box(engine):
    # vesin/tests/neighbors.cpp:225-262
    result = canonical(run_engine(engine, [[0.0, 0.0, 0.0]], np.eye(3) * 0.5, True, 0.6, full=False))
    assert result["pairs"].tolist() == [[0, 0]] * 3
    assert result["shifts"].tolist() == [[0, 0, 1], [0, 1, 0], [1, 0, 0]]
    assert result["vectors"].tolist() == [[0.0, 0.0, 0.5], [0.0, 0.5, 0.0], [0.5, 0.0, 0.0]]
    assert result["distances"].tolist() == [0.5] * 3


@pytest.mark.parametrize("engine", ENGINES)
def test_slanted_box(engine):
    # vesin/tests/neighbors.cpp:264-328: 90 half-list pairs, including shifts (-2, 0..2, 0) between points 0 and 3
    points = [[1.42, 0.0, 0.0], [2.84, 0.0, 0.0], [3.55, -1.22975607, 0.0], [4.97, -1.22975607, 0.0]]
    box = [[4.26, -2.45951215, 0.0], [2.13, 1.22975607, 0.0], [0.0, 0.0, 50.0]]
    result = run_engine(engine, points, box, True, 6.4, full=False, quantities="ijS")
    assert len(result["pairs"]) == 90
    rows = {(int(p[0]), int(p[1]), *map(int, s)) for p, s in zip(result["pairs"], result["shifts"])}
    for shift in ([-2, 0, 0], [-2, 1, 0], [-2, 2, 0]):
        assert (0, 3, *shift) in rows


@pytest.mark.parametrize("engine", ENGINES)
def test_fcc_counts_of_the_allocation_reuse_test(engine):
    # vesin/tests/memory.cpp:36-84: 9 -> 67 -> 134 -> 27 pairs
    box = [[0.0, 1.5, 1.5], [1.5, 0.0, 1.5], [1.5, 1.5, 0.0]]
    point = [[0.0, 0.0, 0.0]]
    assert len(run_engine(engine, point, box, True, 3.4, full=False)["pairs"]) == 9
    assert len(run_engine(engine, point, box, True, 6.0, full=False)["pairs"]) == 67
    assert len(run_engine(engine, point, box, True, 6.0, full=True)["pairs"]) == 134
    assert len(run_engine(engine, point, box, True, 4.5, full=False)["pairs"]) == 27


@pytest.mark.parametrize("engine", ENGINES)
def test_three_points_in_fcc_like_box(engine):
    # vesin/tests/cuda.cpp:22-126: 5 half-list pairs, exact vectors and distances
    points = [[0.0, 0.0, 0.0], [1.0, 1.0, 1.0], [2.0, 2.0, 2.0]]
    box = [[0.0, 3.0, 3.0], [3.0, 0.0, 3.0], [3.0, 3.0, 0.0]]
    result = canonical(run_engine(engine, points, box, True, 3.0, full=False))
    assert result["pairs"].tolist() == [[0, 1], [0, 2], [0, 2], [0, 2], [1, 2]]
    assert result["shifts"].tolist() == [[0, 0, 0], [-1, 0, 0], [0, -1, 0], [0, 0, -1], [0, 0, 0]]
    assert result["vectors"].tolist() == [
        [1.0, 1.0, 1.0], [2.0, -1.0, -1.0], [-1.0, 2.0, -1.0], [-1.0, -1.0, 2.0], [1.0, 1.0, 1.0],
    ]
    assert result["distances"].tolist() == [np.sqrt(3.0), np.sqrt(6.0), np.sqrt(6.0), np.sqrt(6.0), np.sqrt(3.0)]


@pytest.mark.parametrize("engine", ENGINES)
def test_two_points_in_a_cube(engine):
    # fortran/tests/tests.f90:19-82: single-precision literals widened to double, half list, sorted
    f = np.float32
    points = np.array([[0.0, 0.0, 0.0], [0.0, f(1.3), f(1.3)]], dtype=np.float64)
    box = np.eye(3) * float(f(3.2))
    result = run_engine(engine, points, box, True, float(f(3.3)), full=False, sorted=True)
    assert result["pairs"][:, 0].tolist() == sorted(result["pairs"][:, 0].tolist())
    result = canonical(result)
    assert result["pairs"].tolist() == [[0, 0]] * 3 + [[0, 1]] * 4 + [[1, 1]] * 3
    assert result["shifts"].tolist() == [
        [0, 0, 1], [0, 1, 0], [1, 0, 0],
        [0, -1, -1], [0, -1, 0], [0, 0, -1], [0, 0, 0],
        [0, 0, 1], [0, 1, 0], [1, 0, 0],
    ]
    expected = [3.2, 3.2, 3.2, 2.6870059, 2.3021729, 2.3021729, 1.8384775, 3.2, 3.2, 3.2]
    assert np.allclose(result["distances"], expected, atol=1e-6)


@pytest.mark.parametrize("engine", ENGINES)
def test_array_like_pair(engine):
    # python/vesin/tests/test_numpy.py:115-128
    result = canonical(run_engine(engine, [[0.0, 0.0, 0.0], [0.5, 0.0, 0.0]], np.eye(3) * 2.0, False, 1.0))
    assert result["pairs"].tolist() == [[0, 1], [1, 0]]
    assert result["distances"].tolist() == [0.5, 0.5]
    assert result["vectors"].tolist() == [[0.5, 0.0, 0.0], [-0.5, 0.0, 0.0]]


@pytest.mark.parametrize("engine", ENGINES)
def test_gigantic_cell(engine):
    # python/vesin/tests/test_numpy.py:328-340
    points, box, periodic = systems.gigantic_cell()
    assert len(run_engine(engine, points, box, periodic, 8.0, full=True, quantities="ij")["pairs"]) == 412


@pytest.mark.parametrize("engine", ENGINES)
def test_all_negative_coordinates(engine):
    # python/vesin/tests/test_numpy.py:343-370
    points = np.array(
        [[3.87166034, 1.63896135, 22.14371739], [3.19075223, 1.6182371, 22.87858863], [5.01141342, 1.73904134, 20.79729257]]
    )
    expected = [[0, 1], [0, 2], [1, 0], [1, 2], [2, 0], [2, 1]]
    for candidate in (points, points - 15.0):
        result = canonical(run_engine(engine, candidate, np.zeros((3, 3)), False, 8.0, quantities="ij"))
        assert result["pairs"].tolist() == expected


@pytest.mark.parametrize("engine", ENGINES)
def test_diamond_shells(engine):
    # closed form: neighbour shells of the diamond lattice hold 4, 12, 12, 6, 12 sites at
    # a*sqrt(3)/4, a/sqrt(2), a*sqrt(11)/4, a, a*sqrt(19)/4
    points, box, periodic = systems.read_xyz("diamond")
    a = box[0, 0]
    shells = [(np.sqrt(3) / 4, 4), (1 / np.sqrt(2), 12), (np.sqrt(11) / 4, 12), (1.0, 6), (np.sqrt(19) / 4, 12)]
    total = 0
    for radius, count in shells:
        total += count
        result = run_engine(engine, points, box, periodic, a * radius * 1.001, full=True, quantities="ijd")
        assert len(result["pairs"]) == total * len(points)
