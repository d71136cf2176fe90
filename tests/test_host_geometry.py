"""Host logic of the HIP driver (vesin_amd/csrc/geometry.hpp), checked on the CPU through a small g++-built shim:
the normalised box, its inverse and the face distances must carry the same bits as the oracle's (they feed the
shift vectors), and the grid must keep its covering guarantee."""

import ctypes
import os
import subprocess

import numpy as np
import pytest

import oracle
from golden import systems

HERE = os.path.dirname(os.path.realpath(__file__))
ROOT = os.path.dirname(HERE)


@pytest.fixture(scope="module")
def probe(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("probe") / "libprobe.so")
    subprocess.run(
        ["g++", "-std=c++17", "-O2", "-ffp-contract=off", "-fPIC", "-shared", "-I", os.path.join(ROOT, "vesin_amd", "csrc"),
         os.path.join(HERE, "host_probe.cpp"), "-o", out],
        check=True,
    )
    lib = ctypes.CDLL(out)
    lib.probe_box.argtypes = [ctypes.c_void_p] * 5
    lib.probe_grid.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_double, ctypes.c_size_t, ctypes.c_void_p,
                               ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.probe_pruning.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_double, ctypes.c_size_t, ctypes.c_void_p,
                                  ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                  ctypes.c_void_p, ctypes.c_size_t]
    lib.probe_box_guess.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.probe_box_guess.restype = None
    lib.probe_ordered_records_fit.argtypes = [ctypes.c_size_t, ctypes.c_size_t]
    lib.probe_ordered_records_fit.restype = ctypes.c_int
    lib.probe_prefilter.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_double, ctypes.c_size_t, ctypes.c_void_p,
                                    ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    lib.probe_wait_rest.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.probe_wait_rest.restype = None
    lib.probe_candidate_lifetime.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.probe_candidate_lifetime.restype = None
    lib.probe_ordered_share.argtypes = [ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int]
    lib.probe_ordered_share.restype = ctypes.c_uint
    for name in ("probe_ordered_write_split", "probe_ordered_count_split"):
        getattr(lib, name).argtypes = [ctypes.c_size_t, ctypes.c_size_t]
        getattr(lib, name).restype = ctypes.c_uint
    return lib


def run_box_guess(probe, n_points, cutoff, changed):
    n_points = np.ascontiguousarray(n_points, dtype=np.uint64)
    cutoff = np.ascontiguousarray(cutoff, dtype=np.float64)
    changed = np.ascontiguousarray(changed, dtype=np.uint8)
    guessed = np.zeros(len(changed), dtype=np.uint8)
    probe.probe_box_guess(n_points.ctypes.data, cutoff.ctypes.data, changed.ctypes.data, len(changed), guessed.ctypes.data)
    return guessed.astype(bool)


def test_a_constant_box_is_guessed_from_the_second_call_on(probe):
    guessed = run_box_guess(probe, [1000] * 10, [5.0] * 10, [0] * 10)
    assert not guessed[0] and guessed[1:].all()


def test_no_guess_for_another_question(probe):
    # other number of points, other cutoff: the remembered box belongs to another system
    n_points = [1000, 1000, 64, 64, 1000, 1000, 1000, 1000]
    cutoff = [5.0, 5.0, 5.0, 5.0, 5.0, 5.0, 6.0, 6.0]
    guessed = run_box_guess(probe, n_points, cutoff, [0] * 8)
    assert guessed.tolist() == [False, True, False, True, False, True, False, True]
    # and nothing to guess for no points at all
    assert not run_box_guess(probe, [0] * 4, [5.0] * 4, [0] * 4).any()


def test_wrong_guesses_are_made_less_and_less_often(probe):
    # the box changes with every call: guesses at calls 1, 34, 99, 228, ... (32, 64, 128, ... calls of rest after each)
    n = 20000
    guessed = run_box_guess(probe, [1000] * n, [5.0] * n, [1] * n)
    at = np.flatnonzero(guessed)
    assert at[0] == 1
    rests = np.diff(at) - 1
    assert rests[:7].tolist() == [32, 64, 128, 256, 512, 1024, 2048]
    assert (rests[7:] == 4096).all() and len(rests) > 8
    assert guessed.sum() <= 12


def test_a_right_guess_restores_the_short_rest(probe):
    # three wrong guesses (rests 32, 64, 128), then the box stays: guesses on every call; the next change costs 32 again
    changed = [1] * 100 + [0] * 140 + [1] + [0] * 40
    n = len(changed)
    guessed = run_box_guess(probe, [1000] * n, [5.0] * n, changed)
    at = np.flatnonzero(guessed)
    assert at[:4].tolist() == [1, 34, 99, 228]
    assert guessed[228:241].all()
    assert changed[240] == 1
    assert not guessed[241:273].any() and guessed[273]


def run_pruning(probe, box, periodic, cutoff, n_points, lo=(0, 0, 0), hi=(0, 0, 0), single_cell=False):
    """Grid, edge vectors of one cell (rows), and which stencil entries are dropped, as a dict keyed by (dx, dy, dz)."""
    box = np.ascontiguousarray(box, dtype=np.float64)
    periodic = np.ascontiguousarray(periodic, dtype=np.uint8)
    lo = np.ascontiguousarray(lo, dtype=np.float64)
    hi = np.ascontiguousarray(hi, dtype=np.float64)
    n, s = np.zeros(3, dtype=np.int32), np.zeros(3, dtype=np.int32)
    cell = np.zeros((3, 3))
    dropped = np.zeros(1 << 16, dtype=np.uint8)
    status = probe.probe_pruning(box.ctypes.data, periodic.ctypes.data, cutoff, n_points, lo.ctypes.data, hi.ctypes.data,
                                 int(single_cell), n.ctypes.data, s.ctypes.data, cell.ctypes.data, dropped.ctypes.data,
                                 dropped.size)
    assert status == 0
    entries = {}
    at = 0
    for dx in range(-s[0], s[0] + 1):
        for dy in range(-s[1], s[1] + 1):
            for dz in range(-s[2], s[2] + 1):
                entries[(dx, dy, dz)] = bool(dropped[at])
                at += 1
    return n, s, cell, entries


def run_box(probe, box, periodic):
    box = np.ascontiguousarray(box, dtype=np.float64)
    periodic = np.ascontiguousarray(periodic, dtype=np.uint8)
    H, Hinv, face = np.zeros((3, 3)), np.zeros((3, 3)), np.zeros(3)
    status = probe.probe_box(box.ctypes.data, periodic.ctypes.data, H.ctypes.data, Hinv.ctypes.data, face.ctypes.data)
    return status, H, Hinv, face


def run_grid(probe, box, periodic, cutoff, n_points, lo, hi, single_cell=False):
    box = np.ascontiguousarray(box, dtype=np.float64)
    periodic = np.ascontiguousarray(periodic, dtype=np.uint8)
    lo = np.ascontiguousarray(lo, dtype=np.float64)
    hi = np.ascontiguousarray(hi, dtype=np.float64)
    n, s = np.zeros(3, dtype=np.int32), np.zeros(3, dtype=np.int32)
    status = probe.probe_grid(box.ctypes.data, periodic.ctypes.data, cutoff, n_points, lo.ctypes.data, hi.ctypes.data,
                              int(single_cell), n.ctypes.data, s.ctypes.data)
    return status, n, s


@pytest.mark.parametrize("name", list(systems.small_systems()))
@pytest.mark.parametrize("mask", range(8))
def test_box_bits_match_the_oracle(probe, name, mask):
    points, box, _ = systems.small_systems()[name]
    periodic = np.array([(mask >> d) & 1 == 1 for d in range(3)])
    if np.allclose(box, 0) and periodic.any():
        box = systems.transformed((points, np.diag([11.0, 12.0, 13.0]), periodic), 5, False)[1]
    try:
        grid = oracle.neighbors(points, box, periodic, 4.0, return_grid=True)["grid"]
    except RuntimeError as e:
        assert "not invertible" in str(e)
        assert run_box(probe, box, periodic)[0] == 1
        return
    status, H, Hinv, face = run_box(probe, box, periodic)
    assert status == 0
    assert np.array_equal(H, grid["matrix"])
    assert np.array_equal(Hinv, grid["inverse"])
    for d in range(3):
        if periodic[d]:
            assert face[d] == grid["face_distances"][d]


def test_singular_box_is_refused(probe):
    assert run_box(probe, np.zeros((3, 3)), [True, True, True])[0] == 1
    assert run_box(probe, np.zeros((3, 3)), [False, False, False])[0] == 0  # box ignored
    assert run_box(probe, np.diag([4.0, 4.5, 0.0]), [True, True, False])[0] == 0  # python/vesin/tests/_utils.py:186-194


def test_grid_orthorhombic(probe):
    lengths = np.array([10.7, 23.1, 37.9])
    status, n, s = run_grid(probe, np.diag(lengths), [1, 1, 1], 5.0, 10000, [0] * 3, [0] * 3)
    assert status == 0 and n.tolist() == [2, 4, 7] and s.tolist() == [1, 1, 1]
    # cutoff above the box: images on each side
    status, n, s = run_grid(probe, np.diag(lengths), [1, 1, 1], 25.0, 10000, [0] * 3, [0] * 3)
    assert n.tolist() == [1, 1, 1] and s.tolist() == [3, 2, 1]
    # an edge that is an exact multiple of the cutoff gets one cell less, never a cell of exactly the cutoff
    status, n, s = run_grid(probe, np.diag([20.0, 20.0, 20.0]), [1, 1, 1], 5.0, 10000, [0] * 3, [0] * 3)
    assert n.tolist() == [3, 3, 3] and s.tolist() == [1, 1, 1]


def test_grid_covering_guarantee(probe):
    rng = np.random.default_rng(0)
    for _ in range(200):
        box = rng.normal(size=(3, 3)) * rng.uniform(1, 30)
        if abs(np.linalg.det(box)) < 1e-3:
            continue
        cutoff = rng.uniform(0.5, 12)
        n_points = int(rng.integers(1, 100000))
        status, n, s = run_grid(probe, box, [1, 1, 1], cutoff, n_points, [0] * 3, [0] * 3)
        assert status == 0
        _, _, _, face = run_box(probe, box, [1, 1, 1])
        # s cells of width face / n must reach beyond the cutoff
        assert np.all(s * face / n > cutoff)
        assert np.prod(n.astype(np.int64)) <= max(64, 2 * n_points)


def test_grid_open_directions_and_single_cell(probe):
    box = np.diag([300.0, 300.0, 300.0])
    status, n, s = run_grid(probe, box, [1, 1, 0], 4.5, 500000, [0, 0, -20.0], [0, 0, 330.0])
    assert status == 0
    assert n[2] == int(np.floor(350.0 * 1.01 / (4.5 * (1 + 1e-9)))) and s.tolist() == [1, 1, 1]
    # a flat system along an open direction: one cell, nothing to search beyond it
    status, n, s = run_grid(probe, box, [1, 1, 0], 4.5, 1000, [0, 0, 1.0], [0, 0, 1.0])
    assert n[2] == 1 and s[2] == 0
    status, n, s = run_grid(probe, np.diag([7.134] * 3), [1, 1, 1], 10.0, 64, [0] * 3, [0] * 3, single_cell=True)
    assert n.tolist() == [1, 1, 1] and s.tolist() == [2, 2, 2]
    status, n, s = run_grid(probe, box, [0, 0, 0], 4.5, 64, [0] * 3, [100.0] * 3, single_cell=True)
    assert n.tolist() == [1, 1, 1] and s.tolist() == [0, 0, 0]


def test_never_more_cells_than_twice_the_points(probe):
    """The work buffers of a batch are sized for max(64, 2 n) cells per system whatever its points do: a system that
    is long in one direction and thin in the others (a stretched chain, a dissociating pair) must not keep more
    cells along its length than that because the thin directions cannot go below one cell."""
    open_box = np.eye(3)
    cases = [
        (40, 5.0, [1000.0, 3.0, 3.0]),      # 199 cells along x before the limit, 80 allowed
        (1000, 5.0, [20000.0, 0.0, 0.0]),   # a line of points
        (2, 1.0, [1.0e6, 0.5, 0.5]),        # two atoms far apart
        (500, 2.0, [3000.0, 3000.0, 1.0]),  # a sheet
        (33, 0.5, [700.0, 650.0, 600.0]),
        (100000, 3.0, [1.0e5, 1.0e5, 2.0]),
    ]
    for n_points, cutoff, width in cases:
        for order in ([0, 1, 2], [1, 2, 0], [2, 0, 1]):
            hi = [width[k] for k in order]
            status, n, s = run_grid(probe, open_box, [0, 0, 0], cutoff, n_points, [0.0] * 3, hi)
            assert status == 0
            cells = int(np.prod(n.astype(np.int64)))
            assert cells <= max(64, 2 * n_points), (n_points, cutoff, hi, n.tolist())
            # and still cells: the limit does not collapse a long system into a handful of cells
            assert cells >= min(0.4 * max(64, 2 * n_points), np.prod(np.maximum(np.floor(np.array(hi) * 1.01 / cutoff), 1)) * 0.4)
            # cells at least as wide as the cutoff, stencil reaching beyond it or to the last cell
            extent = np.maximum(np.where(np.array(hi) >= 1e-6, np.array(hi), 1.0) * 1.01, 1.0)
            assert np.all((extent / n > cutoff) | (n == 1))
            assert np.all((s * extent / n > cutoff) | (s == n - 1))
    rng = np.random.default_rng(5)
    for _ in range(500):
        n_points = int(rng.integers(1, 5000))
        cutoff = rng.uniform(0.5, 8.0)
        hi = (10.0 ** rng.uniform(-2, 5, size=3)).tolist()
        status, n, s = run_grid(probe, open_box, [0, 0, 0], cutoff, n_points, [0.0] * 3, hi)
        assert status == 0 and int(np.prod(n.astype(np.int64))) <= max(64, 2 * n_points)


def test_too_many_images_is_an_error(probe):
    status, _, _ = run_grid(probe, np.eye(3) * 0.01, [1, 1, 1], 10.0, 10, [0] * 3, [0] * 3)
    assert status == 1


def closest_approach(cell, offset):
    """Smallest distance between a point of the cell at the origin and a point of the cell `offset` cells away: the
    minimum of |(offset + f) . cell| over f in [-1, 1]^3 (f = difference of the two places inside the cells), a
    convex problem with bounds."""
    from scipy.optimize import minimize

    offset = np.asarray(offset, dtype=np.float64)
    gram = cell @ cell.T

    def squared(f):
        t = offset + f
        return t @ gram @ t

    def gradient(f):
        return 2.0 * gram @ (offset + f)

    best = min(
        minimize(squared, start, jac=gradient, bounds=[(-1.0, 1.0)] * 3, method="L-BFGS-B", options={"ftol": 1e-15, "gtol": 1e-12}).fun
        for start in (np.zeros(3), -np.sign(offset) * 1.0, -np.sign(offset) * 0.5)
    )
    return np.sqrt(max(best, 0.0))


def test_dropped_stencil_entries_of_the_small_cell_case(probe):
    # 7.134 A cube, cutoff 10 A: one cell, 5^3 images; those with two components of +-2 are at least sqrt(2) * 7.134 A
    # away and go, the other 81 stay (the distance between two boxes one image apart along a direction is zero)
    n, s, cell, entries = run_pruning(probe, np.eye(3) * 7.134, [1, 1, 1], 10.0, 64)
    assert list(n) == [1, 1, 1] and list(s) == [2, 2, 2]
    kept = [offset for offset, gone in entries.items() if not gone]
    assert len(entries) == 125 and len(kept) == 81
    assert all(sum(abs(c) == 2 for c in offset) <= 1 for offset in kept)
    # radius one: every cell of the stencil touches the centre cell
    n, s, cell, entries = run_pruning(probe, np.eye(3) * 40.0, [1, 1, 1], 5.0, 1000)
    assert list(s) == [1, 1, 1] and not any(entries.values())


@pytest.mark.parametrize("seed", range(12))
def test_dropped_stencil_entries_cannot_hold_a_neighbour(probe, seed):
    # For boxes of every shape: an entry is only dropped when no two points of the two cells are within the cutoff
    # (checked with the true closest approach of the two cells, a bounded convex minimisation), and the bound is
    # not idle: in narrow boxes of orthogonal vectors every entry beyond the cutoff is dropped.
    rng = np.random.default_rng(400 + seed)
    edges = rng.uniform(1.5, 6.0, size=3)
    box = np.diag(edges)
    kind = seed % 4
    if kind == 1:
        q, _ = np.linalg.qr(rng.normal(size=(3, 3)))
        box = box @ q
    elif kind >= 2:
        box = box + rng.normal(scale=0.35 * edges.min(), size=(3, 3))
        if abs(np.linalg.det(box)) < 0.3 * np.prod(edges):
            box = np.diag(edges) + np.triu(box - np.diag(edges)) * 0.3
    periodic = [1, 1, 1] if kind != 3 else [1, 0, 1]
    cutoff = float(rng.uniform(5.0, 9.0))
    n, s, cell, entries = run_pruning(probe, box, periodic, cutoff, 50, lo=(-1.0, -2.0, -3.0), hi=(4.0, 7.5, 2.0))
    assert max(s) >= 2
    n_dropped = 0
    for offset, gone in entries.items():
        apart = closest_approach(cell, offset)
        if gone:
            n_dropped += 1
            assert apart > cutoff, f"entry {offset} is dropped, its cell comes as close as {apart} (cutoff {cutoff})"
        elif kind <= 1:
            # orthogonal vectors: the bound is the closest approach itself, up to the margins
            assert apart <= cutoff * (1 + 1e-5), f"entry {offset} at {apart} is kept (cutoff {cutoff})"
    if kind <= 1 and min(s) >= 2:
        assert n_dropped > 0


# ---------------------------------------------------------------------------------------------------------------------
# How the search that writes a sorted list in order cuts its work into waves (policy.hpp)


def _tile_slots(n_points, n_cells):
    """What the driver holds tiles for: a tile per occupied cell and one more per 32 points, in multiples of 32."""
    slots = min(n_cells, n_points) + n_points // 32 + 1
    return (slots + 31) // 32 * 32


def test_share_of_a_tile_per_wave(probe):
    def share(n_points, n_cells, coarse=False):
        return probe.probe_ordered_share(n_points, n_cells, _tile_slots(n_points, n_cells), int(coarse))

    # large systems: a wave per tile
    assert share(100_000, 4096) == 32
    assert share(1_000_000, 42_875) == 32
    assert share(30_000, 3375) == 32  # 8.9 points per cell, but enough tiles
    # mid-size systems: 8 points, or 4 where shares of 8 would be too few
    assert share(10_000, 1331) == 8
    assert share(10_000, 729) == 8   # 13.7 points per cell: two shares of 8 per tile, 1458 in all
    assert share(6_000, 343) == 4    # 17.5 points per cell: three shares of 8 per tile are only 1029
    assert share(4_000, 512) == 4
    assert share(15_000, 2197) == 8  # more than 2048 cells, few points in each
    assert share(50_000, 2197) == 32  # the same cells well filled: the tiles are worth a wave each
    # the smallest systems: down to a point per wave
    assert share(216, 27) == 1
    assert share(2_000, 343) == 4
    assert share(1, 1) == 1
    # fixed work memory: the coarser rule, which only counts the slots
    assert share(10_000, 1331, coarse=True) == 16
    assert share(6_000, 343, coarse=True) == 8
    assert share(100_000, 4096, coarse=True) == 32
    # always a power of two between 1 and 32
    rng = np.random.default_rng(5)
    for _ in range(2000):
        n_points = int(rng.integers(1, 400_000))
        n_cells = int(rng.integers(1, 2 * n_points + 2))
        for coarse in (False, True):
            found = share(n_points, n_cells, coarse)
            assert found in (1, 2, 4, 8, 16, 32)
            if not coarse:
                assert found <= share(n_points, n_cells, True) or found in (4, 8)


def test_waves_per_tile_of_the_two_passes(probe):
    write = probe.probe_ordered_write_split
    count = probe.probe_ordered_count_split
    # nothing known about the system yet
    assert write(100_000, 0) == 1 and count(100_000, 0) == 1
    # the 100,000-atom benchmark: 4,260 tiles of 23.5 points
    assert write(100_000, 4260) == 4 and count(100_000, 4260) == 2
    # twice and four times the size at the same filling
    assert write(200_000, 9000) == 4 and count(200_000, 9000) == 2
    assert write(400_000, 19_000) == 4 and count(400_000, 19_000) == 1
    assert write(800_000, 39_000) == 1 and count(800_000, 39_000) == 1
    # few tiles: the writing pass has room for all of them at once
    assert write(50_000, 2300) == 1 and count(50_000, 2300) == 2
    # 12 points per tile: one wave each, whatever the number of tiles
    assert write(100_000, 8100) == 1 and count(100_000, 8100) == 1
    assert write(50_000, 4200) == 1 and count(50_000, 4200) == 1
    for tiles in range(1, 40_000, 97):
        for per_tile in (3, 15, 16, 31):
            assert write(tiles * per_tile, tiles) in (1, 4)
            assert count(tiles * per_tile, tiles) in (1, 2)
            if per_tile < 16:
                assert write(tiles * per_tile, tiles) == 1 and count(tiles * per_tile, tiles) == 1


def run_wait_rest(probe, gives_up):
    gives_up = np.ascontiguousarray(gives_up, dtype=np.uint8)
    used = np.zeros(len(gives_up), dtype=np.uint8)
    probe.probe_wait_rest(gives_up.ctypes.data, len(gives_up), used.ctypes.data)
    return used.astype(bool)


def test_a_launch_whose_waves_gave_up_is_left_alone_for_longer_and_longer(probe):
    # never a give-up: used by every call
    assert run_wait_rest(probe, [0] * 50).all()
    # a GPU on which the launch gives up whenever it is tried: tried at calls 0, 65, 194, 451, ... (64, 128, 256 ...
    # calls of rest in between, 4096 at most)
    used = run_wait_rest(probe, [1] * 20000)
    tried = np.flatnonzero(used)
    assert tried[:5].tolist() == [0, 65, 194, 451, 964]
    assert np.diff(tried).max() == 4097 and np.diff(tried)[-1] == 4097
    # one give-up, then fine again: 64 calls of rest once, and the next give-up starts from 64 again
    gives_up = np.zeros(400, dtype=np.uint8)
    gives_up[10] = 1
    gives_up[200] = 1
    used = run_wait_rest(probe, gives_up)
    assert used[:11].all() and not used[11:75].any() and used[75:201].all() and not used[201:265].any() and used[265:].all()




def run_candidate_lifetime(probe, outdated):
    outdated = np.ascontiguousarray(outdated, dtype=np.uint8)
    what = np.zeros(len(outdated), dtype=np.uint8)
    probe.probe_candidate_lifetime(outdated.ctypes.data, len(outdated), what.ctypes.data)
    return what.tolist()


def test_candidates_that_keep_getting_outdated_are_given_up_for_a_while(probe):
    """options.skin > 0: 0 = direct search that keeps nothing, 1 = direct search and new candidates, 2 = filter,
    3 = failed filter, new candidates, filter."""
    # candidates that last: one set, filtered for ever; outdated every tenth call: computed again every time
    assert run_candidate_lifetime(probe, [0] * 30) == [1] + [2] * 29
    every_tenth = [1 if k % 10 == 0 else 0 for k in range(50)]
    assert run_candidate_lifetime(probe, every_tenth) == [1] + [3 if k % 10 == 0 else 2 for k in range(1, 50)]
    # outdated at every call: three sets that served one call each (the one that computed them), then 64 direct
    # searches, then candidates once more
    what = run_candidate_lifetime(probe, [1] * 200)
    assert what[:4] == [1, 3, 3, 0] and what[4:68] == [0] * 64 and what[68:72] == [1, 3, 3, 0]
    # every third call: sets that serve three calls are short-lived as well; every fourth: they are not
    what = run_candidate_lifetime(probe, [1 if k % 3 == 0 else 0 for k in range(40)])
    assert what[:11] == [1, 2, 2, 3, 2, 2, 3, 2, 2, 0, 0]
    what = run_candidate_lifetime(probe, [1 if k % 4 == 0 else 0 for k in range(60)])
    assert 0 not in what
    # two short-lived sets, then one that lasts: the count starts over
    outdated = [0, 1, 1, 0, 0, 0, 0, 0, 1, 1, 1, 0]
    assert run_candidate_lifetime(probe, outdated) == [1, 3, 3, 2, 2, 2, 2, 2, 3, 3, 3, 2]


def test_work_memory_of_the_in_order_search_is_bounded(probe):
    # 12 KB per tile slot. Diamond at cutoff 5: 1,000,000 atoms have about 74,000 slots, 8,000,000 about 600,000
    assert probe.probe_ordered_records_fit(1_000_000, 74_000 * 12288)
    assert probe.probe_ordered_records_fit(8_000_000, 600_000 * 12288)
    # a cell per point: 17,000,000 points would take 212 GB
    assert not probe.probe_ordered_records_fit(17_000_000, 17_300_000 * 12288)
    # small systems always fit
    assert probe.probe_ordered_records_fit(216, 2048 * 12288)
    assert probe.probe_ordered_records_fit(1, 64 * 12288)


def run_prefilter(probe, box, periodic, cutoff, n_points, lo, hi, single_cell=False):
    box = np.ascontiguousarray(box, dtype=np.float64)
    flags = np.ascontiguousarray(periodic, dtype=np.uint8)
    lo = np.ascontiguousarray(lo, dtype=np.float64)
    hi = np.ascontiguousarray(hi, dtype=np.float64)
    n = np.zeros(3, dtype=np.int32)
    s = np.zeros(3, dtype=np.int32)
    out = np.zeros(12)
    status = probe.probe_prefilter(box.ctypes.data, flags.ctypes.data, cutoff, n_points, lo.ctypes.data, hi.ctypes.data,
                                   int(single_cell), n.ctypes.data, s.ctypes.data, out.ctypes.data)
    assert status == 0
    return bool(out[0]), np.float32(out[1]), np.float32(out[2]), out[3:].reshape(3, 3), n, s


@pytest.mark.parametrize("seed", range(6))
def test_single_precision_pre_test_never_decides_a_pair_it_should_not(probe, seed):
    """The counting pass of the in-order search decides a pair in single precision when its squared distance, worked
    out from the places of the two points inside their cells and the offset between the cells, lies below `lo32` or
    above `hi32`. Here that arithmetic is repeated in numpy's float32 for pairs at the cutoff to within a part in a
    million, in boxes of every shape, against the squared distance in double precision (extended precision where
    numpy has it): no pair may be decided the wrong way, and the error stays within half of what the thresholds
    allow (the bound in geometry.hpp is doubled)."""
    rng = np.random.default_rng(100 + seed)
    worst = 0.0
    for case in range(40):
        cutoff = float(rng.uniform(1.0, 9.0))
        kind = case % 4
        if kind == 0:
            box = np.diag(rng.uniform(2.5, 40.0, size=3) * cutoff / 3.0)
        else:
            box = rng.normal(size=(3, 3)) * rng.uniform(3.0, 30.0)
            if abs(np.linalg.det(box)) < 0.2 * np.prod(np.linalg.norm(box, axis=1)):
                continue
        periodic = [1, 1, 1] if kind < 3 else [1, 0, 1]
        use32, lo32, hi32, edges, n, s = run_prefilter(probe, box, periodic, cutoff, 50000, [0, -20.0, 0], [0, 35.0, 0],
                                                      single_cell=(kind == 2))
        if np.prod(2 * s + 1) > 64:
            continue  # (the search with the pre-test is not used for such a stencil)
        assert use32, (box, cutoff)
        assert float(lo32) < cutoff * cutoff < float(hi32)
        allowed = (float(hi32) - float(lo32)) / 2.0
        m = 20000
        # place of the first point in its cell, direction and length of the pair: the second point's cell follows
        inside_i = rng.random((m, 3))
        length = cutoff * (1.0 + rng.uniform(-1e-6, 1e-6, size=m))
        direction = rng.normal(size=(m, 3))
        direction /= np.linalg.norm(direction, axis=1)[:, None]
        in_cells_j = inside_i + (direction * length[:, None]) @ np.linalg.inv(edges)
        offset = np.floor(in_cells_j)
        inside_j = in_cells_j - offset
        reachable = np.all(np.abs(offset) <= s, axis=1)
        inside_i, inside_j, offset = inside_i[reachable], inside_j[reachable], offset[reachable]
        # double (or extended) precision: the vector the reference tests
        wide = np.longdouble
        exact = (inside_j.astype(wide) + offset.astype(wide) - inside_i.astype(wide)) @ edges.astype(wide)
        d2 = np.sum(exact * exact, axis=1).astype(np.float64)
        # single precision, as the kernel does it
        place_i = (inside_i @ edges).astype(np.float32)
        place_j = (inside_j @ edges).astype(np.float32)
        between = (offset @ edges).astype(np.float32)
        seen = (place_j + between).astype(np.float32)
        v = (seen - place_i).astype(np.float32)
        d2_32 = ((v[:, 0] * v[:, 0] + v[:, 1] * v[:, 1]).astype(np.float32) + v[:, 2] * v[:, 2]).astype(np.float32)
        inside_cutoff = d2 < cutoff * cutoff
        assert not np.any(inside_cutoff & (d2_32 > hi32)), (box, cutoff)
        assert not np.any(~inside_cutoff & (d2_32 < lo32)), (box, cutoff)
        worst = max(worst, float(np.max(np.abs(d2_32.astype(np.float64) - d2)) / allowed))
    assert 0.0 < worst <= 0.5, worst


@pytest.mark.parametrize("seed", range(4))
def test_pre_test_of_systems_of_one_cell_stays_within_its_bound(probe, seed):
    """Sorted batches search systems of one cell over their images, and decide a pair in single precision from where
    the two points are after they were moved into the box, seen from a point inside the box (each rounded once), and
    the shift of the image (rounded once): d2_32 = |(u_j - u_i) + q . H|^2 with the squares added by fused
    multiply-adds. The same in numpy's float32 for pairs at the cutoff to within a part in a million, across up to two
    boxes, against double (extended) precision: no pair is decided the wrong way and the error stays within half of
    what the thresholds allow."""
    rng = np.random.default_rng(200 + seed)
    worst = 0.0
    cases = 0
    for case in range(60):
        cutoff = float(rng.uniform(1.0, 9.0))
        if case % 2 == 0:
            box = np.diag(rng.uniform(0.52, 2.5, size=3) * cutoff)
        else:
            box = np.eye(3) * rng.uniform(0.6, 2.0) * cutoff + 0.15 * cutoff * rng.normal(size=(3, 3))
        use32, lo32, hi32, edges, n, s = run_prefilter(probe, box, [1, 1, 1], cutoff, 64, [0] * 3, [0] * 3, single_cell=True)
        if np.prod(2 * s + 1) > 128:
            continue  # (more images than that search keeps)
        assert use32 and np.all(n == 1), (box, cutoff)
        cases += 1
        allowed = (float(hi32) - float(lo32)) / 2.0
        m = 20000
        wide = np.longdouble
        seen_from = rng.random(3) @ box
        inside_i = rng.random((m, 3)) @ box
        length = cutoff * (1.0 + rng.uniform(-1e-6, 1e-6, size=m))
        direction = rng.normal(size=(m, 3))
        direction /= np.linalg.norm(direction, axis=1)[:, None]
        target = inside_i + direction * length[:, None]
        q = np.floor(target @ np.linalg.inv(box))          # the image of j that is meant
        inside_j = target - q @ box
        reachable = np.all(np.abs(q) <= s, axis=1)
        inside_i, inside_j, q = inside_i[reachable], inside_j[reachable], q[reachable]
        exact = (inside_j.astype(wide) - inside_i.astype(wide)) + q.astype(wide) @ box.astype(wide)
        d2 = np.sum(exact * exact, axis=1).astype(np.float64)
        u_i = (inside_i - seen_from).astype(np.float32)
        u_j = (inside_j - seen_from).astype(np.float32)
        shift = (q @ box).astype(np.float32)
        v = ((u_j - u_i).astype(np.float32) + shift).astype(np.float32)
        v64 = v.astype(np.float64)
        xx = (v64[:, 0] * v64[:, 0]).astype(np.float32)                                   # vx * vx
        xy = (v64[:, 1] * v64[:, 1] + xx.astype(np.float64)).astype(np.float32)           # fma(vy, vy, .)
        d2_32 = (v64[:, 2] * v64[:, 2] + xy.astype(np.float64)).astype(np.float32)        # fma(vz, vz, .)
        inside_cutoff = d2 < cutoff * cutoff
        assert not np.any(inside_cutoff & (d2_32 > hi32)), (box, cutoff)
        assert not np.any(~inside_cutoff & (d2_32 < lo32)), (box, cutoff)
        worst = max(worst, float(np.max(np.abs(d2_32.astype(np.float64) - d2)) / allowed))
    assert cases >= 20 and 0.0 < worst <= 0.5, (cases, worst)


def test_pre_test_is_switched_off_where_its_bound_is_no_use(probe):
    # one cell much wider than the cutoff: the margin would be a sizeable part of the squared cutoff
    use32, *_ = run_prefilter(probe, np.eye(3), [0, 0, 0], 1e-3, 100, [0] * 3, [5000.0] * 3, single_cell=True)
    assert not use32
    # an open system very far from the origin: its coordinates have too few digits left for the places
    use32, *_ = run_prefilter(probe, np.eye(3), [0, 0, 0], 3.0, 100000, [1e12] * 3, [1e12 + 100.0] * 3)
    assert not use32
    # a box squeezed almost flat
    flat = np.array([[1.0e4, 0.0, 0.0], [0.0, 1.0e4, 0.0], [1.0e4, 1.0e4, 10.0]])
    use32, *_ = run_prefilter(probe, flat, [1, 1, 1], 3.0, 100000000, [0] * 3, [0] * 3)
    assert not use32
    # ordinary systems have it
    use32, *_ = run_prefilter(probe, np.eye(3) * 178.35, [1, 1, 1], 5.0, 1000000, [0] * 3, [0] * 3)
    assert use32
