"""Systems used by the parity tests.

``data/*.xyz`` are the data files of the reference's own test-suite (python/vesin/tests/data), kept as fixtures. The
generated systems restate the ones of python/vesin/tests/_utils.py:114-195 (same numbers, same seeds), and the
``config*`` entries are reduced-size versions of the benchmark configurations.
"""

import os
import re

import numpy as np

HERE = os.path.dirname(os.path.realpath(__file__))


def read_xyz(name):
    """Minimal extended-XYZ reader: positions, ``Lattice="..."`` (rows = cell vectors) and ``pbc="..."``. Without a
    lattice the cell is zero and nothing is periodic; with a lattice and no pbc flag everything is periodic."""
    with open(os.path.join(HERE, "data", f"{name}.xyz")) as fd:
        lines = fd.read().splitlines()
    n = int(lines[0])
    header = lines[1]
    lattice = re.search(r'Lattice="([^"]*)"', header)
    pbc = re.search(r'pbc="([^"]*)"', header)
    if lattice is not None:
        box = np.array([float(x) for x in lattice.group(1).split()]).reshape(3, 3)
        periodic = np.array([True, True, True])
    else:
        box = np.zeros((3, 3))
        periodic = np.array([False, False, False])
    if pbc is not None:
        periodic = np.array([flag.upper().startswith("T") for flag in pbc.group(1).split()])
    points = np.array([[float(x) for x in line.split()[1:4]] for line in lines[2 : 2 + n]])
    return points, box, periodic


def polymer_chain():
    spacing = 1.54
    points = np.array([[index * spacing, 0.0, 0.0] for index in range(8)])
    return points, np.diag([8 * spacing, 18.0, 18.0]), np.array([True, False, False])


def graphene_sheet():
    a1 = np.array([2.46, 0.0, 0.0])
    a2 = np.array([1.23, 2.13042249, 0.0])
    basis = [np.array([0.0, 0.0, 0.0]), np.array([1.23, 0.71014083, 0.0])]
    points = [i * a1 + j * a2 + atom for i in range(4) for j in range(4) for atom in basis]
    box = np.array([[9.84, 0.0, 0.0], [4.92, 8.52168996, 0.0], [0.0, 0.0, 18.0]])
    return np.array(points), box, np.array([True, True, False])


def diamond_crystal():
    points, box, periodic = read_xyz("diamond")
    # 2x2x2 supercell, cells outermost / atoms innermost
    offsets = np.array([[a, b, c] for a in range(2) for b in range(2) for c in range(2)], dtype=float) @ box
    points = (offsets[:, None, :] + points[None, :, :]).reshape(-1, 3)
    points = points + np.random.default_rng(1234).normal(scale=1.0, size=points.shape)
    return points, 2.0 * box, periodic


def naphthalene_cluster():
    points, _, _ = read_xyz("naphthalene")
    return points, np.diag([30.0, 30.0, 30.0]), np.array([False, False, False])


def issue_153():
    points = np.array([[0.0, 2.5, 0.0], [2.0, 0.0, 0.0]])
    return points, np.diag([4.0, 4.5, 0.0]), np.array([True, True, False])


def mixed_periodic(periodic):
    """100 points in a skewed unit-sized box (python/vesin/tests/test_numpy.py:231-269, with a seeded box)."""
    rng = np.random.default_rng(7)
    box = np.eye(3)[[2, 0, 1]] + 0.1 * rng.normal(size=(3, 3))
    points = np.random.default_rng(0).random((100, 3))
    return points, box, np.array(periodic, dtype=bool)


def gigantic_cell():
    """python/vesin/tests/test_numpy.py:328-340: 3000 points, 1e7 A periodic cell, 412 pairs at cutoff 8."""
    state = np.random.RandomState(34)
    return state.randn(3000, 3) * 100, 1e7 * np.eye(3), np.array([True, True, True])


def rotation(seed):
    """A seeded proper or improper rotation (python/vesin/tests/_utils.py:37-48 uses unseeded ones)."""
    rng = np.random.default_rng(seed)
    q, _ = np.linalg.qr(rng.normal(size=(3, 3)))
    if np.linalg.det(q) < 0:
        q[:, 0] *= -1
    if rng.integers(2):
        q = -q
    return q


def transformed(system, seed, translate):
    points, box, periodic = system
    q = rotation(seed)
    points = points @ q.T
    if translate:
        points = points + np.random.default_rng(seed + 1000).uniform(-100.0, 100.0, size=3)
    return np.ascontiguousarray(points), np.ascontiguousarray(box @ q.T), periodic


XYZ_NAMES = ["water", "diamond", "naphthalene", "carbon", "slab", "Cd2I4O12", "rotated_box"]


def small_systems():
    """name -> (points, box, periodic): the 12 systems of the reference's python tests."""
    systems = {name: read_xyz(name) for name in XYZ_NAMES}
    systems["naphthalene_cluster"] = naphthalene_cluster()
    systems["polymer_chain"] = polymer_chain()
    systems["graphene_sheet"] = graphene_sheet()
    systems["diamond_crystal"] = diamond_crystal()
    systems["issue_153"] = issue_153()
    return systems


LARGE_POINTS = 17_000_000  # more than 2^24


def uniform_large(n_points=LARGE_POINTS, pairs_per_point=4.0, cutoff=1.0, seed=77):
    """Uniformly random points in a periodic cube, at the density that gives every point `pairs_per_point` neighbours
    within `cutoff` on average: a system whose point indices, cells and rows go beyond 2^24 while its list stays
    small enough to check (the reference's own guard for large values: python/vesin/tests/test_cupy.py:339-350)."""
    density = pairs_per_point / (4.0 / 3.0 * np.pi * cutoff**3)
    length = (n_points / density) ** (1.0 / 3.0)
    rng = np.random.default_rng(seed)
    points = rng.random((n_points, 3)) * length
    return points, np.eye(3) * length, np.array([True, True, True])


def golden_cases(full_size=False, large=False):
    """Yield (name, points, box, periodic, cutoff, full_list). Small cases always; with ``full_size`` also the
    benchmark configurations at their real sizes; with ``large`` only the system of more than 2^24 points."""
    from vesin_amd import configs

    if large:
        yield "uniform-17m", *uniform_large(), 1.0, True
        return

    for name, system in small_systems().items():
        for cutoff in (3.0, 5.0, 7.0, 10.0):
            for full in (True, False):
                yield f"{name}-rc{cutoff:g}-{'full' if full else 'half'}", *system, cutoff, full
        for seed, translate in ((11, False), (12, True)):
            moved = transformed(system, seed, translate)
            yield f"{name}-rot{seed}-rc5-full", *moved, 5.0, True

    for mask in range(8):
        periodic = [(mask >> d) & 1 == 1 for d in range(3)]
        tag = "".join("T" if p else "F" for p in periodic)
        yield f"mixed-{tag}-rc0.35-full", *mixed_periodic(periodic), 0.35, True
        yield f"mixed-{tag}-rc0.35-half", *mixed_periodic(periodic), 0.35, False

    yield "gigantic-rc8-full", *gigantic_cell(), 8.0, True

    p, b, per, o = configs.config0()
    yield "config0", p, b, per, o["cutoff"], True
    p, b, per, o = configs.config1(8)
    yield "config1-8cubed", p, b, per, o["cutoff"], True
    p, b, per, o = configs.config2(5000)
    yield "config2-5k", p, b, per, o["cutoff"], False
    for replica in (0, 1, 4095):
        p, b, per, o = configs.config3(replica)
        yield f"config3-replica{replica}", p, b, per, o["cutoff"], True
    p, b, per, o = configs.config4(20000, (False, False, False))
    yield "config4a-20k", p, b, per, o["cutoff"], True
    p, b, per, o = configs.config4(20000, (True, True, False))
    yield "config4b-20k", p, b, per, o["cutoff"], True

    if full_size:
        p, b, per, o = configs.config1()
        yield "config1", p, b, per, o["cutoff"], True
        p, b, per, o = configs.config2()
        yield "config2", p, b, per, o["cutoff"], False
        p, b, per, o = configs.config4(periodic=(False, False, False))
        yield "config4a", p, b, per, o["cutoff"], True
        p, b, per, o = configs.config4(periodic=(True, True, False))
        yield "config4b", p, b, per, o["cutoff"], True


# --------------------------------------------------------------------------------------------------------------
# Order-independent fingerprints: a 64-bit mix of every row, summed modulo 2^64


def _mix(x):
    x = x.astype(np.uint64, copy=True)
    with np.errstate(over="ignore"):
        x ^= x >> np.uint64(30)
        x *= np.uint64(0xBF58476D1CE4E5B9)
        x ^= x >> np.uint64(27)
        x *= np.uint64(0x94D049BB133111EB)
        x ^= x >> np.uint64(31)
    return x


def _combine(h, column):
    with np.errstate(over="ignore"):
        return _mix(h * np.uint64(0x9E3779B97F4A7C15) + column.astype(np.uint64) + np.uint64(0x7F4A7C15))


def fingerprints(result):
    """{"n_pairs", "ijS", "d", "D"}: sums (mod 2^64) over all pairs of a hash of (i, j, S), of (i, j, S, bits of d)
    and of (i, j, S, bits of D). Independent of the order of the pairs; chunked to bound memory."""
    pairs = result["pairs"]
    n = pairs.shape[0]
    out = {"n_pairs": int(n), "ijS": 0, "d": 0, "D": 0}
    chunk = 1 << 22
    for start in range(0, n, chunk):
        stop = min(n, start + chunk)
        h = _combine(np.zeros(stop - start, dtype=np.uint64), pairs[start:stop, 0])
        h = _combine(h, pairs[start:stop, 1])
        if "shifts" in result:
            s = result["shifts"][start:stop].astype(np.int64)
            for d in range(3):
                h = _combine(h, s[:, d].view(np.uint64))
        out["ijS"] = (out["ijS"] + int(h.sum(dtype=np.uint64))) & 0xFFFFFFFFFFFFFFFF
        if "distances" in result:
            hd = _combine(h, np.ascontiguousarray(result["distances"][start:stop]).view(np.uint64))
            out["d"] = (out["d"] + int(hd.sum(dtype=np.uint64))) & 0xFFFFFFFFFFFFFFFF
        if "vectors" in result:
            v = np.ascontiguousarray(result["vectors"][start:stop]) + 0.0  # -0.0 and +0.0 hash alike
            hv = h
            for d in range(3):
                hv = _combine(hv, np.ascontiguousarray(v[:, d]).view(np.uint64))
            out["D"] = (out["D"] + int(hv.sum(dtype=np.uint64))) & 0xFFFFFFFFFFFFFFFF
    return out


def fingerprints_of_systems(per_system):
    """One fingerprint for a batch of systems from the fingerprints of its members: the sum (mod 2^64) of a mix of
    each member's sums with the member's number, so that rows reported under the wrong system change it.
    ``per_system`` is a sequence of ``fingerprints()`` results (or of dicts with the same keys)."""
    out = {"n_systems": len(per_system), "n_pairs": 0, "ijS": 0, "d": 0}
    for number, prints in enumerate(per_system):
        out["n_pairs"] += int(prints["n_pairs"])
        for key in ("ijS", "d"):
            mixed = _mix(np.array([(int(prints[key]) ^ (number + 1)) & 0xFFFFFFFFFFFFFFFF], dtype=np.uint64))[0]
            out[key] = (out[key] + int(mixed)) & 0xFFFFFFFFFFFFFFFF
    return out
