"""Seeded synthetic systems for the benchmark and the parity tests (host side, numpy only).

Every generator returns ``(points, box, periodic, options)`` where ``options`` is a dict with ``cutoff``,
``full_list``, ``sorted`` and ``quantities`` in the vocabulary of ``NeighborList``.
"""

import numpy as np

DIAMOND_A = 3.567
_DIAMOND_BASIS = np.array(
    [
        [0.0, 0.0, 0.0],
        [0.0, 0.5, 0.5],
        [0.5, 0.0, 0.5],
        [0.5, 0.5, 0.0],
        [0.25, 0.25, 0.25],
        [0.25, 0.75, 0.75],
        [0.75, 0.25, 0.75],
        [0.75, 0.75, 0.25],
    ]
)


def diamond(replicas, seed, sigma=0.05):
    """Jittered diamond carbon: the 8-atom conventional cell (a = 3.567 A) replicated ``replicas``^3 times in an
    orthorhombic periodic box; every coordinate gets N(0, sigma^2) noise."""
    n = int(replicas)
    grid = np.stack(np.meshgrid(np.arange(n), np.arange(n), np.arange(n), indexing="ij"), axis=-1).reshape(-1, 3)
    points = (grid[:, None, :] + _DIAMOND_BASIS[None, :, :]).reshape(-1, 3) * DIAMOND_A
    rng = np.random.default_rng(seed)
    points = points + rng.normal(scale=sigma, size=points.shape)
    box = np.eye(3) * (n * DIAMOND_A)
    return np.ascontiguousarray(points), box, np.array([True, True, True])


def triclinic_box(lengths, angles_deg):
    """Crystallographic cell: a along x, b in the xy plane."""
    a, b, c = lengths
    alpha, beta, gamma = np.radians(angles_deg)
    bx = b * np.cos(gamma)
    by = b * np.sin(gamma)
    cx = c * np.cos(beta)
    cy = c * (np.cos(alpha) - np.cos(beta) * np.cos(gamma)) / np.sin(gamma)
    cz = np.sqrt(c * c - cx * cx - cy * cy)
    return np.array([[a, 0.0, 0.0], [bx, by, 0.0], [cx, cy, cz]])


def config0():
    """216-atom diamond, cutoff 5, full, sorted, i j S d."""
    points, box, periodic = diamond(3, seed=0)
    return points, box, periodic, dict(cutoff=5.0, full_list=True, sorted=True, quantities="ijSd")


def config1(replicas=50):
    """The headline case: 50^3 diamond cells = 1,000,000 atoms, cutoff 5, full, unsorted, i j S d."""
    points, box, periodic = diamond(replicas, seed=1)
    return points, box, periodic, dict(cutoff=5.0, full_list=True, sorted=False, quantities="ijSd")


def config2(n_atoms=100_000):
    """Triclinic liquid-like system at 0.1 atoms/A^3, cutoff 6, half list, sorted, i j S d D."""
    box = triclinic_box((100.0, 105.0, 110.0), (70.0, 80.0, 100.0))
    volume = abs(np.linalg.det(box))
    box = box * (n_atoms / 0.1 / volume) ** (1.0 / 3.0)
    rng = np.random.default_rng(2)
    points = rng.random((n_atoms, 3)) @ box
    return np.ascontiguousarray(points), box, np.array([True, True, True]), dict(
        cutoff=6.0, full_list=False, sorted=True, quantities="ijSdD"
    )


def config3(replica):
    """One 64-atom replica of the small-cell case: box 7.134 A, cutoff 10 A (> box / 2), full, i j S d."""
    points, box, periodic = diamond(2, seed=3000 + int(replica))
    return points, box, periodic, dict(cutoff=10.0, full_list=True, sorted=False, quantities="ijSd")


def config4(n_atoms=500_000, periodic=(False, False, False), n_blobs=50):
    """Gaussian blobs (sigma 8 A, centres uniform in a 300 A cube), cutoff 4.5, full, unsorted, i j d.
    ``periodic=(False,)*3`` ignores the box (zeros); otherwise the box is the 300 A cube."""
    rng = np.random.default_rng(4)
    centres = rng.uniform(0.0, 300.0, size=(n_blobs, 3))
    which = rng.integers(0, n_blobs, size=n_atoms)
    points = centres[which] + rng.normal(scale=8.0, size=(n_atoms, 3))
    periodic = np.array(periodic, dtype=bool)
    box = np.eye(3) * 300.0 if periodic.any() else np.zeros((3, 3))
    return np.ascontiguousarray(points), box, periodic, dict(
        cutoff=4.5, full_list=True, sorted=False, quantities="ijd"
    )


def algorithmic_bytes(n_points, n_pairs, quantities):
    """Compulsory traffic of one call: positions read once, every requested output written once."""
    per_pair = 16 + 12 * ("S" in quantities) + 8 * ("d" in quantities) + 24 * ("D" in quantities)
    return 24 * n_points + n_pairs * per_pair
