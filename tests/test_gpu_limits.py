"""The sizes the kernels' packed fields were laid out for, exercised (``-m gpu``): a system of more than 2^24 points
(32-bit point indices in 64-bit sort keys, (points, tiles) packed into one word of the cell scan, a window of original
indices in the ordering of a tile's candidates) and the sorted list of the 1,000,000-atom configuration at full size.
Lists of this size are compared where they are, on the device: order-independent fingerprints against those of the
compiled reference on record (tests/golden/reference_checksums.json, made by tests/golden/make_golden.py), the order
of a sorted list row by row. The reference's own guard for large values: python/vesin/tests/test_cupy.py:339-350."""

import json
import os

import numpy as np
import pytest

from golden import systems
from test_gpu_batch import fingerprints_per_system_on_device
from vesin_amd import NeighborList, configs

pytestmark = pytest.mark.gpu

with open(os.path.join(os.path.dirname(systems.__file__), "reference_checksums.json")) as fd:
    GOLDEN = json.load(fd)


def _prints_on_device(pairs, shifts, distances):
    import torch

    pairs = pairs.view(torch.int64)
    ijS, d = fingerprints_per_system_on_device(pairs, shifts, distances, [0, pairs.shape[0]])
    return {"n_pairs": int(pairs.shape[0]), "ijS": int(ijS[0]), "d": int(d[0])}


def _mirrored_prints_on_device(pairs, shifts, distances):
    import torch

    pairs = pairs.view(torch.int64)
    return _prints_on_device(torch.stack([pairs[:, 1], pairs[:, 0]], dim=1), -shifts, distances)


def _assert_in_order(pairs, shifts, n_points):
    """Rows in strictly increasing (i, j, Sx, Sy, Sz) order, checked on the device."""
    import torch

    if pairs.shape[0] < 2:
        return
    pairs = pairs.view(torch.int64)
    i = pairs[:, 0]
    j = pairs[:, 1]
    assert int(i.max()) < n_points and int(j.max()) < n_points
    # (i, j) in one word, the shift in another: both fit 63 bits
    first = i * n_points + j
    second = ((shifts[:, 0].to(torch.int64) + 1024) * 4096 + (shifts[:, 1].to(torch.int64) + 1024)) * 4096 + (
        shifts[:, 2].to(torch.int64) + 1024
    )
    ascending = (first[1:] > first[:-1]) | ((first[1:] == first[:-1]) & (second[1:] > second[:-1]))
    out_of_order = int((~ascending).sum())
    assert out_of_order == 0, f"{out_of_order} rows are not after the row before them"


def _same_prints(actual, golden, what):
    for key in ("n_pairs", "ijS", "d"):
        assert actual[key] == golden[key], f"{what}: {key} differs from the compiled reference's"


def test_config1_sorted_at_full_size():
    """1,000,000 atoms with sorted=true (the in-order search over about 52,000 tiles, candidates ordered through the
    window of original indices): the rows of the compiled reference, in (i, j, S) order."""
    import torch

    points, box, periodic, options = configs.config1()
    device_points = torch.as_tensor(points, device="cuda:0")
    device_box = torch.as_tensor(box, device="cuda:0")
    calculator = NeighborList(cutoff=options["cutoff"], full_list=True, sorted=True)
    for call in ("first call", "second call"):
        pairs, shifts, distances = calculator.compute(device_points, device_box, periodic, "PSd", copy=False)
        _same_prints(_prints_on_device(pairs, shifts, distances), GOLDEN["config1"], call)
        _assert_in_order(pairs, shifts, len(points))
    # the same atoms in random order: every tile sees indices from all over (candidates ordered through buckets)
    order = np.random.default_rng(1).permutation(len(points))
    inverse = torch.as_tensor(np.argsort(order), device="cuda:0")
    shuffled = torch.as_tensor(points[order], device="cuda:0")
    for call in ("shuffled, first call", "shuffled, second call"):
        pairs, shifts, distances = calculator.compute(shuffled, device_box, periodic, "PSd", copy=False)
        _assert_in_order(pairs, shifts, len(points))
        # in the numbering of the unshuffled points these are the reference's rows
        renumbered = torch.as_tensor(order, device="cuda:0")[pairs.view(torch.int64)]
        _same_prints(_prints_on_device(renumbered, shifts, distances), GOLDEN["config1"], call)
    del inverse


def test_more_than_two_to_the_24_points():
    """17,000,000 points, about four neighbours each: unsorted (the first call of a list goes through count, scan and
    write, the second through the single-pass search), then sorted, full and half."""
    import torch

    golden = GOLDEN["uniform-17m"]
    points, box, periodic = systems.uniform_large()
    assert len(points) == golden["n_points"] > 2**24
    device_points = torch.as_tensor(points, device="cuda:0")
    device_box = torch.as_tensor(box, device="cuda:0")
    del points

    calculator = NeighborList(cutoff=golden["cutoff"], full_list=True)
    for call in ("unsorted, first call", "unsorted, second call"):
        pairs, shifts, distances = calculator.compute(device_points, device_box, True, "PSd", copy=False)
        _same_prints(_prints_on_device(pairs, shifts, distances), golden, call)
        assert int(pairs.view(torch.int64).max()) >= 2**24
    del calculator, pairs, shifts, distances
    torch.cuda.empty_cache()

    calculator = NeighborList(cutoff=golden["cutoff"], full_list=True, sorted=True)
    for call in ("sorted, first call", "sorted, second call"):
        pairs, shifts, distances = calculator.compute(device_points, device_box, True, "PSd", copy=False)
        _same_prints(_prints_on_device(pairs, shifts, distances), golden, call)
        _assert_in_order(pairs, shifts, golden["n_points"])
    del calculator, pairs, shifts, distances
    torch.cuda.empty_cache()

    # a half list holds one row of every pair; with the mirrored rows it is the full list
    calculator = NeighborList(cutoff=golden["cutoff"], full_list=False, sorted=True)
    pairs, shifts, distances = calculator.compute(device_points, device_box, True, "PSd", copy=False)
    assert 2 * pairs.shape[0] == golden["n_pairs"]
    _assert_in_order(pairs, shifts, golden["n_points"])
    kept = _prints_on_device(pairs, shifts, distances)
    mirrored = _mirrored_prints_on_device(pairs, shifts, distances)
    for key in ("ijS", "d"):
        assert (kept[key] + mirrored[key]) % 2**64 == golden[key], f"half list: {key} differs from the compiled reference's"
    i = pairs.view(torch.int64)
    assert bool((i[:, 0] <= i[:, 1]).all())
