"""``vesin_hip_neighbors_batch``: many systems in one call give, per system, the rows of a call on that system alone
(``-m gpu``)."""

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from golden import systems
from vesin_amd import NeighborList, configs

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}


def run_batch(calculator, all_points, all_boxes, letters="PSdD", periodic=True):
    import torch

    first_point = np.cumsum([0] + [len(p) for p in all_points])
    points = torch.as_tensor(np.concatenate(all_points).astype(np.float64), device="cuda:0")
    boxes = torch.as_tensor(np.stack(all_boxes).astype(np.float64), device="cuda:0")
    # the first call of a list sizes its arrays with the two passes, the second goes through the single-pass
    # search: both must give the same rows per system
    results = []
    for _ in range(2):
        outputs, first_pair = calculator.compute_batch(points, first_point, boxes, periodic, letters)
        whole = {NAMES[q]: out.cpu().numpy() for q, out in zip(letters, outputs)}
        per_system = []
        for s in range(len(all_points)):
            rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
            per_system.append({key: value[rows] for key, value in whole.items()})
        assert first_pair[0] == 0 and first_pair[-1] == len(whole["pairs"])
        results.append(per_system)
    first, second = results
    for s, (a, b) in enumerate(zip(first, second)):
        assert len(a["pairs"]) == len(b["pairs"]), f"system {s}: the second call has other rows than the first"
        if "shifts" in a and "distances" in a and "vectors" in a:
            assert_same_list(b, a, what=f"system {s}, second call against the first")
    return second


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_replicas_of_the_small_cell_case(full):
    # 64 atoms, cutoff above the box: one cell, 5^3 images (the multi-image path), 48 systems at once
    replicas = [configs.config3(r) for r in range(48)]
    cutoff = replicas[0][3]["cutoff"]
    calculator = NeighborList(cutoff=cutoff, full_list=full)
    lists = run_batch(calculator, [r[0] for r in replicas], [r[1] for r in replicas])
    for r, (points, box, periodic, _) in enumerate(replicas):
        expected = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
        assert_same_list(lists[r], expected, what=f"replica {r}")


def test_waves_that_give_up_waiting_fall_back_to_the_two_passes(capfd, monkeypatch):
    # a batch places its rows through the chain of workgroup totals; with VESIN_HIP_CHAIN_SPINS=0 every wait gives up
    # at once (the kernels still run to their end) and the second call of the list must notice and start over
    import torch

    monkeypatch.setenv("VESIN_HIP_CHAIN_SPINS", "0")
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    replicas = [configs.config3(r) for r in range(40, 64)]
    cutoff = replicas[0][3]["cutoff"]
    calculator = NeighborList(cutoff=cutoff, full_list=True)
    capfd.readouterr()
    lists = run_batch(calculator, [r[0] for r in replicas], [r[1] for r in replicas])
    launched = [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass (batch)")]
    assert len(launched) == 1 and " timeout 0 " not in launched[0], launched
    for r, (points, box, periodic, _) in enumerate(replicas):
        expected = oracle.neighbors(points, box, periodic, cutoff, True, False, "ijSdD")
        assert_same_list(lists[r], expected, what=f"replica {r}")
    # The list stays away from the launch that gave up: the next 64 calls go to the two passes directly (they do not
    # pay for the wait again), whatever the patience of the waves by then; the call after them is back on it.
    monkeypatch.delenv("VESIN_HIP_CHAIN_SPINS")
    first_point = np.cumsum([0] + [len(r[0]) for r in replicas])
    points = torch.as_tensor(np.concatenate([r[0] for r in replicas]), device="cuda:0")
    boxes = torch.as_tensor(np.stack([r[1] for r in replicas]), device="cuda:0")
    for rest in range(64):
        outputs, first_pair = calculator.compute_batch(points, first_point, boxes, True, "P")
        assert not [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass (batch)")], rest
    assert int(first_pair[-1]) == sum(len(rows["pairs"]) for rows in lists)
    outputs, first_pair = calculator.compute_batch(points, first_point, boxes, True, "PSdD")
    launched = [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass (batch)")]
    assert len(launched) == 1 and " timeout 0 " in launched[0], launched
    whole = {NAMES[q]: out.cpu().numpy() for q, out in zip("PSdD", outputs)}
    for r in range(len(replicas)):
        rows = slice(int(first_pair[r]), int(first_pair[r + 1]))
        assert_same_list({key: value[rows] for key, value in whole.items()}, lists[r], what=f"replica {r}, back on the chain")


def test_systems_of_different_sizes_and_shapes():
    rng = np.random.default_rng(31)
    all_points, all_boxes = [], []
    # a triclinic box with a few hundred points (a real cell list), tiny systems, an empty one, a larger cube
    points, box, _ = systems.read_xyz("carbon")
    all_points.append(points)
    all_boxes.append(box)
    for n in (1, 2, 0, 33, 700):
        edge = 6.0 + 2.0 * rng.random()
        box = np.eye(3) * edge + 0.3 * rng.normal(size=(3, 3))
        all_boxes.append(box)
        all_points.append(rng.random((n, 3)) @ box + rng.integers(-2, 3, size=(n, 3)) @ box)
    big = configs.config1(5)
    all_points.append(big[0])
    all_boxes.append(big[1])
    for full in (True, False):
        calculator = NeighborList(cutoff=4.0, full_list=full)
        lists = run_batch(calculator, all_points, all_boxes)
        for s, (points, box) in enumerate(zip(all_points, all_boxes)):
            expected = oracle.neighbors(points, box, True, 4.0, full, False, "ijSdD")
            assert_same_list(lists[s], expected, what=f"system {s} full={full}")


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_molecules_slabs_and_crystals_in_one_batch(full):
    """Per-system periodicity: free molecules (box ignored, even all zeros), slabs, wires and crystals side by side,
    every one with the rows of a call on it alone."""
    rng = np.random.default_rng(41)
    all_points, all_boxes, all_flags = [], [], []
    for n, flags in (
        (5, (False, False, False)),
        (180, (False, False, False)),
        (64, (True, True, True)),
        (300, (True, True, False)),
        (1, (False, False, False)),
        (90, (False, True, False)),
        (0, (False, False, False)),
        (1200, (False, False, False)),
        (400, (True, False, True)),
    ):
        edge = 7.0 + 3.0 * rng.random()
        box = np.eye(3) * edge + 0.4 * rng.normal(size=(3, 3))
        points = rng.random((n, 3)) @ box * rng.choice([0.6, 1.0, 1.7])
        if not any(flags) and n == 180:
            box = np.zeros((3, 3))  # free molecules need no box at all
        all_points.append(points)
        all_boxes.append(box)
        all_flags.append(flags)
    calculator = NeighborList(cutoff=3.1, full_list=full)
    lists = run_batch(calculator, all_points, all_boxes, periodic=np.array(all_flags))
    for s, (points, box, flags) in enumerate(zip(all_points, all_boxes, all_flags)):
        expected = oracle.neighbors(points, box, list(flags), 3.1, full, False, "ijSdD")
        assert_same_list(lists[s], expected, what=f"system {s} periodic={flags}")


def test_many_free_molecules():
    """2000 molecules of 3 to 40 atoms: the case a batch is for."""
    rng = np.random.default_rng(43)
    all_points = [rng.normal(scale=2.0, size=(int(rng.integers(3, 41)), 3)) + rng.uniform(-50, 50, size=3) for _ in range(2000)]
    all_boxes = [np.zeros((3, 3))] * len(all_points)
    calculator = NeighborList(cutoff=2.4, full_list=True)
    lists = run_batch(calculator, all_points, all_boxes, periodic=False)
    for s in range(0, len(all_points), 37):
        expected = oracle.neighbors(all_points[s], all_boxes[s], [False] * 3, 2.4, True, False, "ijSdD")
        assert_same_list(lists[s], expected, what=f"molecule {s}")
    total = sum(len(rows["pairs"]) for rows in lists)
    brute = 0
    for points in all_points:
        d = np.linalg.norm(points[:, None, :] - points[None, :, :], axis=-1)
        brute += int((d < 2.4).sum()) - len(points)
    assert abs(total - brute) <= 2  # pairs at the cutoff to the last bit aside


def test_single_pass_on_a_reused_list_and_its_fallbacks(capfd, monkeypatch):
    """A list that served a batch goes through the single-pass search on the next one; a larger batch that does
    not fit its arrays, or VESIN_HIP_SEARCH=two-pass, starts over with the two passes."""
    import torch

    def batch(replicas):
        chosen = [configs.config3(r) for r in replicas]
        first_point = np.cumsum([0] + [len(c[0]) for c in chosen])
        points = torch.as_tensor(np.concatenate([c[0] for c in chosen]), device="cuda:0")
        boxes = torch.as_tensor(np.stack([c[1] for c in chosen]), device="cuda:0")
        return chosen, points, first_point, boxes

    def report():
        return [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass (batch):")]

    def check(chosen, outputs, first_pair):
        whole = {NAMES[q]: out.cpu().numpy() for q, out in zip("PSdD", outputs)}
        for s in (0, len(chosen) - 1):
            rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
            expected = oracle.neighbors(chosen[s][0], chosen[s][1], chosen[s][2], 10.0, True, False, "ijSdD")
            assert_same_list({key: value[rows] for key, value in whole.items()}, expected, what=f"system {s}")

    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    calculator = NeighborList(cutoff=10.0, full_list=True)
    small = batch(range(6))
    large = batch(range(6, 30))
    capfd.readouterr()
    check(small[0], *calculator.compute_batch(small[1], small[2], small[3], True, "PSdD"))
    assert not report()  # first call: nothing to write into yet
    check(small[0], *calculator.compute_batch(small[1], small[2], small[3], True, "PSdD"))
    lines = report()
    assert lines and " deferred 0 overflow 0 timeout 0" in lines[-1] and " general 0 " in lines[-1], lines
    check(large[0], *calculator.compute_batch(large[1], large[2], large[3], True, "PSdD"))
    lines = report()
    assert lines and " overflow 0 " not in lines[-1], lines  # four times the rows: did not fit, two passes
    check(large[0], *calculator.compute_batch(large[1], large[2], large[3], True, "PSdD"))
    lines = report()
    assert lines and " overflow 0 " in lines[-1], lines
    monkeypatch.setenv("VESIN_HIP_SEARCH", "two-pass")
    check(small[0], *calculator.compute_batch(small[1], small[2], small[3], True, "PSdD"))
    assert not report()


def test_what_the_host_keeps_between_batches_follows_the_inputs():
    # One list, many batches: the host keeps the grids it derived from the boxes while boxes, flags and division
    # into systems stay what they were. Every change of one of them, and of the points alone, must show in the rows.
    import torch

    rng = np.random.default_rng(91)

    def batch(n_systems, edge, sizes):
        boxes = [np.diag(edge + rng.random(3)) for _ in range(n_systems)]
        points = [rng.random((n, 3)) @ box for n, box in zip(sizes, boxes)]
        return points, boxes

    def check(calculator, points, boxes, periodic, cutoff, what):
        first_point = np.cumsum([0] + [len(p) for p in points])
        outputs, first_pair = calculator.compute_batch(
            torch.as_tensor(np.concatenate(points), device="cuda:0"), first_point,
            torch.as_tensor(np.stack(boxes), device="cuda:0"), periodic, "PSdD",
        )
        whole = {NAMES[q]: out.cpu().numpy() for q, out in zip("PSdD", outputs)}
        flags = np.broadcast_to(np.asarray(periodic, dtype=bool), (len(points), 3)) if not isinstance(periodic, bool) else None
        for s, (p, box) in enumerate(zip(points, boxes)):
            rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
            per = periodic if flags is None else [bool(f) for f in flags[s]]
            expected = oracle.neighbors(p, box, per, cutoff, True, False, "ijSdD")
            assert_same_list({k: v[rows] for k, v in whole.items()}, expected, what=f"{what}, system {s}")

    sizes = [40, 25, 60, 33, 48]
    points, boxes = batch(5, 6.0, sizes)
    calculator = NeighborList(cutoff=4.0, full_list=True)
    check(calculator, points, boxes, True, 4.0, "first batch")
    check(calculator, points, boxes, True, 4.0, "the same batch again")
    # a call on one system uses the same work buffer its own way
    single = calculator.compute(
        torch.as_tensor(points[2], device="cuda:0"), torch.as_tensor(boxes[2], device="cuda:0"), True, "PSdD"
    )
    assert_same_list(
        {NAMES[q]: out.cpu().numpy() for q, out in zip("PSdD", single)},
        oracle.neighbors(points[2], boxes[2], True, 4.0, True, False, "ijSdD"), what="one system between two batches",
    )
    check(calculator, points, boxes, True, 4.0, "the same batch after a call on one system")
    moved = [p + 0.3 * rng.normal(size=p.shape) for p in points]
    check(calculator, moved, boxes, True, 4.0, "same boxes, moved points")
    other_boxes = [box.copy() for box in boxes]
    other_boxes[3] = np.diag([9.0, 5.5, 7.0])
    check(calculator, moved, other_boxes, True, 4.0, "one box changed")
    regrouped = [moved[0][:30], np.concatenate([moved[0][30:], moved[1]]), moved[2], moved[3], moved[4]]
    check(calculator, regrouped, other_boxes, True, 4.0, "same boxes, other division into systems")
    slab = np.array([[True, True, True]] * 4 + [[True, True, False]])
    check(calculator, regrouped, other_boxes, slab, 4.0, "one system opened along z")
    check(calculator, [p * 1.0 for p in regrouped], other_boxes, slab, 4.0, "open direction: never kept")
    check(calculator, regrouped, other_boxes, True, 4.0, "closed again")
    wider = NeighborList(cutoff=4.0, full_list=True)
    check(wider, points, boxes, True, 4.0, "another list, first cutoff")
    wider.cutoff = 7.5
    check(wider, points, boxes, True, 7.5, "same list and boxes, larger cutoff")


def test_batch_of_one_equals_the_single_call():
    points, box, periodic, _ = configs.config1(8)
    calculator = NeighborList(cutoff=5.0, full_list=True)
    (alone,) = run_batch(calculator, [points], [box])
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    assert_same_list(alone, expected)
    # the same struct then serves a single call
    import torch

    out = calculator.compute(torch.as_tensor(points, device="cuda:0"), torch.as_tensor(box, device="cuda:0"), True, "PSdD")
    single = {NAMES[q]: t.cpu().numpy() for q, t in zip("PSdD", out)}
    assert_same_list(single, expected)


def test_batch_errors():
    import torch

    points, box, periodic, _ = configs.config3(0)
    device_points = torch.as_tensor(points, device="cuda:0")
    boxes = torch.as_tensor(box[None], device="cuda:0")
    with pytest.raises(RuntimeError, match="non-finite coordinate along axis 1"):
        flags = torch.as_tensor([[True, False, True]], device="cuda:0")
        broken = device_points.clone()
        broken[5, 1] = float("nan")
        NeighborList(cutoff=5.0, full_list=True).compute_batch(broken, [0, len(points)], boxes, flags)
    with pytest.raises(RuntimeError, match="must not decrease"):
        NeighborList(cutoff=5.0, full_list=True).compute_batch(device_points, [0, 70, len(points)], torch.cat([boxes, boxes]))
    singular = boxes.clone()
    singular[0, 2] = singular[0, 1]
    with pytest.raises(RuntimeError, match="the box matrix is not invertible"):
        NeighborList(cutoff=5.0, full_list=True).compute_batch(device_points, [0, len(points)], singular)


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_sorted_batch_equals_sorted_single_calls(full, capfd, monkeypatch):
    """sorted=True in a batch: every system's rows in the order vesin_neighbors gives for that system alone
    ((i, j, shift) lexicographic), compared in place with the oracle's rows put in that order and with single calls.
    Systems of one cell and of several: the rows come out of the two searches that write them in order, and
    through the two passes and the radix sort when VESIN_HIP_SORT=radix asks for that."""
    import torch

    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")

    rng = np.random.default_rng(57)
    all_points, all_boxes, all_flags = [], [], []
    for replica in (0, 1, 2):
        points, box, _, _ = configs.config3(replica)  # many images of every pair
        all_points.append(points)
        all_boxes.append(box)
        all_flags.append((True, True, True))
    for n, flags in ((0, (True, True, True)), (1, (True, True, True)), (150, (False, False, False)), (400, (True, False, True)),
                     (700, (True, True, True))):
        # (at most 0.08 points per cubic A: the search that writes rows in order holds 1024 candidates around a tile)
        edge = max(7.0 + 3.0 * rng.random(), (n / 0.08) ** (1.0 / 3.0))
        box = np.eye(3) * edge + 0.4 * rng.normal(size=(3, 3))
        all_points.append(rng.random((n, 3)) @ box + rng.integers(-1, 2, size=(n, 3)) @ box)
        all_boxes.append(box)
        all_flags.append(flags)
    cutoff = 4.2
    complete = None
    for way in ("in order", "radix"):
        if way == "radix":
            monkeypatch.setenv("VESIN_HIP_SORT", "radix")
        calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
        for letters in ("PSdD", "Pd"):
            capfd.readouterr()
            lists = run_batch(calculator, all_points, all_boxes, letters=letters, periodic=np.array(all_flags))
            taken = [line for line in capfd.readouterr().err.splitlines() if line.startswith("in-order search (batch)")]
            if way == "radix":
                assert not taken
            else:
                assert len(taken) == 2 and all(line.endswith(": used") for line in taken), taken
            for s, (points, box, flags) in enumerate(zip(all_points, all_boxes, all_flags)):
                expected = oracle.canonicalize(oracle.neighbors(points, box, list(flags), cutoff, full, False, "ijSdD"))
                for key in lists[s]:
                    assert np.array_equal(lists[s][key], expected[key]), f"system {s}, {letters}, {way}: {key} differ or are out of order"
            complete = complete or lists
    monkeypatch.delenv("VESIN_HIP_SORT")
    # the same through one call per system
    single = NeighborList(cutoff=cutoff, full_list=full, sorted=True)
    for s in (0, 6, 7):
        pairs, shifts, distances = single.compute(
            torch.as_tensor(all_points[s], device="cuda:0"), torch.as_tensor(all_boxes[s], device="cuda:0"),
            list(all_flags[s]), "PSd",
        )
        assert np.array_equal(pairs.cpu().numpy(), complete[s]["pairs"])
        assert np.array_equal(shifts.cpu().numpy(), complete[s]["shifts"])
        assert np.array_equal(distances.cpu().numpy(), complete[s]["distances"])


def test_outputs_on_request_only():
    replicas = [configs.config3(r) for r in range(4)]
    calculator = NeighborList(cutoff=10.0, full_list=True)
    lists = run_batch(calculator, [r[0] for r in replicas], [r[1] for r in replicas], letters="Pd")
    for r, (points, box, periodic, _) in enumerate(replicas):
        expected = oracle.neighbors(points, box, periodic, 10.0, True, False, "ijSd")
        assert len(lists[r]["pairs"]) == len(expected["pairs"])
        assert np.array_equal(np.sort(lists[r]["distances"]), np.sort(expected["distances"]))


# ---- the full batch of the small-cell configuration: 4096 replicas in one call

_SIGNED = 1 << 63


def _signed(value):
    """A 64-bit pattern as the int64 that torch keeps it in."""
    value &= 0xFFFFFFFFFFFFFFFF
    return value - (1 << 64) if value >= _SIGNED else value


def _mix_on_device(x):
    """systems._mix on int64 tensors (same bits; shifts made logical by masking)."""
    x = x ^ ((x >> 30) & ((1 << 34) - 1))
    x = x * _signed(0xBF58476D1CE4E5B9)
    x = x ^ ((x >> 27) & ((1 << 37) - 1))
    x = x * _signed(0x94D049BB133111EB)
    return x ^ ((x >> 31) & ((1 << 33) - 1))


def _combine_on_device(h, column):
    return _mix_on_device(h * _signed(0x9E3779B97F4A7C15) + column + _signed(0x7F4A7C15))


def fingerprints_per_system_on_device(pairs, shifts, distances, first_pair):
    """The sums of ``systems.fingerprints`` (hash of (i, j, S) and of (i, j, S, bits of d), modulo 2^64) for every
    system of a batch, computed where the rows are: 190 million rows do not have to cross to the host."""
    import torch

    h = _combine_on_device(torch.zeros(pairs.shape[0], dtype=torch.int64, device=pairs.device), pairs[:, 0].view(torch.int64))
    h = _combine_on_device(h, pairs[:, 1].view(torch.int64))
    for d in range(3):
        h = _combine_on_device(h, shifts[:, d].to(torch.int64))
    hd = _combine_on_device(h, distances.view(torch.int64))
    edges = torch.as_tensor(np.asarray(first_pair, dtype=np.int64), device=pairs.device)
    out = []
    for hashes in (h, hd):
        running = torch.cat([torch.zeros(1, dtype=torch.int64, device=pairs.device), torch.cumsum(hashes, 0)])
        out.append((running[edges[1:]] - running[edges[:-1]]).cpu().numpy().view(np.uint64))
    return out


def test_the_device_side_fingerprints_are_those_of_the_host():
    import torch

    points, box, periodic, options = configs.config3(7)
    rows = oracle.neighbors(points, box, periodic, options["cutoff"], True, False, "ijSd")
    expected = systems.fingerprints(rows)
    n = len(rows["pairs"])
    ijS, d = fingerprints_per_system_on_device(
        torch.as_tensor(rows["pairs"].astype(np.int64), device="cuda:0"), torch.as_tensor(rows["shifts"], device="cuda:0"),
        torch.as_tensor(rows["distances"], device="cuda:0"), [0, n // 3, n],
    )
    with np.errstate(over="ignore"):
        assert int(ijS.sum(dtype=np.uint64)) == expected["ijS"] and int(d.sum(dtype=np.uint64)) == expected["d"]
    first = systems.fingerprints({key: value[: n // 3] for key, value in rows.items()})
    assert int(ijS[0]) == first["ijS"] and int(d[0]) == first["d"]


def test_config3_full_batch_of_4096_replicas():
    """64 atoms, box 7.134 A, cutoff 10 A, 4096 seeded replicas in ONE call: every system's rows against the oracle
    (fingerprints of (i, j, S) and of the distances' bits), both for the first call of a list (count, scan, write) and
    for the second (single-pass search); the whole batch against the compiled reference's fingerprint on record."""
    import json
    import os

    import torch

    replicas = [configs.config3(r) for r in range(4096)]
    cutoff = replicas[0][3]["cutoff"]
    expected = []
    for points, box, periodic, _ in replicas:
        expected.append(systems.fingerprints(oracle.neighbors(points, box, periodic, cutoff, True, False, "ijSd")))
    with open(os.path.join(os.path.dirname(systems.__file__), "reference_checksums.json")) as fd:
        golden = json.load(fd)["config3-batch4096"]
    assert systems.fingerprints_of_systems(expected) == golden

    first_point = np.cumsum([0] + [len(r[0]) for r in replicas])
    points = torch.as_tensor(np.concatenate([r[0] for r in replicas]), device="cuda:0")
    boxes = torch.as_tensor(np.stack([r[1] for r in replicas]), device="cuda:0")
    calculator = NeighborList(cutoff=cutoff, full_list=True)
    for call in ("first call", "second call"):
        (pairs, shifts, distances), first_pair = calculator.compute_batch(points, first_point, boxes, True, "PSd", copy=False)
        assert pairs.shape[0] == golden["n_pairs"] == 190477980
        assert first_pair[0] == 0 and first_pair[-1] == pairs.shape[0]
        assert int(pairs.view(torch.int64).max()) == 63  # indices count inside each system
        ijS, d = fingerprints_per_system_on_device(pairs, shifts, distances, first_pair)
        per_system = []
        for s, prints in enumerate(expected):
            rows = int(first_pair[s + 1] - first_pair[s])
            assert rows == prints["n_pairs"], f"{call}, system {s}: {rows} rows, expected {prints['n_pairs']}"
            assert int(ijS[s]) == prints["ijS"], f"{call}, system {s}: pairs or shifts differ from the oracle's"
            assert int(d[s]) == prints["d"], f"{call}, system {s}: distances differ from the oracle's"
            per_system.append({"n_pairs": rows, "ijS": int(ijS[s]), "d": int(d[s])})
        assert systems.fingerprints_of_systems(per_system) == golden, call
        del pairs, shifts, distances, ijS, d


def test_boxes_are_compared_on_the_device_and_a_change_is_never_missed(capfd, monkeypatch):
    """A batch whose other inputs are those of the call before starts from the grids it has while a kernel compares
    the boxes; a box that changed by one bit makes the call start over, and the list then reads the boxes first for
    32 calls. The rows are the oracle's every time."""
    import torch

    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(92)
    sizes = [40, 25, 60, 33, 48, 52]
    boxes = [np.diag(6.0 + rng.random(3)) + 0.3 * np.triu(rng.normal(size=(3, 3)), 1).T for _ in sizes]
    points = [rng.random((n, 3)) @ box for n, box in zip(sizes, boxes)]
    first_point = np.cumsum([0] + sizes)
    calculator = NeighborList(cutoff=4.0, full_list=True)
    started_over = []

    def run(boxes, check=True):
        capfd.readouterr()
        outputs, first_pair = calculator.compute_batch(
            torch.as_tensor(np.concatenate(points), device="cuda:0"), first_point,
            torch.as_tensor(np.stack(boxes), device="cuda:0"), True, "PSdD",
        )
        err = capfd.readouterr().err.splitlines()
        lines = [line for line in err if line.startswith("single pass (batch):")]
        started_over.append(any(line.startswith("batch: the boxes are not those of the call before") for line in err))
        if check:
            whole = {NAMES[q]: out.cpu().numpy() for q, out in zip("PSdD", outputs)}
            for s, (p, box) in enumerate(zip(points, boxes)):
                rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
                expected = oracle.neighbors(p, box, True, 4.0, True, False, "ijSdD")
                assert_same_list({k: v[rows] for k, v in whole.items()}, expected, what=f"system {s}")
        return [("grids of the call before" in line) for line in lines]

    assert run(boxes) == []            # sizes the arrays with the two passes
    assert run(boxes) == [True]
    assert run(boxes) == [True]
    nudged = [box.copy() for box in boxes]
    nudged[4][1, 1] = np.nextafter(nudged[4][1, 1], 10.0)  # one bit of one box
    # started from the old grids, found the box changed, started over with the boxes on the host
    assert run(nudged) == [False] and started_over == [False, False, False, True]
    guessed = [run(nudged, check=step in (0, 31, 32)) for step in range(34)]
    assert guessed[:31] == [[False]] * 31 and guessed[32:] == [[True]] * 2, guessed
    assert not any(started_over[4:])
    # a box that keeps changing: every wrong guess doubles the time until the next one
    del started_over[:]
    for step in range(70):
        other = [box.copy() for box in nudged]
        other[0][0, 0] += 1e-3 * (step + 1)
        assert run(other, check=step % 23 == 0) == [False]
    assert started_over[0] and sum(started_over) <= 2, started_over


@pytest.mark.parametrize("algorithm", ["auto", "cell_list", "brute_force"])
def test_free_molecules_get_their_grids_on_the_device(algorithm, capfd, monkeypatch):
    """A batch of systems without any periodic direction: from the second call with arrays on, the grids are picked
    on the device from the extent of this call's points. Molecules that drift, stretch and collapse, from one atom
    to a few hundred; the rows are the oracle's every time, and a flag that changes is noticed."""
    import torch

    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(93)
    sizes = [1, 2, 5, 17, 40, 64, 90, 300, 33, 3, 31, 32, 700]
    molecules = [rng.normal(scale=1.0 + 0.1 * n ** (1 / 3), size=(n, 3)) + rng.uniform(-40, 40, size=3) for n in sizes]
    first_point = np.cumsum([0] + sizes)
    boxes = np.zeros((len(sizes), 3, 3))
    calculator = NeighborList(cutoff=3.2, full_list=True, algorithm=algorithm)

    def run(molecules, flags, check=True):
        capfd.readouterr()
        outputs, first_pair = calculator.compute_batch(
            torch.as_tensor(np.concatenate(molecules), device="cuda:0"), first_point,
            torch.as_tensor(boxes, device="cuda:0"), flags, "PSdD",
        )
        err = capfd.readouterr().err.splitlines()
        if check:
            whole = {NAMES[q]: out.cpu().numpy() for q, out in zip("PSdD", outputs)}
            per_system = np.broadcast_to(np.asarray(flags, dtype=bool), (len(sizes), 3))
            for s, points in enumerate(molecules):
                rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
                box = np.eye(3) * 500.0 if per_system[s].any() else boxes[s]
                expected = oracle.neighbors(points, box, [bool(f) for f in per_system[s]], 3.2, True, False, "ijSdD")
                assert_same_list({k: v[rows] for k, v in whole.items()}, expected, what=f"system {s}")
        return sum("grids picked on the device" in line for line in err)

    assert run(molecules, False) == 0  # sizes the arrays
    assert run(molecules, False) == 1
    for step in range(6):
        if step == 2:
            molecules = [(m - m.mean(axis=0)) * 2.5 + m.mean(axis=0) for m in molecules]  # stretch
        elif step == 4:
            molecules = [(m - m.mean(axis=0)) * 0.2 + m.mean(axis=0) + 300.0 for m in molecules]  # collapse, far away
        else:
            molecules = [m + rng.normal(scale=0.2, size=m.shape) for m in molecules]
        assert run(molecules, False) == 1, step
    # one system becomes periodic along z: the flags are others, the call starts over with the boxes on the host
    flags = np.zeros((len(sizes), 3), dtype=bool)
    flags[4, 2] = True
    boxes[4] = np.eye(3) * 500.0
    assert run(molecules, flags) == 0
    assert run(molecules, flags) == 0
    # a coordinate that is not finite is reported by the kernels that pick the grids as by any other
    calculator2 = NeighborList(cutoff=3.2, full_list=True, algorithm=algorithm)
    calculator, kept = calculator2, calculator
    boxes[4] = 0.0
    assert run(molecules, False) == 0
    assert run(molecules, False) == 1
    broken = [m.copy() for m in molecules]
    broken[7][5, 1] = np.nan
    with pytest.raises(RuntimeError, match="point"):
        run(broken, False, check=False)
    assert run(molecules, False) in (0, 1)


@pytest.mark.parametrize("algorithm", ["auto", "cell_list"])
def test_stretched_open_systems_keep_to_the_room_for_their_cells(algorithm, capfd, monkeypatch):
    """Systems that are long in one direction and thin in the others (stretched chains, a pair of atoms moving apart)
    must not get more cells than the batch's buffers were sized for (64, or twice the points, per system), also when
    the grids are picked on the device: a chain that keeps getting longer from call to call, checked against the
    oracle on every call."""
    import torch

    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(11)
    sizes = [40, 2, 1000, 33, 64, 7]
    first_point = np.cumsum([0] + sizes)
    boxes = np.zeros((len(sizes), 3, 3))
    cutoff = 5.0
    calculator = NeighborList(cutoff=cutoff, full_list=True, algorithm=algorithm)

    def systems(stretch):
        out = []
        for k, n in enumerate(sizes):
            axis = k % 3
            points = rng.uniform(0.0, 3.0, size=(n, 3))
            # 1.5 points per cutoff along the chain at stretch 1: neighbours stay, cells multiply
            points[:, axis] = np.sort(rng.uniform(0.0, n * cutoff / 1.5 * stretch, size=n))
            out.append(points + rng.uniform(-50, 50, size=3))
        return out

    # (the longest chain stays below 100,000 cutoffs: beyond that many cells the reference's own grid, which the
    # oracle restates, has no cells left in the thin directions, vesin/src/cpu_cell_list.cpp:294-304)
    for call, stretch in enumerate([1.0, 1.0, 4.0, 25.0, 0.1, 100.0]):
        molecules = systems(stretch)
        capfd.readouterr()
        outputs, first_pair = calculator.compute_batch(
            torch.as_tensor(np.concatenate(molecules), device="cuda:0"), first_point,
            torch.as_tensor(boxes, device="cuda:0"), False, "PSdD",
        )
        err = capfd.readouterr().err
        assert ("grids picked on the device" in err) == (call >= 1), (call, err)
        whole = {NAMES[q]: out.cpu().numpy() for q, out in zip("PSdD", outputs)}
        for s, points in enumerate(molecules):
            rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
            expected = oracle.neighbors(points, np.eye(3) * 500.0, [False] * 3, cutoff, True, False, "ijSdD")
            assert_same_list({k: v[rows] for k, v in whole.items()}, expected, what=f"call {call}, system {s}")


def test_five_thousand_systems_of_every_kind_and_other_ones_with_every_call():
    """Enough systems for the host to go over them on several threads (boxes, grids), with open directions among
    them (extents of the points in between), and another set of systems with every call; a singular box among them is
    the error it always is."""
    rng = np.random.default_rng(91)
    calculator = NeighborList(cutoff=3.0, full_list=True)
    for call in range(3):
        all_points, all_boxes, all_flags = [], [], []
        for _ in range(5000):
            n = int(rng.integers(0, 24))
            edge = 4.0 + 4.0 * rng.random()
            box = np.eye(3) * edge + 0.2 * rng.normal(size=(3, 3))
            kind = rng.integers(0, 4)
            flags = [(True, True, True), (True, True, False), (False, False, False), (True, True, True)][kind]
            all_points.append(rng.random((n, 3)) @ box)
            all_boxes.append(box)
            all_flags.append(flags)
        if call == 2:
            all_boxes[4321] = all_boxes[4321].copy()
            all_boxes[4321][2] = all_boxes[4321][0]
            all_flags[4321] = (True, True, True)
            with pytest.raises(RuntimeError, match="the box matrix is not invertible"):
                run_batch(calculator, all_points, all_boxes, periodic=np.array(all_flags))
            continue
        lists = run_batch(calculator, all_points, all_boxes, periodic=np.array(all_flags))
        for s in rng.choice(5000, size=150, replace=False):
            expected = oracle.neighbors(all_points[s], all_boxes[s], list(all_flags[s]), 3.0, True, False, "ijSdD")
            assert_same_list(lists[s], expected, what=f"call {call}, system {s}")
