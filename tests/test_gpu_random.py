"""Randomised differential test of the HIP path against the CPU oracle (``-m gpu``): many small systems with random
boxes, periodicity, densities and cutoffs go through ONE reused list per option set, so that consecutive calls
exercise the single-pass search, its fallbacks (growth, crowded tiles, wrapped points), the remembered box and the
sliced small-system layout in whatever order the generator produces them."""

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from vesin_amd import NeighborList

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}


def random_system(rng, larger=False):
    kind = rng.integers(0, 6)
    n = int(rng.choice([1, 2, 3, 17, 64, 65, 200, 700, 1500]))
    edge = float(rng.uniform(3.0, 14.0))
    if larger:
        # beyond the 2048 points that one launch takes: the searches of the large systems, at a liquid's density
        n = int(rng.choice([2100, 3000, 5000, 9000]))
        edge = float((n / rng.uniform(0.03, 0.12)) ** (1.0 / 3.0))
    if kind == 0:  # cubic
        box = np.eye(3) * edge
    elif kind == 1:  # orthorhombic, one short axis (several images along it)
        box = np.diag([edge, edge * rng.uniform(0.2, 0.5), edge * rng.uniform(0.8, 1.6)])
    else:  # triclinic
        box = np.eye(3) * edge + rng.normal(scale=0.25 * edge, size=(3, 3)) * (np.arange(3)[:, None] > np.arange(3)[None, :])
    periodic = [bool(b) for b in rng.integers(0, 2, size=3)] if rng.random() < 0.5 else [True, True, True]
    points = rng.random((n, 3)) @ box
    if kind == 3:  # a crowded corner
        points[: n // 2] = points[: n // 2] * 0.15
    if kind == 4:  # points far outside the box
        points = points + rng.integers(-3, 4, size=(n, 3)) @ box
    if kind == 5 and n > 3:  # coincident points
        points[1] = points[0]
        points[-1] = points[-2]
    return points, box, periodic


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
@pytest.mark.parametrize("seed", range(8))
def test_random_systems_on_one_reused_list(seed, full):
    import torch

    rng = np.random.default_rng(1000 + seed)
    cutoff = float(rng.choice([1.5, 2.5, 3.7]))
    calculator = NeighborList(cutoff=cutoff, full_list=full)
    for step in range(14):
        points, box, periodic = random_system(rng)
        expected = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
        for repeat in range(2):  # the second call on the same input meets the remembered box and kept arrays
            outputs = calculator.compute(
                torch.as_tensor(points, device="cuda:0"), torch.as_tensor(box, device="cuda:0"), periodic, "PSdD"
            )
            actual = {NAMES[q]: t.cpu().numpy() for q, t in zip("PSdD", outputs)}
            assert_same_list(actual, expected, what=f"seed {seed} step {step} repeat {repeat} n={len(points)} periodic={periodic}")


@pytest.mark.parametrize("seed", range(60))
def test_random_options_and_moves_on_one_reused_list(seed):
    """Sorted or not, half or full, with or without a skin; a system is followed for a few small moves (which the
    Verlet filter and the remembered box meet) before the next one replaces it."""
    import torch

    rng = np.random.default_rng(50_000 + seed)
    cutoff = float(rng.choice([1.1, 1.5, 2.5, 3.7]))
    full = bool(rng.integers(0, 2))
    is_sorted = bool(rng.integers(0, 2))
    skin = float(rng.choice([0.0, 0.0, 0.3, 0.9]))
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=is_sorted, skin=skin)
    points = None
    for step in range(8):
        if points is None or rng.random() < 0.5:
            # (every third sequence mixes in systems of a few thousand points)
            points, box, periodic = random_system(rng, larger=seed % 3 == 2 and rng.random() < 0.5)
        else:
            points = points + rng.normal(scale=rng.choice([0.01, 0.1, 0.6]), size=points.shape)
            if rng.random() < 0.3:
                box = box + rng.normal(scale=0.02, size=(3, 3)) * (np.abs(box) > 0)
        expected = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
        outputs = calculator.compute(
            torch.as_tensor(points, device="cuda:0"), torch.as_tensor(box, device="cuda:0"), periodic, "PSdD"
        )
        actual = {NAMES[q]: t.cpu().numpy() for q, t in zip("PSdD", outputs)}
        what = f"seed {seed} step {step} n={len(points)} sorted={is_sorted} skin={skin} periodic={periodic}"
        if is_sorted:
            in_order = oracle.canonicalize(expected)
            assert actual["pairs"].shape == in_order["pairs"].shape, what
            for key in actual:
                assert np.array_equal(actual[key], in_order[key]), (what, key)
        else:
            assert_same_list(actual, expected, what=what)


def test_random_batches():
    import torch

    rng = np.random.default_rng(77)
    for trial in range(4):
        cutoff = float(rng.choice([2.0, 3.0]))
        full = bool(rng.integers(0, 2))
        n_systems = int(rng.integers(1, 12))
        all_points, all_boxes = [], []
        for _ in range(n_systems):
            points, box, _ = random_system(rng)
            all_points.append(points)
            all_boxes.append(box)
        first_point = np.cumsum([0] + [len(p) for p in all_points])
        calculator = NeighborList(cutoff=cutoff, full_list=full)
        outputs, first_pair = calculator.compute_batch(
            torch.as_tensor(np.concatenate(all_points), device="cuda:0"),
            first_point,
            torch.as_tensor(np.stack(all_boxes), device="cuda:0"),
            True,
            "PSdD",
        )
        whole = {NAMES[q]: t.cpu().numpy() for q, t in zip("PSdD", outputs)}
        for s in range(n_systems):
            rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
            expected = oracle.neighbors(all_points[s], all_boxes[s], True, cutoff, full, False, "ijSdD")
            assert_same_list({k: v[rows] for k, v in whole.items()}, expected, what=f"trial {trial} system {s}")


@pytest.mark.parametrize("seed", range(32))
def test_random_batches_on_one_reused_list(seed):
    """Batches of random systems, each with its own periodicity, sorted or not, on one reused list: a batch is
    followed for a few small moves (the set-up kept from the call before, boxes compared on the device, grids of open
    systems picked on the device, the searches that write sorted rows in order and their fallbacks) before another
    replaces it. Sorted rows are compared in place with the oracle's rows in (i, j, shift) order."""
    import torch

    rng = np.random.default_rng(90_000 + seed)
    cutoff = float(rng.choice([1.5, 2.5, 3.7]))
    full = bool(rng.integers(0, 2))
    is_sorted = bool(rng.integers(0, 4) > 0)
    all_open = seed % 4 == 3
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=is_sorted)
    systems = None
    for step in range(7):
        if systems is None or rng.random() < 0.35:
            systems = []
            for _ in range(int(rng.integers(1, 10))):
                points, box, periodic = random_system(rng, larger=seed % 8 == 5 and rng.random() < 0.2)
                if all_open:
                    periodic = [False, False, False]
                systems.append([points, box, periodic])
        else:
            for system in systems:
                system[0] = system[0] + rng.normal(scale=rng.choice([0.01, 0.1, 0.5]), size=system[0].shape)
        first_point = np.cumsum([0] + [len(s[0]) for s in systems])
        outputs, first_pair = calculator.compute_batch(
            torch.as_tensor(np.concatenate([s[0] for s in systems]).reshape(-1, 3), device="cuda:0"),
            first_point,
            torch.as_tensor(np.stack([s[1] for s in systems]), device="cuda:0"),
            np.array([s[2] for s in systems], dtype=bool),
            "PSdD",
        )
        whole = {NAMES[q]: t.cpu().numpy() for q, t in zip("PSdD", outputs)}
        assert first_pair[0] == 0 and first_pair[-1] == len(whole["pairs"])
        for k, (points, box, periodic) in enumerate(systems):
            rows = slice(int(first_pair[k]), int(first_pair[k + 1]))
            expected = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
            actual = {key: value[rows] for key, value in whole.items()}
            what = f"seed {seed} step {step} system {k} n={len(points)} sorted={is_sorted} periodic={periodic}"
            if is_sorted:
                in_order = oracle.canonicalize(expected)
                assert actual["pairs"].shape == in_order["pairs"].shape, what
                for key in actual:
                    assert np.array_equal(actual[key], in_order[key]), (what, key)
            else:
                assert_same_list(actual, expected, what=what)


@pytest.mark.parametrize("seed", range(24))
def test_every_kind_of_call_on_one_calculator(seed):
    """Every way of calling one calculator, in random order: ``compute`` with copies (which take the list's arrays
    over) and with views, batches, queued calls and queued batches, with ``sorted``, ``full_list`` and ``skin``
    changing in between. Every result against the oracle; what a queued call said on the device is either pending or
    the number of rows; results of earlier calls are checked again later (arrays that were handed over stay what
    they were whatever the list goes on to do)."""
    import torch

    rng = np.random.default_rng(430_000 + seed)
    cutoff = float(rng.choice([1.5, 2.5, 3.7]))
    calc = NeighborList(cutoff=cutoff, full_list=True)
    kept = []  # (tensors, expected dict, ordered, what)
    single = None
    batch = None
    for step in range(14):
        if rng.random() < 0.25:
            calc.sorted = bool(rng.integers(0, 2))
        if rng.random() < 0.15:
            calc.full_list = bool(rng.integers(0, 2))
        if rng.random() < 0.15:
            calc.skin = float(rng.choice([0.0, 0.0, 0.4]))
        full, is_sorted = calc.full_list, calc.sorted
        kinds = ["compute", "views", "batch", "enqueue", "enqueue_batch"]
        kind = rng.choice(kinds, p=[0.3, 0.1, 0.25, 0.2, 0.15])
        letters = "PSdD"
        what = f"seed {seed} step {step} {kind} sorted={is_sorted} full={full} skin={calc.skin}"
        if kind in ("compute", "views", "enqueue"):
            if single is None or rng.random() < 0.5:
                single = random_system(rng, larger=seed % 5 == 4 and rng.random() < 0.3)
            else:
                moved = single[0] + rng.normal(scale=rng.choice([0.01, 0.3]), size=single[0].shape)
                single = (moved, single[1], single[2])
            points, box, periodic = single
            tp = torch.as_tensor(points, device="cuda:0")
            tb = torch.as_tensor(box, device="cuda:0")
            expected = oracle.neighbors(points, box, periodic, cutoff, full, False, "ijSdD")
            if kind == "enqueue":
                flags = torch.as_tensor(np.array(periodic, dtype=bool), device="cuda:0")
                word = calc.enqueue(tp.contiguous(), tb.contiguous(), flags, letters)
                seen = word.clone()
                outputs = calc.collect(copy=bool(rng.integers(0, 2)))
                assert int(seen.item()) in (-1, len(outputs[0])), what
                assert int(word.item()) == len(outputs[0]), what
            else:
                outputs = calc.compute(tp, tb, periodic, letters, copy=(kind == "compute"))
            actual = {NAMES[q]: t.cpu().numpy() for q, t in zip(letters, outputs)}
            assert_same_list(actual, expected, ordered=is_sorted, what=what + f" n={len(points)} periodic={periodic}")
            if kind == "compute" and len(kept) < 6:
                kept.append((outputs, [expected], None, is_sorted, what))
        else:
            if batch is None or rng.random() < 0.5:
                batch = []
                free = rng.random() < 0.3
                for _ in range(int(rng.integers(1, 9))):
                    p, b, f = random_system(rng)
                    if free:
                        f = [False] * 3
                        p = p[: int(rng.integers(1, 60))]
                    batch.append([p, b, f])
            else:
                for s in batch:
                    s[0] = s[0] + rng.normal(scale=rng.choice([0.01, 0.3]), size=s[0].shape)
            first_point = np.cumsum([0] + [len(s[0]) for s in batch])
            args = (
                torch.as_tensor(np.concatenate([s[0] for s in batch]).reshape(-1, 3), device="cuda:0"),
                first_point,
                torch.as_tensor(np.stack([s[1] for s in batch]), device="cuda:0"),
                np.array([s[2] for s in batch], dtype=bool),
            )
            if kind == "enqueue_batch":
                word = calc.enqueue_batch(*args, letters)
                seen = word.clone()
                outputs, first_pair = calc.collect(copy=bool(rng.integers(0, 2)))
                assert int(seen.item()) in (-1, int(first_pair[-1])), what
                assert int(word.item()) == int(first_pair[-1]), what
                on_device = calc.first_pair_on_device()
                if first_point[-1] > 0:
                    assert np.array_equal(on_device.cpu().numpy().astype(np.uint64), first_pair), what
            else:
                copy = bool(rng.integers(0, 2))
                outputs, first_pair = calc.compute_batch(*args, letters, copy=copy)
            whole = {NAMES[q]: t.cpu().numpy() for q, t in zip(letters, outputs)}
            assert first_pair[0] == 0 and first_pair[-1] == len(whole["pairs"]), what
            exps = []
            for k, (p, b, f) in enumerate(batch):
                rows = slice(int(first_pair[k]), int(first_pair[k + 1]))
                exp = oracle.neighbors(p, b, f, cutoff, full, False, "ijSdD")
                exps.append(exp)
                assert_same_list(
                    {key: v[rows] for key, v in whole.items()}, exp, ordered=is_sorted,
                    what=what + f" system {k} n={len(p)} periodic={f}",
                )
        # results of earlier calls that were copies (or took the arrays over) are what they were
        if kept and rng.random() < 0.4:
            outputs, exps, fp, was_sorted, was = kept[int(rng.integers(0, len(kept)))]
            actual = {NAMES[q]: t.cpu().numpy() for q, t in zip("PSdD", outputs)}
            assert_same_list(actual, exps[0], ordered=was_sorted, what="kept result of " + was + " after " + what)
