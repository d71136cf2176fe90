"""vesin_hip_neighbors_batch_enqueue / vesin_hip_neighbors_collect: a batch in two halves (``-m gpu``). The first
queues what the batch can do before the host needs an answer from the GPU and comes back, the second completes the
call. Per system the rows must be those of a call on that system alone, whatever part of the call was queued (a
list's first call, the same division into systems again, other systems, other boxes). The reference ends every GPU
call with a device synchronisation (vesin/src/vesin_cuda.cpp:793-803, :899) and has no batched call: no counterpart."""

import threading

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from vesin_amd import NeighborList, configs

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}


def _on_device(all_points, all_boxes, all_flags):
    import torch

    first_point = np.cumsum([0] + [len(p) for p in all_points])
    points = torch.as_tensor(np.concatenate(all_points).astype(np.float64).reshape(-1, 3), device="cuda:0")
    boxes = torch.as_tensor(np.stack(all_boxes).astype(np.float64), device="cuda:0")
    flags = torch.as_tensor(np.asarray(all_flags, dtype=bool), device="cuda:0")
    return points, first_point, boxes, flags


def _per_system(outputs, first_pair, letters="PSdD"):
    whole = {NAMES[q]: out.cpu().numpy() for q, out in zip(letters, outputs)}
    assert first_pair[0] == 0 and first_pair[-1] == len(whole["pairs"])
    return [
        {key: value[int(first_pair[s]) : int(first_pair[s + 1])] for key, value in whole.items()}
        for s in range(len(first_pair) - 1)
    ]


def _check(lists, all_points, all_boxes, all_flags, cutoff, full, is_sorted, what):
    assert len(lists) == len(all_points)
    for s, (points, box, flags) in enumerate(zip(all_points, all_boxes, all_flags)):
        expected = oracle.neighbors(points, box, list(flags), cutoff, full, False, "ijSdD")
        if is_sorted:
            expected = oracle.canonicalize(expected)
        assert_same_list(lists[s], expected, ordered=is_sorted, what=f"{what}, system {s} periodic={flags}")


def _mixed_systems(rng, sizes):
    all_points, all_boxes, all_flags = [], [], []
    kinds = [(False, False, False), (True, True, True), (True, True, False), (False, True, False), (True, False, True)]
    for k, n in enumerate(sizes):
        flags = kinds[k % len(kinds)]
        edge = 7.0 + 3.0 * rng.random()
        box = np.eye(3) * edge + 0.4 * rng.normal(size=(3, 3))
        all_points.append(rng.random((n, 3)) @ box * rng.choice([0.6, 1.0, 1.7]))
        all_boxes.append(box)
        all_flags.append(flags)
    return all_points, all_boxes, all_flags


@pytest.mark.parametrize("is_sorted", [False, True], ids=["unsorted", "sorted"])
@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_a_batch_in_two_halves_gives_the_rows_of_the_blocking_call(full, is_sorted):
    """Molecules, slabs and crystals in one batch, on one list: its first call, the same systems again (what a list
    keeps between batches applies), moved points, other boxes, another division into systems. Between the two halves
    more work is queued on the stream, and the word on the device says that the rows are pending until collect."""
    import torch

    rng = np.random.default_rng(97 + 2 * full + is_sorted)
    cutoff = 3.1
    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=is_sorted)
    sizes = (5, 180, 64, 300, 1, 90, 0, 700, 400, 33)
    systems = _mixed_systems(rng, sizes)
    stream = torch.cuda.Stream()
    for step in range(6):
        if step == 2:
            systems = (
                [p + 0.05 * rng.normal(size=p.shape) for p in systems[0]],
                systems[1],
                systems[2],
            )
        elif step == 3:
            systems = (systems[0], [b * 1.02 for b in systems[1]], systems[2])
        elif step == 4:
            systems = _mixed_systems(rng, (40, 12, 256, 90, 7))
        inputs = _on_device(*systems)
        with torch.cuda.stream(stream):
            busy = torch.ones(1 << 20, device="cuda:0").cumsum(0)  # (something ahead of the batch on its stream)
            word = calculator.enqueue_batch(*inputs, quantities="PSdD")
            seen = word.clone()  # queued behind the batch, no host synchronisation in between
            with pytest.raises(RuntimeError, match="pending"):
                calculator.enqueue_batch(*inputs, quantities="PSdD")
            outputs, first_pair = calculator.collect()
        lists = _per_system(outputs, first_pair)
        _check(lists, *systems, cutoff, full, is_sorted, f"step {step}")
        stream.synchronize()
        # (systems with open directions beside periodic ones: the host picks the grids from the points of every call,
        # so the queued part never is the whole call)
        assert int(seen.item()) == -1
        assert int(word.item()) == int(first_pair[-1])
        assert np.array_equal(calculator.first_pair_on_device().cpu().numpy().astype(np.uint64), first_pair)
        assert float(busy[-1]) == float(1 << 20)
        # the blocking call on the same list gives the same rows (and leaves the list fit for the next queued call)
        again, first_again = calculator.compute_batch(*inputs, quantities="PSdD")
        assert np.array_equal(first_again, first_pair)
        for s, (a, b) in enumerate(zip(_per_system(again, first_again), lists)):
            assert_same_list(a, b, ordered=is_sorted, what=f"step {step}, system {s}: blocking call after the queued one")


@pytest.mark.parametrize("is_sorted", [False, True], ids=["unsorted", "sorted"])
def test_free_molecules_and_a_skin(is_sorted):
    """Batches of small free molecules (kernels of their own) and batches with a skin (kept candidates, filtered) are
    queued the same way."""
    rng = np.random.default_rng(5 + is_sorted)
    cutoff = 2.4
    molecules = [rng.normal(size=(int(n), 3)) * 1.6 for n in rng.integers(1, 40, size=300)]
    boxes = [np.zeros((3, 3))] * len(molecules)
    flags = [(False, False, False)] * len(molecules)
    for skin in (0.0, 0.5):
        calculator = NeighborList(cutoff=cutoff, full_list=True, sorted=is_sorted, skin=skin)
        systems = (molecules, boxes, flags)
        for step in range(4):
            if step > 0:
                # small moves: a list with a skin filters its candidates, until the last step moves too far
                move = 0.04 if step < 3 else 0.6
                systems = ([p + move * rng.normal(size=p.shape) for p in systems[0]], boxes, flags)
            inputs = _on_device(*systems)
            word = calculator.enqueue_batch(*inputs, quantities="PSdD")
            seen = word.clone()  # queued behind the batch, no host synchronisation in between
            on_device = calculator.first_pair_on_device()
            seen_first_pair = on_device.clone() if on_device is not None else None
            outputs, first_pair = calculator.collect()
            _check(_per_system(outputs, first_pair), *systems, cutoff, True, is_sorted, f"skin {skin} step {step}")
            total = int(first_pair[-1])
            assert int(word.item()) == total
            assert int(seen.item()) in (-1, total), f"skin {skin} step {step}"
            if skin == 0.0 and step == 1:
                # other molecules than those of the call before, and still the whole call is queued: work behind it
                # finds the number of rows and every system's first row on the device
                assert int(seen.item()) == total
            if int(seen.item()) == total and skin == 0.0:
                assert np.array_equal(seen_first_pair.cpu().numpy().astype(np.uint64), first_pair)
            assert np.array_equal(calculator.first_pair_on_device().cpu().numpy().astype(np.uint64), first_pair)


def test_errors_other_threads_and_lists_dropped_with_a_batch_pending():
    import torch

    rng = np.random.default_rng(11)
    cutoff = 3.0
    systems = _mixed_systems(rng, (50, 120, 64, 9))
    inputs = _on_device(*systems)
    calculator = NeighborList(cutoff=cutoff, full_list=True)
    for _ in range(2):
        calculator.enqueue_batch(*inputs, quantities="PSdD")
        outputs, first_pair = calculator.collect()
    _check(_per_system(outputs, first_pair), *systems, cutoff, True, False, "before the error")

    # an error of the calculation comes out of collect, and the list stays usable
    bad = inputs[0].clone()
    bad[60, 2] = float("nan")
    calculator.enqueue_batch(bad, *inputs[1:], quantities="PSdD")
    with pytest.raises(RuntimeError, match="finite|NaN|nan"):
        calculator.collect()
    with pytest.raises(RuntimeError, match="no call pending"):
        calculator.collect()

    # an error of the inputs comes out of the first half, with nothing pending afterwards
    with pytest.raises(RuntimeError, match="first_point"):
        calculator.enqueue_batch(inputs[0], np.array([0, 5, 3, 10, 20]), *inputs[2:], quantities="P")
    outputs, first_pair = calculator.compute_batch(*inputs, quantities="PSdD")
    _check(_per_system(outputs, first_pair), *systems, cutoff, True, False, "after the errors")

    # every other entry point refuses a list with a batch pending; collect on another host thread
    calculator.enqueue_batch(*inputs, quantities="PSdD")
    with pytest.raises(RuntimeError, match="pending|queued"):
        calculator.compute_batch(*inputs, quantities="PSdD")
    collected = {}

    def collect():
        try:
            collected["result"] = calculator.collect()
        except Exception as error:  # noqa: BLE001
            collected["error"] = error

    thread = threading.Thread(target=collect)
    thread.start()
    thread.join()
    assert "error" not in collected, collected.get("error")
    outputs, first_pair = collected["result"]
    _check(_per_system(outputs, first_pair), *systems, cutoff, True, False, "collected on another thread")

    # a calculator dropped with a batch pending completes it first
    calculator.enqueue_batch(*inputs, quantities="PSdD")
    del calculator
    torch.cuda.synchronize()


def test_the_small_cell_batch_queued():
    """Replicas of the 64-atom cell with a cutoff above the box (one cell, 125 images): the shape of the batched
    benchmark, first call and reused list."""
    replicas = 24
    all_points, all_boxes = [], []
    for r in range(replicas):
        points, box, periodic, options = configs.config3(r)
        all_points.append(points)
        all_boxes.append(box)
    flags = [(True, True, True)] * replicas
    cutoff = options["cutoff"]
    inputs = _on_device(all_points, all_boxes, flags)
    for is_sorted in (False, True):
        calculator = NeighborList(cutoff=cutoff, full_list=True, sorted=is_sorted)
        counts = []
        for call in range(4):
            word = calculator.enqueue_batch(*inputs, quantities="PSdD")
            seen = word.clone()
            on_device = calculator.first_pair_on_device()
            seen_first_pair = on_device.clone() if on_device is not None else None
            outputs, first_pair = calculator.collect()
            _check(_per_system(outputs, first_pair), all_points, all_boxes, flags, cutoff, True, is_sorted, f"call {call}")
            counts.append(int(seen.item()))
            assert int(word.item()) == int(first_pair[-1])
            if counts[-1] != -1:
                assert np.array_equal(seen_first_pair.cpu().numpy().astype(np.uint64), first_pair)
        total = int(first_pair[-1])
        if is_sorted:
            # (the search that writes the rows in order has a second wait: its queued part is never the whole call)
            assert counts == [-1] * 4
        else:
            # the list's first batch sizes the arrays; from then on the same systems and boxes are queued whole
            assert counts == [-1, total, total, total]
    # a call on a single system in between: no batch, nothing to point at
    points, box, periodic, _ = configs.config3(0)
    import torch

    calculator.compute(torch.tensor(points, device="cuda:0"), torch.tensor(box, device="cuda:0"), True, "P")
    assert calculator.first_pair_on_device() is None
