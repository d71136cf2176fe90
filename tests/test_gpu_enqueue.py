"""vesin_hip_neighbors_enqueue / vesin_hip_neighbors_collect: a call in two halves. The first queues what a list in
its steady state needs (cell list, search, rows) on the caller's stream and comes back without waiting, so the caller
can queue the consumer of the rows right behind; the second looks at what the kernels found and completes the list
when the queued part did not (first call, arrays too small, another box). The reference ends every GPU call with a
device synchronisation (vesin/src/vesin_cuda.cpp:793-803, :899) and has no counterpart."""

import ctypes
import threading

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from vesin_amd import configs
from vesin_amd._c_api import VesinCUDA, VesinDevice, VesinNeighborList, VesinOptions, get_library

pytestmark = pytest.mark.gpu

ROWS_PENDING = 2**64 - 1


def _options(cutoff, full=True, sorted=False):
    options = VesinOptions()
    options.cutoff = cutoff
    options.full = full
    options.sorted = sorted
    options.return_shifts = True
    options.return_distances = True
    options.return_vectors = True
    return options


def _device(points, box, periodic):
    import torch

    return (
        torch.tensor(np.ascontiguousarray(points, dtype=np.float64), device="cuda:0"),
        torch.tensor(np.ascontiguousarray(box, dtype=np.float64), device="cuda:0"),
        torch.tensor(np.asarray(periodic, dtype=bool), device="cuda:0"),
    )


def _view(pointer, shape, typestr, owner):
    import torch

    from vesin_amd._neighbors import _DeviceView

    return torch.as_tensor(_DeviceView(pointer, shape, typestr, owner), device="cuda:0")


def _blocking(lib, inputs, options, neighbors, stream=None):
    points, box, periodic = inputs
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_on_stream(
        points.data_ptr(), points.shape[0], box.data_ptr(), periodic.data_ptr(), VesinDevice(VesinCUDA, 0), options,
        ctypes.byref(neighbors), stream, ctypes.byref(message),
    )
    assert status == 0, message.value


def _enqueue(lib, inputs, options, neighbors, stream):
    points, box, periodic = inputs
    message = ctypes.c_char_p()
    word = ctypes.c_void_p()
    status = lib.vesin_hip_neighbors_enqueue(
        points.data_ptr(), points.shape[0], box.data_ptr(), periodic.data_ptr(), VesinDevice(VesinCUDA, 0), options,
        ctypes.byref(neighbors), stream, ctypes.byref(word), ctypes.byref(message),
    )
    assert status == 0, message.value
    assert message.value is None and word.value
    return word.value


def _collect(lib, neighbors, expect_failure=False):
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_collect(ctypes.byref(neighbors), ctypes.byref(message))
    if expect_failure:
        assert status == 1
        return message.value.decode()
    assert status == 0, message.value
    assert message.value is None
    return None


def _rows(neighbors):
    n = neighbors.length
    return {
        "pairs": _view(neighbors.pairs, (n, 2), "<u8", neighbors).cpu().numpy(),
        "shifts": _view(neighbors.shifts, (n, 3), "<i4", neighbors).cpu().numpy(),
        "distances": _view(neighbors.distances, (n,), "<f8", neighbors).cpu().numpy(),
        "vectors": _view(neighbors.vectors, (n, 3), "<f8", neighbors).cpu().numpy(),
    }


class Consumer:
    """What a caller queues behind the list on the same stream, with nothing but tensor operations (no value comes to
    the host in between): a copy of the device word, and sums over the rows below that count of what identifies a
    row. `room` rows of the arrays are looked at (the arrays of the list hold that many)."""

    def __init__(self, neighbors, word, room):
        import torch

        count = _view(word, (1,), "<i8", neighbors)
        self.count = count.clone()
        there = (torch.arange(room, device="cuda:0") < count).to(torch.int64)  # all zero while the word says pending
        pairs = _view(neighbors.pairs, (room, 2), "<i8", neighbors)
        shifts = _view(neighbors.shifts, (room, 3), "<i4", neighbors).to(torch.int64)
        distances = _view(neighbors.distances, (room,), "<f8", neighbors)
        self.sums = torch.stack([
            (pairs[:, 0] * there).sum(), (pairs[:, 1] * there).sum(), (pairs[:, 0] * pairs[:, 1] % 1000003 * there).sum(),
            ((shifts[:, 0] * 3 + shifts[:, 1] * 5 + shifts[:, 2] * 7) * (pairs[:, 1] % 97) * there).sum(),
        ])
        self.distance_sum = torch.where(there.to(torch.bool), distances, torch.zeros_like(distances)).sum()

    def check(self, rows):
        """Against the rows the host finally reads: the consumer saw exactly these, through the word it was given."""
        n = len(rows["pairs"])
        assert int(self.count.item()) == n
        i = rows["pairs"][:, 0].astype(np.int64)
        j = rows["pairs"][:, 1].astype(np.int64)
        s = rows["shifts"].astype(np.int64)
        expected = [i.sum(), j.sum(), (i * j % 1000003).sum(), ((s[:, 0] * 3 + s[:, 1] * 5 + s[:, 2] * 7) * (j % 97)).sum()]
        assert self.sums.cpu().numpy().tolist() == [int(v) for v in expected]
        assert np.isclose(float(self.distance_sum.item()), rows["distances"].sum(), rtol=1e-12)

    def saw_nothing(self):
        assert int(self.count.item()) == -1  # VESIN_HIP_ROWS_PENDING read as a signed word
        assert self.sums.cpu().numpy().tolist() == [0, 0, 0, 0]


def _busy(stream):
    """Keeps `stream` busy for a few milliseconds, so that whatever is queued behind has certainly not run when the
    host looks right after queueing it."""
    import torch

    with torch.cuda.stream(stream):
        filler = torch.zeros((16384, 8192), device="cuda:0")
        for _ in range(12):
            filler = filler * 1.0001 + 1.0
    return filler


CASES = [
    pytest.param(12, 5.0, True, False, id="13824 atoms, unsorted: single-pass search"),
    pytest.param(12, 5.0, False, False, id="13824 atoms, half list, unsorted"),
    pytest.param(12, 5.0, True, True, id="13824 atoms, sorted: in-order search"),
    pytest.param(3, 5.0, True, True, id="216 atoms, sorted: one launch"),
    pytest.param(4, 4.0, False, False, id="512 atoms, half list, unsorted: one launch"),
]


@pytest.mark.parametrize("cells, cutoff, full, sorted", CASES)
def test_a_list_in_its_steady_state_is_queued_whole(cells, cutoff, full, sorted):
    import torch

    lib = get_library()
    options = _options(cutoff, full, sorted)
    stream = torch.cuda.Stream()
    neighbors = VesinNeighborList()
    try:
        # two calls that size the arrays and remember the box
        first = configs.diamond(cells, seed=40)
        inputs = _device(*first)
        torch.cuda.synchronize()
        for _ in range(2):
            _blocking(lib, inputs, options, neighbors, stream.cuda_stream)
        room = neighbors.length
        arrays_before = (neighbors.pairs, neighbors.shifts, neighbors.distances, neighbors.vectors)
        for step in range(3):
            # other positions in the same box: the rows are others every time
            points, box, periodic = configs.diamond(cells, seed=41 + step, sigma=0.04)
            expected = oracle.neighbors(points, box, periodic, cutoff, full, sorted, "ijSdD")
            assert len(expected["pairs"]) <= room + room // 8
            inputs = _device(points, box, periodic)
            torch.cuda.synchronize()
            _busy(stream)
            word = _enqueue(lib, inputs, options, neighbors, stream.cuda_stream)
            queued = not stream.query()
            with torch.cuda.stream(stream):
                consumer = Consumer(neighbors, word, room + room // 8)
            still_queued = not stream.query()
            _collect(lib, neighbors)
            assert queued and still_queued, "the call waited for the stream instead of queueing its work"
            assert (neighbors.pairs, neighbors.shifts, neighbors.distances, neighbors.vectors) == arrays_before
            stream.synchronize()
            rows = _rows(neighbors)
            assert_same_list(rows, expected, ordered=sorted, what=f"step {step}")
            consumer.check(rows)
            assert int(_view(word, (1,), "<i8", neighbors).item()) == neighbors.length
    finally:
        lib.vesin_free(ctypes.byref(neighbors))


@pytest.mark.parametrize("sorted", [False, True], ids=["unsorted", "sorted"])
def test_a_list_with_a_skin_is_queued_whole_while_its_candidates_hold(sorted):
    """options.skin > 0: a call that only filters the kept candidates is two launches, all queued; when a point has
    moved too far the word stays pending and collect computes the candidates again."""
    import torch

    lib = get_library()
    options = _options(5.0, True, sorted)
    options.skin = 1.0
    stream = torch.cuda.Stream()
    neighbors = VesinNeighborList()
    try:
        inputs = _device(*configs.diamond(6, seed=60, sigma=0.02))
        torch.cuda.synchronize()
        for _ in range(2):
            _blocking(lib, inputs, options, neighbors, stream.cuda_stream)  # the search and the candidates; a filter
        room = neighbors.length
        for step, sigma in enumerate([0.02, 0.02, 0.02, 0.6, 0.6]):
            points, box, periodic = configs.diamond(6, seed=61 + (step if sigma < 0.1 else 3), sigma=sigma)
            expected = oracle.neighbors(points, box, periodic, 5.0, True, sorted, "ijSdD")
            inputs = _device(points, box, periodic)
            torch.cuda.synchronize()
            _busy(stream)
            word = _enqueue(lib, inputs, options, neighbors, stream.cuda_stream)
            queued = not stream.query()
            with torch.cuda.stream(stream):
                consumer = Consumer(neighbors, word, min(room, len(expected["pairs"])))
            _collect(lib, neighbors)
            assert queued, "the call waited for the stream instead of queueing its work"
            stream.synchronize()
            rows = _rows(neighbors)
            assert_same_list(rows, expected, ordered=sorted, what=f"step {step}")
            assert int(_view(word, (1,), "<i8", neighbors).item()) == neighbors.length
            if step < 3 or step == 4:
                # within the skin of the candidates (step 4: of the candidates that step 3 computed)
                assert len(expected["pairs"]) <= room + room // 8
                if len(expected["pairs"]) <= room:
                    consumer.check(rows)
            else:
                consumer.saw_nothing()
            room = max(room, neighbors.length)
    finally:
        lib.vesin_free(ctypes.byref(neighbors))


def test_what_the_queued_part_cannot_finish_is_finished_by_collect():
    """The first call of a list (no arrays yet), rows that outgrow the arrays, and a box that is not the one of the
    call before: the consumer queued in between finds the word pending and touches nothing; after collect the list is
    the oracle's and the word holds its length."""
    import torch

    lib = get_library()
    options = _options(5.0, True, False)
    stream = torch.cuda.Stream()
    neighbors = VesinNeighborList()
    try:
        small = configs.diamond(8, seed=50)
        squeezed = (small[0] * 0.8, small[1], small[2])  # the same points in half the volume: twice the rows
        compressed = (small[0] * 0.97, small[1] * 0.97, small[2])
        systems = [
            ("first call", small),
            ("steady", small),
            ("rows outgrow the arrays", squeezed),
            ("steady with the new rows", squeezed),
            ("another box", compressed),
            ("the call after a box that changed", compressed),
        ]
        complete_when_queued = []
        for what, (points, box, periodic) in systems:
            expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
            inputs = _device(points, box, periodic)
            torch.cuda.synchronize()
            room = 0 if neighbors.pairs is None else min(neighbors.length, len(expected["pairs"]))
            word = _enqueue(lib, inputs, options, neighbors, stream.cuda_stream)
            consumer = None
            if room > 0:
                with torch.cuda.stream(stream):
                    consumer = Consumer(neighbors, word, room)
            else:
                with torch.cuda.stream(stream):
                    seen = _view(word, (1,), "<i8", neighbors).clone()
            _collect(lib, neighbors)
            stream.synchronize()
            rows = _rows(neighbors)
            assert_same_list(rows, expected, what=what)
            assert int(_view(word, (1,), "<i8", neighbors).item()) == len(expected["pairs"]), what
            if consumer is None:
                complete_when_queued.append(int(seen.item()) != -1)
            else:
                complete_when_queued.append(int(consumer.count.item()) != -1)
                if complete_when_queued[-1]:
                    assert int(consumer.count.item()) == len(expected["pairs"]), what
                else:
                    consumer.saw_nothing()
        # (after a box that changed the list reads the box first for a while, as every blocking call does as well)
        assert complete_when_queued == [False, True, False, True, False, False], complete_when_queued
    finally:
        lib.vesin_free(ctypes.byref(neighbors))


def test_errors_come_out_of_collect_and_the_list_stays_usable():
    import torch

    lib = get_library()
    options = _options(5.0, True, False)
    stream = torch.cuda.Stream()
    neighbors = VesinNeighborList()
    try:
        points, box, periodic = configs.diamond(8, seed=60)
        expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
        good = _device(points, box, periodic)
        for _ in range(2):
            _blocking(lib, good, options, neighbors, stream.cuda_stream)
        broken_points = points.copy()
        broken_points[1234, 2] = np.nan
        broken = _device(broken_points, box, periodic)
        torch.cuda.synchronize()
        word = _enqueue(lib, broken, options, neighbors, stream.cuda_stream)
        with torch.cuda.stream(stream):
            seen = _view(word, (1,), "<i8", neighbors).clone()
        # the list is taken until the queued call was collected
        message = ctypes.c_char_p()
        status = lib.vesin_hip_neighbors_on_stream(
            good[0].data_ptr(), good[0].shape[0], good[1].data_ptr(), good[2].data_ptr(), VesinDevice(VesinCUDA, 0),
            options, ctypes.byref(neighbors), stream.cuda_stream, ctypes.byref(message),
        )
        assert status == 1 and b"vesin_hip_neighbors_collect" in message.value
        text = _collect(lib, neighbors, expect_failure=True)
        assert "point 1234 has non-finite coordinate along axis 2" in text
        assert int(seen.item()) == -1
        # collecting twice is harmless; the list works as before
        _collect(lib, neighbors)
        word = _enqueue(lib, good, options, neighbors, stream.cuda_stream)
        _collect(lib, neighbors)
        assert_same_list(_rows(neighbors), expected, what="after the error")
    finally:
        lib.vesin_free(ctypes.byref(neighbors))
    # a list that never queued anything has nothing to collect
    other = VesinNeighborList()
    message = ctypes.c_char_p()
    assert lib.vesin_hip_neighbors_collect(ctypes.byref(other), ctypes.byref(message)) == 1
    assert b"no calculation was queued" in message.value


def test_collect_on_another_host_thread_free_with_a_call_pending_and_no_points():
    import torch

    lib = get_library()
    options = _options(5.0, True, True)
    stream = torch.cuda.Stream()
    neighbors = VesinNeighborList()
    points, box, periodic = configs.diamond(6, seed=70)
    expected = oracle.neighbors(points, box, periodic, 5.0, True, True, "ijSdD")
    inputs = _device(points, box, periodic)
    torch.cuda.synchronize()
    for _ in range(2):
        _blocking(lib, inputs, options, neighbors, stream.cuda_stream)
    _enqueue(lib, inputs, options, neighbors, stream.cuda_stream)
    failures = []

    def collect():
        try:
            _collect(lib, neighbors)
        except BaseException as error:  # noqa: BLE001 - reported by the main thread
            failures.append(repr(error))

    thread = threading.Thread(target=collect)
    thread.start()
    thread.join()
    assert not failures, failures
    assert_same_list(_rows(neighbors), expected, ordered=True, what="collected by another thread")

    # no points: nothing to wait for, the call is complete when enqueue returns (collect is still fine to call)
    empty = torch.zeros((0, 3), dtype=torch.float64, device="cuda:0")
    message = ctypes.c_char_p()
    word = ctypes.c_void_p()
    status = lib.vesin_hip_neighbors_enqueue(
        inputs[0].data_ptr(), 0, inputs[1].data_ptr(), inputs[2].data_ptr(), VesinDevice(VesinCUDA, 0), options,
        ctypes.byref(neighbors), stream.cuda_stream, ctypes.byref(word), ctypes.byref(message),
    )
    assert status == 0, message.value
    _collect(lib, neighbors)
    assert neighbors.length == 0
    stream.synchronize()
    assert int(_view(word.value, (1,), "<i8", neighbors).item()) == 0
    del empty

    # freed with a call pending: the call is completed first
    _enqueue(lib, inputs, options, neighbors, stream.cuda_stream)
    lib.vesin_free(ctypes.byref(neighbors))
    assert neighbors.pairs is None and neighbors.opaque is None
    torch.cuda.synchronize()


def test_the_python_caller_in_two_halves():
    """NeighborList.enqueue / collect: the word on the device as a tensor that work on torch's current stream reads,
    the rows of compute, a pending call refused, an error raised by collect."""
    import torch

    from vesin_amd import NeighborList

    points, box, periodic, options = configs.config0()
    inputs = _device(points, box, [bool(p) for p in np.broadcast_to(periodic, 3)])
    expected = oracle.canonicalize(oracle.neighbors(points, box, periodic, options["cutoff"], True, False, "ijSd"))
    calculator = NeighborList(cutoff=options["cutoff"], full_list=True, sorted=True)
    counts = []
    for call in range(3):
        word = calculator.enqueue(*inputs, quantities="PSd")
        seen = word.clone()  # queued on the same stream, no host synchronisation in between
        with pytest.raises(RuntimeError, match="pending"):
            calculator.enqueue(*inputs, quantities="PSd")
        pairs, shifts, distances = calculator.collect()
        counts.append(int(seen.item()))
        assert np.array_equal(pairs.cpu().numpy(), expected["pairs"]), call
        assert np.array_equal(shifts.cpu().numpy(), expected["shifts"]), call
        assert np.array_equal(distances.cpu().numpy(), expected["distances"]), call
        assert int(word.item()) == len(expected["pairs"])
    # the list's first call cannot be queued whole, its later calls are
    assert counts == [-1, len(expected["pairs"]), len(expected["pairs"])]
    with pytest.raises(RuntimeError, match="no call pending"):
        calculator.collect()
    bad = inputs[0].clone()
    bad[7, 1] = float("nan")
    calculator.enqueue(bad, inputs[1], inputs[2], quantities="P")
    with pytest.raises(RuntimeError, match="finite|NaN|nan"):
        calculator.collect()
    # and the calculator is as usable as before
    (pairs,) = calculator.compute(inputs[0], inputs[1], periodic, "P")
    assert np.array_equal(pairs.cpu().numpy(), expected["pairs"])
