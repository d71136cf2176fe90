"""vesin_hip_neighbors_no_alloc: the rows of vesin_hip_neighbors_on_stream, written into arrays of the caller's, with
work memory that is part of the library instead of allocations. Every call is compared with the allocating entry
point on the same inputs (bit for bit, as sets of rows for unsorted lists and in place for sorted ones) and, for the
small systems, with the CPU oracle."""

import ctypes

import numpy as np
import pytest

import oracle
from _helpers import _fully_ordered
from vesin_amd import configs
from vesin_amd._c_api import VesinCUDA, VesinDevice, VesinNeighborList, VesinOptions, get_library

pytestmark = pytest.mark.gpu

KEYS = ("pairs", "shifts", "distances", "vectors")


def _options(cutoff, full, sorted, quantities="SdD"):
    options = VesinOptions()
    options.cutoff = cutoff
    options.full = full
    options.sorted = sorted
    options.return_shifts = "S" in quantities
    options.return_distances = "d" in quantities
    options.return_vectors = "D" in quantities
    return options


class CallerArrays:
    """Output arrays the caller owns: allocated once, before any call of the entry point under test."""

    def __init__(self, capacity):
        import torch

        self.capacity = capacity
        self.pairs = torch.full((capacity, 2), -1, dtype=torch.int64, device="cuda:0")
        self.shifts = torch.full((capacity, 3), 77, dtype=torch.int32, device="cuda:0")
        self.distances = torch.full((capacity,), -1.0, dtype=torch.float64, device="cuda:0")
        self.vectors = torch.full((capacity, 3), -1.0, dtype=torch.float64, device="cuda:0")

    def reset(self):
        self.pairs.fill_(-1)
        self.shifts.fill_(77)
        self.distances.fill_(-1.0)
        self.vectors.fill_(-1.0)

    def rows(self, n, options):
        out = {"pairs": self.pairs[:n].cpu().numpy().astype(np.uint64)}
        if options.return_shifts:
            out["shifts"] = self.shifts[:n].cpu().numpy()
        if options.return_distances:
            out["distances"] = self.distances[:n].cpu().numpy()
        if options.return_vectors:
            out["vectors"] = self.vectors[:n].cpu().numpy()
        return out


def _no_alloc(lib, points, box, periodic, options, arrays, stream=None, expect_failure=False):
    length = ctypes.c_size_t(0)
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_no_alloc(
        points.data_ptr(), points.shape[0], box.data_ptr(), periodic.data_ptr(), VesinDevice(VesinCUDA, 0), options,
        arrays.pairs.data_ptr(), arrays.shifts.data_ptr(), arrays.distances.data_ptr(), arrays.vectors.data_ptr(),
        arrays.capacity, ctypes.byref(length), stream, ctypes.byref(message),
    )
    if expect_failure:
        assert status == 1
        return length.value, message.value.decode()
    assert status == 0, message.value
    assert message.value is None
    return length.value


def _allocating(lib, points, box, periodic, options):
    """The existing entry point on the same inputs; two calls, so that the second goes the way of a reused list."""
    import torch

    from vesin_amd._neighbors import _DeviceView

    neighbors = VesinNeighborList()
    message = ctypes.c_char_p()
    try:
        for _ in range(2):
            status = lib.vesin_hip_neighbors_on_stream(
                points.data_ptr(), points.shape[0], box.data_ptr(), periodic.data_ptr(), VesinDevice(VesinCUDA, 0),
                options, ctypes.byref(neighbors), None, ctypes.byref(message),
            )
            assert status == 0, message.value
        n = neighbors.length
        out = {}
        for name, pointer, shape, typestr in (
            ("pairs", neighbors.pairs, (n, 2), "<u8"),
            ("shifts", neighbors.shifts, (n, 3), "<i4"),
            ("distances", neighbors.distances, (n,), "<f8"),
            ("vectors", neighbors.vectors, (n, 3), "<f8"),
        ):
            if pointer:
                out[name] = torch.as_tensor(_DeviceView(pointer, shape, typestr, neighbors), device="cuda:0").cpu().numpy()
        return out
    finally:
        lib.vesin_free(ctypes.byref(neighbors))


def _same_rows(actual, expected, in_place):
    assert set(actual) == set(expected)
    if not in_place:
        actual, expected = _fully_ordered(actual), _fully_ordered(expected)
    for key in actual:
        assert actual[key].shape == expected[key].shape, (key, actual[key].shape, expected[key].shape)
        assert np.array_equal(actual[key], expected[key]), key


def _device(points, box, periodic):
    import torch

    return (
        torch.tensor(np.ascontiguousarray(points), device="cuda:0"),
        torch.tensor(np.ascontiguousarray(box), device="cuda:0"),
        torch.tensor(np.asarray(periodic, dtype=bool), device="cuda:0"),
    )


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
@pytest.mark.parametrize("sorted", [False, True], ids=["unsorted", "sorted"])
def test_two_calls_in_a_row_the_second_smaller(full, sorted):
    """A 13,824-atom system, then a 1,728-atom one through the same work memory: what the first call left there must
    not show in the second. Then the first again."""
    import torch

    lib = get_library()
    arrays = CallerArrays(1_400_000)
    torch.cuda.synchronize()
    options = _options(5.0, full, sorted)
    for cells, seed in ((12, 5), (6, 6), (12, 5)):
        points, box, periodic = configs.diamond(cells, seed=seed)
        d_points, d_box, d_periodic = _device(points, box, periodic)
        expected = _allocating(lib, d_points, d_box, d_periodic, options)
        arrays.reset()
        torch.cuda.synchronize()
        n = _no_alloc(lib, d_points, d_box, d_periodic, options, arrays)
        assert n == len(expected["pairs"])
        _same_rows(arrays.rows(n, options), expected, in_place=sorted)
        if cells == 6:
            reference = oracle.neighbors(points, box, periodic, 5.0, full, sorted, "ijSdD")
            _same_rows(
                oracle.canonicalize(arrays.rows(n, options)), oracle.canonicalize(reference), in_place=True
            )
        # nothing beyond the rows was written
        assert int(arrays.pairs[n, 0]) == -1 and float(arrays.distances[n]) == -1.0


def test_unrequested_arrays_are_left_alone_and_shapes_vary():
    """Clustered points without periodic directions, a small triclinic cell with many images, a handful of points;
    only distances requested."""
    lib = get_library()
    arrays = CallerArrays(600_000)
    rng = np.random.default_rng(11)
    systems = [
        (rng.normal(0.0, 6.0, (4000, 3)), np.zeros((3, 3)), (False, False, False), 3.0),
        (rng.uniform(0.0, 4.0, (40, 3)), np.array([[4.0, 0.0, 0.0], [1.0, 4.0, 0.0], [0.5, 0.7, 4.0]]), (True, True, True), 7.5),
        (rng.uniform(0.0, 10.0, (3, 3)), np.eye(3) * 10.0, (True, False, True), 6.0),
    ]
    for points, box, periodic, cutoff in systems:
        options = _options(cutoff, True, False, "d")
        d_points, d_box, d_periodic = _device(points, box, periodic)
        expected = _allocating(lib, d_points, d_box, d_periodic, options)
        n = _no_alloc(lib, d_points, d_box, d_periodic, options, arrays)
        assert n == len(expected["pairs"])
        _same_rows(arrays.rows(n, options), expected, in_place=False)
        reference = oracle.neighbors(points, box, periodic, cutoff, True, False, "ijd")
        _same_rows(arrays.rows(n, options), reference, in_place=False)
        assert int(arrays.shifts[0, 0]) == 77 and float(arrays.vectors[0, 0]) == -1.0


@pytest.mark.parametrize("sorted", [False, True], ids=["unsorted", "sorted"])
def test_small_systems_take_one_launch_here_too(sorted, capfd, monkeypatch):
    """Systems of at most 2048 points go through the one launch that builds the cells, searches and writes (its two
    meeting words live in the library's work array); several in a row through the same array, each against the
    allocating entry point and the oracle."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    lib = get_library()
    arrays = CallerArrays(400_000)
    rng = np.random.default_rng(19)
    systems = [configs.diamond(3, seed=1), configs.diamond(4, seed=2), configs.diamond(3, seed=3)]
    systems.append((rng.uniform(0.0, 9.0, (150, 3)), np.zeros((3, 3)), (False, False, False)))
    used = 0
    for points, box, periodic in systems:
        periodic = [bool(p) for p in np.broadcast_to(np.asarray(periodic), (3,))]
        options = _options(4.5, True, sorted)
        d_points, d_box, d_periodic = _device(points, box, periodic)
        expected = _allocating(lib, d_points, d_box, d_periodic, options)
        arrays.reset()
        capfd.readouterr()
        n = _no_alloc(lib, d_points, d_box, d_periodic, options, arrays)
        used += sum(line.startswith("one launch:") and "gave up 0" in line for line in capfd.readouterr().err.splitlines())
        assert n == len(expected["pairs"])
        _same_rows(arrays.rows(n, options), expected, in_place=sorted)
        reference = oracle.neighbors(points, box, periodic, 4.5, True, False, "ijSdD")
        _same_rows(arrays.rows(n, options), oracle.canonicalize(reference) if sorted else reference, in_place=sorted)
        assert int(arrays.pairs[n, 0]) == -1
    assert used == len(systems)


def test_device_memory_in_use_does_not_change():
    """The contract is that nothing is allocated or freed: the free memory of the device (hipMemGetInfo) is, byte for
    byte, what it was, after calls of every kind through the same work array: a large system unsorted and sorted, small
    ones through the one launch, a system without periodic directions, and a sorted list that needs the radix sort (a
    cell of many images). One call of each kind comes first: the runtime itself sets up what it needs for a kernel or
    a copy (code objects, staging) the first time that one is used."""
    import torch

    lib = get_library()
    arrays = CallerArrays(1_400_000)
    rng = np.random.default_rng(23)
    cases = []
    for points, box, periodic, cutoff in (
        (*configs.diamond(12, seed=5), 5.0),
        (*configs.diamond(3, seed=1), 5.0),
        (rng.normal(0.0, 6.0, (4000, 3)), np.zeros((3, 3)), (False, False, False), 3.0),
        (rng.uniform(0.0, 9.0, (150, 3)), np.zeros((3, 3)), (False, False, False), 4.5),
        (rng.uniform(0.0, 4.0, (40, 3)), np.array([[4.0, 0.0, 0.0], [1.0, 4.0, 0.0], [0.5, 0.7, 4.0]]), (True, True, True), 7.5),
    ):
        periodic = [bool(p) for p in np.broadcast_to(np.asarray(periodic), (3,))]
        for sorted in (False, True):
            cases.append((_device(points, box, periodic), _options(cutoff, True, sorted)))
    counts = []
    for (d_points, d_box, d_periodic), options in cases:  # warm-up
        counts.append(_no_alloc(lib, d_points, d_box, d_periodic, options, arrays))
    torch.cuda.synchronize()
    free_before, total = torch.cuda.mem_get_info()
    for repeat in range(3):
        for k, ((d_points, d_box, d_periodic), options) in enumerate(cases):
            assert _no_alloc(lib, d_points, d_box, d_periodic, options, arrays) == counts[k]
            free_now, _ = torch.cuda.mem_get_info()
            assert free_now == free_before, (repeat, k, free_before - free_now)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info() == (free_before, total)


def test_on_a_stream_of_the_caller():
    import torch

    lib = get_library()
    arrays = CallerArrays(200_000)
    points, box, periodic = configs.diamond(6, seed=3)
    d_points, d_box, d_periodic = _device(points, box, periodic)
    options = _options(5.0, True, True)
    expected = _allocating(lib, d_points, d_box, d_periodic, options)
    stream = torch.cuda.Stream()
    torch.cuda.synchronize()
    n = _no_alloc(lib, d_points, d_box, d_periodic, options, arrays, stream=stream.cuda_stream)
    _same_rows(arrays.rows(n, options), expected, in_place=True)


def test_limits_are_errors_with_a_message():
    import torch

    lib = get_library()
    points, box, periodic = configs.diamond(6, seed=3)
    d_points, d_box, d_periodic = _device(points, box, periodic)
    options = _options(5.0, True, False)
    expected = _allocating(lib, d_points, d_box, d_periodic, options)
    n_rows = len(expected["pairs"])

    # arrays that are too small: the message and `length` say how many rows there are; a second call with enough
    # room succeeds
    small = CallerArrays(1000)
    length, message = _no_alloc(lib, d_points, d_box, d_periodic, options, small, expect_failure=True)
    assert length == n_rows
    assert f"the neighbor list has {n_rows} pairs, the output arrays of the caller hold 1000" in message
    arrays = CallerArrays(n_rows)
    assert _no_alloc(lib, d_points, d_box, d_periodic, options, arrays) == n_rows
    _same_rows(arrays.rows(n_rows, options), expected, in_place=False)

    # too many points
    many = torch.zeros((262_145, 3), dtype=torch.float64, device="cuda:0")
    _, message = _no_alloc(lib, many, d_box, d_periodic, options, arrays, expect_failure=True)
    assert "at most 262144 points" in message

    # a skin needs memory that outlives the call
    with_skin = _options(5.0, True, False)
    with_skin.skin = 0.5
    _, message = _no_alloc(lib, d_points, d_box, d_periodic, with_skin, arrays, expect_failure=True)
    assert "skin" in message

    # a requested array that is missing
    length = ctypes.c_size_t(0)
    error = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_no_alloc(
        d_points.data_ptr(), d_points.shape[0], d_box.data_ptr(), d_periodic.data_ptr(), VesinDevice(VesinCUDA, 0),
        options, arrays.pairs.data_ptr(), None, arrays.distances.data_ptr(), arrays.vectors.data_ptr(),
        arrays.capacity, ctypes.byref(length), None, ctypes.byref(error),
    )
    assert status == 1 and b"`shifts` is requested" in error.value


def test_the_largest_system_it_takes():
    """262,144 points (the limit) at the density of the other tests: the work memory holds it."""
    lib = get_library()
    points, box, periodic = configs.diamond(32, seed=9)
    assert len(points) == 262_144
    d_points, d_box, d_periodic = _device(points, box, periodic)
    options = _options(5.0, True, False, "Sd")
    expected = _allocating(lib, d_points, d_box, d_periodic, options)
    arrays = CallerArrays(len(expected["pairs"]) + 64)
    n = _no_alloc(lib, d_points, d_box, d_periodic, options, arrays)
    assert n == len(expected["pairs"])
    from golden import systems

    assert systems.fingerprints(arrays.rows(n, options)) == systems.fingerprints(expected)
