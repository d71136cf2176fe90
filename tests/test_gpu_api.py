"""Behaviour of the C ABI and of the Python caller on a real GPU (``-m gpu``): buffer reuse, ownership of the
outputs, error paths that need a device, concurrency, dtypes and shapes."""

import ctypes
import os
import threading

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from golden import systems
from vesin_amd import NeighborList, _c_api, enable_timings

pytestmark = pytest.mark.gpu


def device_inputs(points, box, periodic):
    import torch

    return (
        torch.as_tensor(np.ascontiguousarray(points, dtype=np.float64), device="cuda:0"),
        torch.as_tensor(np.ascontiguousarray(box, dtype=np.float64), device="cuda:0"),
        torch.as_tensor(np.asarray(periodic, dtype=np.bool_), device="cuda:0"),
    )


def raw_call(lib, neighbors, points, box, periodic, **kwargs):
    options = _c_api.VesinOptions()
    options.cutoff = kwargs.get("cutoff", 3.4)
    options.full = kwargs.get("full", False)
    options.sorted = kwargs.get("sorted", False)
    options.algorithm = kwargs.get("algorithm", 0)
    options.return_shifts = kwargs.get("shifts", False)
    options.return_distances = kwargs.get("distances", False)
    options.return_vectors = kwargs.get("vectors", False)
    message = ctypes.c_char_p()
    status = lib.vesin_neighbors(
        points.data_ptr() if hasattr(points, "data_ptr") else points, kwargs.get("n_points", 1),
        box.data_ptr() if hasattr(box, "data_ptr") else box,
        periodic.data_ptr() if hasattr(periodic, "data_ptr") else periodic,
        _c_api.VesinDevice(_c_api.VesinCUDA, kwargs.get("device_id", 0)), options, ctypes.byref(neighbors),
        ctypes.byref(message),
    )
    return status, (message.value.decode() if message.value else None)


def test_allocations_are_reused_and_unrequested_outputs_are_null():
    # vesin/tests/memory.cpp:5-87 on the GPU
    import torch

    lib = _c_api.get_library()
    points, box, periodic = device_inputs([[0.0, 0.0, 0.0]], [[0.0, 1.5, 1.5], [1.5, 0.0, 1.5], [1.5, 1.5, 0.0]], [True] * 3)
    neighbors = _c_api.VesinNeighborList()

    status, message = raw_call(lib, neighbors, points, box, periodic, cutoff=3.4, distances=True)
    assert (status, message) == (0, None)
    assert neighbors.length == 9
    assert neighbors.pairs and neighbors.distances and not neighbors.shifts and not neighbors.vectors
    first_pairs = neighbors.pairs

    assert raw_call(lib, neighbors, points, box, periodic, cutoff=6.0, distances=True) == (0, None)
    assert neighbors.length == 67 and neighbors.pairs == first_pairs  # no reallocation for a list that still fits

    assert raw_call(lib, neighbors, points, box, periodic, cutoff=6.0, full=True, distances=True) == (0, None)
    assert neighbors.length == 134

    assert raw_call(lib, neighbors, points, box, periodic, cutoff=4.5, shifts=True) == (0, None)
    assert neighbors.length == 27
    assert neighbors.pairs and neighbors.shifts and not neighbors.distances and not neighbors.vectors

    lib.vesin_free(ctypes.byref(neighbors))
    assert neighbors.length == 0 and not neighbors.pairs and not neighbors.opaque and neighbors.device.type == 0
    torch.cuda.synchronize()


def test_pointer_checks():
    # vesin/src/vesin_cuda.cpp:831-854
    lib = _c_api.get_library()
    points, box, periodic = device_inputs(np.zeros((4, 3)), np.eye(3) * 5, [True] * 3)
    host = np.zeros(16)
    neighbors = _c_api.VesinNeighborList()
    assert raw_call(lib, neighbors, host.ctypes.data, box, periodic) == (1, "`points` pointer is not allocated on a CUDA device")
    assert raw_call(lib, neighbors, points, host.ctypes.data, periodic) == (1, "`box` pointer is not allocated on a CUDA device")
    assert raw_call(lib, neighbors, points, box, host.ctypes.data) == (1, "`periodic` pointer is not allocated on a CUDA device")
    # a list is bound to the device of its first call; a fresh one asked for a GPU that does not exist fails
    fresh = _c_api.VesinNeighborList()
    status, message = raw_call(lib, fresh, points, box, periodic, device_id=77)
    assert status == 1 and "device_id" in message
    # the list is still usable afterwards
    neighbors = _c_api.VesinNeighborList()
    assert raw_call(lib, neighbors, points, box, periodic, n_points=4) == (0, None)
    lib.vesin_free(ctypes.byref(neighbors))


def test_errors_through_the_python_caller():
    import torch

    calculator = NeighborList(cutoff=1.0, full_list=True)
    points = torch.zeros((3, 3), dtype=torch.float64, device="cuda:0")
    with pytest.raises(RuntimeError, match="the box matrix is not invertible"):
        calculator.compute(points, torch.zeros((3, 3), dtype=torch.float64, device="cuda:0"), True, "ij")
    bad = points.clone()
    bad[2, 1] = float("inf")
    with pytest.raises(RuntimeError, match="point 2 has non-finite coordinate along axis 1: inf"):
        calculator.compute(bad, torch.eye(3, dtype=torch.float64, device="cuda:0") * 4, True, "ij")
    with pytest.raises(RuntimeError, match="point 2 has non-finite coordinate along axis 1: inf"):
        calculator.compute(bad, torch.eye(3, dtype=torch.float64, device="cuda:0") * 4, False, "ij")
    with pytest.raises(ValueError, match="n_threads must be zero or a positive integer"):
        NeighborList(cutoff=1.0, full_list=True, n_threads=-1)
    with pytest.raises(ValueError, match="Unknown algorithm"):
        NeighborList(cutoff=1.0, full_list=True, algorithm="magic")
    with pytest.raises(RuntimeError, match="cutoff must be a finite, positive number"):
        NeighborList(cutoff=-1.0, full_list=True).compute(points, torch.eye(3, dtype=torch.float64, device="cuda:0"), True)
    # and the calculator survives its errors
    i, j = calculator.compute(points, torch.eye(3, dtype=torch.float64, device="cuda:0") * 4, True, "ij")
    assert len(i) == 6


def test_pairs_per_point_limit_from_the_environment():
    # python/vesin/tests/test_cupy.py:292-336: the variable is honoured as a user-imposed limit, with the same texts
    box = np.eye(3) * 3.0
    points = np.random.default_rng(0).random((100, 3)) * 3.0
    calculator = NeighborList(cutoff=4, full_list=True)
    assert len(calculator.compute(points, box, True, "ijSDd")[0]) > 12800  # no default capacity to overflow
    try:
        os.environ["VESIN_CUDA_MAX_PAIRS_PER_POINT"] = "1000"
        calculator.compute(points, box, True, "ijSDd")
        os.environ["VESIN_CUDA_MAX_PAIRS_PER_POINT"] = "10"
        message = (
            "The number of neighbor pairs exceeds the maximum capacity of 1000 "
            "\\(max_pairs_per_point=10; n_points=100\\). Consider reducing the "
            "cutoff distance, or explicitly setting VESIN_CUDA_MAX_PAIRS_PER_POINT as "
            "an environment variable."
        )
        with pytest.raises(RuntimeError, match=message):
            calculator.compute(points, box, True, "ijSDd")
        for invalid in ["-3", "44 ABC", "0", "-1", "1.5", ""]:
            os.environ["VESIN_CUDA_MAX_PAIRS_PER_POINT"] = invalid
            with pytest.raises(RuntimeError, match=f"Invalid value for VESIN_CUDA_MAX_PAIRS_PER_POINT: '{invalid}'"):
                calculator.compute(points, box, True, "ijSDd")
    finally:
        os.environ.pop("VESIN_CUDA_MAX_PAIRS_PER_POINT", None)


def test_ten_host_threads_at_once():
    # vesin/tests/cuda.cpp:141-157: independent lists from concurrent host threads
    points, box, periodic = systems.diamond_crystal()
    expected = oracle.neighbors(points, box, periodic, 5.0, False, False, "ijSdD")
    failures = []

    def worker():
        try:
            import torch

            calculator = NeighborList(cutoff=5.0, full_list=False)
            for _ in range(5):
                outputs = calculator.compute(
                    torch.as_tensor(points, device="cuda:0"), torch.as_tensor(box, device="cuda:0"), periodic, "PSdD"
                )
                actual = dict(zip(("pairs", "shifts", "distances", "vectors"), (o.cpu().numpy() for o in outputs)))
                assert_same_list(actual, expected)
        except Exception as e:  # noqa: BLE001
            failures.append(e)

    threads = [threading.Thread(target=worker) for _ in range(10)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures[0]


def test_dtypes_shapes_and_views():
    # python/vesin/tests/test_numpy.py:272-284, test_cupy.py:277-289, _neighbors.py:295-305
    import torch

    box = torch.eye(3, dtype=torch.float64, device="cuda:0") * 3.0
    points = torch.as_tensor(np.random.default_rng(0).random((100, 3)) * 3.0, device="cuda:0")
    calculator = NeighborList(cutoff=1, full_list=True)
    i, j, s, D, d, P = calculator.compute(points, box, True, "ijSDdP")
    assert i.dtype == torch.uint64 and j.dtype == torch.uint64 and P.dtype == torch.uint64
    assert s.dtype == torch.int32 and D.dtype == torch.float64 and d.dtype == torch.float64
    assert i.device.type == "cuda"
    assert P.shape == (len(i), 2) and s.shape == (len(i), 3) and D.shape == (len(i), 3) and d.shape == (len(i),)
    assert torch.equal(P[:, 0].to(torch.int64), i.to(torch.int64))

    # float32 in, float32 out (the calculation itself is always fp64)
    i32, d32 = calculator.compute(points.float(), box.float(), True, "id")
    assert d32.dtype == torch.float32

    # views alias the library's buffers
    (view,) = calculator.compute(points, box, True, "d", copy=False)
    (copy,) = calculator.compute(points, box, True, "d", copy=True)
    assert torch.equal(view, copy)

    # empty result
    i, j, s, D, d = calculator.compute(points[:1], box, False, "ijSDd")
    assert i.shape == (0,) and s.shape == (0, 3) and D.shape == (0, 3) and d.shape == (0,)
    # no points at all
    (P,) = calculator.compute(points[:0], box, True, "P")
    assert P.shape == (0, 2)

    # numpy in, numpy out
    i, S = NeighborList(cutoff=1, full_list=True).compute(points.cpu().numpy(), box.cpu().numpy(), True, "iS")
    assert isinstance(i, np.ndarray) and i.dtype == np.uint64 and S.dtype == np.int32

    with pytest.raises(ValueError, match="`box` must be a 3x3 matrix"):
        calculator.compute(points, box[:2], True, "ij")
    with pytest.raises(ValueError, match="`points` must be a nx3 array"):
        calculator.compute(points[:, :2], box, True, "ij")
    with pytest.raises(RuntimeError, match="same dtype"):
        calculator.compute(points, box.float(), True, "ij")


def test_stage_timings_are_reported():
    import torch

    enable_timings(True)
    try:
        points, box, periodic = systems.diamond_crystal()
        calculator = NeighborList(cutoff=5.0, full_list=True, sorted=True)
        calculator.compute(torch.as_tensor(points, device="cuda:0"), torch.as_tensor(box, device="cuda:0"), periodic, "ijS")
        timings = calculator.timings()
        assert timings is not None and timings["total"] > 0 and timings["write"] > 0 and timings["sort"] > 0
    finally:
        enable_timings(False)
