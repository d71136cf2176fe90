"""vesin_hip_neighbors_on_stream and vesin_hip_neighbors_batch_on_stream: the same calculations issued on a stream
of the caller's instead of the null stream (the reference works on the null stream only,
vesin/src/vesin_cuda.cpp:793-803)."""

import ctypes
import threading

import numpy as np
import pytest

import oracle
from vesin_amd import configs
from vesin_amd._c_api import VesinCUDA, VesinDevice, VesinNeighborList, VesinOptions, get_library

pytestmark = pytest.mark.gpu


def _options(cutoff, full=True, sorted=True):
    options = VesinOptions()
    options.cutoff = cutoff
    options.full = full
    options.sorted = sorted
    options.return_shifts = True
    options.return_distances = True
    options.return_vectors = True
    return options


def _call(lib, points, box, periodic, options, neighbors, stream):
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_on_stream(
        points.data_ptr(), points.shape[0], box.data_ptr(), periodic.data_ptr(), VesinDevice(VesinCUDA, 0), options,
        ctypes.byref(neighbors), stream, ctypes.byref(message),
    )
    assert status == 0, message.value
    assert message.value is None


def _to_host(neighbors):
    import torch

    from vesin_amd._neighbors import _DeviceView  # the Python caller's own zero-copy wrapper

    n = neighbors.length
    out = {}
    for name, pointer, shape, typestr in (
        ("pairs", neighbors.pairs, (n, 2), "<u8"),
        ("shifts", neighbors.shifts, (n, 3), "<i4"),
        ("distances", neighbors.distances, (n,), "<f8"),
        ("vectors", neighbors.vectors, (n, 3), "<f8"),
    ):
        out[name] = torch.as_tensor(_DeviceView(pointer, shape, typestr, neighbors), device="cuda:0").cpu().numpy()
    return out


def test_inputs_produced_on_the_same_stream_need_no_synchronisation():
    import torch

    lib = get_library()
    points, box, periodic = configs.diamond(6, seed=21)
    expected = oracle.canonicalize(oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD"))
    host_points = torch.tensor(points).pin_memory()
    device_box = torch.tensor(box, device="cuda:0")
    device_periodic = torch.tensor(periodic, device="cuda:0")
    torch.cuda.synchronize()

    stream = torch.cuda.Stream()
    neighbors = VesinNeighborList()
    try:
        for _ in range(3):  # two-pass first, then the single-pass search; sorted so that rows compare in place
            with torch.cuda.stream(stream):
                # a long chain of kernels, then the copy the list depends on: all of it only queued so far
                filler = torch.zeros((4096, 4096), device="cuda:0")
                for _ in range(20):
                    filler = filler * 1.0001 + 1.0
                device_points = host_points.to("cuda:0", non_blocking=True) + 0.0
            _call(lib, device_points, device_box, device_periodic, _options(5.0), neighbors, stream.cuda_stream)
            result = _to_host(neighbors)
            for key in ("pairs", "shifts", "distances", "vectors"):
                assert np.array_equal(result[key], expected[key]), key
    finally:
        lib.vesin_free(ctypes.byref(neighbors))


def test_two_host_threads_on_two_streams():
    import torch

    lib = get_library()
    systems = [configs.diamond(4, seed=31), configs.diamond(5, seed=32)]
    expected = [
        oracle.canonicalize(oracle.neighbors(points, box, periodic, 4.0, False, False, "ijSdD"))
        for points, box, periodic in systems
    ]
    on_device = [
        (torch.tensor(points, device="cuda:0"), torch.tensor(box, device="cuda:0"), torch.tensor(periodic, device="cuda:0"))
        for points, box, periodic in systems
    ]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    failures = []

    def work(k):
        neighbors = VesinNeighborList()
        try:
            for _ in range(20):
                _call(lib, *on_device[k], _options(4.0, full=False), neighbors, streams[k].cuda_stream)
                result = _to_host(neighbors)
                for key in ("pairs", "shifts", "distances", "vectors"):
                    if not np.array_equal(result[key], expected[k][key]):
                        failures.append((k, key))
        except Exception as error:  # noqa: BLE001 - reported by the main thread
            failures.append((k, repr(error)))
        finally:
            lib.vesin_free(ctypes.byref(neighbors))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(2)]
    for thread in threads:
        thread.start()
    for thread in threads:
        thread.join()
    assert not failures, failures


def test_null_stream_handle_is_the_plain_call():
    import torch

    lib = get_library()
    points, box, periodic = configs.diamond(3, seed=0)
    expected = oracle.canonicalize(oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD"))
    neighbors = VesinNeighborList()
    try:
        _call(
            lib, torch.tensor(points, device="cuda:0"), torch.tensor(box, device="cuda:0"),
            torch.tensor(periodic, device="cuda:0"), _options(5.0), neighbors, None,
        )
        result = _to_host(neighbors)
        for key in ("pairs", "shifts", "distances", "vectors"):
            assert np.array_equal(result[key], expected[key]), key
    finally:
        lib.vesin_free(ctypes.byref(neighbors))


def test_batch_with_inputs_produced_on_the_same_stream():
    import torch

    lib = get_library()
    rng = np.random.default_rng(33)
    systems = []
    for s in range(40):
        n = int(rng.integers(1, 90))
        box = np.diag(rng.uniform(6.0, 12.0, size=3)) + rng.uniform(-0.5, 0.5, size=(3, 3))
        flags = [True, True, True] if s % 3 else [bool(f) for f in rng.integers(0, 2, size=3)]
        systems.append((rng.random((n, 3)) @ box, box, flags))
    first_point = np.zeros(len(systems) + 1, dtype=np.uint64)
    first_point[1:] = np.cumsum([len(p) for p, _, _ in systems])
    host_points = torch.tensor(np.concatenate([p for p, _, _ in systems])).pin_memory()
    host_boxes = torch.tensor(np.stack([b for _, b, _ in systems])).pin_memory()
    host_flags = torch.tensor(np.array([f for _, _, f in systems], dtype=np.bool_)).pin_memory()
    expected = [oracle.canonicalize(oracle.neighbors(p, b, f, 4.0, False, False, "ijSdD")) for p, b, f in systems]
    torch.cuda.synchronize()

    options = _options(4.0, full=False, sorted=False)
    stream = torch.cuda.Stream()
    neighbors = VesinNeighborList()
    first_pair = np.zeros(len(systems) + 1, dtype=np.uint64)
    try:
        for _ in range(3):  # two passes first, then the single pass into the arrays that are kept
            with torch.cuda.stream(stream):
                filler = torch.zeros((4096, 4096), device="cuda:0")
                for _ in range(20):
                    filler = filler * 1.0001 + 1.0
                device_points = host_points.to("cuda:0", non_blocking=True) + 0.0
                device_boxes = host_boxes.to("cuda:0", non_blocking=True) + 0.0
                device_flags = host_flags.to("cuda:0", non_blocking=True).clone()
            message = ctypes.c_char_p()
            status = lib.vesin_hip_neighbors_batch_on_stream(
                device_points.data_ptr(), first_point.ctypes.data_as(ctypes.POINTER(ctypes.c_size_t)), len(systems),
                device_boxes.data_ptr(), device_flags.data_ptr(), VesinDevice(VesinCUDA, 0), options,
                ctypes.byref(neighbors), first_pair.ctypes.data_as(ctypes.POINTER(ctypes.c_size_t)), stream.cuda_stream,
                ctypes.byref(message),
            )
            assert status == 0, message.value
            result = _to_host(neighbors)
            assert first_pair[-1] == neighbors.length
            for s, want in enumerate(expected):
                rows = slice(int(first_pair[s]), int(first_pair[s + 1]))
                got = oracle.canonicalize({key: value[rows] for key, value in result.items()})
                for key in ("pairs", "shifts", "distances", "vectors"):
                    assert np.array_equal(got[key], want[key]), (s, key)
    finally:
        lib.vesin_free(ctypes.byref(neighbors))
