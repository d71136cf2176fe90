"""Output arrays from the caller's allocator, handed over instead of copied (vesin_hip_set_output_allocator,
vesin_hip_detach_outputs, vesin_hip_output_capacity). The reference copies every array out of the list's memory for a
caller that wants to keep it (python/vesin/vesin/_neighbors.py:343-381, vesin-torch/src/vesin_torch.cpp:214-256) and
has no counterpart; the rows must be the ones a copy would have held, and stay what they are when the list goes on."""

import ctypes
import gc

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from vesin_amd import NeighborList, configs
from vesin_amd._c_api import VesinCUDA, VesinDevice, VesinNeighborList, VesinOptions, get_library

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}

# PyTorch's allocator counts the blocks it hands out, and hands out a cached block of up to 1 MB more than was asked
# for without splitting it: the memory in use after the same calls differs by what its cache held. Arrays that stayed
# behind would add 0.8 MB per call and array in the loops below, 32 MB in all at least.
SLACK = 16 << 20


def _device(points, box, periodic):
    import torch

    return (
        torch.tensor(np.ascontiguousarray(points, dtype=np.float64), device="cuda:0"),
        torch.tensor(np.ascontiguousarray(box, dtype=np.float64), device="cuda:0"),
        torch.tensor(np.asarray(periodic, dtype=bool), device="cuda:0"),
    )


def _options(cutoff, full=True, sorted=False, quantities="SdD"):
    options = VesinOptions()
    options.cutoff = cutoff
    options.full = full
    options.sorted = sorted
    options.return_shifts = "S" in quantities
    options.return_distances = "d" in quantities
    options.return_vectors = "D" in quantities
    return options


def _host(outputs, letters):
    return {NAMES[q]: out.cpu().numpy() for q, out in zip(letters, outputs)}


class CountingAllocator:
    """An allocator of the caller's own behind the two C callbacks: device memory from PyTorch's caching allocator,
    with a record of what is out."""

    def __init__(self):
        import torch

        self.out = {}
        self.calls = 0
        self.fail = False

        def allocate(size, context):
            self.calls += 1
            if self.fail:
                return None
            pointer = torch.cuda.caching_allocator_alloc(max(int(size), 1), device=0)
            self.out[pointer] = int(size)
            return pointer

        def release(pointer, context):
            assert pointer in self.out, "released an array this allocator never made"
            del self.out[pointer]
            torch.cuda.caching_allocator_delete(pointer)

        self.allocate = ctypes.CFUNCTYPE(ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p)(allocate)
        self.release = ctypes.CFUNCTYPE(None, ctypes.c_void_p, ctypes.c_void_p)(release)

    def give_back(self, pointer):
        self.release(pointer, None)


def _call(lib, neighbors, device_arrays, options):
    points, box, periodic = device_arrays
    message = ctypes.c_char_p()
    status = lib.vesin_neighbors(
        points.data_ptr(), points.shape[0], box.data_ptr(), periodic.data_ptr(), VesinDevice(VesinCUDA, 0), options,
        ctypes.byref(neighbors), ctypes.byref(message),
    )
    return status, message.value


def _rows(neighbors):
    """The list as the struct holds it, on the host."""
    import torch

    from vesin_amd._neighbors import _DeviceView

    n = neighbors.length
    out = {}
    for name, pointer, shape, typestr in (
        ("pairs", neighbors.pairs, (n, 2), "<u8"), ("shifts", neighbors.shifts, (n, 3), "<i4"),
        ("distances", neighbors.distances, (n,), "<f8"), ("vectors", neighbors.vectors, (n, 3), "<f8"),
    ):
        if pointer:
            out[name] = torch.as_tensor(_DeviceView(pointer, shape, typestr, neighbors), device="cuda:0").cpu().numpy()
    return out


def test_allocator_of_the_caller_through_the_c_abi():
    import torch

    lib = get_library()
    points, box, periodic, settings = configs.config1(6)
    arrays = _device(points, box, periodic)
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    allocator = CountingAllocator()
    neighbors = VesinNeighborList()
    message = ctypes.c_char_p()

    # one function without the other is refused, and so is a device that is no GPU
    status = lib.vesin_hip_set_output_allocator(
        ctypes.byref(neighbors), VesinDevice(VesinCUDA, 0), ctypes.cast(allocator.allocate, ctypes.c_void_p), None, None,
        ctypes.byref(message),
    )
    assert status != 0 and b"come together" in message.value
    assert neighbors.device.type == 0, "a refused call leaves a zeroed list zeroed"
    status = lib.vesin_hip_set_output_allocator(
        ctypes.byref(neighbors), VesinDevice(1, 0), ctypes.cast(allocator.allocate, ctypes.c_void_p),
        ctypes.cast(allocator.release, ctypes.c_void_p), None, ctypes.byref(message),
    )
    assert status != 0

    status = lib.vesin_hip_set_output_allocator(
        ctypes.byref(neighbors), VesinDevice(VesinCUDA, 0), ctypes.cast(allocator.allocate, ctypes.c_void_p),
        ctypes.cast(allocator.release, ctypes.c_void_p), None, ctypes.byref(message),
    )
    assert status == 0, message.value
    assert lib.vesin_hip_output_capacity(ctypes.byref(neighbors)) == 0

    options = _options(5.0)
    status, text = _call(lib, neighbors, arrays, options)
    assert status == 0, text
    assert len(allocator.out) == 4 and {neighbors.pairs, neighbors.shifts, neighbors.distances, neighbors.vectors} == set(allocator.out)
    capacity = lib.vesin_hip_output_capacity(ctypes.byref(neighbors))
    assert capacity >= neighbors.length
    assert allocator.out[neighbors.pairs] == 16 * capacity and allocator.out[neighbors.distances] == 8 * capacity
    assert_same_list(_rows(neighbors), expected, what="arrays of the caller's allocator")

    # the arrays become the caller's: the struct forgets them, nothing is released
    mine = (neighbors.pairs, neighbors.shifts, neighbors.distances, neighbors.vectors)
    length = neighbors.length
    reported = ctypes.c_size_t()
    assert lib.vesin_hip_detach_outputs(ctypes.byref(neighbors), ctypes.byref(reported), ctypes.byref(message)) == 0
    assert reported.value == capacity and neighbors.length == length
    assert not any((neighbors.pairs, neighbors.shifts, neighbors.distances, neighbors.vectors))
    assert set(mine) == set(allocator.out)
    assert lib.vesin_hip_output_capacity(ctypes.byref(neighbors)) == 0

    # the next call gets arrays of the same size before it starts (it is the list's steady state: one pass), other
    # points this time; the arrays that were handed over keep their rows
    moved = points + np.random.default_rng(5).normal(scale=0.05, size=points.shape)
    arrays_moved = _device(moved, box, periodic)
    calls_before = allocator.calls
    status, text = _call(lib, neighbors, arrays_moved, options)
    assert status == 0, text
    assert allocator.calls == calls_before + 4 and len(allocator.out) == 8
    assert lib.vesin_hip_output_capacity(ctypes.byref(neighbors)) == capacity
    assert_same_list(_rows(neighbors), oracle.neighbors(moved, box, periodic, 5.0, True, False, "ijSdD"), what="after the hand-over")
    kept = VesinNeighborList()
    kept.length = length
    kept.pairs, kept.shifts, kept.distances, kept.vectors = mine
    assert_same_list(_rows(kept), expected, what="the arrays that were handed over")
    for pointer in mine:
        allocator.give_back(pointer)

    # fewer outputs: the arrays nobody asks for go back; a sorted list through the same arrays
    status, text = _call(lib, neighbors, arrays, _options(5.0, sorted=True, quantities="d"))
    assert status == 0, text
    assert len(allocator.out) == 2 and not neighbors.shifts and not neighbors.vectors
    rows = _rows(neighbors)
    assert_same_list(rows, oracle.neighbors(points, box, periodic, 5.0, True, True, "ijd"), ordered=True, what="sorted")

    # an allocator that has nothing: the call fails as when hipMalloc does, and the list goes on afterwards
    assert lib.vesin_hip_detach_outputs(ctypes.byref(neighbors), None, ctypes.byref(message)) == 0
    for pointer in list(allocator.out):
        allocator.give_back(pointer)
    allocator.fail = True
    status, text = _call(lib, neighbors, arrays, options)
    assert status != 0 and text == b"failed to allocate memory"
    assert not allocator.out
    allocator.fail = False
    status, text = _call(lib, neighbors, arrays, options)
    assert status == 0, text
    assert_same_list(_rows(neighbors), expected, what="after a failed allocation")

    # back to the runtime's own allocation: what the list holds returns to the allocator it came from
    status = lib.vesin_hip_set_output_allocator(ctypes.byref(neighbors), VesinDevice(VesinCUDA, 0), None, None, None, ctypes.byref(message))
    assert status == 0 and not allocator.out and not neighbors.pairs
    status, text = _call(lib, neighbors, arrays, options)
    assert status == 0, text
    assert_same_list(_rows(neighbors), expected, what="hipMalloc again")
    status = lib.vesin_hip_set_output_allocator(
        ctypes.byref(neighbors), VesinDevice(VesinCUDA, 0), ctypes.cast(allocator.allocate, ctypes.c_void_p),
        ctypes.cast(allocator.release, ctypes.c_void_p), None, ctypes.byref(message),
    )
    assert status == 0
    status, text = _call(lib, neighbors, arrays, options)
    assert status == 0 and len(allocator.out) == 4

    # vesin_free gives everything back
    lib.vesin_free(ctypes.byref(neighbors))
    assert not allocator.out
    torch.cuda.synchronize()


def test_detach_on_lists_without_arrays_and_with_a_call_pending():
    import torch

    lib = get_library()
    message = ctypes.c_char_p()
    neighbors = VesinNeighborList()
    reported = ctypes.c_size_t(7)
    assert lib.vesin_hip_detach_outputs(ctypes.byref(neighbors), ctypes.byref(reported), ctypes.byref(message)) == 0
    assert reported.value == 0
    assert lib.vesin_hip_detach_outputs(None, None, ctypes.byref(message)) != 0

    points, box, periodic, _ = configs.config1(4)
    arrays = _device(points, box, periodic)
    options = _options(5.0)
    for _ in range(2):
        status, text = _call(lib, neighbors, arrays, options)
        assert status == 0, text
    word = ctypes.c_void_p()
    status = lib.vesin_hip_neighbors_enqueue(
        arrays[0].data_ptr(), arrays[0].shape[0], arrays[1].data_ptr(), arrays[2].data_ptr(), VesinDevice(VesinCUDA, 0),
        options, ctypes.byref(neighbors), torch.cuda.current_stream().cuda_stream, ctypes.byref(word), ctypes.byref(message),
    )
    assert status == 0, message.value
    held = neighbors.pairs
    assert lib.vesin_hip_detach_outputs(ctypes.byref(neighbors), None, ctypes.byref(message)) != 0
    assert b"vesin_hip_neighbors_collect" in message.value and neighbors.pairs == held
    assert lib.vesin_hip_neighbors_collect(ctypes.byref(neighbors), ctypes.byref(message)) == 0
    # without an allocator the arrays are hipMalloc's: the caller frees them with hipFree
    mine = [neighbors.pairs, neighbors.shifts, neighbors.distances, neighbors.vectors]
    assert lib.vesin_hip_detach_outputs(ctypes.byref(neighbors), None, ctypes.byref(message)) == 0
    # (the HIP runtime this process already uses: the one PyTorch brought along)
    with open("/proc/self/maps") as maps:
        runtime = next(line.split()[-1] for line in maps if "libamdhip64" in line)
    hip = ctypes.CDLL(runtime)
    hip.hipFree.argtypes = [ctypes.c_void_p]
    for pointer in mine:
        assert hip.hipFree(pointer) == 0
    status, text = _call(lib, neighbors, arrays, options)
    assert status == 0 and neighbors.pairs
    assert_same_list(_rows(neighbors), oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD"), what="after hipFree by the caller")
    lib.vesin_free(ctypes.byref(neighbors))


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
@pytest.mark.parametrize("is_sorted", [False, True], ids=["unsorted", "sorted"])
def test_results_that_took_the_arrays_over_are_those_of_a_copy(full, is_sorted):
    import torch

    from vesin_amd import _neighbors

    assert _neighbors._torch_handover(), "lib/libvesin_torch.so must be there: arrays are handed over through it"
    letters = "PSdD"
    systems = [configs.config1(5)[:3], configs.config2(20_000)[:3], configs.config0()[:3]]
    cutoffs = [5.0, 6.0, 5.0]
    taking = NeighborList(cutoff=5.0, full_list=full, sorted=is_sorted)
    copying = NeighborList(cutoff=5.0, full_list=full, sorted=is_sorted)
    copying.hand_over = False
    kept = []
    for round_ in range(3):
        for (points, box, periodic), cutoff in zip(systems, cutoffs):
            taking.cutoff = copying.cutoff = cutoff
            moved = points + np.random.default_rng(round_).normal(scale=0.02 * round_, size=points.shape)
            arrays = _device(moved, box, periodic)
            owned = taking.compute(arrays[0], arrays[1], arrays[2], letters, copy=True)
            copied = copying.compute(arrays[0], arrays[1], arrays[2], letters, copy=True)
            assert copying._neighbors.pairs and not copying._allocator_set
            expected = oracle.neighbors(moved, box, periodic, cutoff, full, is_sorted, "ijSdD")
            assert_same_list(_host(owned, letters), expected, ordered=is_sorted, what="arrays taken over")
            assert_same_list(_host(copied, letters), expected, ordered=is_sorted, what="arrays copied")
            for tensor, other in zip(owned, copied):
                assert tensor.dtype == other.dtype and tensor.shape == other.shape and tensor.is_contiguous()
            kept.append((owned, expected))
    # nothing a later call did touched what earlier calls returned
    for owned, expected in kept:
        assert_same_list(_host(owned, letters), expected, ordered=is_sorted, what="kept over later calls")
    # the 216 atoms after 20,000: arrays with room for many times their rows are copied, not handed over
    small = kept[-1][0]
    assert small[0].untyped_storage().nbytes() == small[0].numel() * 8
    large = kept[-2][0]
    assert large[0].data_ptr() != taking._neighbors.pairs
    del kept, owned, copied, small, large
    torch.cuda.synchronize()


def test_views_single_quantities_other_dtypes_and_numpy():
    import torch

    points, box, periodic, _ = configs.config1(5)
    arrays = _device(points, box, periodic)
    expected = oracle.neighbors(points, box, periodic, 5.0, True, True, "ijSdD")
    calculator = NeighborList(cutoff=5.0, full_list=True, sorted=True)

    # only distances: the pairs nobody took go back to the allocator; memory in use does not grow over the calls
    for _ in range(3):
        (distances,) = calculator.compute(arrays[0], arrays[1], arrays[2], "d", copy=True)
    gc.collect()
    torch.cuda.synchronize()
    in_use = torch.cuda.memory_allocated()
    for _ in range(40):
        (distances,) = calculator.compute(arrays[0], arrays[1], arrays[2], "d", copy=True)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() <= in_use + SLACK, "an array per call (0.8 MB at least) stays behind"
    assert np.array_equal(distances.cpu().numpy(), oracle.canonicalize(expected)["distances"])

    # views after results that took the arrays, and the other way round
    i, j, shifts = calculator.compute(arrays[0], arrays[1], arrays[2], "ijS", copy=False)
    assert i.data_ptr() == calculator._neighbors.pairs
    view = {"pairs": torch.stack([i, j], dim=1).cpu().numpy(), "shifts": shifts.cpu().numpy()}
    assert_same_list(view, {k: expected[k] for k in ("pairs", "shifts")}, ordered=True, what="views")
    pairs, vectors = calculator.compute(arrays[0], arrays[1], arrays[2], "PD", copy=True)
    assert not calculator._neighbors.pairs
    assert_same_list({"pairs": pairs.cpu().numpy(), "vectors": vectors.cpu().numpy()},
                     {k: expected[k] for k in ("pairs", "vectors")}, ordered=True, what="after views")

    # single precision in, single precision out; numpy in, numpy out
    i32, d32 = calculator.compute(arrays[0].float(), arrays[1].float(), arrays[2], "id", copy=True)
    assert d32.dtype == torch.float32 and len(i32) == len(d32)
    as_numpy = calculator.compute(points, box, [True, True, True], "PSdD", copy=True)
    assert all(isinstance(a, np.ndarray) for a in as_numpy)
    assert_same_list(dict(zip(("pairs", "shifts", "distances", "vectors"), as_numpy)), expected, ordered=True, what="numpy")

    # no rows at all
    far = _device(np.array([[0.0, 0.0, 0.0], [50.0, 0.0, 0.0]]), np.eye(3) * 200.0, [False] * 3)
    empty = calculator.compute(far[0], far[1], far[2], "PSd", copy=True)
    assert [tuple(t.shape) for t in empty] == [(0, 2), (0, 3), (0,)]
    full_again = calculator.compute(arrays[0], arrays[1], arrays[2], "PSdD", copy=True)
    assert_same_list(_host(full_again, "PSdD"), expected, ordered=True, what="after an empty list")


def test_batches_queued_calls_and_a_skin_hand_their_arrays_over():
    import torch

    rng = np.random.default_rng(11)
    systems = []
    for n in (40, 64, 200, 9, 120):
        edge = (n / 0.05) ** (1.0 / 3.0)
        box = np.eye(3) * edge + 0.05 * edge * rng.normal(size=(3, 3))
        systems.append((rng.random((n, 3)) @ box, box))
    first_point = np.cumsum([0] + [len(p) for p, _ in systems]).astype(np.uint64)
    all_points = torch.tensor(np.concatenate([p for p, _ in systems]), device="cuda:0")
    boxes = torch.tensor(np.stack([b for _, b in systems]), device="cuda:0")

    calculator = NeighborList(cutoff=5.0, full_list=True, sorted=True)
    kept = []
    for _ in range(3):
        outputs, first_pair = calculator.compute_batch(all_points, first_point, boxes, True, "PSdD", copy=True)
        assert not calculator._neighbors.pairs, "the batch's arrays went to the tensors"
        kept.append((outputs, first_pair))
    for outputs, first_pair in kept:
        rows = _host(outputs, "PSdD")
        for s, (points, box) in enumerate(systems):
            part = {k: v[int(first_pair[s]):int(first_pair[s + 1])] for k, v in rows.items()}
            assert_same_list(part, oracle.neighbors(points, box, [True] * 3, 5.0, True, True, "ijSdD"), ordered=True,
                             what=f"system {s} of the batch")

    # a queued call: the arrays exist before the kernels are queued, and go to the tensors when it is collected
    points, box, periodic, _ = configs.config1(5)
    arrays = _device(points, box, periodic)
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    queued = NeighborList(cutoff=5.0, full_list=True)
    for _ in range(3):
        word = queued.enqueue(arrays[0], arrays[1], arrays[2], "PSdD")
        rows = queued.collect(copy=True)
        assert int(word.item()) in (-1, len(rows[0]))
        assert not queued._neighbors.pairs
        assert_same_list(_host(rows, "PSdD"), expected, what="queued call")

    # with a skin the candidates stay the list's own, the rows go to the caller
    skinned = NeighborList(cutoff=5.0, full_list=True, sorted=True, skin=0.5)
    moving = points.copy()
    for step in range(4):
        moving = moving + np.random.default_rng(step).normal(scale=0.02, size=moving.shape)
        here = _device(moving, box, periodic)
        rows = skinned.compute(here[0], here[1], here[2], "PSdD", copy=True)
        assert_same_list(_host(rows, "PSdD"), oracle.neighbors(moving, box, periodic, 5.0, True, True, "ijSdD"),
                         ordered=True, what=f"skin, step {step}")


def test_scripted_class_hands_its_arrays_over():
    import torch

    from vesin_amd.torchscript import NeighborList as ScriptedList

    points, box, periodic, _ = configs.config1(5)
    arrays = _device(points, box, periodic)
    expected = oracle.neighbors(points, box, periodic, 5.0, True, True, "ijSdD")
    calculator = ScriptedList(cutoff=5.0, full_list=True, sorted=True)
    kept = []
    for _ in range(3):
        kept.append(calculator.compute(arrays[0], arrays[1], arrays[2], "PSdD", copy=True))
    views = calculator.compute(arrays[0], arrays[1], arrays[2], "PSdD", copy=False)
    kept.append([t.clone() for t in views])
    for outputs in kept:
        assert outputs[0].dtype == torch.int64
        rows = _host(outputs, "PSdD")
        rows["pairs"] = rows["pairs"].astype(np.uint64)
        assert_same_list(rows, expected, ordered=True, what="scripted class")
    assert len({out[0].data_ptr() for out in kept}) == len(kept), "every result has memory of its own"

    # gradients flow through results that took the arrays over
    p = arrays[0].clone().requires_grad_(True)
    b = arrays[1].clone().requires_grad_(True)
    i, j, shifts, distances = calculator.compute(p, b, arrays[2], "ijSd", copy=True)
    distances.sum().backward()
    reference = (p.detach()[j] - p.detach()[i] + shifts.to(torch.float64) @ b.detach())
    wanted = torch.zeros_like(p)
    unit = reference / reference.norm(dim=1, keepdim=True)
    wanted.index_add_(0, j, unit)
    wanted.index_add_(0, i, -unit)
    assert torch.allclose(p.grad, wanted, atol=1e-9)
    # (what earlier tests left behind goes first: only this loop is to be seen)
    del kept, views, p, b, i, j, shifts, distances, reference, wanted, unit
    gc.collect()
    in_use = None
    for _ in range(40):
        out = calculator.compute(arrays[0], arrays[1], arrays[2], "PSdD", copy=True)
        torch.cuda.synchronize()
        if in_use is None:
            in_use = torch.cuda.memory_allocated()
    assert torch.cuda.memory_allocated() <= in_use + SLACK, "an array per call (0.8 MB at least) stays behind"
