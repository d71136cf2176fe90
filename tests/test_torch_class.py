"""The TorchScript class ``torch.classes.vesin._NeighborList`` and its Python front (vesin_amd.torchscript).

The cases follow the reference's own tests of its class (python/vesin_torch/tests/test_neighbors.py:14-168,
test_autograd.py:8-28), run on a HIP device. What needs no device (registration, argument checks, scripting,
pickled state) runs everywhere.
"""

import io
import os
from typing import List

import numpy as np
import pytest
import torch

import oracle
from vesin_amd.torchscript import NeighborList


def test_errors_that_need_no_device():
    points = torch.tensor([[0.0, 0.0, 0.0], [0.0, 0.0, 2.0]], dtype=torch.float64)
    box = torch.zeros((3, 3), dtype=torch.float64)
    calculator = NeighborList(cutoff=2.8, full_list=True)

    message = "expected `points` and `box` to have the same device, got cpu and meta"
    with pytest.raises(ValueError, match=message):
        calculator.compute(points, box.to(device="meta"), periodic=False, quantities="ij")

    with pytest.raises(ValueError, match="unexpected character in `quantities`: Q"):
        calculator.compute(points, box, periodic=False, quantities="ijQ")

    with pytest.raises(RuntimeError, match="device meta is not supported in vesin"):
        calculator.compute(points.to(device="meta"), box.to(device="meta"), periodic=False, quantities="ij")

    with pytest.raises(ValueError, match="n_threads must be zero or a positive integer"):
        NeighborList(cutoff=2.8, full_list=True, n_threads=-1)

    with pytest.raises(RuntimeError, match="must have the same dtype"):
        calculator.compute(points, box.to(torch.float32), periodic=False, quantities="ij")

    with pytest.raises(ValueError, match="`points` must be n x 3 tensor"):
        calculator.compute(points.reshape(3, 2), box, periodic=False, quantities="ij")

    with pytest.raises(ValueError, match="`box` must be 3 x 3 tensor"):
        calculator.compute(points, box[:2], periodic=False, quantities="ij")

    with pytest.raises(ValueError, match="`periodic` must be a tensor of bool"):
        calculator.compute(points, box, periodic=torch.tensor([1, 1, 1]), quantities="ij")

    with pytest.raises(ValueError, match="either a single bool or a tensor of 3 bool"):
        calculator.compute(points, box, periodic=torch.tensor([True, True]), quantities="ij")

    # there is no CPU engine behind the class: the library says so instead of computing something else
    with pytest.raises(RuntimeError, match="failed to compute neighbors: this library only implements GPU devices"):
        calculator.compute(points, box, periodic=False, quantities="ij")

    with pytest.raises(RuntimeError, match="unknown algorithm 'fastest'"):
        NeighborList(cutoff=2.8, full_list=True, algorithm="fastest").compute(points, box, False, "ij")


class NeighborListWrap:
    def __init__(self, cutoff: float, full_list: bool, sorted: bool):
        self._c = NeighborList(cutoff=cutoff, full_list=full_list, sorted=sorted)

    def compute(
        self, points: torch.Tensor, box: torch.Tensor, periodic: bool, quantities: str, copy: bool
    ) -> List[torch.Tensor]:
        return self._c.compute(points=points, box=box, periodic=periodic, quantities=quantities, copy=copy)


class Distances(torch.nn.Module):
    def __init__(self, cutoff: float):
        super().__init__()
        self.calculator = torch.classes.vesin._NeighborList(cutoff, True, True)

    def forward(self, points: torch.Tensor, box: torch.Tensor) -> List[torch.Tensor]:
        periodic = torch.ones(3, dtype=torch.bool, device=points.device)
        return self.calculator.compute(points, box, periodic, "ijSd", True)


def test_script():
    class TestModule(torch.nn.Module):
        def forward(self, x: NeighborListWrap) -> NeighborListWrap:
            return x

    torch.jit.script(TestModule())


def test_scripted_module_keeps_the_options_when_saved():
    module = torch.jit.script(Distances(3.5))
    buffer = io.BytesIO()
    torch.jit.save(module, buffer)
    buffer.seek(0)
    loaded = torch.jit.load(buffer)
    state, _class_name = loaded.calculator.__getstate__()
    assert state == {"cutoff": 3.5, "full_list": True, "sorted": True, "algorithm": "auto", "n_threads": 0}


def _system(n=48, seed=11):
    rng = np.random.default_rng(seed)
    box = np.diag(5.0 * rng.random(3) + 2.0) + rng.random((3, 3))
    points = rng.random((n, 3)) @ box
    return points, box


@pytest.mark.gpu
@pytest.mark.parametrize("full_list", [True, False])
@pytest.mark.parametrize("copy", [True, False])
def test_outputs_equal_the_oracle(full_list, copy):
    points, box = _system()
    calculator = NeighborList(cutoff=4.2, full_list=full_list, sorted=True)
    i, j, P, S, d, D = calculator.compute(
        torch.tensor(points, device="cuda:0"), torch.tensor(box, device="cuda:0"), True, "ijPSdD", copy=copy
    )
    assert i.dtype == torch.int64 and j.dtype == torch.int64 and P.dtype == torch.int64
    assert S.dtype == torch.int32 and d.dtype == torch.float64 and D.dtype == torch.float64
    expected = oracle.canonicalize(oracle.neighbors(points, box, [True] * 3, 4.2, full_list, False, "ijSdD"))
    assert np.array_equal(P.cpu().numpy(), expected["pairs"].astype(np.int64))
    assert np.array_equal(i.cpu().numpy(), expected["pairs"][:, 0].astype(np.int64))
    assert np.array_equal(j.cpu().numpy(), expected["pairs"][:, 1].astype(np.int64))
    assert np.array_equal(S.cpu().numpy(), expected["shifts"])
    assert np.array_equal(d.cpu().numpy(), expected["distances"])
    assert np.array_equal(D.cpu().numpy(), expected["vectors"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_dtype(dtype):
    box = torch.eye(3, dtype=dtype, device="cuda:0") * 3.0
    points = torch.rand((100, 3), dtype=dtype, device="cuda:0") * 3.0
    calculator = NeighborList(cutoff=1, full_list=True)
    i, j, s, D, d = calculator.compute(points, box, True, "ijSDd")
    assert i.dtype == torch.int64
    assert j.dtype == torch.int64
    assert s.dtype == torch.int32
    assert D.dtype == dtype
    assert d.dtype == dtype
    assert i.device == points.device and D.device == points.device


@pytest.mark.gpu
@pytest.mark.parametrize("quantities", ["ijS", "D", "d", "ijSDd"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_all_alone_no_neighbors(quantities, dtype):
    points = torch.tensor([[0.0, 0.0, 0.0], [0.5, 0.5, 0.5]], dtype=dtype, device="cuda:0")
    box = torch.eye(3, dtype=dtype, device="cuda:0")
    calculator = NeighborList(cutoff=0.1, full_list=True)

    for requires_grad in (False, True):
        points.requires_grad_(requires_grad)
        box.requires_grad_(requires_grad)
        outputs = calculator.compute(points, box, True, quantities)
        if "ij" in quantities:
            assert list(outputs[quantities.index("i")].shape) == [0]
            assert list(outputs[quantities.index("j")].shape) == [0]
        if "S" in quantities:
            assert list(outputs[quantities.index("S")].shape) == [0, 3]
        if "D" in quantities:
            assert list(outputs[quantities.index("D")].shape) == [0, 3]
            assert outputs[quantities.index("D")].requires_grad == requires_grad
        if "d" in quantities:
            assert list(outputs[quantities.index("d")].shape) == [0]
            assert outputs[quantities.index("d")].requires_grad == requires_grad


@pytest.mark.gpu
@pytest.mark.parametrize("full_list", [True, False])
@pytest.mark.parametrize("requires_grad", [(True, True), (False, True), (True, False)])
@pytest.mark.parametrize("quantities", ["ijS", "D", "d", "ijSDd"])
def test_autograd(full_list, requires_grad, quantities):
    """Finite differences against the backward kernel. The list is sorted so that the rows keep their places
    while gradcheck moves the inputs; the kernel sums with atomics, so two runs may differ in the last bits."""
    torch.manual_seed(0xDEADBEEF)
    points_fractional = torch.rand((34, 3), dtype=torch.float64)
    box = torch.diag(5 * torch.rand(3, dtype=torch.float64))
    box += torch.rand((3, 3), dtype=torch.float64)
    points = (points_fractional @ box).to("cuda:0")
    box = box.to("cuda:0")
    points.requires_grad_(requires_grad[0])
    box.requires_grad_(requires_grad[1])

    calculator = NeighborList(cutoff=7.8, full_list=full_list, sorted=True)

    def compute(points, box):
        return calculator.compute(points, box, periodic=True, quantities=quantities)

    torch.autograd.gradcheck(compute, (points, box), fast_mode=True, nondet_tol=1e-10)


def _backward_with_tensor_operations(pairs, shifts, distances, vectors, distances_grad, vectors_grad, n_points):
    """The formulas of the reference's backward step (vesin-torch/src/vesin_torch.cpp:437-468)."""
    g = vectors_grad + distances_grad[:, None] * vectors / distances[:, None]
    points_grad = torch.zeros((n_points, 3), dtype=torch.float64, device=g.device)
    points_grad = torch.index_add(points_grad, 0, pairs[:, 1], g)
    points_grad = torch.index_add(points_grad, 0, pairs[:, 0], g, alpha=-1.0)
    box_grad = shifts.to(torch.float64).t().matmul(g)
    return points_grad, box_grad


@pytest.mark.gpu
@pytest.mark.parametrize("sorted_rows", [True, False])
@pytest.mark.parametrize("n_cells", [2, 12, 30])
def test_backward_kernel_equals_tensor_operations(sorted_rows, n_cells):
    """An energy that uses both distances and vectors, on a jittered diamond crystal: forces and box gradient
    from the kernel against the reference's formulas evaluated with tensor operations. Sums of about a hundred
    terms in another order: equal within 1e-12 of the largest component."""
    from vesin_amd import configs

    points, box, _ = configs.diamond(n_cells, seed=5)
    points = torch.tensor(points, device="cuda:0", requires_grad=True)
    box = torch.tensor(box, device="cuda:0", requires_grad=True)
    calculator = NeighborList(cutoff=5.0, full_list=True, sorted=sorted_rows)
    P, S, d, D = calculator.compute(points, box, True, "PSdD")
    weights = torch.tensor([0.3, -1.1, 0.7], dtype=torch.float64, device="cuda:0")
    energy = torch.exp(-d).sum() + (torch.tanh(D) @ weights).sum()
    distances_grad, vectors_grad = torch.autograd.grad(energy, (d, D), retain_graph=True)
    points_grad, box_grad = torch.autograd.grad(energy, (points, box))

    expected_points, expected_box = _backward_with_tensor_operations(
        P, S, d.detach(), D.detach(), distances_grad, vectors_grad, len(points)
    )
    scale = float(expected_points.abs().max())
    assert float((points_grad - expected_points).abs().max()) <= 1e-12 * scale
    scale = float(expected_box.abs().max())
    assert float((box_grad - expected_box).abs().max()) <= 1e-12 * scale


@pytest.mark.gpu
@pytest.mark.parametrize("n_points", [7, 3000, 200_000])
def test_backward_with_rows_in_no_order(n_points):
    """Rows that name points at random: with many points a workgroup meets more of them than its table in LDS
    holds, and the rest goes to memory directly; with 7 points every addition collides."""
    import ctypes

    from vesin_amd._c_api import VesinCUDA, VesinDevice, get_library

    lib = get_library()
    generator = torch.Generator(device="cuda:0").manual_seed(n_points)
    n_pairs = 70_001
    pairs = torch.randint(0, n_points, (n_pairs, 2), dtype=torch.int64, device="cuda:0", generator=generator)
    shifts = torch.randint(-2, 3, (n_pairs, 3), dtype=torch.int32, device="cuda:0", generator=generator)
    vectors = torch.randn((n_pairs, 3), dtype=torch.float64, device="cuda:0", generator=generator)
    distances = vectors.norm(dim=1)
    distances_grad = torch.randn(n_pairs, dtype=torch.float64, device="cuda:0", generator=generator)
    vectors_grad = torch.randn((n_pairs, 3), dtype=torch.float64, device="cuda:0", generator=generator)
    points_grad = torch.zeros((n_points, 3), dtype=torch.float64, device="cuda:0")
    box_grad = torch.zeros((3, 3), dtype=torch.float64, device="cuda:0")
    message = ctypes.c_char_p()
    status = lib.vesin_hip_pairs_backward(
        pairs.data_ptr(), shifts.data_ptr(), distances.data_ptr(), vectors.data_ptr(), n_pairs,
        distances_grad.data_ptr(), vectors_grad.data_ptr(), n_points, VesinDevice(VesinCUDA, 0),
        points_grad.data_ptr(), box_grad.data_ptr(), None, ctypes.byref(message),
    )
    assert status == 0, message.value
    expected_points, expected_box = _backward_with_tensor_operations(
        pairs, shifts, distances, vectors, distances_grad, vectors_grad, n_points
    )
    assert float((points_grad - expected_points).abs().max()) <= 1e-12 * float(expected_points.abs().max())
    assert float((box_grad - expected_box).abs().max()) <= 1e-12 * float(expected_box.abs().max())


@pytest.mark.gpu
def test_backward_after_the_calculator_moved_on():
    """With gradients the outputs are copies even when views were asked for: a later calculation on the same
    calculator must not change what the backward step of an earlier one reads."""
    from vesin_amd import configs

    calculator = NeighborList(cutoff=4.0, full_list=True, sorted=True)
    first, box, _ = configs.diamond(3, seed=1)
    first = torch.tensor(first, device="cuda:0", requires_grad=True)
    box = torch.tensor(box, device="cuda:0")
    P, d, D = calculator.compute(first, box, True, "PdD", copy=False)
    kept = (P.clone(), d.detach().clone(), D.detach().clone())
    energy = (d**2).sum() + D[:, 0].sum()

    other, other_box, _ = configs.diamond(4, seed=2)
    calculator.compute(torch.tensor(other, device="cuda:0"), torch.tensor(other_box, device="cuda:0"), True, "PdD", copy=False)

    (points_grad,) = torch.autograd.grad(energy, (first,))
    distances_grad = 2.0 * kept[1]
    vectors_grad = torch.zeros_like(kept[2])
    vectors_grad[:, 0] = 1.0
    shifts = torch.zeros((len(kept[0]), 3), dtype=torch.int32, device="cuda:0")
    expected, _ = _backward_with_tensor_operations(kept[0], shifts, kept[1], kept[2], distances_grad, vectors_grad, len(first))
    assert float((points_grad - expected).abs().max()) <= 1e-12 * float(expected.abs().max())


@pytest.mark.gpu
def test_backward_refuses_rows_of_another_system():
    """The entry point checks the indices it is given instead of writing outside `points_grad`."""
    import ctypes

    from vesin_amd._c_api import VesinCUDA, VesinDevice, get_library

    lib = get_library()
    pairs = torch.tensor([[0, 1], [1, 7]], dtype=torch.int64, device="cuda:0")
    vectors_grad = torch.ones((2, 3), dtype=torch.float64, device="cuda:0")
    points_grad = torch.zeros((2, 3), dtype=torch.float64, device="cuda:0")
    message = ctypes.c_char_p()
    status = lib.vesin_hip_pairs_backward(
        pairs.data_ptr(), None, None, None, 2, None, vectors_grad.data_ptr(), 2, VesinDevice(VesinCUDA, 0),
        points_grad.data_ptr(), None, None, ctypes.byref(message),
    )
    assert status == 1
    assert message.value == b"`pairs` names a point beyond `n_points`"


@pytest.mark.gpu
def test_scripted_module_on_the_gpu():
    points, box = _system()
    module = torch.jit.script(Distances(4.2))
    i, j, S, d = module(torch.tensor(points, device="cuda:0"), torch.tensor(box, device="cuda:0"))
    expected = oracle.canonicalize(oracle.neighbors(points, box, [True] * 3, 4.2, True, False, "ijSd"))
    assert np.array_equal(torch.stack([i, j], dim=1).cpu().numpy(), expected["pairs"].astype(np.int64))
    assert np.array_equal(S.cpu().numpy(), expected["shifts"])
    assert np.array_equal(d.cpu().numpy(), expected["distances"])


@pytest.mark.gpu
def test_caller_on_another_stream():
    """Inputs produced on a side stream are complete before the library (on the null stream) reads them."""
    points, box = _system(n=4000, seed=3)
    expected = oracle.canonicalize(oracle.neighbors(points, box, [True] * 3, 1.5, True, False, "ijSd"))
    calculator = NeighborList(cutoff=1.5, full_list=True, sorted=True)
    host_points = torch.tensor(points).pin_memory()
    device_box = torch.tensor(box, device="cuda:0")
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        device_points = host_points.to("cuda:0", non_blocking=True) * 1.0
        P, S, d = calculator.compute(device_points, device_box, True, "PSd")
    torch.cuda.synchronize()
    assert np.array_equal(P.cpu().numpy(), expected["pairs"].astype(np.int64))
    assert np.array_equal(d.cpu().numpy(), expected["distances"])
