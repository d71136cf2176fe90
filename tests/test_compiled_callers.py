"""Compiled callers of the C ABI: a C program and the reference's own TorchScript class.

* ``tests/abi_caller.c`` includes ``vesin.h`` and links ``-lvesin`` like any C user of vesin. It is compiled and
  linked on every machine (CPU test) and run on the GPU (``-m gpu``): the cases of the reference's GPU test program
  (vesin/tests/cuda.cpp:22-226), with exact ``==`` on distances and vectors and ten host threads at once.
* ``tests/call_loop.c`` calls ``vesin_neighbors`` a few thousand times on one small system, like a simulation code
  without any wrapper, and prints the time per call; the test checks the number of rows against the oracle.
* The reference's ``vesin-torch/src/vesin_torch.cpp`` is compiled UNMODIFIED against this repository's header and
  linked to this repository's library (``oracle/Makefile``, target ``ref_torch``; output in ``oracle/_ref/``, which
  is not part of the repository's history). The CPU test does that where the reference checkout exists; the GPU test
  loads the prebuilt class in a process of its own (it registers the same class name as this package's own
  TorchScript class) and compares its lists and gradients with the oracle.
"""

import os
import subprocess
import sys
import textwrap

import pytest

import oracle

HERE = os.path.dirname(os.path.realpath(__file__))
ROOT = os.path.dirname(HERE)
LIB_DIR = os.path.join(ROOT, "vesin_amd", "lib")
REFERENCE = "/root/reference"


def build_c_caller(directory, name="abi_caller"):
    out = os.path.join(str(directory), name)
    command = [
        "gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
        "-I" + os.path.join(ROOT, "include"), os.path.join(HERE, name + ".c"), "-o", out,
        "-L" + LIB_DIR, "-lvesin", "-L/opt/rocm/lib", "-lamdhip64", "-lpthread", "-lm",
        "-Wl,-rpath," + LIB_DIR, "-Wl,-rpath,/opt/rocm/lib",
    ]
    result = subprocess.run(command, capture_output=True, text=True)
    assert result.returncode == 0, result.stderr
    return out


def test_c_caller_compiles_and_links(tmp_path):
    program = build_c_caller(tmp_path)
    symbols = subprocess.run(["nm", "-D", "--undefined-only", program], capture_output=True, text=True, check=True).stdout
    assert " U vesin_neighbors" in symbols and " U vesin_free" in symbols


@pytest.mark.gpu
def test_c_caller_runs(tmp_path):
    program = build_c_caller(tmp_path)
    result = subprocess.run([program], capture_output=True, text=True, timeout=100)
    assert result.returncode == 0, result.stdout + result.stderr
    assert result.stdout.strip() == "ok"


def test_call_loop_compiles_and_links(tmp_path):
    build_c_caller(tmp_path, "call_loop")


def _call_loop_system(cells):
    """The atoms tests/call_loop.c makes: diamond with the jitter of its linear congruential generator."""
    import numpy as np

    a = 3.567
    basis = np.array([[0, 0, 0], [0, .5, .5], [.5, 0, .5], [.5, .5, 0], [.25, .25, .25], [.25, .75, .75], [.75, .25, .75],
                      [.75, .75, .25]])
    points = []
    state = 12345
    for x in range(cells):
        for y in range(cells):
            for z in range(cells):
                for b in range(8):
                    point = []
                    for d, corner in enumerate((x, y, z)):
                        state = (state * 1664525 + 1013904223) % 2**32
                        point.append((corner + basis[b][d]) * a + 0.05 * ((state >> 8) / 16777216.0 - 0.5))
                    points.append(point)
    return np.array(points), np.eye(3) * cells * a


@pytest.mark.gpu
@pytest.mark.parametrize("cells, sorted_rows", [(3, 1), (3, 0), (2, 0), (5, 1)])
def test_call_loop_runs(tmp_path, cells, sorted_rows):
    program = build_c_caller(tmp_path, "call_loop")
    result = subprocess.run([program, str(cells), str(sorted_rows), "300"], capture_output=True, text=True, timeout=100)
    assert result.returncode == 0, result.stdout + result.stderr
    points, box = _call_loop_system(cells)
    expected = oracle.neighbors(points, box, [True, True, True], 5.0, True, False, "ij")
    assert f"{len(points)} atoms, sorted {sorted_rows}: {len(expected['pairs'])} rows, " in result.stdout, result.stdout
    # the same as a queued call and its completion, the word on the device checked after every call
    result = subprocess.run([program, str(cells), str(sorted_rows), "300", "queued"], capture_output=True, text=True, timeout=100)
    assert result.returncode == 0, result.stdout + result.stderr
    assert f"{len(expected['pairs'])} rows, queued: " in result.stdout, result.stdout


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "vesin-torch", "src")), reason="needs the reference checkout")
def test_reference_torch_class_compiles_and_links_unchanged():
    """The reference's vesin_torch.cpp against include/vesin.h and libvesin.so, no undefined symbol left over."""
    library = oracle.build_ref_torch(REFERENCE)
    assert os.path.exists(library)
    wanted = subprocess.run(["nm", "-D", "--undefined-only", library], capture_output=True, text=True, check=True).stdout
    assert " U vesin_neighbors" in wanted and " U vesin_free" in wanted
    needed = subprocess.run(["readelf", "-d", library], capture_output=True, text=True, check=True).stdout
    assert "libvesin.so" in needed
    # its source is the reference's, untouched: nothing of it is in this repository
    tracked = subprocess.run(["git", "-C", ROOT, "ls-files"], capture_output=True, text=True).stdout
    assert "vesin_torch.cpp" not in tracked


REFERENCE_CLASS_SCRIPT = textwrap.dedent(
    """
    import sys
    sys.path.insert(0, {root!r}); sys.path.insert(0, {tests!r})
    import numpy as np
    import torch
    import oracle
    from vesin_amd import configs
    from vesin_amd._c_api import get_library

    get_library()  # one HIP runtime in the process: PyTorch's
    torch.ops.load_library({library!r})
    NeighborList = torch.classes.vesin._NeighborList

    # ---- lists: the class's outputs against the oracle's, sorted lists element by element
    points, box, periodic, options = configs.config0()
    for full in (True, False):
        calculator = NeighborList({cutoff}, full, True, "auto", 0)
        d_points = torch.tensor(points, device="cuda:0")
        d_box = torch.tensor(box, device="cuda:0")
        for call in range(2):
            i, j, S, d, D = calculator.compute(d_points, d_box, torch.tensor(periodic), "ijSdD", True)
        expected = oracle.canonicalize(oracle.neighbors(points, box, periodic, {cutoff}, full, False, "ijSdD"))
        assert i.dtype == torch.int64 and S.dtype == torch.int32 and d.dtype == torch.float64 and i.is_cuda
        pairs = torch.stack([i, j], dim=1).cpu().numpy()
        assert np.array_equal(pairs, expected["pairs"].astype(np.int64)), "pairs"
        assert np.array_equal(S.cpu().numpy(), expected["shifts"]), "shifts"
        assert np.array_equal(d.cpu().numpy(), expected["distances"]), "distances"
        assert np.array_equal(D.cpu().numpy(), expected["vectors"]), "vectors"

    # ---- gradients through the class's own backward (tensor operations of the reference)
    d_points = torch.tensor(points, device="cuda:0", requires_grad=True)
    d_box = torch.tensor(box, device="cuda:0", requires_grad=True)
    calculator = NeighborList({cutoff}, True, True, "auto", 0)
    P, S, d, D = calculator.compute(d_points, d_box, torch.tensor(periodic), "PSdD", True)
    ((d ** 2).sum() + (D * D).sum()).backward()
    expected = oracle.canonicalize(oracle.neighbors(points, box, periodic, {cutoff}, True, False, "ijSdD"))
    gradient = np.zeros_like(points)
    np.add.at(gradient, expected["pairs"][:, 1].astype(np.int64), 4.0 * expected["vectors"])
    np.add.at(gradient, expected["pairs"][:, 0].astype(np.int64), -4.0 * expected["vectors"])
    assert np.abs(d_points.grad.cpu().numpy() - gradient).max() <= 1e-11 * max(1.0, np.abs(gradient).max())
    box_gradient = 4.0 * expected["shifts"].astype(np.float64).T @ expected["vectors"]
    assert np.abs(d_box.grad.cpu().numpy() - box_gradient).max() <= 1e-11 * max(1.0, np.abs(box_gradient).max())

    # ---- a scripted module holding the class
    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.calculator = torch.classes.vesin._NeighborList({cutoff}, True, False, "auto", 0)

        def forward(self, points: torch.Tensor, box: torch.Tensor, periodic: torch.Tensor) -> torch.Tensor:
            return self.calculator.compute(points, box, periodic, "d", True)[0].sum()

    scripted = torch.jit.script(Model())
    total = scripted(torch.tensor(points, device="cuda:0"), torch.tensor(box, device="cuda:0"), torch.tensor(periodic))
    assert abs(float(total) - float(expected["distances"].sum())) <= 1e-9 * float(expected["distances"].sum())
    print("reference class ok")
    """
)


@pytest.mark.gpu
def test_reference_torch_class_runs_on_this_library(tmp_path):
    """The reference's TorchScript class, as compiled in this repository's build container from the reference's
    untouched source, on a HIP device: lists identical to the oracle's, gradients with respect to points and box,
    a scripted module. Skipped when that build is not in the tree."""
    if not os.path.exists(oracle.REF_TORCH_LIB):
        pytest.skip("oracle/_ref/libvesin_torch_ref.so was not built (it needs the reference checkout)")
    script = REFERENCE_CLASS_SCRIPT.format(root=ROOT, tests=HERE, library=oracle.REF_TORCH_LIB, cutoff=5.0)
    program = tmp_path / "reference_class.py"  # a file: TorchScript reads the source of what it compiles
    program.write_text(script)
    result = subprocess.run([sys.executable, str(program)], capture_output=True, text=True, timeout=110)
    assert result.returncode == 0, result.stdout[-2000:] + result.stderr[-4000:]
    assert "reference class ok" in result.stdout
