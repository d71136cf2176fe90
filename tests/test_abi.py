"""The drop-in boundary, checked without a GPU: struct layouts (against vesin/include/vesin.h:49-78,103-108,129-163
as documented in include/vesin.h), exported symbols, and the argument validation of vesin_neighbors
(vesin/src/vesin.cpp:51-105) which runs before any GPU call."""

import ctypes
import os
import re
import subprocess

import pytest

from vesin_amd import _c_api

HERE = os.path.dirname(os.path.realpath(__file__))
ROOT = os.path.dirname(HERE)
HEADER = os.path.join(ROOT, "include", "vesin.h")

PROBE = r"""
#include <stdio.h>
#include <stddef.h>
#include "vesin.h"
int main(void) {
    printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(struct VesinOptions),
        offsetof(struct VesinOptions, cutoff), offsetof(struct VesinOptions, full), offsetof(struct VesinOptions, sorted),
        offsetof(struct VesinOptions, algorithm), offsetof(struct VesinOptions, n_threads),
        offsetof(struct VesinOptions, return_shifts), offsetof(struct VesinOptions, return_distances),
        offsetof(struct VesinOptions, return_vectors), offsetof(struct VesinOptions, skin));
    printf("%zu %zu %zu\n", sizeof(struct VesinDevice), offsetof(struct VesinDevice, type), offsetof(struct VesinDevice, device_id));
    printf("%zu %zu %zu %zu %zu %zu %zu %zu\n", sizeof(struct VesinNeighborList),
        offsetof(struct VesinNeighborList, length), offsetof(struct VesinNeighborList, device),
        offsetof(struct VesinNeighborList, pairs), offsetof(struct VesinNeighborList, shifts),
        offsetof(struct VesinNeighborList, distances), offsetof(struct VesinNeighborList, vectors),
        offsetof(struct VesinNeighborList, opaque));
    printf("%d %d %d %d %d %d\n", VesinAutoAlgorithm, VesinBruteForce, VesinCellList, VesinUnknownDevice, VesinCPU, VesinCUDA);
    return 0;
}
"""


@pytest.mark.parametrize("compiler,std", [("gcc", "-std=c11"), ("g++", "-std=c++17")])
def test_struct_layout(tmp_path, compiler, std):
    source = tmp_path / ("probe.c" if compiler == "gcc" else "probe.cpp")
    source.write_text(PROBE)
    exe = tmp_path / "probe"
    subprocess.run([compiler, std, "-I", os.path.join(ROOT, "include"), str(source), "-o", str(exe)], check=True)
    lines = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines()
    assert lines[0].split() == ["32", "0", "8", "9", "12", "16", "20", "21", "22", "24"]
    assert lines[1].split() == ["8", "0", "4"]
    assert lines[2].split() == ["56", "0", "8", "16", "24", "32", "40", "48"]
    assert lines[3].split() == ["0", "1", "2", "0", "1", "2"]


def test_ctypes_mirror_has_the_same_layout():
    assert ctypes.sizeof(_c_api.VesinOptions) == 32
    assert [getattr(_c_api.VesinOptions, f).offset for f, _ in _c_api.VesinOptions._fields_] == [0, 8, 9, 12, 16, 20, 21, 22, 24]
    assert ctypes.sizeof(_c_api.VesinDevice) == 8
    assert ctypes.sizeof(_c_api.VesinNeighborList) == 56
    assert [getattr(_c_api.VesinNeighborList, f).offset for f, _ in _c_api.VesinNeighborList._fields_] == [0, 8, 16, 24, 32, 40, 48]


def test_library_exports_every_declared_symbol():
    with open(HEADER) as fd:
        text = fd.read()
    declared = re.findall(r"^\w[\w *]*\bVESIN_API\s+(\w+)\s*\(", text, flags=re.M)
    assert set(declared) >= {"vesin_neighbors", "vesin_free"}
    lib = _c_api.get_library()
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/vesin.h but not exported"


def call(lib, points=1, n_points=1, box=1, periodic=1, device=(2, 0), cutoff=1.0, n_threads=0, skin=0.0, neighbors="new",
         with_message=True):
    """Drive vesin_neighbors with dummy non-null pointers: every case here must fail before they are touched."""
    options = _c_api.VesinOptions()
    options.cutoff = cutoff
    options.full = True
    options.n_threads = n_threads
    options.skin = skin
    dummy = (ctypes.c_double * 16)()
    address = ctypes.addressof(dummy)
    if neighbors == "new":
        neighbors = _c_api.VesinNeighborList()
    message = ctypes.c_char_p()
    lib.vesin_neighbors.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p, _c_api.VesinDevice,
                                    _c_api.VesinOptions, ctypes.c_void_p, ctypes.c_void_p]
    status = lib.vesin_neighbors(
        address if points else None, n_points, address if box else None, address if periodic else None,
        _c_api.VesinDevice(*device), options,
        ctypes.addressof(neighbors) if neighbors is not None else None,
        ctypes.addressof(message) if with_message else None,
    )
    return status, (message.value.decode() if message.value else None)


def test_validation_messages():
    lib = _c_api.get_library()
    assert call(lib, with_message=False) == (1, None)
    assert call(lib, points=0) == (1, "`points` can not be a NULL pointer")
    assert call(lib, box=0) == (1, "`cell` can not be a NULL pointer")
    assert call(lib, neighbors=None) == (1, "`neighbors` can not be a NULL pointer")
    for cutoff in (0.0, -1.0, float("nan"), float("inf")):
        assert call(lib, cutoff=cutoff) == (1, "cutoff must be a finite, positive number")
    assert call(lib, cutoff=1e-7) == (1, "cutoff is too small")
    assert call(lib, skin=-1.0) == (1, "skin must be a finite, non-negative number")
    assert call(lib, n_threads=-1) == (1, "n_threads must be zero or a positive integer")
    assert call(lib, device=(0, 0)) == (1, "got an unknown device type")

    existing = _c_api.VesinNeighborList()
    existing.device = _c_api.VesinDevice(_c_api.VesinCPU, 0)
    assert call(lib, neighbors=existing) == (1, "`neighbors` device and data `device` do not match, free the neighbors first")

    status, message = call(lib, device=(_c_api.VesinCPU, 0))
    assert status == 1 and "no CPU engine" in message
    # a skin is accepted (Verlet caching); without a GPU the call gets as far as looking for one
    status, message = call(lib, skin=0.5)
    assert status == 1 and message == "no HIP device is available to this process"


def test_free_accepts_null_and_zeroed_lists():
    lib = _c_api.get_library()
    lib.vesin_free(None)
    neighbors = _c_api.VesinNeighborList()
    lib.vesin_free(ctypes.byref(neighbors))
    assert neighbors.length == 0 and neighbors.pairs is None


def test_validation_of_the_additions():
    """The entry points this library adds check their arguments like vesin_neighbors does, before any GPU work."""
    lib = _c_api.get_library()
    dummy = (ctypes.c_double * 16)()
    address = ctypes.addressof(dummy)
    gpu = _c_api.VesinDevice(_c_api.VesinCUDA, 0)
    cpu = _c_api.VesinDevice(_c_api.VesinCPU, 0)
    options = _c_api.VesinOptions()
    options.cutoff = 1.0

    def text(message):
        return message.value.decode() if message.value else None

    # the calculation on a stream: same checks, same texts
    neighbors = _c_api.VesinNeighborList()
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_on_stream(
        None, 1, address, address, gpu, options, ctypes.byref(neighbors), None, ctypes.byref(message)
    )
    assert (status, text(message)) == (1, "`points` can not be a NULL pointer")
    bad = _c_api.VesinOptions()
    bad.cutoff = -2.0
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_on_stream(
        address, 1, address, address, gpu, bad, ctypes.byref(neighbors), None, ctypes.byref(message)
    )
    assert (status, text(message)) == (1, "cutoff must be a finite, positive number")
    assert lib.vesin_hip_neighbors_on_stream(address, 1, address, address, gpu, options, ctypes.byref(neighbors), None, None) == 1

    # the gradient
    message = ctypes.c_char_p()
    status = lib.vesin_hip_pairs_backward(
        address, None, None, None, 1, None, address, 1, cpu, address, None, None, ctypes.byref(message)
    )
    assert status == 1 and "only computed on a GPU device" in text(message)
    message = ctypes.c_char_p()
    status = lib.vesin_hip_pairs_backward(
        address, None, None, None, 0, None, address, 1, gpu, address, None, None, ctypes.byref(message)
    )
    assert (status, text(message)) == (0, None)  # no rows: nothing to do, no device needed
    assert lib.vesin_hip_pairs_backward(address, None, None, None, 1, None, address, 1, gpu, address, None, None, None) == 1

    # the batch
    first_point = (ctypes.c_size_t * 2)(0, 1)
    first_pair = (ctypes.c_size_t * 2)()
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_batch(
        address, None, 1, address, address, gpu, options, ctypes.byref(neighbors), first_pair, ctypes.byref(message)
    )
    assert (status, text(message)) == (1, "`first_point` can not be a NULL pointer")
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_batch(
        address, first_point, 1, address, address, cpu, options, ctypes.byref(neighbors), first_pair, ctypes.byref(message)
    )
    assert status == 1 and "only computed on a GPU device" in text(message)
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_batch_on_stream(
        address, first_point, 1, address, address, gpu, options, ctypes.byref(neighbors), None, None, ctypes.byref(message)
    )
    assert (status, text(message)) == (1, "`first_pair` can not be a NULL pointer")
    with_skin = _c_api.VesinOptions()
    with_skin.cutoff = 1.0
    with_skin.skin = -0.2
    message = ctypes.c_char_p()
    status = lib.vesin_hip_neighbors_batch(
        address, first_point, 1, address, address, gpu, with_skin, ctypes.byref(neighbors), first_pair, ctypes.byref(message)
    )
    assert (status, text(message)) == (1, "skin must be a finite, non-negative number")
    lib.vesin_free(ctypes.byref(neighbors))
