"""CPU checkers for the neighbor-list path: TEST INFRASTRUCTURE ONLY.

Two shared libraries are driven from here through ctypes:

* ``liboracle.so``: this repository's C restatement of vesin's CPU algorithm (``vesin_oracle.c``);
* ``_ref/libvesin_ref.so``: the reference's own CPU path, compiled unmodified by ``oracle/Makefile`` from the
  reference checkout when that is present (it is not on the GPU box, where the prebuilt file is used).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module.
The shipped library never does.
"""

import ctypes
import os
import subprocess
import time

import numpy as np

HERE = os.path.dirname(os.path.realpath(__file__))
ORACLE_LIB = os.path.join(HERE, "liboracle.so")
REF_LIB = os.path.join(HERE, "_ref", "libvesin_ref.so")
REF_TORCH_LIB = os.path.join(HERE, "_ref", "libvesin_torch_ref.so")


def build(reference="/root/reference"):
    """Compile liboracle.so and, when the reference checkout exists, _ref/libvesin_ref.so."""
    subprocess.run(["make", "-C", HERE, "-s", "liboracle.so", "ref", f"REFERENCE={reference}"], check=True)


def build_ref_torch(reference="/root/reference"):
    """Compile the reference's TorchScript class, unmodified, against this repository's header and library
    (_ref/libvesin_torch_ref.so); needs the reference checkout and a built vesin_amd/lib/libvesin.so."""
    subprocess.run(["make", "-C", HERE, "-s", "ref_torch", f"REFERENCE={reference}"], check=True)
    return REF_TORCH_LIB


class _Options(ctypes.Structure):
    _fields_ = [
        ("cutoff", ctypes.c_double),
        ("full", ctypes.c_int32),
        ("sorted", ctypes.c_int32),
        ("return_shifts", ctypes.c_int32),
        ("return_distances", ctypes.c_int32),
        ("return_vectors", ctypes.c_int32),
        ("n_threads", ctypes.c_int32),
    ]


class _List(ctypes.Structure):
    _fields_ = [
        ("length", ctypes.c_size_t),
        ("pairs", ctypes.POINTER(ctypes.c_size_t)),
        ("shifts", ctypes.POINTER(ctypes.c_int32)),
        ("distances", ctypes.POINTER(ctypes.c_double)),
        ("vectors", ctypes.POINTER(ctypes.c_double)),
    ]


class _Grid(ctypes.Structure):
    _fields_ = [
        ("n_cells", ctypes.c_int32 * 3),
        ("n_search", ctypes.c_int32 * 3),
        ("face_distances", ctypes.c_double * 3),
        ("matrix", ctypes.c_double * 9),
        ("inverse", ctypes.c_double * 9),
    ]


_oracle = None

# wall-clock seconds spent inside the C call of the most recent neighbors() / ref_neighbors()
last_call_seconds = 0.0


def _load_oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_LIB):
            build()
        lib = ctypes.CDLL(ORACLE_LIB)
        lib.vesin_oracle_neighbors.restype = ctypes.c_int
        lib.vesin_oracle_neighbors.argtypes = [
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.POINTER(_Options),
            ctypes.POINTER(_List),
            ctypes.POINTER(_Grid),
            ctypes.c_char_p,
            ctypes.c_size_t,
        ]
        lib.vesin_oracle_free.restype = None
        lib.vesin_oracle_free.argtypes = [ctypes.POINTER(_List)]
        lib.vesin_oracle_half_list_keeps.restype = ctypes.c_int
        lib.vesin_oracle_half_list_keeps.argtypes = [ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p]
        _oracle = lib
    return _oracle


def _prepare(points, box, periodic):
    points = np.ascontiguousarray(points, dtype=np.float64).reshape(-1, 3)
    box = np.ascontiguousarray(box, dtype=np.float64).reshape(3, 3)
    if isinstance(periodic, (bool, np.bool_)):
        periodic = [periodic] * 3
    periodic = np.ascontiguousarray(periodic, dtype=np.uint8).reshape(3)
    return points, box, periodic


def _collect(length, pairs, shifts, distances, vectors, want_S, want_d, want_D):
    def take(pointer, count, dtype):
        if count == 0:
            return np.zeros(0, dtype=dtype)
        return np.ctypeslib.as_array(pointer, shape=(count,)).astype(dtype, copy=True)

    result = {"pairs": take(pairs, 2 * length, np.uint64).reshape(-1, 2)}
    if want_S:
        result["shifts"] = take(shifts, 3 * length, np.int32).reshape(-1, 3)
    if want_d:
        result["distances"] = take(distances, length, np.float64)
    if want_D:
        result["vectors"] = take(vectors, 3 * length, np.float64).reshape(-1, 3)
    return result


def neighbors(points, box, periodic, cutoff, full=True, sorted=False, quantities="ijSdD", n_threads=0,
              return_grid=False):
    """Run the C restatement. Returns a dict with ``pairs`` (n,2) uint64 and, as requested by the letters
    S / d / D in ``quantities``, ``shifts`` (n,3) int32, ``distances`` (n,), ``vectors`` (n,3)."""
    lib = _load_oracle()
    points, box, periodic = _prepare(points, box, periodic)
    options = _Options(float(cutoff), int(full), int(sorted), int("S" in quantities), int("d" in quantities),
                       int("D" in quantities), int(n_threads))
    out = _List()
    grid = _Grid()
    error = ctypes.create_string_buffer(512)
    global last_call_seconds
    start = time.perf_counter()
    status = lib.vesin_oracle_neighbors(points.ctypes.data, points.shape[0], box.ctypes.data, periodic.ctypes.data,
                                        ctypes.byref(options), ctypes.byref(out), ctypes.byref(grid), error, 512)
    last_call_seconds = time.perf_counter() - start
    if status != 0:
        raise RuntimeError(error.value.decode("utf8"))
    try:
        result = _collect(out.length, out.pairs, out.shifts, out.distances, out.vectors,
                          "S" in quantities, "d" in quantities, "D" in quantities)
    finally:
        lib.vesin_oracle_free(ctypes.byref(out))
    if return_grid:
        result["grid"] = {
            "n_cells": np.array(grid.n_cells[:], dtype=np.int32),
            "n_search": np.array(grid.n_search[:], dtype=np.int32),
            "face_distances": np.array(grid.face_distances[:]),
            "matrix": np.array(grid.matrix[:]).reshape(3, 3),
            "inverse": np.array(grid.inverse[:]).reshape(3, 3),
        }
    return result


def half_list_keeps(first, second, shift):
    lib = _load_oracle()
    shift = np.ascontiguousarray(shift, dtype=np.int32)
    return bool(lib.vesin_oracle_half_list_keeps(int(first), int(second), shift.ctypes.data))


# --------------------------------------------------------------------------------------------------------------
# The compiled reference (vesin's own vesin_neighbors with device = VesinCPU)


class _RefOptions(ctypes.Structure):
    _fields_ = [
        ("cutoff", ctypes.c_double),
        ("full", ctypes.c_bool),
        ("sorted", ctypes.c_bool),
        ("algorithm", ctypes.c_int),
        ("n_threads", ctypes.c_int32),
        ("return_shifts", ctypes.c_bool),
        ("return_distances", ctypes.c_bool),
        ("return_vectors", ctypes.c_bool),
        ("skin", ctypes.c_double),
    ]


class _RefDevice(ctypes.Structure):
    _fields_ = [("type", ctypes.c_int), ("device_id", ctypes.c_int)]


class _RefList(ctypes.Structure):
    _fields_ = [
        ("length", ctypes.c_size_t),
        ("device", _RefDevice),
        ("pairs", ctypes.POINTER(ctypes.c_size_t)),
        ("shifts", ctypes.POINTER(ctypes.c_int32)),
        ("distances", ctypes.POINTER(ctypes.c_double)),
        ("vectors", ctypes.POINTER(ctypes.c_double)),
        ("opaque", ctypes.c_void_p),
    ]


_ref = None


def have_ref():
    return os.path.exists(REF_LIB)


def _load_ref():
    global _ref
    if _ref is None:
        lib = ctypes.CDLL(REF_LIB)
        lib.vesin_neighbors.restype = ctypes.c_int
        lib.vesin_neighbors.argtypes = [
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            _RefDevice,
            _RefOptions,
            ctypes.POINTER(_RefList),
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_free.restype = None
        lib.vesin_free.argtypes = [ctypes.POINTER(_RefList)]
        _ref = lib
    return _ref


def ref_neighbors(points, box, periodic, cutoff, full=True, sorted=False, quantities="ijSdD", n_threads=0):
    """Run the compiled reference CPU path; same return convention as :func:`neighbors`."""
    lib = _load_ref()
    points, box, periodic = _prepare(points, box, periodic)
    options = _RefOptions(float(cutoff), bool(full), bool(sorted), 0, int(n_threads), "S" in quantities,
                          "d" in quantities, "D" in quantities, 0.0)
    out = _RefList()
    message = ctypes.c_char_p()
    global last_call_seconds
    start = time.perf_counter()
    status = lib.vesin_neighbors(points.ctypes.data, points.shape[0], box.ctypes.data, periodic.ctypes.data,
                                 _RefDevice(1, 0), options, ctypes.byref(out), ctypes.byref(message))
    last_call_seconds = time.perf_counter() - start
    if status != 0:
        raise RuntimeError(message.value.decode("utf8"))
    try:
        return _collect(out.length, out.pairs, out.shifts, out.distances, out.vectors,
                        "S" in quantities, "d" in quantities, "D" in quantities)
    finally:
        lib.vesin_free(ctypes.byref(out))


# --------------------------------------------------------------------------------------------------------------
# Canonical order shared by every comparison


def canonical_order(pairs, shifts=None):
    """Permutation putting a list in lexicographic (i, j, Sx, Sy, Sz) order."""
    pairs = np.asarray(pairs).reshape(-1, 2)
    keys = []
    if shifts is not None:
        shifts = np.asarray(shifts).reshape(-1, 3)
        keys += [shifts[:, 2], shifts[:, 1], shifts[:, 0]]
    keys += [pairs[:, 1], pairs[:, 0]]
    return np.lexsort(keys)


def canonicalize(result):
    """Return a copy of a result dict reordered to lexicographic (i, j, S) order (needs ``shifts`` to be a total
    order whenever one pair of points has several images)."""
    order = canonical_order(result["pairs"], result.get("shifts"))
    return {key: value[order] for key, value in result.items() if key != "grid"}
