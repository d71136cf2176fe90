"""ctypes mirror of include/vesin.h (layouts asserted in tests/test_abi.py)."""

import ctypes
import os

VesinAutoAlgorithm = 0
VesinBruteForce = 1
VesinCellList = 2

VesinUnknownDevice = 0
VesinCPU = 1
VesinCUDA = 2


class VesinDevice(ctypes.Structure):
    _fields_ = [("type", ctypes.c_int), ("device_id", ctypes.c_int)]


class VesinOptions(ctypes.Structure):
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


class VesinNeighborList(ctypes.Structure):
    _fields_ = [
        ("length", ctypes.c_size_t),
        ("device", VesinDevice),
        ("pairs", ctypes.c_void_p),
        ("shifts", ctypes.c_void_p),
        ("distances", ctypes.c_void_p),
        ("vectors", ctypes.c_void_p),
        ("opaque", ctypes.c_void_p),
    ]


class VesinHipTimings(ctypes.Structure):
    _fields_ = [
        ("total", ctypes.c_float),
        ("cell_build", ctypes.c_float),
        ("count", ctypes.c_float),
        ("scan", ctypes.c_float),
        ("write", ctypes.c_float),
        ("sort", ctypes.c_float),
        ("candidates", ctypes.c_uint64),
    ]


LIB_PATH = os.path.join(os.path.dirname(os.path.realpath(__file__)), "lib", "libvesin.so")

_LIBRARY = None


def get_library():
    """Load libvesin.so. There is no fallback: without the compiled HIP library nothing can be computed."""
    global _LIBRARY
    if _LIBRARY is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it first with `python -m vesin_amd._build` "
                "(hipcc, --offload-arch=gfx950)"
            )
        # PyTorch-ROCm ships its own HIP runtime. A process must use one runtime only (device pointers and streams
        # of one are unknown to another): torch goes first, so that the library's HIP symbols resolve to the
        # runtime that owns the caller's tensors.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = ctypes.CDLL(LIB_PATH)
        lib.vesin_neighbors.restype = ctypes.c_int
        lib.vesin_neighbors.argtypes = [
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            VesinDevice,
            VesinOptions,
            ctypes.POINTER(VesinNeighborList),
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_free.restype = None
        lib.vesin_free.argtypes = [ctypes.POINTER(VesinNeighborList)]
        lib.vesin_hip_neighbors_batch.restype = ctypes.c_int
        lib.vesin_hip_neighbors_batch.argtypes = [
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_size_t),
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            VesinDevice,
            VesinOptions,
            ctypes.POINTER(VesinNeighborList),
            ctypes.POINTER(ctypes.c_size_t),
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_neighbors_batch_on_stream.restype = ctypes.c_int
        lib.vesin_hip_neighbors_batch_on_stream.argtypes = [
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_size_t),
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            VesinDevice,
            VesinOptions,
            ctypes.POINTER(VesinNeighborList),
            ctypes.POINTER(ctypes.c_size_t),
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_neighbors_batch_enqueue.restype = ctypes.c_int
        lib.vesin_hip_neighbors_batch_enqueue.argtypes = [
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_size_t),
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            VesinDevice,
            VesinOptions,
            ctypes.POINTER(VesinNeighborList),
            ctypes.POINTER(ctypes.c_size_t),
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_void_p),
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_batch_first_pair_on_device.restype = ctypes.c_void_p
        lib.vesin_hip_batch_first_pair_on_device.argtypes = [ctypes.POINTER(VesinNeighborList)]
        lib.vesin_hip_pairs_backward.restype = ctypes.c_int
        lib.vesin_hip_pairs_backward.argtypes = [
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_size_t,
            VesinDevice,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_neighbors_on_stream.restype = ctypes.c_int
        lib.vesin_hip_neighbors_on_stream.argtypes = [
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            VesinDevice,
            VesinOptions,
            ctypes.POINTER(VesinNeighborList),
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_neighbors_enqueue.restype = ctypes.c_int
        lib.vesin_hip_neighbors_enqueue.argtypes = [
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            VesinDevice,
            VesinOptions,
            ctypes.POINTER(VesinNeighborList),
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_void_p),
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_neighbors_collect.restype = ctypes.c_int
        lib.vesin_hip_neighbors_collect.argtypes = [ctypes.POINTER(VesinNeighborList), ctypes.POINTER(ctypes.c_char_p)]
        lib.vesin_hip_neighbors_no_alloc.restype = ctypes.c_int
        lib.vesin_hip_neighbors_no_alloc.argtypes = [
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.c_void_p,
            ctypes.c_void_p,
            VesinDevice,
            VesinOptions,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_size_t,
            ctypes.POINTER(ctypes.c_size_t),
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_set_output_allocator.restype = ctypes.c_int
        lib.vesin_hip_set_output_allocator.argtypes = [
            ctypes.POINTER(VesinNeighborList),
            VesinDevice,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.c_void_p,
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_detach_outputs.restype = ctypes.c_int
        lib.vesin_hip_detach_outputs.argtypes = [
            ctypes.POINTER(VesinNeighborList),
            ctypes.POINTER(ctypes.c_size_t),
            ctypes.POINTER(ctypes.c_char_p),
        ]
        lib.vesin_hip_output_capacity.restype = ctypes.c_size_t
        lib.vesin_hip_output_capacity.argtypes = [ctypes.POINTER(VesinNeighborList)]
        lib.vesin_hip_enable_timings.restype = None
        lib.vesin_hip_enable_timings.argtypes = [ctypes.c_int]
        lib.vesin_hip_last_timings.restype = ctypes.c_int
        lib.vesin_hip_last_timings.argtypes = [ctypes.POINTER(VesinNeighborList), ctypes.POINTER(VesinHipTimings)]
        _LIBRARY = lib
    return _LIBRARY
