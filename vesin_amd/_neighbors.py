"""``NeighborList``: the Python caller of the C ABI, with the interface of the reference's
``vesin.NeighborList`` (python/vesin/vesin/_neighbors.py:69-381): same constructor arguments, same
``compute(points, box, periodic, quantities, copy)`` contract, same dtypes and shapes of the results.

The calculation always runs on a GPU through ``vesin_neighbors`` with ``device = {VesinCUDA, index}``:

* torch tensors on a ``cuda`` device (what PyTorch-ROCm calls a HIP GPU) are used in place, and the results are
  torch tensors on the same device (zero-copy views of the library's buffers when ``copy=False``);
* device arrays of other libraries (cupy on ROCm, numba: anything that is not a torch tensor and has a
  ``__cuda_array_interface__``; the reference takes ``cupy.ndarray`` at python/vesin/vesin/_neighbors.py:173-183,
  436-452) are used in place too, and the results are arrays of the same library, made by its ``asarray`` from
  objects with that interface (views of the library's buffers when ``copy=False``);
* numpy arrays (or anything numpy can convert) are uploaded to ``device`` (default ``cuda:0``) and the results come
  back as numpy arrays.

With ``copy=True`` (the default) the reference copies every array out of the list's memory
(python/vesin/vesin/_neighbors.py:343-381, 513-574). Here the list takes its arrays from PyTorch's caching allocator
(``vesin_hip_set_output_allocator``, through the two functions ``lib/libvesin_torch.so`` exports) and the tensors that
go to the caller take them over (``vesin_hip_detach_outputs``): nothing is copied, the next call gets arrays of the
same size from the allocator's cache. Arrays with room for more than twice their rows are copied as before, and so is
everything when ``lib/libvesin_torch.so`` was not built.

torch is only used to hold device memory; nothing is computed with it.
"""

import ctypes
from typing import Sequence, Union

import numpy as np

from ._c_api import (
    VesinAutoAlgorithm,
    VesinBruteForce,
    VesinCellList,
    VesinCUDA,
    VesinDevice,
    VesinHipTimings,
    VesinNeighborList,
    VesinOptions,
    VesinUnknownDevice,
    get_library,
)

_HANDOVER = None


def _torch_handover():
    """What taking arrays over needs, or False when ``lib/libvesin_torch.so`` is not there: the library itself (for
    its ``vesin_amd_torch_release``), the addresses of its allocate and release functions, and the operator that
    makes a tensor the owner of an array from that allocator."""
    global _HANDOVER
    if _HANDOVER is None:
        try:
            import torch

            from .torchscript import TORCH_LIB_PATH, load_torch_library

            load_torch_library()
            hooks = ctypes.CDLL(TORCH_LIB_PATH)
            hooks.vesin_amd_torch_release.restype = None
            hooks.vesin_amd_torch_release.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
            allocate = ctypes.cast(hooks.vesin_amd_torch_allocate, ctypes.c_void_p).value
            release = ctypes.cast(hooks.vesin_amd_torch_release, ctypes.c_void_p).value
            _HANDOVER = (hooks, allocate, release, torch.ops.vesin_amd.adopt)
        except Exception:
            _HANDOVER = False
    return _HANDOVER


_ALGORITHMS = {
    "auto": VesinAutoAlgorithm,
    "brute_force": VesinBruteForce,
    "cell_list": VesinCellList,
}


class _DeviceView:
    """Expose a raw device pointer through ``__cuda_array_interface__`` so torch (or any array library that reads
    the interface) can wrap it without a copy. ``owner`` is kept alive as long as the view."""

    def __init__(self, pointer, shape, typestr, owner, strides=None):
        self._owner = owner
        self.__cuda_array_interface__ = {
            "shape": tuple(shape),
            "typestr": typestr,
            "data": (int(pointer), False),
            "version": 2,
            "strides": strides,
        }


_TYPESTR = {"torch.uint64": "<u8", "torch.int32": "<i4", "torch.float64": "<f8", "torch.float32": "<f4",
            "torch.float16": "<f2"}


def _export(tensor, namespace):
    """Hand a torch GPU tensor to another array library: ``namespace.asarray`` of a view of the same memory."""
    itemsize = tensor.element_size()
    strides = None if tensor.is_contiguous() else tuple(stride * itemsize for stride in tensor.stride())
    pointer = tensor.data_ptr() if tensor.numel() > 0 else 0
    return namespace.asarray(_DeviceView(pointer, tensor.shape, _TYPESTR[str(tensor.dtype)], tensor, strides))


def _namespace_of(array):
    """The top-level module of the library an array comes from (``cupy`` for a ``cupy.ndarray``)."""
    import importlib

    namespace = importlib.import_module(type(array).__module__.split(".")[0])
    if not hasattr(namespace, "asarray"):
        raise TypeError(f"can not return results as {type(array)}: its module `{namespace.__name__}` has no `asarray`")
    return namespace


def _device_index_of(array, default):
    """GPU index of a device array: ``array.device.id`` (cupy), ``array.device.index``, else ``default``."""
    device = getattr(array, "device", None)
    for name in ("id", "index"):
        index = getattr(device, name, None)
        if isinstance(index, int):
            return index
    return default


class NeighborList:
    """A neighbor list calculator running on an AMD GPU."""

    def __init__(
        self,
        cutoff: float,
        full_list: bool,
        sorted: bool = False,
        algorithm: str = "auto",
        skin: float = 0.0,
        n_threads: int = 0,
        device: str = "cuda:0",
    ):
        """
        :param cutoff: spherical cutoff; pairs strictly closer than this are returned
        :param full_list: return each pair twice (``i-j`` and ``j-i``) or only once
        :param sorted: order the pairs by ``i`` (this implementation orders by ``(i, j, shift)``)
        :param algorithm: ``"auto"``, ``"brute_force"`` or ``"cell_list"``
        :param skin: Verlet skin: with a positive value, candidates computed at ``cutoff + skin`` are kept and
            filtered at the cutoff while no point moved further than half of it; the result is that of ``skin=0``
        :param n_threads: accepted for compatibility (must be ``>= 0``); the GPU path does not use it
        :param device: GPU used for inputs that are not already torch GPU tensors
        """
        self._lib = get_library()
        self.cutoff = float(cutoff)
        self.full_list = bool(full_list)
        self.sorted = bool(sorted)
        self.skin = float(skin)
        self.algorithm = algorithm
        self.n_threads = int(n_threads)
        if self.n_threads < 0:
            raise ValueError("n_threads must be zero or a positive integer")
        self.device = device
        self._neighbors = VesinNeighborList()
        # whether results with ``copy=True`` take the list's arrays over instead of copying them
        self.hand_over = True
        self._allocator_set = False

    def _torch_allocator(self, c_device):
        """Make the list take its arrays from PyTorch's caching allocator (once per list); returns what
        ``_torch_handover`` does, or None when arrays are not handed over."""
        if not self.hand_over:
            return None
        handover = _torch_handover()
        if not handover:
            return None
        if not self._allocator_set:
            error_message = ctypes.c_char_p()
            status = self._lib.vesin_hip_set_output_allocator(
                ctypes.byref(self._neighbors), c_device, handover[1], handover[2], None, ctypes.byref(error_message)
            )
            if status != 0:
                raise RuntimeError(error_message.value.decode("utf8"))
            self._allocator_set = True
        return handover

    def _take_arrays(self, handover):
        """The arrays of the list become the caller's (None when they stay: no allocator, no rows, or room for more
        than twice the rows): returns a function ``(pointer, shape, dtype, index) -> tensor`` that makes a tensor the
        owner of one of them, and a function that releases those no tensor took."""
        n_pairs = self._neighbors.length
        if not handover or not self._allocator_set or n_pairs == 0:
            return None
        if 2 * n_pairs < self._lib.vesin_hip_output_capacity(ctypes.byref(self._neighbors)):
            return None
        arrays = [self._neighbors.pairs, self._neighbors.shifts, self._neighbors.distances, self._neighbors.vectors]
        error_message = ctypes.c_char_p()
        if self._lib.vesin_hip_detach_outputs(ctypes.byref(self._neighbors), None, ctypes.byref(error_message)) != 0:
            return None
        hooks, adopt = handover[0], handover[3]
        left = {pointer for pointer in arrays if pointer}

        def owned(pointer, shape, dtype, index):
            left.discard(pointer)
            return adopt(pointer, list(shape), dtype, index)

        def release_rest():
            for pointer in left:
                hooks.vesin_amd_torch_release(pointer, None)
            left.clear()

        return owned, release_rest

    def __del__(self):
        if hasattr(self, "_lib") and hasattr(self, "_neighbors"):
            self._lib.vesin_free(ctypes.byref(self._neighbors))

    @property
    def algorithm(self) -> str:
        return self._algorithm

    @algorithm.setter
    def algorithm(self, value: str):
        algorithm = value.lower()
        if algorithm not in _ALGORITHMS:
            raise ValueError(
                f"Unknown algorithm '{algorithm}'. Must be one of 'auto', 'brute_force', or 'cell_list'."
            )
        self._algorithm = algorithm
        self._c_algorithm = _ALGORITHMS[algorithm]

    def compute(
        self,
        points,
        box,
        periodic: Union[bool, Sequence[bool]],
        quantities: str = "ij",
        copy: bool = True,
    ):
        """Compute the neighbor list and return the requested ``quantities``, any of: ``i``, ``j``, ``P`` (both
        indices), ``S`` (shifts), ``d`` (distances), ``D`` (vectors), as a tuple in the order asked for.

        With ``copy=False`` the returned torch tensors alias the calculator's buffers and are invalidated by the
        next ``compute`` or when the calculator is collected.
        """
        import torch

        is_torch = isinstance(points, torch.Tensor)
        if is_torch and points.device.type != "cuda":
            raise RuntimeError(
                "this implementation only computes on GPU tensors; move `points` to a cuda (HIP) device"
            )
        device = points.device if is_torch else torch.device(self.device)
        namespace = None
        if not is_torch and hasattr(points, "__cuda_array_interface__"):
            # a device array of another library: used in place, results go back through its own `asarray`
            namespace = _namespace_of(points)
            device = torch.device("cuda", _device_index_of(points, device.index if device.index is not None else 0))
            points = torch.as_tensor(points, device=device)
            if hasattr(box, "__cuda_array_interface__"):
                box = torch.as_tensor(box, device=device)
            else:
                box = torch.from_numpy(np.ascontiguousarray(np.asarray(box))).to(device=device)
            if hasattr(periodic, "__cuda_array_interface__"):
                periodic = torch.as_tensor(periodic, device=device)
            is_torch = True

        if isinstance(periodic, (bool, np.bool_)):
            periodic = [bool(periodic)] * 3

        if is_torch:
            if not isinstance(box, torch.Tensor):
                box = torch.as_tensor(box)
            initial_dtype = points.dtype
            if box.dtype != initial_dtype:
                raise RuntimeError(
                    f"`points` and `box` must have the same dtype, got {points.dtype} and {box.dtype}"
                )
            if points.requires_grad or box.requires_grad:
                raise RuntimeError("NeighborList.compute does not support autograd for torch tensors")
            float_dtype = initial_dtype if initial_dtype.is_floating_point else torch.float64
            if namespace is None:
                to_result = lambda t: t  # noqa: E731
            else:
                to_result = lambda t: _export(t, namespace)  # noqa: E731
        else:
            points = np.asarray(points)
            box = np.asarray(box)
            initial_dtype = points.dtype
            if box.dtype != initial_dtype:
                raise RuntimeError(
                    f"`points` and `box` must have the same dtype, got {points.dtype} and {box.dtype}"
                )
            np_float = initial_dtype if np.issubdtype(initial_dtype, np.floating) else np.float64
            float_dtype = {np.dtype(np.float32): torch.float32, np.dtype(np.float64): torch.float64}.get(
                np.dtype(np_float), torch.float64
            )
            points = torch.from_numpy(np.ascontiguousarray(points))
            box = torch.from_numpy(np.ascontiguousarray(box))
            to_result = lambda t: t.cpu().numpy()  # noqa: E731

        if tuple(box.shape) != (3, 3):
            raise ValueError("`box` must be a 3x3 matrix")
        if points.dim() != 2 or points.shape[1] != 3:
            raise ValueError("`points` must be a nx3 array")

        if isinstance(periodic, torch.Tensor):
            periodic = periodic.to(dtype=torch.bool, device=device).contiguous()
        else:
            # the three flags rarely change between calls: keep their device copy (a list or tuple of three plain
            # booleans, the usual argument, is recognised without going through numpy)
            plain = type(periodic) in (list, tuple) and len(periodic) == 3 and all(type(f) is bool for f in periodic)
            key = (tuple(periodic), device) if plain else None
            cached = getattr(self, "_periodic_on_device", None)
            if key is None or cached is None or cached[0] != key:
                flags = np.asarray(periodic).astype(np.bool_)
                key = (tuple(bool(f) for f in flags), device) if flags.shape == (3,) else (flags.tobytes(), flags.shape, device)
                if cached is None or cached[0] != key:
                    cached = (key, torch.as_tensor(flags).to(device=device))
                    self._periodic_on_device = cached
            periodic = cached[1]
        if tuple(periodic.shape) != (3,):
            raise ValueError(
                f"`periodic` must be a single boolean or a sequence of three booleans, got {periodic}"
            )

        if points.dtype != torch.float64 or points.device != device or not points.is_contiguous():
            points = points.to(device=device, dtype=torch.float64).contiguous()
        if box.dtype != torch.float64 or box.device != device or not box.is_contiguous():
            box = box.to(device=device, dtype=torch.float64).contiguous()

        index = device.index if device.index is not None else torch.cuda.current_device()

        # options and device of the call: the same objects while nothing they are made of changes
        settings = (self.cutoff, self.full_list, self.sorted, self._c_algorithm, self.n_threads, self.skin, quantities, index)
        kept = self.__dict__.get("_call_settings")
        if kept is None or kept[0] != settings:
            options = VesinOptions()
            options.cutoff = self.cutoff
            options.full = self.full_list
            options.sorted = self.sorted
            options.algorithm = self._c_algorithm
            options.n_threads = self.n_threads
            options.return_shifts = "S" in quantities
            options.return_distances = "d" in quantities
            options.return_vectors = "D" in quantities
            options.skin = self.skin
            kept = (settings, options, VesinDevice(VesinCUDA, index))
            self._call_settings = kept
        options, c_device = kept[1], kept[2]

        if self._neighbors.device.type != VesinUnknownDevice and (
            self._neighbors.device.type != c_device.type or self._neighbors.device.device_id != c_device.device_id
        ):
            # the list lives on another GPU: release it and start from a zeroed struct
            self._lib.vesin_free(ctypes.byref(self._neighbors))
            ctypes.memset(ctypes.byref(self._neighbors), 0, ctypes.sizeof(self._neighbors))
            self._allocator_set = False
        handover = self._torch_allocator(c_device) if copy else None

        # inputs may still be in flight on torch's current stream. The library works on the null stream, which waits
        # for everything earlier on torch's default stream by itself; only a stream of the caller's own does not
        stream = torch.cuda.current_stream(device)
        if stream.cuda_stream != 0:
            stream.synchronize()

        # an empty tensor has no storage; the ABI still wants a device pointer
        points_ptr = points.data_ptr() if points.shape[0] > 0 else box.data_ptr()

        error_message = ctypes.c_char_p()
        status = self._lib.vesin_neighbors(
            points_ptr,
            points.shape[0],
            box.data_ptr(),
            periodic.data_ptr(),
            c_device,
            options,
            ctypes.byref(self._neighbors),
            ctypes.byref(error_message),
        )
        if status != 0:
            raise RuntimeError(error_message.value.decode("utf8"))

        n_pairs = self._neighbors.length
        pointers = (self._neighbors.pairs, self._neighbors.shifts, self._neighbors.distances, self._neighbors.vectors)
        taken = self._take_arrays(handover) if copy else None
        if not copy:
            # views of arrays that did not move, asked for in the same way: the tuple of the call before
            result_key = (
                quantities, n_pairs, *pointers, float_dtype, index,
                # (distances and vectors in another precision are converted copies, made again on every call)
                namespace is None and is_torch and float_dtype == torch.float64,
            )
            last = self.__dict__.get("_last_views")
            if last is not None and last[0] == result_key and result_key[-1]:
                return last[1]
        device_str = f"cuda:{index}"

        views = self.__dict__.setdefault("_views", {})

        def wrap(pointer, shape, typestr, dtype):
            if n_pairs == 0:
                return torch.empty(shape, dtype=dtype, device=device_str)
            if taken is not None:
                return taken[0](pointer, shape, dtype, index)
            if copy:
                return torch.as_tensor(_DeviceView(pointer, shape, typestr, self), device=device_str).clone()
            # the arrays are kept between calls: the same pointer and shape give the same view (views refer to
            # the calculator, so only callers who asked for views make it refer to itself)
            key = (pointer, shape, typestr, device_str)
            cached = views.get(typestr + str(len(shape)))
            if cached is None or cached[0] != key:
                cached = (key, torch.as_tensor(_DeviceView(pointer, shape, typestr, self), device=device_str))
                views[typestr + str(len(shape))] = cached
            return cached[1]

        pairs = shifts = distances = vectors = None
        if any(q in quantities for q in "ijP"):
            pairs = wrap(pointers[0], (n_pairs, 2), "<u8", torch.uint64)
        if "S" in quantities:
            shifts = wrap(pointers[1], (n_pairs, 3), "<i4", torch.int32)
        if "d" in quantities:
            distances = wrap(pointers[2], (n_pairs,), "<f8", torch.float64).to(float_dtype)
        if "D" in quantities:
            vectors = wrap(pointers[3], (n_pairs, 3), "<f8", torch.float64).to(float_dtype)
        if taken is not None:
            taken[1]()  # (the pairs of a call that asked for none of "ijP")

        data = []
        for quantity in quantities:
            if quantity == "P":
                data.append(to_result(pairs))
            elif quantity == "i":
                data.append(to_result(pairs[:, 0]))
            elif quantity == "j":
                data.append(to_result(pairs[:, 1]))
            elif quantity == "S":
                data.append(to_result(shifts))
            elif quantity == "d":
                data.append(to_result(distances))
            elif quantity == "D":
                data.append(to_result(vectors))
        data = tuple(data)
        if not copy and n_pairs != 0:
            self._last_views = (result_key, data)
        return data

    def compute_batch(self, points, first_point, boxes, periodic=True, quantities: str = "ij", copy: bool = True):
        """Neighbor lists of many systems in one go (``vesin_hip_neighbors_batch``).

        ``points``: (N, 3) GPU tensor with the systems one after the other; ``first_point``: n_systems + 1 integers,
        where each system starts; ``boxes``: (n_systems, 3, 3) GPU tensor; ``periodic``: one flag for everything, or an
        (n_systems, 3) boolean tensor (free molecules, slabs and crystals can share a batch). Returns ``(outputs, first_pair)``: the requested quantities for all systems
        (indices count inside each system) and the n_systems + 1 row offsets of the systems as a numpy array.
        """
        import torch

        device, index, first_point, n_systems, points, boxes, periodic, options = self._batch_arguments(
            points, first_point, boxes, periodic, quantities
        )
        handover = self._torch_allocator(VesinDevice(VesinCUDA, index)) if copy else None
        torch.cuda.current_stream(device).synchronize()
        first_pair = np.zeros(n_systems + 1, dtype=np.uint64)
        error_message = ctypes.c_char_p()
        status = self._lib.vesin_hip_neighbors_batch(
            points.data_ptr() if points.shape[0] > 0 else boxes.data_ptr(),
            first_point.ctypes.data_as(ctypes.POINTER(ctypes.c_size_t)),
            n_systems,
            boxes.data_ptr(),
            periodic.data_ptr(),
            VesinDevice(VesinCUDA, index),
            options,
            ctypes.byref(self._neighbors),
            first_pair.ctypes.data_as(ctypes.POINTER(ctypes.c_size_t)),
            ctypes.byref(error_message),
        )
        if status != 0:
            self._last_batch_systems = None
            raise RuntimeError(error_message.value.decode("utf8"))
        self._last_batch_systems = n_systems

        return self._results(quantities, index, copy, handover), first_pair

    def _batch_arguments(self, points, first_point, boxes, periodic, quantities):
        """The inputs of a batch as the library takes them (tensors on the points' device, the division into systems
        as a numpy array, the options), on a list of that device."""
        import torch

        if not isinstance(points, torch.Tensor) or points.device.type != "cuda":
            raise RuntimeError("a batch takes torch tensors on a cuda (HIP) device")
        device = points.device
        first_point = np.ascontiguousarray(first_point, dtype=np.uint64)
        n_systems = len(first_point) - 1
        points = points.to(dtype=torch.float64).contiguous()
        boxes = torch.as_tensor(boxes).to(device=device, dtype=torch.float64).contiguous()
        if tuple(boxes.shape) != (n_systems, 3, 3):
            raise ValueError("`boxes` must hold one 3x3 matrix per system")
        if isinstance(periodic, (bool, np.bool_)):
            # one flag for everything: the tensor of flags is kept for the next batch of this size
            key = (n_systems, bool(periodic), str(device))
            kept = getattr(self, "_batch_flags", None)
            if kept is None or kept[0] != key:
                kept = (key, torch.full((n_systems, 3), bool(periodic), dtype=torch.bool, device=device))
                self._batch_flags = kept
            periodic = kept[1]
        else:
            periodic = torch.as_tensor(periodic).to(device=device, dtype=torch.bool).contiguous()
        if tuple(periodic.shape) != (n_systems, 3):
            raise ValueError("`periodic` must hold three flags per system")

        options = VesinOptions()
        options.cutoff = self.cutoff
        options.full = self.full_list
        options.sorted = self.sorted
        options.algorithm = self._c_algorithm
        options.n_threads = self.n_threads
        options.return_shifts = "S" in quantities
        options.return_distances = "d" in quantities
        options.return_vectors = "D" in quantities
        options.skin = self.skin

        index = device.index if device.index is not None else torch.cuda.current_device()
        if self._neighbors.device.type != VesinUnknownDevice and self._neighbors.device.device_id != index:
            self._lib.vesin_free(ctypes.byref(self._neighbors))
            ctypes.memset(ctypes.byref(self._neighbors), 0, ctypes.sizeof(self._neighbors))
            self._allocator_set = False
        return device, index, first_point, n_systems, points, boxes, periodic, options

    def _results(self, quantities, index, copy, handover):
        """The requested quantities of the call that just ended, as torch tensors: views of the list's arrays, or
        (``copy``) tensors of their own, which take the arrays over when they can."""
        import torch

        n_pairs = self._neighbors.length
        device_str = f"cuda:{index}"
        pointers = (self._neighbors.pairs, self._neighbors.shifts, self._neighbors.distances, self._neighbors.vectors)
        taken = self._take_arrays(handover) if copy else None

        def wrap(pointer, shape, typestr, dtype):
            if n_pairs == 0:
                return torch.empty(shape, dtype=dtype, device=device_str)
            if taken is not None:
                return taken[0](pointer, shape, dtype, index)
            view = torch.as_tensor(_DeviceView(pointer, shape, typestr, self), device=device_str)
            return view.clone() if copy else view

        data = []
        pairs = None
        for quantity in quantities:
            if quantity in "ijP" and pairs is None:
                pairs = wrap(pointers[0], (n_pairs, 2), "<u8", torch.uint64)
            if quantity == "P":
                data.append(pairs)
            elif quantity == "i":
                data.append(pairs[:, 0])
            elif quantity == "j":
                data.append(pairs[:, 1])
            elif quantity == "S":
                data.append(wrap(pointers[1], (n_pairs, 3), "<i4", torch.int32))
            elif quantity == "d":
                data.append(wrap(pointers[2], (n_pairs,), "<f8", torch.float64))
            elif quantity == "D":
                data.append(wrap(pointers[3], (n_pairs, 3), "<f8", torch.float64))
        if taken is not None:
            taken[1]()
        return tuple(data)

    def enqueue(self, points, box, periodic, quantities: str = "ij"):
        """``compute`` in two halves (``vesin_hip_neighbors_enqueue``): queues the calculation on torch's current
        stream and returns without waiting for it, so that the caller can queue whatever consumes the list right
        behind. Takes contiguous float64 torch tensors on the GPU (``points`` (N, 3), ``box`` (3, 3)) and a boolean
        tensor of three flags on the GPU for ``periodic``; they must stay as they are until ``collect``.

        Returns a one-element int64 tensor that views the word in GPU memory where work queued on the same stream
        finds the number of rows, or -1 when the queued kernels did not leave the complete list (a list's first call,
        another box, rows that outgrew the arrays): then nothing may be read before ``collect`` has returned.
        """
        import torch

        for name, tensor in (("points", points), ("box", box), ("periodic", periodic)):
            if not isinstance(tensor, torch.Tensor) or tensor.device.type != "cuda" or not tensor.is_contiguous():
                raise RuntimeError(f"enqueue takes contiguous torch tensors on a cuda (HIP) device, `{name}` is not one")
        if points.dtype != torch.float64 or box.dtype != torch.float64 or periodic.dtype != torch.bool:
            raise RuntimeError("enqueue takes float64 `points` and `box` and boolean `periodic`")
        if points.dim() != 2 or points.shape[1] != 3 or tuple(box.shape) != (3, 3) or tuple(periodic.shape) != (3,):
            raise ValueError("`points` must be a nx3 array, `box` a 3x3 matrix, `periodic` three flags")
        if self.__dict__.get("_queued") is not None:
            raise RuntimeError("this calculator has a call pending: collect() it first")
        device = points.device
        index = device.index if device.index is not None else torch.cuda.current_device()
        options = VesinOptions()
        options.cutoff = self.cutoff
        options.full = self.full_list
        options.sorted = self.sorted
        options.algorithm = self._c_algorithm
        options.n_threads = self.n_threads
        options.return_shifts = "S" in quantities
        options.return_distances = "d" in quantities
        options.return_vectors = "D" in quantities
        options.skin = self.skin
        if self._neighbors.device.type != VesinUnknownDevice and self._neighbors.device.device_id != index:
            self._lib.vesin_free(ctypes.byref(self._neighbors))
            ctypes.memset(ctypes.byref(self._neighbors), 0, ctypes.sizeof(self._neighbors))
            self._allocator_set = False
        self._torch_allocator(VesinDevice(VesinCUDA, index))
        word = ctypes.c_void_p()
        error_message = ctypes.c_char_p()
        status = self._lib.vesin_hip_neighbors_enqueue(
            points.data_ptr() if points.shape[0] > 0 else box.data_ptr(), points.shape[0], box.data_ptr(),
            periodic.data_ptr(), VesinDevice(VesinCUDA, index), options, ctypes.byref(self._neighbors),
            torch.cuda.current_stream(device).cuda_stream, ctypes.byref(word), ctypes.byref(error_message),
        )
        if status != 0:
            raise RuntimeError(error_message.value.decode("utf8"))
        # (the inputs are referred to until the call is collected)
        self._queued = (quantities, index, points, box, periodic)
        return torch.as_tensor(_DeviceView(word.value, (1,), "<i8", self), device=f"cuda:{index}")

    def enqueue_batch(self, points, first_point, boxes, periodic=True, quantities: str = "ij"):
        """``compute_batch`` in two halves (``vesin_hip_neighbors_batch_enqueue``): queues the batch on torch's
        current stream and returns without waiting for the GPU; ``collect`` completes it and returns what
        ``compute_batch`` would have, ``(outputs, first_pair)``. The inputs must not be changed in between. The
        tensor returned here holds -1 until ``collect`` has set it to the number of rows."""
        import torch

        if self.__dict__.get("_queued") is not None:
            raise RuntimeError("this calculator has a call pending: collect() it first")
        device, index, first_point, n_systems, points, boxes, periodic, options = self._batch_arguments(
            points, first_point, boxes, periodic, quantities
        )
        self._torch_allocator(VesinDevice(VesinCUDA, index))
        first_pair = np.zeros(n_systems + 1, dtype=np.uint64)
        word = ctypes.c_void_p()
        error_message = ctypes.c_char_p()
        status = self._lib.vesin_hip_neighbors_batch_enqueue(
            points.data_ptr() if points.shape[0] > 0 else boxes.data_ptr(),
            first_point.ctypes.data_as(ctypes.POINTER(ctypes.c_size_t)),
            n_systems,
            boxes.data_ptr(),
            periodic.data_ptr(),
            VesinDevice(VesinCUDA, index),
            options,
            ctypes.byref(self._neighbors),
            first_pair.ctypes.data_as(ctypes.POINTER(ctypes.c_size_t)),
            torch.cuda.current_stream(device).cuda_stream,
            ctypes.byref(word),
            ctypes.byref(error_message),
        )
        if status != 0:
            self._last_batch_systems = None
            raise RuntimeError(error_message.value.decode("utf8"))
        self._last_batch_systems = n_systems
        # (the inputs and the two host arrays are referred to until the call is collected)
        self._queued = (quantities, index, points, boxes, periodic, first_point, first_pair)
        return torch.as_tensor(_DeviceView(word.value, (1,), "<i8", self), device=f"cuda:{index}")

    def first_pair_on_device(self):
        """The first row of every system of the last batch as the kernels left it on the GPU
        (``vesin_hip_batch_first_pair_on_device``): a tensor of n_systems + 1 int64 that refers to the calculator's
        memory and holds these values until the next call; None when the last call was no batch or had no points. For
        work queued behind ``enqueue_batch`` that goes through the rows system by system without the host."""
        import torch

        pointer = self._lib.vesin_hip_batch_first_pair_on_device(ctypes.byref(self._neighbors))
        n_systems = self.__dict__.get("_last_batch_systems")
        if not pointer or n_systems is None:
            return None
        index = self._neighbors.device.device_id
        return torch.as_tensor(_DeviceView(pointer, (n_systems + 1,), "<i8", self), device=f"cuda:{index}")

    def collect(self, copy: bool = True):
        """Completes the call that ``enqueue`` or ``enqueue_batch`` started (``vesin_hip_neighbors_collect``) and
        returns what ``compute`` or ``compute_batch`` would have. Errors of the calculation are raised here."""
        import torch

        queued = self.__dict__.get("_queued")
        if queued is None:
            raise RuntimeError("this calculator has no call pending")
        self._queued = None
        quantities, index = queued[0], queued[1]
        error_message = ctypes.c_char_p()
        if self._lib.vesin_hip_neighbors_collect(ctypes.byref(self._neighbors), ctypes.byref(error_message)) != 0:
            self._last_batch_systems = None
            raise RuntimeError(error_message.value.decode("utf8"))
        handover = _torch_handover() if copy and self.hand_over and self._allocator_set else None
        results = self._results(quantities, index, copy, handover)
        return (results, queued[6]) if len(queued) == 7 else results

    def timings(self):
        """Per-stage GPU times (ms) of the last ``compute``; needs ``enable_timings(True)`` beforehand."""
        timings = VesinHipTimings()
        if self._lib.vesin_hip_last_timings(ctypes.byref(self._neighbors), ctypes.byref(timings)) != 0:
            return None
        return {name: getattr(timings, name) for name, _ in VesinHipTimings._fields_ if name != "candidates"}


def enable_timings(enabled: bool = True):
    """Make every later call record HIP events between its stages."""
    get_library().vesin_hip_enable_timings(1 if enabled else 0)
