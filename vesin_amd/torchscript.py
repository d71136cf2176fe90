"""TorchScript-compatible calculator, mirroring ``vesin_torch.NeighborList`` (reference:
python/vesin_torch/vesin_torch/_neighbors.py:6-107). The work is done by the custom class
``torch.classes.vesin._NeighborList`` of ``lib/libvesin_torch.so``, which calls this library's C ABI: the same class
name, arguments and pickled state as the reference's, so that scripted modules written for it run unchanged on a
HIP device. Outputs follow the dtype of ``points`` for distances and vectors, int64 for indices, int32 for shifts;
distances and vectors carry gradients with respect to ``points`` and ``box``.
"""

import os
from typing import List, Union

import torch

from ._c_api import get_library

TORCH_LIB_PATH = os.path.join(os.path.dirname(os.path.realpath(__file__)), "lib", "libvesin_torch.so")

_LOADED = False


def load_torch_library():
    """Register ``torch.classes.vesin._NeighborList``. There is no fallback when the library was not built."""
    global _LOADED
    if not _LOADED:
        if not os.path.exists(TORCH_LIB_PATH):
            raise RuntimeError(
                f"{TORCH_LIB_PATH} is missing: build it first with `python -m vesin_amd._build`"
            )
        get_library()
        torch.ops.load_library(TORCH_LIB_PATH)
        _LOADED = True


load_torch_library()


class NeighborList:
    """Calculator usable from TorchScript code; thin front of ``torch.classes.vesin._NeighborList``."""

    def __init__(self, cutoff: float, full_list: bool, sorted: bool = False, algorithm: str = "auto", n_threads: int = 0):
        """
        :param cutoff: spherical cutoff
        :param full_list: return every pair twice (``i-j`` and ``j-i``) or once
        :param sorted: sort the pairs (by ``i``, then ``j``, then shift)
        :param algorithm: accepted for compatibility (``"auto"``, ``"brute_force"``, ``"cell_list"``): one engine
            covers every case on the GPU
        :param n_threads: accepted for compatibility, must be zero or positive
        """
        if int(n_threads) < 0:
            raise ValueError("n_threads must be zero or a positive integer")
        self._c = torch.classes.vesin._NeighborList(cutoff, full_list, sorted, algorithm, int(n_threads))

    def compute(
        self,
        points: torch.Tensor,
        box: torch.Tensor,
        periodic: Union[bool, torch.Tensor],
        quantities: str = "ij",
        copy: bool = True,
    ) -> List[torch.Tensor]:
        """
        Neighbor list of ``points`` in ``box``; ``quantities`` is any combination of ``i``, ``j``, ``P`` (both
        indices), ``S`` (shifts), ``d`` (distances), ``D`` (vectors). With ``copy=False`` the tensors are views of
        memory the calculator owns, valid until its next calculation (outputs that carry gradients are always
        copies). The library computes in float64: other floating-point inputs are converted on the way in, and
        distances and vectors come back in the dtype of ``points``.
        """
        dtype = points.dtype
        if box.dtype != dtype:
            raise RuntimeError(f"`points` and `box` must have the same dtype, got {points.dtype} and {box.dtype}")
        flags = torch.as_tensor(periodic) if isinstance(periodic, bool) else periodic

        outputs = self._c.compute(points.to(torch.float64), box.to(torch.float64), flags, quantities, copy)
        if dtype == torch.float64:
            return outputs
        back: List[torch.Tensor] = []
        for position in range(len(outputs)):
            letter = quantities[position]
            tensor = outputs[position]
            back.append(tensor.to(dtype) if letter in ("d", "D") else tensor)
        return back
