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
    """A neighbor list calculator that can be used with TorchScript."""

    def __init__(
        self,
        cutoff: float,
        full_list: bool,
        sorted: bool = False,
        algorithm: str = "auto",
        n_threads: int = 0,
    ):
        """
        :param cutoff: spherical cutoff
        :param full_list: return every pair twice (``i-j`` and ``j-i``) or once
        :param sorted: sort the pairs (by ``i``, then ``j``, then shift)
        :param algorithm: accepted for compatibility (``"auto"``, ``"brute_force"``, ``"cell_list"``): one engine
            covers every case on the GPU
        :param n_threads: accepted for compatibility, must be zero or positive
        """
        n_threads = int(n_threads)
        if n_threads < 0:
            raise ValueError("n_threads must be zero or a positive integer")

        self._c = torch.classes.vesin._NeighborList(
            cutoff=cutoff,
            full_list=full_list,
            sorted=sorted,
            algorithm=algorithm,
            n_threads=n_threads,
        )

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
        memory the calculator owns, valid until its next calculation.
        """
        if isinstance(periodic, bool):
            periodic = torch.as_tensor(periodic)

        initial_dtype = points.dtype
        if box.dtype != initial_dtype:
            raise RuntimeError(
                f"`points` and `box` must have the same dtype, got {points.dtype} and {box.dtype}"
            )

        results = self._c.compute(
            points=points.to(torch.float64),
            box=box.to(torch.float64),
            periodic=periodic,
            quantities=quantities,
            copy=copy,
        )

        converted: List[torch.Tensor] = []
        for index, result in enumerate(results):
            letter = quantities[index]
            if letter == "d" or letter == "D":
                result = result.to(initial_dtype)
            converted.append(result)
        return converted
