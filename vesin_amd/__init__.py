"""MI355X-native neighbor lists behind vesin's C ABI.

``NeighborList`` mirrors the reference's Python calculator; the work is done by ``lib/libvesin.so`` (hand-written
gfx950 HIP kernels, built by ``vesin_amd._build.build``). Importing this package does not load the library;
creating a ``NeighborList`` does, and fails loudly when it has not been built.
"""

from ._ase import ase_neighbor_list  # noqa: F401
from ._neighbors import NeighborList, enable_timings  # noqa: F401

__all__ = ["NeighborList", "ase_neighbor_list", "enable_timings"]
