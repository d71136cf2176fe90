"""``ase_neighbor_list``: the calling convention of ``ase.neighborlist.neighbor_list`` on top of ``NeighborList``,
as the reference offers it (python/vesin/vesin/_ase.py:9-55): same arguments, same refusals, a full list sorted by
``i``, results as numpy arrays. The calculation itself runs on the GPU."""

import numbers

from ._neighbors import NeighborList

try:
    import ase
except ImportError:  # the wrapper then says so when called
    ase = None


def ase_neighbor_list(quantities, a, cutoff, self_interaction=False, max_nbins=0, device="cuda:0"):
    """Neighbor list of an ``ase.Atoms`` with the interface of ``ase.neighborlist.neighbor_list``.

    :param quantities: any of ``i``, ``j``, ``d``, ``D``, ``S``, with ASE's meaning
    :param a: the ``ase.Atoms``
    :param cutoff: one cutoff radius for all atoms (ASE's per-element dictionaries are not supported)
    :param self_interaction: must stay ``False``
    :param max_nbins: accepted and ignored, as in the reference
    :param device: the GPU that computes (this implementation has no CPU engine)
    """
    if ase is None:
        raise ImportError("could not import ase, this function requires ase")
    if self_interaction:
        raise ValueError("self_interaction=True is not implemented")
    if isinstance(cutoff, bool) or not isinstance(cutoff, numbers.Real):
        raise ValueError("only a single float cutoff is supported")
    if not isinstance(a, ase.Atoms):
        raise TypeError(f"`a` should be ase.Atoms, got {type(a)} instead")

    # ASE gives every pair twice, ordered by the first atom
    calculator = NeighborList(cutoff=float(cutoff), full_list=True, sorted=True, device=device)
    return calculator.compute(points=a.positions, box=a.cell[:], periodic=a.pbc, quantities=quantities, copy=True)
