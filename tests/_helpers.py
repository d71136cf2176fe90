"""Shared helpers of the test-suite: run the GPU path through the C ABI, compare with the CPU oracle."""

import numpy as np

import oracle


def gpu_neighbors(points, box, periodic, cutoff, full=True, sorted=False, quantities="ijSdD", algorithm="auto"):
    """Run the HIP path (vesin_neighbors through ctypes, inputs as torch GPU tensors) and bring the result to the
    host in the layout of ``oracle.neighbors``."""
    import torch

    from vesin_amd import NeighborList

    calculator = NeighborList(cutoff=cutoff, full_list=full, sorted=sorted, algorithm=algorithm)
    letters = "P" + "".join(q for q in "SdD" if q in quantities)
    outputs = calculator.compute(
        torch.as_tensor(np.ascontiguousarray(points, dtype=np.float64), device="cuda:0"),
        torch.as_tensor(np.ascontiguousarray(box, dtype=np.float64), device="cuda:0"),
        periodic,
        letters,
        copy=True,
    )
    names = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}
    result = {names[q]: out.cpu().numpy() for q, out in zip(letters, outputs)}
    del calculator
    return result


def near_cutoff_count(result, cutoff):
    """Pairs whose distance is within 1e-12 * cutoff of the cutoff (reported, never excluded silently)."""
    if "distances" not in result:
        return 0
    return int(np.sum(np.abs(result["distances"] - cutoff) <= 1e-12 * cutoff))


def assert_same_list(actual, expected, ordered=False, what=""):
    """(i, j, S) must be identical; distances and vectors must be bit-identical (stricter than the 1e-12 relative
    tolerance the acceptance bar allows). With ``ordered`` the actual list must already BE in canonical
    (i, j, Sx, Sy, Sz) order: it is compared element-wise without being re-sorted."""
    expected = oracle.canonicalize(expected)
    if not ordered:
        actual = oracle.canonicalize(actual)
    assert actual["pairs"].shape == expected["pairs"].shape, (
        f"{what}: {actual['pairs'].shape[0]} pairs, expected {expected['pairs'].shape[0]}"
    )
    assert np.array_equal(actual["pairs"], expected["pairs"]), f"{what}: pairs differ"
    for key in ("shifts", "distances", "vectors"):
        if key in expected and key in actual:
            if not np.array_equal(actual[key], expected[key]):
                if key == "shifts":
                    raise AssertionError(f"{what}: shifts differ")
                scale = np.maximum(np.abs(expected[key]), 1e-300)
                worst = float(np.max(np.abs(actual[key] - expected[key]) / scale))
                raise AssertionError(f"{what}: {key} not bit-identical, worst relative difference {worst:.3e}")


import pytest  # noqa: E402

ENGINES = [pytest.param("oracle", id="oracle"), pytest.param("gpu", id="gpu", marks=pytest.mark.gpu)]


def run_engine(engine, points, box, periodic, cutoff, full=True, sorted=False, quantities="ijSdD", algorithm="auto"):
    """Same call against the CPU oracle or the HIP path."""
    if engine == "oracle":
        return oracle.neighbors(points, box, periodic, cutoff, full, sorted, quantities)
    return gpu_neighbors(points, box, periodic, cutoff, full, sorted, quantities, algorithm)


def ulp_close(actual, expected, ulps=4):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    spacing = np.spacing(np.maximum(np.abs(actual), np.abs(expected)))
    return bool(np.all(np.abs(actual - expected) <= ulps * spacing))
