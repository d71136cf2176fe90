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
    names = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}
    device_points = torch.as_tensor(np.ascontiguousarray(points, dtype=np.float64), device="cuda:0")
    device_box = torch.as_tensor(np.ascontiguousarray(box, dtype=np.float64), device="cuda:0")

    # The first call of a list sizes the outputs with the two-pass search; later calls of an unsorted list go
    # through the single-pass search into the arrays they kept. Both must give the same rows.
    results = []
    for _ in range(2):
        outputs = calculator.compute(device_points, device_box, periodic, letters, copy=True)
        results.append({names[q]: out.cpu().numpy() for q, out in zip(letters, outputs)})
    del calculator
    first, second = results
    if sorted:
        for key in first:
            assert np.array_equal(first[key], second[key]), f"second call differs from the first: {key}"
    elif len(first["pairs"]) > 2_000_000:
        # too many rows to sort twice within a test's time: order-independent fingerprints of the rows
        from golden import systems

        assert systems.fingerprints(first) == systems.fingerprints(second), "second call differs from the first"
    else:
        a = _fully_ordered(first)
        b = _fully_ordered(second)
        for key in a:
            assert a[key].shape == b[key].shape, (
                f"second call has {b[key].shape[0]} rows of {key}, the first had {a[key].shape[0]}"
            )
            assert np.array_equal(a[key], b[key]), f"second call differs from the first: {key}"
    return second


def _fully_ordered(result):
    """Rows sorted by every column present, so that two row orders of one list compare equal even when the shifts
    that tell the images of a pair apart were not requested."""
    n = len(result["pairs"])
    columns = []
    for key in ("vectors", "distances", "shifts", "pairs"):
        if key in result:
            block = result[key].reshape(n, -1)
            columns += [block[:, c] for c in range(block.shape[1] - 1, -1, -1)]
    order = np.lexsort(columns) if n else np.arange(0)
    return {key: value[order] for key, value in result.items()}


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
