"""The two ways the HIP path produces an unsorted list must agree (``-m gpu``).

A list's first call sizes the output arrays with the two-pass search (count, scan, write). Later calls go through the
single-pass search (sweep with hit columns, chained row offsets, replay) straight into the arrays they kept, and fall
back to the two passes when the rows do not fit or the problem has a shape the single pass does not cover. Every
branch of that decision is driven here and compared with the CPU oracle."""

import os

import numpy as np
import pytest

import oracle
from _helpers import assert_same_list
from golden import systems
from vesin_amd import NeighborList, configs, enable_timings

pytestmark = pytest.mark.gpu

NAMES = {"P": "pairs", "S": "shifts", "d": "distances", "D": "vectors"}


def on_device(points, box):
    import torch

    return (
        torch.as_tensor(np.ascontiguousarray(points, dtype=np.float64), device="cuda:0"),
        torch.as_tensor(np.ascontiguousarray(box, dtype=np.float64), device="cuda:0"),
    )


def call(calculator, points, box, periodic, letters="PSdD"):
    device_points, device_box = on_device(points, box)
    outputs = calculator.compute(device_points, device_box, periodic, letters, copy=True)
    return {NAMES[q]: out.cpu().numpy() for q, out in zip(letters, outputs)}


@pytest.fixture(autouse=True)
def separate_launches(monkeypatch):
    """Small systems with arrays from earlier calls would go through the one launch of tests/test_gpu_small_*.py
    instead; here they are what drives the single-pass search through its branches."""
    monkeypatch.setenv("VESIN_HIP_LAUNCHES", "separate")


@pytest.fixture
def timings():
    enable_timings(True)
    yield
    enable_timings(False)


def used_single_pass(calculator):
    stages = calculator.timings()
    return stages["count"] == 0 and stages["scan"] == 0 and stages["write"] > 0


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_second_call_is_single_pass_and_matches(timings, full):
    points, box, periodic, _ = configs.config1(10)
    expected = oracle.neighbors(points, box, periodic, 5.0, full, False, "ijSdD")
    calculator = NeighborList(cutoff=5.0, full_list=full)
    first = call(calculator, points, box, periodic)
    assert not used_single_pass(calculator)
    assert_same_list(first, expected, what="first call")
    for repeat in range(3):
        again = call(calculator, points, box, periodic)
        assert used_single_pass(calculator)
        assert_same_list(again, expected, what=f"call {repeat + 2}")


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_ordered_rows_are_the_same_on_every_run(timings, monkeypatch, full):
    # VESIN_HIP_ROWS=ordered: rows in work-item order, placed by the chain of workgroup totals
    monkeypatch.setenv("VESIN_HIP_ROWS", "ordered")
    points, box, periodic, _ = configs.config1(12)
    expected = oracle.neighbors(points, box, periodic, 5.0, full, False, "ijSdD")
    calculator = NeighborList(cutoff=5.0, full_list=full)
    call(calculator, points, box, periodic)
    second = call(calculator, points, box, periodic)
    third = call(calculator, points, box, periodic)
    assert used_single_pass(calculator)
    for key in second:
        assert np.array_equal(second[key], third[key]), key
    assert_same_list(second, expected)


def test_ordered_rows_with_crowded_tiles_and_growth(timings, monkeypatch):
    monkeypatch.setenv("VESIN_HIP_ROWS", "ordered")
    rng = np.random.default_rng(22)
    points = np.concatenate([rng.random((3000, 3)) * 30.0, rng.random((3000, 3)) * 2.5 + 10.0])
    box = np.eye(3) * 30.0
    expected = oracle.neighbors(points, box, True, 2.5, True, False, "ijSdD")
    calculator = NeighborList(cutoff=2.5, full_list=True)
    small = configs.config1(4)
    call(calculator, *small[:3])
    assert_same_list(call(calculator, points, box, True), expected, what="grown")
    assert_same_list(call(calculator, points, box, True), expected, what="single pass")
    assert used_single_pass(calculator)


def test_waves_that_give_up_waiting_fall_back_to_the_two_passes(timings, capfd, monkeypatch):
    # the ordered placement waits for the rows of other workgroups, with a bound: VESIN_HIP_CHAIN_SPINS=0 makes every
    # such wait give up at once (all kernels still run to their end), and the call must notice and start over
    monkeypatch.setenv("VESIN_HIP_ROWS", "ordered")
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    points, box, periodic, _ = configs.config1(12)
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    calculator = NeighborList(cutoff=5.0, full_list=True)
    call(calculator, points, box, periodic)
    assert_same_list(call(calculator, points, box, periodic), expected, what="patient")
    assert used_single_pass(calculator)
    capfd.readouterr()
    monkeypatch.setenv("VESIN_HIP_CHAIN_SPINS", "0")
    assert_same_list(call(calculator, points, box, periodic), expected, what="impatient")
    assert not used_single_pass(calculator)
    gave_up = [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass:")]
    assert len(gave_up) == 1 and " timeout 0 " not in gave_up[0], gave_up
    # a launch whose waves gave up is not tried again for 64 calls, however patient its waves would be by now
    monkeypatch.delenv("VESIN_HIP_CHAIN_SPINS")
    for rest in range(64):
        result = call(calculator, points, box, periodic, "P")
        assert not used_single_pass(calculator), rest
    assert_same_list(result, {"pairs": expected["pairs"]}, what="while the chain rests")
    assert not [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass:")]
    assert_same_list(call(calculator, points, box, periodic), expected, what="patient again")
    assert used_single_pass(calculator)


def test_environment_switch_keeps_the_two_passes(timings):
    points, box, periodic, _ = configs.config1(8)
    calculator = NeighborList(cutoff=5.0, full_list=True)
    call(calculator, points, box, periodic)
    os.environ["VESIN_HIP_SEARCH"] = "two-pass"
    try:
        call(calculator, points, box, periodic)
        assert not used_single_pass(calculator)
    finally:
        del os.environ["VESIN_HIP_SEARCH"]
    call(calculator, points, box, periodic)
    assert used_single_pass(calculator)


def test_rows_that_do_not_fit_fall_back(timings):
    # same list, then a system with eight times the rows: the single pass finds the arrays too small, writes nothing
    # out of bounds, and the two passes start over
    small = configs.config1(6)
    large = configs.config1(12)
    calculator = NeighborList(cutoff=5.0, full_list=True)
    call(calculator, *small[:3])
    grown = call(calculator, *large[:3])
    assert not used_single_pass(calculator)
    assert_same_list(grown, oracle.neighbors(*large[:3], 5.0, True, False, "ijSdD"), what="grown")
    # and back: the small system now fits with room to spare
    shrunk = call(calculator, *small[:3])
    assert used_single_pass(calculator)
    assert_same_list(shrunk, oracle.neighbors(*small[:3], 5.0, True, False, "ijSdD"), what="shrunk")


def test_crowded_tiles_are_left_to_the_write_pass(timings, capfd, monkeypatch):
    # a dense blob inside a sparse gas: tiles of the blob see more candidates (2048) than the single pass keeps
    # columns for; they are counted and placed by it and written by the write pass
    rng = np.random.default_rng(21)
    gas = rng.random((4000, 3)) * 40.0
    blob = rng.random((4000, 3)) * 3.0 + 18.0
    points = np.concatenate([gas, blob])
    box = np.eye(3) * 40.0
    expected = oracle.neighbors(points, box, True, 2.5, True, False, "ijSdD")
    calculator = NeighborList(cutoff=2.5, full_list=True)
    first = call(calculator, points, box, True)
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    capfd.readouterr()
    # (the list's first call with arrays tries the cell build with 32 slots per cell, which the blob overflows: the
    # call starts over with the packed build and the two passes, and the list stays away from that build)
    learning = call(calculator, points, box, True)
    report = [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass:")]
    assert report and "one-pass cell build, crowded" in report[-1] and "crowded 0," not in report[-1], report
    second = call(calculator, points, box, True)
    report = [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass:")]
    assert report and " deferred 0 " not in report[-1] and "packed cells" in report[-1], report
    assert used_single_pass(calculator)
    assert_same_list(first, expected, what="two-pass")
    assert_same_list(learning, expected, what="after an overflowing cell")
    assert_same_list(second, expected, what="single pass with deferred tiles")


def test_stencil_corners_are_dropped_and_the_switch_keeps_them(capfd, monkeypatch):
    # 64 atoms in a 7.134 A cube, cutoff 10 A: 5^3 = 125 images, of which those with two components of +-2 are more
    # than sqrt(2) * 7.134 A > 10 A away from the box: 81 stay (27 without a 2, 54 with one). A sheared box of the
    # same volume drops fewer. VESIN_HIP_STENCIL=full keeps all of them; the rows are the same either way.
    points, box, periodic, options = configs.config3(5)
    sheared = box.copy()
    sheared[1, 0] = 2.0
    sheared[2, 1] = -1.5
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    for matrix, kept in ((box, "81 of 125"), (sheared, None)):
        expected = oracle.neighbors(points, matrix, periodic, options["cutoff"], True, False, "ijSdD")
        for switch in (None, "full"):
            if switch is None:
                monkeypatch.delenv("VESIN_HIP_STENCIL", raising=False)
            else:
                monkeypatch.setenv("VESIN_HIP_STENCIL", switch)
            calculator = NeighborList(cutoff=options["cutoff"], full_list=True)
            call(calculator, points, matrix, periodic)
            capfd.readouterr()
            again = call(calculator, points, matrix, periodic)
            report = [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass:")]
            assert report, "the second call of a list goes through the single-pass search"
            stencil = report[-1].split("stencil ")[1].rstrip(")")
            if switch == "full":
                assert stencil == "125 of 125", report[-1]
            elif kept is not None:
                assert stencil == kept, report[-1]
            else:
                n_kept = int(stencil.split(" of ")[0])
                assert 81 <= n_kept < 125, report[-1]
            assert_same_list(again, expected, what=f"stencil {stencil}")


def test_shifts_beyond_the_packing_fall_back():
    # points thousands of boxes away: their shifts do not fit the 10-bit fields of the single pass
    rng = np.random.default_rng(6)
    points, box, periodic = systems.read_xyz("carbon")
    points = points + rng.integers(-3000, 3000, size=(len(points), 3)).astype(float) @ box
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    calculator = NeighborList(cutoff=5.0, full_list=True)
    for repeat in range(3):
        assert_same_list(call(calculator, points, box, periodic), expected, what=f"call {repeat + 1}")


@pytest.mark.parametrize("letters", ["P", "PS", "Pd", "PD", "PSdD"])
def test_single_pass_with_every_output(letters):
    points, box, periodic = systems.read_xyz("carbon")
    quantities = "ij" + letters[1:]
    expected = oracle.neighbors(points, box, periodic, 4.0, True, False, "ijSdD")
    calculator = NeighborList(cutoff=4.0, full_list=True)
    call(calculator, points, box, periodic, letters)
    again = call(calculator, points, box, periodic, letters)
    if "S" in letters:
        assert_same_list(again, {k: v for k, v in expected.items() if k in again}, what=quantities)
    else:
        # without shifts the images of one pair have no order of their own: compare as multisets
        assert len(again["pairs"]) == len(expected["pairs"])
        keys = ["pairs"] + [k for k in ("distances", "vectors") if k in again]
        for key in keys:
            a = np.sort(again[key].reshape(len(again["pairs"]), -1), axis=0)
            b = np.sort(expected[key].reshape(len(expected["pairs"]), -1), axis=0)
            assert np.array_equal(a, b), key


def test_wrapped_tiles_in_the_single_pass(timings):
    # half of the points sit one or two boxes away: their tiles take the per-point shift path of both searches
    rng = np.random.default_rng(9)
    points, box, periodic, _ = configs.config1(6)
    points = points + rng.integers(-2, 3, size=(len(points), 3)).astype(float) @ box
    expected = oracle.neighbors(points, box, periodic, 5.0, False, False, "ijSdD")
    calculator = NeighborList(cutoff=5.0, full_list=False)
    call(calculator, points, box, periodic)
    again = call(calculator, points, box, periodic)
    assert used_single_pass(calculator)
    assert_same_list(again, expected)


def test_a_box_that_changes_between_calls():
    # later calls of a list start with the box of the call before and check it when they synchronise: a changed box
    # must be noticed and the call redone, whatever the sequence
    rng = np.random.default_rng(12)
    points, box, periodic, _ = configs.config1(6)
    boxes = [box, box, box, box * 1.03, box * 1.03, box, box * 0.99, box * 0.99, box * 0.99]
    calculator = NeighborList(cutoff=5.0, full_list=True)
    for step, current in enumerate(boxes):
        moved = points * (current[0, 0] / box[0, 0]) + rng.normal(scale=0.01, size=points.shape)
        expected = oracle.neighbors(moved, current, periodic, 5.0, True, False, "ijSdD")
        assert_same_list(call(calculator, moved, current, periodic), expected, what=f"step {step}")
    # the flags are part of what is remembered
    open_box = oracle.neighbors(points, box, [True, False, True], 5.0, True, False, "ijSdD")
    assert_same_list(call(calculator, points, box, [True, False, True]), open_box, what="periodicity changed")
    assert_same_list(call(calculator, points, box, [True, False, True]), open_box, what="periodicity kept")


def test_a_box_that_changes_with_every_call():
    # a trajectory at constant pressure, or structures of a dataset one after the other: every guess is wrong, the list
    # guesses less and less often, and every call still returns the rows of its own box
    rng = np.random.default_rng(13)
    points, box, periodic, _ = configs.config1(4)
    calculator = NeighborList(cutoff=5.0, full_list=True)
    for step in range(75):
        scale = 1.0 + 0.002 * step
        current = box * scale
        moved = points * scale
        result = call(calculator, moved, current, periodic)
        if step % 8 == 0 or step in (33, 34, 66, 67):
            expected = oracle.neighbors(moved, current, periodic, 5.0, True, False, "ijSdD")
            assert_same_list(result, expected, what=f"step {step}")
    # another system through the same list (other number of points, much larger box): never searched with the small box
    other = configs.config1(7)
    expected = oracle.neighbors(*other[:3], 5.0, True, False, "ijSdD")
    assert_same_list(call(calculator, *other[:3]), expected, what="another system")
    del rng


def test_a_box_that_becomes_singular():
    points, box, periodic, _ = configs.config1(4)
    calculator = NeighborList(cutoff=5.0, full_list=True)
    for _ in range(3):
        call(calculator, points, box, periodic)
    flat = box.copy()
    flat[2] = flat[1]
    with pytest.raises(RuntimeError, match="the box matrix is not invertible"):
        call(calculator, points, flat, periodic)
    # and the list is still usable
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    assert_same_list(call(calculator, points, box, periodic), expected)


def test_stencils_larger_than_the_single_pass_tables(timings):
    # cutoff almost three box lengths: 7^3 images, more stencil entries than the single pass keeps in LDS; every
    # call of the list falls back to the two passes (which walk the stencil in batches)
    rng = np.random.default_rng(41)
    box = np.array([[3.1, 0.0, 0.0], [0.4, 2.9, 0.0], [-0.3, 0.5, 3.3]])
    points = rng.random((40, 3)) @ box
    expected = oracle.neighbors(points, box, True, 8.0, True, False, "ijSdD")
    calculator = NeighborList(cutoff=8.0, full_list=True)
    for repeat in range(3):
        assert_same_list(call(calculator, points, box, True), expected, what=f"call {repeat + 1}")
        assert not used_single_pass(calculator)


def test_the_single_pass_is_tried_again_after_its_rest(timings):
    """A list that met a system the single pass does not cover leaves it alone for 64 calls, whatever comes, and
    takes it up again afterwards: rows right at every step."""
    rng = np.random.default_rng(42)
    small_box = np.array([[3.1, 0.0, 0.0], [0.4, 2.9, 0.0], [-0.3, 0.5, 3.3]])
    awkward = rng.random((40, 3)) @ small_box  # cutoff 8: 7^3 images, beyond the single pass's tables
    points, box, periodic, _ = configs.config1(4)
    expected = oracle.neighbors(points, box, periodic, 8.0, True, False, "ijSdD")
    calculator = NeighborList(cutoff=8.0, full_list=True)
    call(calculator, points, box, periodic)
    call(calculator, points, box, periodic)
    assert used_single_pass(calculator)
    for _ in range(2):  # the first of these tries the single pass and finds the stencil too large
        call(calculator, awkward, small_box, True)
        assert not used_single_pass(calculator)
    used = []
    for step in range(70):
        result = call(calculator, points, box, periodic)
        used.append(used_single_pass(calculator))
        if step in (0, 30, 62, 63, 64, 69):
            assert_same_list(result, expected, what=f"step {step}")
    assert not any(used[:63]) and all(used[63:]), used


def _single_pass_reports(capfd):
    return [line for line in capfd.readouterr().err.splitlines() if line.startswith("single pass:")]


@pytest.mark.parametrize("full", [True, False], ids=["full", "half"])
def test_one_pass_cell_build(full, capfd, monkeypatch):
    """Large systems with cells of ordinary occupation (here 64,000 atoms, 23 per cell) build their cells in one
    pass, every cell owning 32 slots; VESIN_HIP_CELLS=packed keeps the counting sort. Same rows either way, also
    with points that were moved out of the box by whole box vectors."""
    points, box, periodic, _ = configs.config1(20)
    rng = np.random.default_rng(3)
    points = points + rng.integers(-1, 2, size=points.shape) @ box * (rng.random((len(points), 1)) < 0.05)
    expected = oracle.neighbors(points, box, periodic, 5.0, full, False, "ijSdD")
    calculator = NeighborList(cutoff=5.0, full_list=full)
    call(calculator, points, box, periodic)
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    capfd.readouterr()
    assert_same_list(call(calculator, points, box, periodic), expected, what="one-pass cell build")
    reports = _single_pass_reports(capfd)
    assert reports and "one-pass cell build, crowded 0," in reports[-1], reports
    monkeypatch.setenv("VESIN_HIP_CELLS", "packed")
    assert_same_list(call(calculator, points, box, periodic), expected, what="packed cells")
    reports = _single_pass_reports(capfd)
    assert reports and "packed cells" in reports[-1], reports


def test_one_pass_cell_build_with_a_cell_too_full(capfd, monkeypatch):
    """One cell holds more points than it has slots: the call's result comes from the packed layout and the two
    passes, and the list stays away from the one-pass build afterwards."""
    points, box, periodic, _ = configs.config1(20)
    rng = np.random.default_rng(4)
    points[:40] = points[0] + 0.3 * rng.random((40, 3))
    expected = oracle.neighbors(points, box, periodic, 5.0, True, False, "ijSdD")
    calculator = NeighborList(cutoff=5.0, full_list=True)
    call(calculator, points, box, periodic)
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    capfd.readouterr()
    assert_same_list(call(calculator, points, box, periodic), expected, what="after the overflow")
    reports = _single_pass_reports(capfd)
    assert reports and "one-pass cell build, crowded" in reports[-1] and "crowded 0," not in reports[-1], reports
    assert_same_list(call(calculator, points, box, periodic), expected, what="next call")
    reports = _single_pass_reports(capfd)
    assert reports and "packed cells" in reports[-1], reports


@pytest.mark.parametrize("n_points", [1, 31, 33, 700, 2048, 2049])
@pytest.mark.parametrize("periodic", [(True, True, True), (True, False, True)])
def test_cell_build_of_small_systems(n_points, periodic, monkeypatch):
    """Up to 2048 points the packed cell build is one launch of one workgroup (above, and with
    VESIN_HIP_CELLS=packed, the four launches): same rows, first call and reused list, points outside the box
    included."""
    rng = np.random.default_rng(n_points)
    box = np.array([[13.0, 0.0, 0.0], [1.5, 12.0, 0.0], [-1.0, 0.8, 14.0]])
    points = rng.random((n_points, 3)) @ box + (rng.integers(-1, 2, size=(n_points, 3)) * (rng.random((n_points, 1)) < 0.2)) @ box
    expected = oracle.neighbors(points, box, list(periodic), 3.0, True, False, "ijSdD")
    for mode in ("default", "packed"):
        if mode == "packed":
            monkeypatch.setenv("VESIN_HIP_CELLS", "packed")
        else:
            monkeypatch.delenv("VESIN_HIP_CELLS", raising=False)
        calculator = NeighborList(cutoff=3.0, full_list=True)
        for repeat in range(3):
            assert_same_list(call(calculator, points, box, list(periodic)), expected, what=f"{mode} call {repeat}")


def test_the_one_pass_cell_build_is_tried_again_after_its_rest(capfd, monkeypatch):
    """A list that met a cell of more than 32 points stays with the packed cell build for 1024 calls that would have
    taken the one-pass build, and takes that up again afterwards: rows right at every step looked at."""
    monkeypatch.setenv("VESIN_HIP_DEBUG", "1")
    rng = np.random.default_rng(43)
    box = np.eye(3) * 40.0
    gas = rng.random((3000, 3)) * 40.0
    with_blob = gas.copy()
    with_blob[:300] = rng.random((300, 3)) * 2.0 + 11.0  # 300 points in one or two cells
    expected = oracle.neighbors(gas, box, True, 4.0, True, False, "ijSdD")
    expected_blob = oracle.neighbors(with_blob, box, True, 4.0, True, False, "ijSdD")
    calculator = NeighborList(cutoff=4.0, full_list=True)

    def build_of(result_expected=None, points=gas):
        capfd.readouterr()
        result = call(calculator, points, box, True)
        lines = _single_pass_reports(capfd)
        if result_expected is not None:
            assert_same_list(result, result_expected)
        assert len(lines) == 1, lines
        return "one-pass" if "one-pass cell build" in lines[0] else "packed"

    call(calculator, gas, box, True)  # sizes the arrays
    assert build_of(expected) == "one-pass"
    assert build_of(expected_blob, with_blob) == "one-pass"  # tried, a cell overflowed, the call started over
    builds = [build_of(expected if step in (0, 1, 500, 1023, 1024, 1029) else None) for step in range(1030)]
    assert builds[:1024] == ["packed"] * 1024 and builds[1024:] == ["one-pass"] * 6, (builds[:3], builds[1020:])
