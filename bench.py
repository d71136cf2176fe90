"""Headline benchmark: neighbor pairs per second of the HIP path on one MI355X.

One "step" is one ``vesin_neighbors`` call (the whole job: cell list, single-pass search into the arrays the list
kept from its first call, final device sync) on the 1,000,000-atom jittered diamond configuration, cutoff 5 A, full list, unsorted, returning i, j, S, d,
with the inputs already resident in HBM. Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-other-configs]

The line carries, next to the throughput:
* ``roofline``: the dominant kernel (the single-pass search, fused_search_kernel) against the 8 TB/s HBM peak, from its
  algorithmic bytes (24 B per point read + 36 B per pair written) and its launch duration measured with HIP events
  on the stream it runs on (``vesin_hip_last_timings``);
* ``other_configs``: steady-state time per call, pairs per second and fraction of the HBM peak (algorithmic bytes over
  the whole call) of the other configurations of the baseline, measured after the timed region: the 216-atom sorted
  case, the triclinic sorted half list, the batch of 4096 small cells, the clustered system without and with periodic
  directions. They are parity cases (tests/test_gpu_parity.py), timed here for the record;
* ``cpu_baseline``: the reference's CPU path (the compiled reference in oracle/_ref when present, otherwise the C
  restatement in oracle/) timed in the same run on the host cores.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.realpath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes moved by ONE launch of the single-pass search kernel on this workload, from rocprofv3 --pmc FETCH_SIZE
# and WRITE_SIZE runs scaled by a device copy of known size (profiles/fused_search_config1_pmc.txt):
# 171.1 MB fetched + 3214.8 MB written. Only meaningful for the default 1M-atom workload.
SEARCH_KERNEL_TRAFFIC_BYTES = 3_385_800_000


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=10)
    parser.add_argument("--replicas", type=int, default=50, help="diamond cells per edge (50 = the 1M-atom workload)")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-other-configs", action="store_true", help="only the headline workload (profiling runs)")
    args = parser.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the neighbor-list path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from vesin_amd import NeighborList, configs, enable_timings

    points, box, periodic, options = configs.config1(args.replicas)
    n_points = len(points)
    quantities = options["quantities"]
    d_points = torch.as_tensor(points, device="cuda:0")
    d_box = torch.as_tensor(box, device="cuda:0")

    calculator = NeighborList(cutoff=options["cutoff"], full_list=options["full_list"], sorted=options["sorted"])

    first_start = time.perf_counter()
    outputs = calculator.compute(d_points, d_box, True, quantities, copy=False)
    torch.cuda.synchronize()
    first_call_ms = (time.perf_counter() - first_start) * 1e3
    n_pairs = int(outputs[0].shape[0])

    for _ in range(args.warmup):
        calculator.compute(d_points, d_box, True, quantities, copy=False)
    torch.cuda.synchronize()

    # ---- the timed region: exactly K calls
    start = time.perf_counter()
    for _ in range(args.steps):
        calculator.compute(d_points, d_box, True, quantities, copy=False)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    ms_per_step = elapsed / args.steps * 1e3

    # ---- per-kernel durations with HIP events, same calls, outside the timed region
    enable_timings(True)
    stage_sums = {}
    timed_calls = max(5, min(args.steps, 20))
    for _ in range(timed_calls):
        calculator.compute(d_points, d_box, True, quantities, copy=False)
        for name, value in calculator.timings().items():
            stage_sums[name] = stage_sums.get(name, 0.0) + value
    enable_timings(False)
    stages = {name: value / timed_calls for name, value in stage_sums.items()}

    # ---- what this GPU's HBM delivers to plain streaming kernels in the same run (context for the 8 TB/s peak)
    scratch = torch.empty(1 << 28, dtype=torch.float64, device="cuda:0")  # 2 GiB
    other = torch.empty_like(scratch)
    for _ in range(3):
        other.copy_(scratch)
        scratch.fill_(1.0)
    torch.cuda.synchronize()
    begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    begin.record()
    for _ in range(10):
        other.copy_(scratch)
    end.record()
    torch.cuda.synchronize()
    copy_gbs = 10 * 2 * scratch.numel() * 8 / (begin.elapsed_time(end) * 1e-3) / 1e9
    begin.record()
    for _ in range(10):
        scratch.fill_(2.0)
    end.record()
    torch.cuda.synchronize()
    fill_gbs = 10 * scratch.numel() * 8 / (begin.elapsed_time(end) * 1e-3) / 1e9
    del scratch, other

    algorithmic_bytes = configs.algorithmic_bytes(n_points, n_pairs, quantities)
    write_ms = stages["write"]
    achieved = algorithmic_bytes / (write_ms * 1e-3) / 1e9
    roofline = {
        "bound": "hbm",
        "kernel": "fused_search_kernel (single-pass search)" if stages["count"] == 0 else "search_kernel<WRITE> (write pass)",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": SEARCH_KERNEL_TRAFFIC_BYTES if (args.replicas == 50 and stages["count"] == 0) else None,
        "algorithmic_bytes": algorithmic_bytes,
        "kernel_ms": round(write_ms, 4),
        "whole_call_frac": round(algorithmic_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
    }

    result = {
        "metric": "neighbor_pairs_per_second",
        "value": n_pairs / (ms_per_step * 1e-3),
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {
            "workload": f"config1: jittered diamond {args.replicas}^3 cells = {n_points} atoms, periodic cube, "
                        "cutoff 5 A, full list, unsorted, returns i j S d",
            "n_points": n_points,
            "n_pairs": n_pairs,
            "quantities": quantities,
        },
        "roofline": roofline,
        "stages_ms": {name: round(value, 4) for name, value in stages.items()},
        "first_call_ms": round(first_call_ms, 2),
        "device_copy_GBs": round(copy_gbs, 1),
        "device_fill_GBs": round(fill_gbs, 1),
    }

    if not args.no_other_configs:
        del outputs, calculator, d_points
        try:
            result["other_configs"] = other_configs(np, torch)
        except Exception as error:  # the headline line is printed whatever happens to the extra measurements
            result["other_configs_error"] = f"{type(error).__name__}: {error}"

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(points, box, periodic, options, n_pairs, np)

    print(json.dumps(result))


def other_configs(np, torch):
    """Steady-state figures of the baseline's other configurations: wall clock around the blocking call, inputs in
    HBM, median of 10 calls after the list's first call and 3 more."""
    from vesin_amd import NeighborList, configs

    def timed(call):
        rows = call()
        for _ in range(3):
            call()
        torch.cuda.synchronize()
        times = []
        for _ in range(10):
            start = time.perf_counter()
            call()
            torch.cuda.synchronize()
            times.append((time.perf_counter() - start) * 1e3)
        return rows, float(np.median(times))

    def entry(name, n_points, rows, ms, quantities):
        algorithmic = configs.algorithmic_bytes(n_points, rows, quantities)
        return {
            "config": name,
            "n_points": n_points,
            "n_pairs": rows,
            "ms_per_call": round(ms, 4),
            "pairs_per_second": rows / (ms * 1e-3),
            "algorithmic_bytes": algorithmic,
            "hbm_frac": round(algorithmic / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        }

    results = []
    single = [
        ("config0: 216 atoms, cutoff 5 A, full, sorted, i j S d", configs.config0()),
        ("config2: 100000 atoms, triclinic, cutoff 6 A, half, sorted, i j S d D", configs.config2()),
        ("config4a: 500000 clustered atoms, no periodic direction, cutoff 4.5 A, full, i j d",
         configs.config4(periodic=(False, False, False))),
        ("config4b: the same atoms, periodic (T, T, F)", configs.config4(periodic=(True, True, False))),
    ]
    for name, (points, box, periodic, options) in single:
        d_points = torch.as_tensor(points, device="cuda:0")
        d_box = torch.as_tensor(box, device="cuda:0")
        calculator = NeighborList(cutoff=options["cutoff"], full_list=options["full_list"], sorted=options["sorted"])
        quantities = options["quantities"]
        rows, ms = timed(lambda: int(calculator.compute(d_points, d_box, periodic, quantities, copy=False)[0].shape[0]))
        results.append(entry(name, len(points), rows, ms, quantities))
        del calculator, d_points

    replicas = [configs.config3(r) for r in range(4096)]
    options = replicas[0][3]
    first_point = np.cumsum([0] + [len(r[0]) for r in replicas])
    d_points = torch.as_tensor(np.concatenate([r[0] for r in replicas]), device="cuda:0")
    d_boxes = torch.as_tensor(np.stack([r[1] for r in replicas]), device="cuda:0")
    calculator = NeighborList(cutoff=options["cutoff"], full_list=options["full_list"])
    letters = "P" + options["quantities"].replace("i", "").replace("j", "")
    rows, ms = timed(
        lambda: int(calculator.compute_batch(d_points, first_point, d_boxes, True, letters, copy=False)[0][0].shape[0])
    )
    results.insert(2, entry(
        "config3: 4096 replicas of 64 atoms, box 7.134 A, cutoff 10 A, full, i j S d, one batched call",
        int(first_point[-1]), rows, ms, options["quantities"],
    ))
    return results


def cpu_baseline(points, box, periodic, options, n_pairs, np):
    """The reference's CPU path on the host cores, one call on the same arrays (a few seconds)."""
    import oracle

    cores = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1)
    if oracle.have_ref():
        kind = "reference"
        run = oracle.ref_neighbors
    else:
        kind = "port"
        run = oracle.neighbors
    result = run(points, box, periodic, options["cutoff"], options["full_list"], options["sorted"],
                 options["quantities"], n_threads=cores)
    seconds = oracle.last_call_seconds  # the C call alone, not the copy of its result into numpy
    pairs = int(len(result["pairs"]))
    return {
        "value": pairs / seconds,
        "unit": "pairs/s",
        "cores": cores,
        "kind": kind,
        "sample": f"1 call on the full workload ({len(points)} atoms, {pairs} pairs), {seconds:.2f} s inside the library",
        "pairs_match_gpu": pairs == n_pairs,
    }


if __name__ == "__main__":
    main()
