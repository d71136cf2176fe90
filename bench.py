"""Headline benchmark: neighbor pairs per second of the HIP path on one MI355X.

One "step" is one ``vesin_neighbors`` call (the whole job: cell list, single-pass search into the arrays the list
kept from its first call, final device sync) on the 1,000,000-atom jittered diamond configuration, cutoff 5 A, full
list, unsorted, returning i, j, S, d, with the inputs already resident in HBM. Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME] [--no-cpu-baseline] [--no-other-configs]

The line carries, next to the throughput:
* ``roofline``: the dominant kernel of the workload against the 8 TB/s HBM peak, from its algorithmic bytes (24 B per
  point read + the bytes of every requested row written) and its launch duration measured with HIP events on the
  stream it runs on (``vesin_hip_last_timings``);
* ``ms_median`` / ``ms_min`` / ``gpu_ms_median``: every timed call also timed on its own (wall clock around the
  blocking call) and, in a second series, between HIP events on the GPU (first launch to last kernel end);
* ``near_cutoff_pairs``: rows whose distance lies within 1e-12 x cutoff of the cutoff (the only rows whose membership
  may legitimately differ from the CPU path's);
* ``other_configs``: the same figures for the other configurations of the baseline (the 216-atom sorted case, the
  triclinic sorted half list, the batch of 4096 small cells, the clustered system without and with periodic
  directions) and for four variants of the headline workload (atoms in random order; a box that changes with every
  call; sorted=true; vectors returned as well). They are parity cases (tests/test_gpu_parity.py), timed here for the record, each next to the CPU path;
* ``cpu_baseline``: the reference's CPU path (the compiled reference in oracle/_ref when present, otherwise the C
  restatement in oracle/) timed in the same run on the host cores, in a child process with a time limit: all cores,
  and one thread on a bounded sample of the same workload.

``--config NAME`` makes another configuration the workload of the line (profiling runs use it):
config0, config1 (default), config1_shuffled, config1_sorted, config1_vectors, config2, config3, config3_sorted,
config3_single, config4a, config4b.
"""

import argparse
import hashlib
import json
import os
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.realpath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# HBM bytes moved by ONE launch of the single-pass search kernel on the 1M-atom workload, from rocprofv3 --pmc
# FETCH_SIZE and WRITE_SIZE runs scaled by a device copy of known size (166.7 MB fetched + 3238.2 MB written). The figure belongs to the kernel sources whose
# digest is recorded with it: a run with other sources reports no traffic instead of a stale one.
SEARCH_KERNEL_TRAFFIC = {
    "bytes": 3_405_000_000,
    "profile": "profiles/fused_search_config1_pmc.txt",
    "kernel_sources_sha256": "328c98660c2d928e30d4d9bc2d87d4aae0645b39d27bfb959108c77a834d4a2f",
}
KERNEL_SOURCES = ["device_common.cuh", "geometry.hpp", "cells.cuh", "search.cuh", "fused.cuh"]

CONFIG_NAMES = ["config0", "config1", "config1_shuffled", "config1_sorted", "config1_vectors", "config2", "config3", "config3_sorted", "config3_single", "config4a",
                "config4b"]
DESCRIPTIONS = {
    "config0": "config0: 216 atoms, cutoff 5 A, full, sorted, i j S d",
    "config1": "config1: jittered diamond {replicas}^3 cells = {n_points} atoms, periodic cube, cutoff 5 A, full list, "
               "unsorted, returns i j S d",
    "config1_shuffled": "config1 with its atoms in random order",
    "config1_box_changes": "config1 with a box that differs from the call before on every call",
    "config1_sorted": "config1 with sorted=true (rows in the order of i, j, S)",
    "config1_vectors": "config1 returning i j S d D (vectors beside the distances: 60 bytes per row)",
    "config2": "config2: 100000 atoms, triclinic, cutoff 6 A, half, sorted, i j S d D",
    "config3": "config3: 4096 replicas of 64 atoms, box 7.134 A, cutoff 10 A, full, i j S d, one batched call",
    "config3_sorted": "config3 with sorted=true (every replica's rows in the order of i, j, S)",
    "config3_single": "one replica of config3 in a call of its own: 64 atoms, box 7.134 A, cutoff 10 A, full, i j S d",
    "config4a": "config4a: 500000 clustered atoms, no periodic direction, cutoff 4.5 A, full, i j d",
    "config4b": "config4b: the same atoms, periodic (T, T, F)",
}
BATCH_REPLICAS = 4096


def kernel_sources_digest():
    digest = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "vesin_amd", "csrc", name), "rb") as source:
            digest.update(source.read())
    return digest.hexdigest()


def host_system(name, replicas=50):
    """(points, box, periodic, options) of a single-system configuration, as host arrays."""
    import numpy as np

    from vesin_amd import configs

    if name == "config0":
        return configs.config0()
    if name in ("config1", "config1_box_changes"):
        return configs.config1(replicas)
    if name == "config1_shuffled":
        points, box, periodic, options = configs.config1(replicas)
        return points[np.random.default_rng(1).permutation(len(points))], box, periodic, options
    if name == "config1_sorted":
        points, box, periodic, options = configs.config1(replicas)
        return points, box, periodic, dict(options, sorted=True)
    if name == "config1_vectors":
        points, box, periodic, options = configs.config1(replicas)
        return points, box, periodic, dict(options, quantities="ijSdD")
    if name == "config2":
        return configs.config2()
    if name == "config3_single":
        return configs.config3(0)
    if name == "config4a":
        return configs.config4(periodic=(False, False, False))
    if name == "config4b":
        return configs.config4(periodic=(True, True, False))
    raise ValueError(f"unknown configuration {name}")


class Workload:
    """One configuration resident on the GPU: ``call()`` is one step and returns the outputs."""

    def __init__(self, name, replicas=50):
        import numpy as np
        import torch

        from vesin_amd import NeighborList, configs

        self.name = name
        self.batch = name in ("config3", "config3_sorted")
        if self.batch:
            systems = [configs.config3(r) for r in range(BATCH_REPLICAS)]
            self.options = dict(systems[0][3], sorted=name == "config3_sorted")
            self.first_point = np.cumsum([0] + [len(s[0]) for s in systems])
            self.n_points = int(self.first_point[-1])
            self.points = torch.as_tensor(np.concatenate([s[0] for s in systems]), device="cuda:0")
            self.box = torch.as_tensor(np.stack([s[1] for s in systems]), device="cuda:0")
            self.periodic = True
            self.letters = "P" + self.options["quantities"].replace("i", "").replace("j", "")
        else:
            points, box, periodic, self.options = host_system(name, replicas)
            self.n_points = len(points)
            self.points = torch.as_tensor(points, device="cuda:0")
            self.box = torch.as_tensor(box, device="cuda:0")
            self.periodic = periodic
            self.letters = self.options["quantities"]
            self.boxes = None
            if name == "config1_box_changes":
                # two boxes one rounding step apart, taken in turns: same rows, and never the box of the call before
                other = box.copy()
                other[0, 0] = np.nextafter(other[0, 0], np.inf)
                self.boxes = [self.box, torch.as_tensor(other, device="cuda:0")]
        self.calls = 0
        self.description = DESCRIPTIONS[name].format(replicas=replicas, n_points=self.n_points)
        self.calculator = NeighborList(
            cutoff=self.options["cutoff"], full_list=self.options["full_list"], sorted=self.options["sorted"]
        )

    def call(self):
        self.calls += 1
        if self.batch:
            outputs, _ = self.calculator.compute_batch(
                self.points, self.first_point, self.box, True, self.letters, copy=False
            )
            return outputs
        box = self.box if self.boxes is None else self.boxes[self.calls % 2]
        return self.calculator.compute(self.points, box, self.periodic, self.letters, copy=False)

    def rows_of(self, outputs):
        return int(outputs[0].shape[0])

    def near_cutoff(self, outputs):
        """Rows within 1e-12 x cutoff of the cutoff, counted on the GPU from the distances of the call."""
        if "d" not in self.letters:
            return None
        distances = outputs[self.letters.index("d")]
        cutoff = self.options["cutoff"]
        return int(((distances - cutoff).abs() <= 1e-12 * cutoff).sum().item())


def measure(workload, steps, warmup, torch, np):
    """First call, warm-up, the timed region of exactly `steps` calls, then per-call series (wall clock; HIP events)."""
    from vesin_amd import configs, enable_timings

    start = time.perf_counter()
    outputs = workload.call()
    torch.cuda.synchronize()
    first_call_ms = (time.perf_counter() - start) * 1e3
    n_pairs = workload.rows_of(outputs)
    near_cutoff = workload.near_cutoff(outputs)
    del outputs

    for _ in range(warmup):
        workload.call()
    torch.cuda.synchronize()

    start = time.perf_counter()
    for _ in range(steps):
        workload.call()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - start) / steps * 1e3

    per_call = []
    for _ in range(max(5, min(steps, 20))):
        start = time.perf_counter()
        workload.call()
        torch.cuda.synchronize()
        per_call.append((time.perf_counter() - start) * 1e3)

    stages = None
    gpu_ms = []
    if not workload.batch:
        enable_timings(True)
        sums = {}
        for _ in range(max(5, min(steps, 20))):
            workload.call()
            timings = workload.calculator.timings()
            gpu_ms.append(timings["total"])
            for name, value in timings.items():
                sums[name] = sums.get(name, 0.0) + value
        enable_timings(False)
        stages = {name: value / len(gpu_ms) for name, value in sums.items()}

    algorithmic = configs.algorithmic_bytes(workload.n_points, n_pairs, workload.options["quantities"])
    return {
        "n_pairs": n_pairs,
        "near_cutoff_pairs": near_cutoff,
        "first_call_ms": first_call_ms,
        "ms_per_step": ms_per_step,
        "ms_median": float(np.median(per_call)),
        "ms_min": float(np.min(per_call)),
        "gpu_ms_median": float(np.median(gpu_ms)) if gpu_ms else None,
        "stages": stages,
        "algorithmic_bytes": algorithmic,
    }


def roofline_of(workload, measured, replicas):
    """The dominant kernel of the workload against the HBM peak: the search kernel that writes the rows."""
    stages = measured["stages"]
    algorithmic = measured["algorithmic_bytes"]
    whole_call = algorithmic / (measured["ms_per_step"] * 1e-3) / 1e9
    if stages is None:
        # a batch has no per-stage events: the whole call stands in for its search kernel
        return {
            "bound": "hbm", "kernel": "whole call (fused_search_kernel<batch> and the cell build)",
            "achieved": round(whole_call, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(whole_call / HBM_PEAK_GBS, 4), "traffic": None, "algorithmic_bytes": algorithmic,
            "kernel_ms": round(measured["ms_per_step"], 4), "whole_call_frac": round(whole_call / HBM_PEAK_GBS, 4),
        }
    write_ms = stages["write"]
    achieved = algorithmic / (write_ms * 1e-3) / 1e9
    single_pass = stages["count"] == 0
    if workload.options["sorted"]:
        kernel = "ordered_search_kernel<WRITE> (in-order search, write pass)"
    elif single_pass:
        kernel = "fused_search_kernel (single-pass search)"
    else:
        kernel = "search_kernel<WRITE> (write pass)"
    traffic = None
    traffic_note = "no counter run on record for this workload"
    if workload.name == "config1" and replicas == 50 and single_pass:
        if kernel_sources_digest() == SEARCH_KERNEL_TRAFFIC["kernel_sources_sha256"]:
            traffic = SEARCH_KERNEL_TRAFFIC["bytes"]
            traffic_note = f"from {SEARCH_KERNEL_TRAFFIC['profile']}, measured on these kernel sources"
        else:
            traffic_note = f"the kernel sources changed since {SEARCH_KERNEL_TRAFFIC['profile']} was measured"
    return {
        "bound": "hbm",
        "kernel": kernel,
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        "traffic": traffic,
        "traffic_note": traffic_note,
        "algorithmic_bytes": algorithmic,
        "kernel_ms": round(write_ms, 4),
        "whole_call_frac": round(whole_call / HBM_PEAK_GBS, 4),
    }


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=10)
    parser.add_argument("--replicas", type=int, default=50, help="diamond cells per edge (50 = the 1M-atom workload)")
    parser.add_argument("--config", default="config1", choices=CONFIG_NAMES, help="workload of the line")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-other-configs", action="store_true", help="only the workload of the line (profiling runs)")
    args = parser.parse_args()

    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the neighbor-list path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    workload = Workload(args.config, args.replicas)
    measured = measure(workload, args.steps, args.warmup, torch, np)
    n_pairs = measured["n_pairs"]
    roofline = roofline_of(workload, measured, args.replicas)
    config = {
        "workload": workload.description,
        "n_points": workload.n_points,
        "n_pairs": n_pairs,
        "quantities": workload.options["quantities"],
    }
    del workload

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

    result = {
        "metric": "neighbor_pairs_per_second",
        "value": n_pairs / (measured["ms_per_step"] * 1e-3),
        "unit": "pairs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(measured["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": config,
        "roofline": roofline,
        "ms_median": round(measured["ms_median"], 4),
        "ms_min": round(measured["ms_min"], 4),
        "gpu_ms_median": None if measured["gpu_ms_median"] is None else round(measured["gpu_ms_median"], 4),
        "near_cutoff_pairs": measured["near_cutoff_pairs"],
        "stages_ms": None if measured["stages"] is None else {k: round(v, 4) for k, v in measured["stages"].items()},
        "first_call_ms": round(measured["first_call_ms"], 2),
        "device_copy_GBs": round(copy_gbs, 1),
        "device_fill_GBs": round(fill_gbs, 1),
    }

    if not args.no_other_configs:
        try:
            result["other_configs"] = other_configs(args, torch, np)
        except Exception as error:  # the headline line is printed whatever happens to the extra measurements
            result["other_configs_error"] = f"{type(error).__name__}: {error}"

    if not args.no_cpu_baseline:
        # after the GPU work, so that the host threads of the timed calls never compete with it for cores
        wanted = [args.config] + [entry["name"] for entry in result.get("other_configs", []) if entry["name"] in DESCRIPTIONS
                                  and not entry["name"].startswith("config1_") and entry["name"] != "config3_sorted"]
        collected = CpuBaselines(wanted, args.replicas).collect()
        own = collected.get(args.config)
        if own is not None:
            own["pairs_match_gpu"] = own.get("pairs") == n_pairs if own.get("sample_is_full_workload") else None
            result["cpu_baseline"] = own
        for entry in result.get("other_configs", []):
            if entry["name"] in collected:
                baseline = collected[entry["name"]]
                baseline["pairs_match_gpu"] = (
                    baseline.get("pairs") == entry["n_pairs"] if baseline.get("sample_is_full_workload") else None
                )
                entry["cpu_baseline"] = baseline
                if baseline.get("value"):
                    entry["gpu_over_cpu"] = round(entry["pairs_per_second"] / baseline["value"], 1)

    print(json.dumps(result))


def other_configs(args, torch, np):
    """Steady-state figures of the other configurations: after the list's first call and 5 more, a timed region of 20
    calls, then 20 calls timed one by one (the median of those is `ms_per_call`) and 20 between HIP events."""
    results = []
    names = [name for name in ["config0", "config2", "config3", "config3_sorted", "config3_single", "config4a", "config4b"]
             if name != args.config]
    if args.config == "config1":
        names += ["config1_shuffled", "config1_box_changes", "config1_sorted", "config1_vectors"]
    for name in names:
        workload = Workload(name, args.replicas)
        measured = measure(workload, 20, 5, torch, np)
        ms = measured["ms_median"]
        entry = {
            "name": name,
            "config": workload.description,
            "n_points": workload.n_points,
            "n_pairs": measured["n_pairs"],
            "ms_per_call": round(ms, 4),
            "ms_mean": round(measured["ms_per_step"], 4),
            "ms_min": round(measured["ms_min"], 4),
            "gpu_ms_median": None if measured["gpu_ms_median"] is None else round(measured["gpu_ms_median"], 4),
            "pairs_per_second": measured["n_pairs"] / (ms * 1e-3),
            "near_cutoff_pairs": measured["near_cutoff_pairs"],
            "algorithmic_bytes": measured["algorithmic_bytes"],
            "hbm_frac": round(measured["algorithmic_bytes"] / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "stages_ms": None if measured["stages"] is None else {k: round(v, 4) for k, v in measured["stages"].items()},
        }
        results.append(entry)
        del workload
        torch.cuda.empty_cache()
    return results


# ---- the CPU path, timed beside the GPU

CPU_TIME_LIMIT = 150.0  # seconds a child may take before it is given up on
ONE_THREAD_SAMPLE = {
    # a smaller system of the same kind for the one-thread figure (same density and cutoff: the same work per atom)
    "config1": "jittered diamond 20^3 cells = 64000 atoms",
    "config4a": "100000 atoms of the same 50 blobs",
    "config4b": "100000 atoms of the same 50 blobs",
}


def cpu_child(name, replicas):
    """Runs in a child process: times the CPU path on one configuration and prints a JSON object."""
    import numpy as np

    import oracle
    from vesin_amd import configs

    cores = int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1)
    if oracle.have_ref():
        kind, run = "reference", oracle.ref_neighbors
    else:
        kind, run = "port", oracle.neighbors

    def timed(system, threads):
        points, box, periodic, options = system
        result = run(points, box, periodic, options["cutoff"], options["full_list"], options["sorted"],
                     options["quantities"], n_threads=threads)
        return int(len(result["pairs"])), oracle.last_call_seconds  # the C call alone, not the copy into numpy

    out = {"unit": "pairs/s", "cores": cores, "kind": kind}
    if name == "config3":
        # one cell per replica, which the CPU path searches with one thread: a sample of replicas one after the
        # other, as a caller without a batched entry point would run them
        sample = 256
        pairs, seconds = 0, 0.0
        for r in range(sample):
            p, s = timed(configs.config3(r), 1)
            pairs, seconds = pairs + p, seconds + s
        out.update({
            "value": pairs / seconds, "cores": 1, "pairs": pairs, "sample_is_full_workload": False,
            "seconds_for_the_whole_batch": seconds / sample * BATCH_REPLICAS,
            "sample": f"{sample} of the {BATCH_REPLICAS} replicas, one call each, one after the other ({seconds:.2f} s); "
                      "one cell per replica means one thread per call",
        })
        print(json.dumps(out), flush=True)
        return
    system = host_system(name, replicas)
    pairs, seconds = timed(system, cores)
    out.update({
        "value": pairs / seconds, "pairs": pairs, "sample_is_full_workload": True,
        "sample": f"1 call on the full workload ({len(system[0])} atoms, {pairs} pairs), {seconds:.2f} s inside the library",
    })
    print(json.dumps(out), flush=True)  # a first line in case the one-thread run is cut short
    if name == "config1":
        small = configs.config1(min(20, replicas))
    elif name in ("config4a", "config4b"):
        small = configs.config4(100_000, periodic=system[2])
    else:
        small = system
    pairs_1, seconds_1 = timed(small, 1)
    out["one_thread"] = {
        "value": pairs_1 / seconds_1, "cores": 1,
        "sample": f"{ONE_THREAD_SAMPLE.get(name, 'the full workload')}: {len(small[0])} atoms, {pairs_1} pairs, "
                  f"{seconds_1:.2f} s",
    }
    print(json.dumps(out), flush=True)


class CpuBaselines:
    """A child process timing the CPU path, one configuration after the other, under one time limit."""

    def __init__(self, names, replicas):
        self.names = names
        code = (
            "import sys; sys.path.insert(0, %r); import bench\n"
            "for name in sys.argv[2:]:\n"
            "    print('BEGIN ' + name, flush=True)\n"
            "    bench.cpu_child(name, int(sys.argv[1]))\n"
        ) % ROOT
        environment = dict(os.environ)
        environment["HIP_VISIBLE_DEVICES"] = ""  # nothing in the child touches the GPU
        self.started = time.perf_counter()
        self.process = subprocess.Popen(
            [sys.executable, "-c", code, str(replicas)] + names, stdout=subprocess.PIPE, stderr=subprocess.PIPE,
            text=True, env=environment,
        )

    def collect(self):
        remaining = max(5.0, CPU_TIME_LIMIT - (time.perf_counter() - self.started))
        try:
            stdout, stderr = self.process.communicate(timeout=remaining)
            cut_short = False
        except subprocess.TimeoutExpired:
            self.process.kill()
            stdout, stderr = self.process.communicate()
            cut_short = True
        collected = {}
        current = None
        for line in stdout.splitlines():
            if line.startswith("BEGIN "):
                current = line[6:]
            elif current is not None and line.startswith("{"):
                collected[current] = json.loads(line)
        for name in self.names:
            if name not in collected:
                reason = f"not measured within {CPU_TIME_LIMIT:.0f} s" if cut_short else "failed: " + stderr[-300:]
                collected[name] = {"value": None, "unit": "pairs/s", "sample": reason}
        return collected


if __name__ == "__main__":
    main()
