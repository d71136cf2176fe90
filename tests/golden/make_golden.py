"""Regenerate reference_checksums.json: run the COMPILED reference CPU path (oracle/_ref/libvesin_ref.so, built by
oracle/Makefile from the reference's own sources) on every golden case and store order-independent fingerprints.

Needs the reference checkout (for the build); run from the repository root:

    python -m tests.golden.make_golden [--full-size | --large]

Small cases are always regenerated; full-size benchmark configurations are kept from the existing file unless
--full-size is given (they take minutes and several GB of host memory). --large regenerates nothing but the system
of 17,000,000 points (minutes as well: the reference's grid holds at most 100,000 cells).
"""

import json
import os
import sys

import oracle
from tests.golden import systems

OUT = os.path.join(os.path.dirname(os.path.realpath(__file__)), "reference_checksums.json")


def main():
    full_size = "--full-size" in sys.argv
    large = "--large" in sys.argv
    oracle.build()
    if not oracle.have_ref():
        raise SystemExit("oracle/_ref/libvesin_ref.so is missing: the reference checkout is needed to build it")

    golden = {}
    if os.path.exists(OUT):
        with open(OUT) as fd:
            golden = json.load(fd)

    for name, points, box, periodic, cutoff, full in systems.golden_cases(full_size=full_size, large=large):
        result = oracle.ref_neighbors(points, box, periodic, cutoff, full, False, "ijSd" if large else "ijSdD")
        entry = systems.fingerprints(result)
        entry.update(cutoff=cutoff, full=full, n_points=int(len(points)))
        golden[name] = entry
        print(name, entry["n_pairs"], flush=True)
        del result

    if full_size:
        # the batch of 4096 small cells (every replica one call of the reference)
        from vesin_amd import configs

        per_system = []
        for replica in range(4096):
            points, box, periodic, options = configs.config3(replica)
            result = oracle.ref_neighbors(points, box, periodic, options["cutoff"], True, False, "ijSd")
            per_system.append(systems.fingerprints(result))
        golden["config3-batch4096"] = systems.fingerprints_of_systems(per_system)
        print("config3-batch4096", golden["config3-batch4096"]["n_pairs"], flush=True)

    with open(OUT, "w") as fd:
        json.dump(golden, fd, indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
