"""Build recipe for libvesin.so: hipcc, gfx950 only, no FMA contraction (pair membership depends on it)."""

import os
import subprocess

HERE = os.path.dirname(os.path.realpath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libvesin.so")

SOURCES = ["driver.hip", "api.cpp"]

FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-ffp-contract=off",
    "-fPIC",
    "-shared",
    "-fvisibility=hidden",
    "-DVESIN_SHARED",
    "-DVESIN_EXPORTS",
    # keep the compiler from forming packed fp32 instructions
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def build(verbose=False):
    """Compile the library in-tree (vesin_amd/lib/libvesin.so). Always recompiles."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    command = [hipcc, *FLAGS, "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    command += [os.path.join(CSRC, source) for source in SOURCES]
    command += ["-o", LIB_PATH]
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + result.stdout + result.stderr)
    if verbose:
        print(result.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
