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

# Arrays indexed with wave-uniform values (the hit columns of the single-pass search: 32 registers) stay in registers
# whatever occupancy a kernel asks for; by default the compiler moves an array larger than a quarter of the kernel's
# register budget to scratch memory. These are options of the compiler's back end, not of its command line: another
# release may not know them, and an unknown one is an error. They are tried on an empty kernel first and left out when
# the compiler refuses them (the kernels are as correct without them, only slower).
TUNING_FLAGS = [
    ["-mllvm", "-amdgpu-promote-alloca-to-vector-vgpr-ratio=1"],
    ["-mllvm", "-amdgpu-promote-alloca-to-vector-max-regs=64"],
]


def _accepted(hipcc, flags):
    import tempfile

    with tempfile.TemporaryDirectory() as scratch:
        source = os.path.join(scratch, "probe.hip")
        with open(source, "w") as out:
            out.write("#include <hip/hip_runtime.h>\n__global__ void probe() {}\n")
        command = [hipcc, "--offload-arch=gfx950", "-c", *flags, source, "-o", os.path.join(scratch, "probe.o")]
        return subprocess.run(command, capture_output=True, text=True).returncode == 0


def extra_flags():
    """What the environment adds to the command line, for developers only: VESIN_EXTRA_FLAGS (measurements with other
    code generation) is read when VESIN_BUILD_DEBUG=1 says that this is meant, so that a variable left over in a
    user's environment does not change the code of a library whose results are compared bit for bit;
    VESIN_HIP_ROCTX=1 compiles the named ranges for profilers in (see TraceRange in driver.hip)."""
    flags = []
    if os.environ.get("VESIN_BUILD_DEBUG") == "1":
        flags += os.environ.get("VESIN_EXTRA_FLAGS", "").split()
    if os.environ.get("VESIN_HIP_ROCTX") == "1":
        flags += ["-DVESIN_HIP_ROCTX", "-L/opt/rocm/lib", "-lrocprofiler-sdk-roctx", "-Wl,-rpath,/opt/rocm/lib"]
    return flags


TORCH_SOURCE = os.path.join(CSRC, "torch", "neighbor_list_class.cpp")
TORCH_LIB_PATH = os.path.join(LIB_DIR, "libvesin_torch.so")


def build_torch(verbose=False):
    """Compile the TorchScript class (vesin_amd/lib/libvesin_torch.so) against the installed PyTorch and against
    libvesin.so, which must have been built before. Host code only: the kernels are all in libvesin.so."""
    import torch
    from torch.utils import cpp_extension

    compiler = os.environ.get("CXX", "g++")
    command = [
        compiler,
        "-O2",
        "-std=c++17",
        "-fPIC",
        "-shared",
        "-fvisibility=hidden",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        "-D__HIP_PLATFORM_AMD__",
        "-DUSE_ROCM",
        "-DVESIN_SHARED",
        "-I" + os.path.join(ROOT, "include"),
        "-I/opt/rocm/include",
    ]
    command += ["-I" + path for path in cpp_extension.include_paths()]
    command += [TORCH_SOURCE, "-o", TORCH_LIB_PATH]
    # libvesin.so is found next to this library; PyTorch's libraries are in the process before this one is loaded
    command += ["-L" + LIB_DIR, "-lvesin", "-Wl,-rpath,$ORIGIN"]
    command += ["-L" + path for path in cpp_extension.library_paths()]
    command += ["-ltorch", "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip"]
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError(f"{compiler} failed:\n" + result.stdout + result.stderr)
    if verbose:
        print(result.stderr)
    return TORCH_LIB_PATH


def build(verbose=False):
    """Compile the library in-tree (vesin_amd/lib/libvesin.so). Always recompiles."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    os.makedirs(LIB_DIR, exist_ok=True)
    flags = list(FLAGS)
    for tuning in TUNING_FLAGS:
        if _accepted(hipcc, tuning):
            flags += tuning
        elif verbose:
            print("left out (the compiler does not know it): " + " ".join(tuning))
    flags += extra_flags()
    command = [hipcc, *flags, "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    command += [os.path.join(CSRC, source) for source in SOURCES]
    command += ["-o", LIB_PATH]
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + result.stdout + result.stderr)
    # what the library was built with, next to it
    with open(LIB_PATH + ".flags", "w") as record:
        record.write(" ".join(flags) + "\n")
    if verbose:
        print(result.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_torch(verbose=True))
