"""Builds libfairring_hip.so (kernels + pipeline + C ABI) for gfx950 with hipcc.

Run as ``python -m fairring_amd.build``; hipcc cross-compiles without a GPU.
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libfairring_hip.so")

SOURCES = ["ksum_kernels.hip", "compress_kernels.hip", "static_scratch.hip", "pipeline.cc",
           "schedule_resident.cc", "schedule_gathered.cc", "schedule_host_staged.cc", "capi.cc"]

# Bit-exactness depends on: no FMA contraction, IEEE fp32 division, fp32
# denormals kept, and no packed-fp32 instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-ffp-contract=off",
    "-fno-gpu-flush-denormals-to-zero",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fvisibility=hidden",
    "-pthread",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found; set HIPCC or install ROCm")


def build(extra_flags=(), output=LIB_PATH, verbose=False):
    cmd = [hipcc_path()] + HIPCC_FLAGS + list(extra_flags) + ["-shared", "-o", output]
    for src in SOURCES:
        cmd += ["-x", "hip", os.path.join(CSRC, src)]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the packed-fp32 feature name and says so
    # on every file; that line is harmless and only hides real diagnostics.
    out = "\n".join(l for l in proc.stdout.splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if out.strip() and verbose:
        print(out)
    return output


def build_c_client(output=None):
    """The plain-C client of the ABI used by the tests (tests/host/abi_client.c):
    gcc, linked against the library above and the HIP runtime, no PyTorch."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "host", "abi_client.c")
    output = output or os.path.join(root, "tests", "host", "abi_client")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-std=c99", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(rocm, "include"),
           "-o", output, src, "-L", HERE, "-lfairring_hip", "-L", os.path.join(rocm, "lib"),
           "-lamdhip64", "-Wl,-rpath,$ORIGIN/../../fairring_amd", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("gcc failed:\n" + proc.stdout)
    return output


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
