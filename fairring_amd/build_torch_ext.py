"""Builds the c10d backend extension fairring_amd/_fairring*.so with g++.

Host-only C++ (no device code): it links against PyTorch-ROCm and against
libfairring_hip.so in the same directory (rpath $ORIGIN).
Run as ``python -m fairring_amd.build_torch_ext``.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "torch_ext")
EXT_SUFFIX = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
OUT = os.path.join(HERE, "_fairring" + EXT_SUFFIX)


def build(verbose=False, jobs=2):
    import torch
    from torch.utils import cpp_extension as ce

    tdir = os.path.dirname(torch.__file__)
    inc = ce.include_paths(device_type="cuda") if "device_type" in ce.include_paths.__code__.co_varnames \
        else ce.include_paths(cuda=True)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    flags = ["-O2", "-fPIC", "-std=c++17", "-Wall", "-Wno-sign-compare", "-Wno-unused-function",
             "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_fairring",
             "-DTORCH_API_INCLUDE_EXTENSION_H",
             "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch.compiled_with_cxx11_abi()),
             "-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(rocm, "include")]
    flags += ["-I" + p for p in inc]
    objs = []
    procs = []
    for name in ("process_group.cc", "bindings.cc"):
        obj = os.path.join(HERE, "csrc", "torch_ext", name[:-3] + ".o")
        cmd = ["g++"] + flags + ["-c", os.path.join(SRC, name), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((name, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                                             text=True)))
        objs.append(obj)
    for name, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            raise RuntimeError("g++ failed on %s:\n%s" % (name, out))
    libdir = os.path.join(tdir, "lib")
    link = ["g++", "-shared", "-o", OUT] + objs + [
        "-L" + libdir, "-L" + HERE, "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + libdir,
        "-lfairring_hip", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
        "-ltorch_python"]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    for o in objs:
        os.remove(o)
    return OUT


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
