"""Build recipe of libamem_nccl.so.1: every source under csrc/ compiled for gfx950 by hipcc.

The library is built in-tree (asystem-amem_amd/lib/) so that it travels with the source
tree; nothing is installed. Run as `python asystem-amem_amd/build.py`.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIBNAME = "libamem_nccl.so.1"
HOOK_NAME = "libamem_rccl_hook.so"
HIP_SOURCES = ["kernels.hip"]
CXX_SOURCES = ["capi.cpp", "engine.cpp", "ipc.cpp", "log.cpp", "slab_pool.cpp", "vmm.cpp"]
# The packed-fp32 target feature is switched off for all device code of this project.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
COMMON = ["-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-result", "-D__HIP_PLATFORM_AMD__"]


def lib_path():
    return os.path.join(LIBDIR, LIBNAME)


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    for src in HIP_SOURCES + CXX_SOURCES:
        obj = os.path.join(objdir, src.rsplit(".", 1)[0] + ".o")
        cmd = [hipcc] + COMMON
        if src.endswith(".hip"):
            cmd += DEVICE_FLAGS
        cmd += ["-c", os.path.join(CSRC, src), "-o", obj]
        _run(cmd, verbose)
        objs.append(obj)
    out = lib_path()
    cmd = [hipcc, "-shared", "-fPIC", "-Wl,-soname," + LIBNAME, "--offload-arch=gfx950", "-o", out] + objs + ["-lpthread"]
    _run(cmd, verbose)
    # the allocator hook for an unpatched RCCL: host code only, placed in front of the HIP runtime
    hook = os.path.join(LIBDIR, HOOK_NAME)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall", "-D__HIP_PLATFORM_AMD__",
           "-I" + os.path.join(rocm, "include"), os.path.join(CSRC, "rccl_hook.cpp"), "-o", hook,
           "-L" + LIBDIR, "-l:" + LIBNAME, "-L" + os.path.join(rocm, "lib"), "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", "-ldl", "-lpthread"]
    _run(cmd, verbose)
    return out


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass does not know the device-only target feature and says so; harmless.
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip() and (verbose or r.returncode):
        print(out, flush=True)
    if r.returncode:
        raise RuntimeError("build failed: " + " ".join(cmd))


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
