"""Builds the test-only host stand-in of libamem_nccl: the library's own host sources, unchanged, linked
with fake_hip.cpp (the HIP calls on host memory) and kernels_host.cpp (host twins of the kernel launchers)
instead of the HIP runtime and the gfx950 code object. Used by CPU tests that need several real processes
to go through pause and resume; the shipped library in asystem-amem_amd/lib is never built this way."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
CSRC = os.path.join(ROOT, "asystem-amem_amd", "csrc")
PRODUCT_SOURCES = ["capi.cpp", "engine.cpp", "ipc.cpp", "log.cpp", "slab_pool.cpp", "vmm.cpp"]
STANDIN_SOURCES = ["fake_hip.cpp", "kernels_host.cpp"]
LIB_NAME = "libamem_nccl_hoststandin.so"


def build(outdir, sanitize=None):
    """Compile into `outdir`; returns the path of the shared object. Recompiles only what is older than its source."""
    os.makedirs(outdir, exist_ok=True)
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    flags = ["-O1", "-g", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-Wall", "-Wno-unused-result",
             "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(rocm, "include")]
    if sanitize:
        flags += ["-fsanitize=" + sanitize, "-fno-omit-frame-pointer"]
    tag = "." + sanitize.replace(",", "_") if sanitize else ""
    objs, deps = [], [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    deps += [os.path.join(ROOT, "include", f) for f in os.listdir(os.path.join(ROOT, "include"))]
    newest_dep = max(os.path.getmtime(d) for d in deps)
    for d, names in ((CSRC, PRODUCT_SOURCES), (HERE, STANDIN_SOURCES)):
        for name in names:
            src, obj = os.path.join(d, name), os.path.join(outdir, name + tag + ".o")
            if not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src), newest_dep):
                subprocess.run(["g++"] + flags + ["-c", src, "-o", obj], check=True, capture_output=True, text=True)
            objs.append(obj)
    lib = os.path.join(outdir, LIB_NAME.replace(".so", tag + ".so"))
    if not os.path.exists(lib) or os.path.getmtime(lib) < max(os.path.getmtime(o) for o in objs):
        cmd = ["g++", "-shared", "-fPIC"] + (["-fsanitize=" + sanitize] if sanitize else []) + ["-o", lib] + objs + ["-lpthread"]
        subprocess.run(cmd, check=True, capture_output=True, text=True)
    return lib


if __name__ == "__main__":
    import sys
    print(build(sys.argv[1] if len(sys.argv) > 1 else os.path.join(HERE, "_build")))
