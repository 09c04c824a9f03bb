"""The host side of the library under ThreadSanitizer and AddressSanitizer (the reference has no
sanitizer runs and leaves its registry unguarded against its own worker thread,
amem_nccl.cpp:303, :342, :365, :391). The library's own sources are rebuilt with the sanitizer on
the host pass only and linked with tests/host_race/registry_hammer.cpp; nothing touches a GPU."""
import os
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "asystem-amem_amd", "csrc")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
SOURCES = ["capi.cpp", "engine.cpp", "ipc.cpp", "log.cpp", "slab_pool.cpp", "vmm.cpp"]


def build(kind, outdir):
    san = ["-Xarch_host", "-fsanitize=" + kind]
    common = ["-O1", "-g", "-std=c++17", "-fPIC", "-D__HIP_PLATFORM_AMD__", "-fno-omit-frame-pointer"]
    objs = []
    for src in SOURCES:
        obj = os.path.join(outdir, src + "." + kind + ".o")
        subprocess.run([HIPCC] + common + san + ["-c", os.path.join(CSRC, src), "-o", obj], check=True,
                       capture_output=True, text=True)
        objs.append(obj)
    kobj = os.path.join(outdir, "kernels." + kind + ".o")
    subprocess.run([HIPCC] + common + san + ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
                   "-packed-fp32-ops", "-c", os.path.join(CSRC, "kernels.hip"), "-o", kobj], check=True,
                   capture_output=True, text=True)
    hobj = os.path.join(outdir, "hammer." + kind + ".o")
    subprocess.run([HIPCC] + common + san + ["-c", os.path.join(ROOT, "tests", "host_race", "registry_hammer.cpp"),
                   "-o", hobj], check=True, capture_output=True, text=True)
    exe = os.path.join(outdir, "hammer_" + kind)
    subprocess.run([HIPCC] + san + ["--offload-arch=gfx950", hobj, kobj] + objs + ["-o", exe, "-lpthread"],
                   check=True, capture_output=True, text=True)
    return exe


@pytest.mark.parametrize("kind", ["thread", "address"])
def test_registry_hammer_under_sanitizer(kind):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc not found")
    outdir = tempfile.mkdtemp(prefix="amem_san_")
    try:
        exe = build(kind, outdir)
        env = dict(os.environ, GMM_LOG="1", GMM_IPC_DIR=outdir, AMEM_GROUPID=str(0x7000 + os.getpid() % 1000),
                   TSAN_OPTIONS="exitcode=66 halt_on_error=0 report_signal_unsafe=0",
                   ASAN_OPTIONS="exitcode=67 detect_leaks=0 protect_shadow_gap=0")
        r = subprocess.run([exe], env=env, capture_output=True, text=True, timeout=180)
        report = (r.stdout + r.stderr)[-6000:]
        assert r.returncode == 0, report
        assert "hammer done: 0 errors" in r.stdout, report
        assert "WARNING: ThreadSanitizer" not in r.stderr and "ERROR: AddressSanitizer" not in r.stderr, report
    finally:
        shutil.rmtree(outdir, ignore_errors=True)


@pytest.fixture(scope="module")
def standin_builds():
    """The host stand-in build of the library per sanitizer, compiled once for the tests below."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "tests", "host_standin"))
    import build_standin
    outdir = tempfile.mkdtemp(prefix="amem_san_standin_")
    built = {}

    def get(kind):
        if kind not in built:
            built[kind] = build_standin.build(outdir, sanitize=kind)
        return built[kind], outdir

    yield get
    shutil.rmtree(outdir, ignore_errors=True)


@pytest.mark.parametrize("kind", ["thread", "address"])
def test_whole_cycles_with_imports_under_sanitizer(kind, standin_builds):
    """The engine's own pause and resume under the sanitizers: the library's sources linked with the host
    stand-in of the HIP calls (tests/host_standin), driven by tests/host_standin/cycle_driver.cpp through six
    cycles with two importing ranks in the process, while three more threads hammer the hook and inspection
    entry points. Every thread the engine starts (copy launcher, unmapper, releaser, three socket services)
    is in the picture."""
    lib, libdir = standin_builds(kind)
    outdir = tempfile.mkdtemp(prefix="amem_san_cycle_")
    try:
        exe = os.path.join(outdir, "cycle_driver_" + kind)
        subprocess.run(["g++", "-O1", "-g", "-std=c++17", "-fsanitize=" + kind, "-fno-omit-frame-pointer",
                        os.path.join(ROOT, "tests", "host_standin", "cycle_driver.cpp"), "-o", exe, lib,
                        "-Wl,-rpath," + libdir, "-lpthread"], check=True, capture_output=True, text=True)
        env = dict(os.environ, AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=outdir, AMEM_GROUPID=str(0x7800 + os.getpid() % 1000),
                   TSAN_OPTIONS="exitcode=66 halt_on_error=0 report_signal_unsafe=0",
                   ASAN_OPTIONS="exitcode=67 detect_leaks=0 protect_shadow_gap=0")
        r = subprocess.run([exe], env=env, capture_output=True, text=True, timeout=600)
        report = (r.stdout + r.stderr)[-8000:]
        assert r.returncode == 0, report
        assert "cycle driver done: 0 errors" in r.stdout, report
        assert "WARNING: ThreadSanitizer" not in r.stderr and "ERROR: AddressSanitizer" not in r.stderr, report
    finally:
        shutil.rmtree(outdir, ignore_errors=True)


def test_allocator_hook_beside_the_engine_under_thread_sanitizer(standin_builds):
    """The RCCL allocator hook's own lock against the registry's: an exporting "proxy thread" in a file named
    librccl_*.so runs beside pause/resume cycles whose tables regrow (the engine then calls hipFree, which
    the hook interposes, while holding the registry's locks). ThreadSanitizer's lock-order checker must
    stay silent: the hook makes no call into the registry or the runtime while it holds its lock."""
    lib, libdir = standin_builds("thread")
    outdir = tempfile.mkdtemp(prefix="amem_san_hook_")
    try:
        rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
        common = ["g++", "-O1", "-g", "-std=c++17", "-fPIC", "-fsanitize=thread", "-fno-omit-frame-pointer",
                  "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(rocm, "include")]
        hook = os.path.join(outdir, "libamem_rccl_hook_tsan.so")
        subprocess.run(common + ["-shared", "-fvisibility=hidden", os.path.join(CSRC, "rccl_hook.cpp"), "-o", hook, lib,
                                 "-Wl,-rpath," + libdir, "-ldl", "-lpthread"], check=True, capture_output=True, text=True)
        rccl = os.path.join(outdir, "librccl_standin.so")
        subprocess.run(common + ["-shared", "-fvisibility=hidden", os.path.join(ROOT, "tests", "rccl_standin", "librccl_standin.cpp"),
                                 "-o", rccl, hook, lib, "-Wl,-rpath," + outdir + ":" + libdir], check=True, capture_output=True, text=True)
        exe = os.path.join(outdir, "hook_race")
        # the hook comes before the stand-in of the runtime in the lookup order, as LD_PRELOAD puts it before libamdhip64
        subprocess.run(common + [os.path.join(ROOT, "tests", "host_race", "hook_race.cpp"), "-o", exe, hook, lib,
                                 "-Wl,-rpath," + outdir + ":" + libdir, "-ldl", "-lpthread"], check=True, capture_output=True, text=True)
        # (the socket service is on: without a slot of its own the hook has nothing to note about an export)
        env = dict(os.environ, AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=outdir, AMEM_HOOK_PLAIN_ALLOC=str(1 << 20),
                   AMEM_GROUPID=str(0x7c00 + os.getpid() % 1000),
                   TSAN_OPTIONS="exitcode=66 halt_on_error=0 report_signal_unsafe=0 detect_deadlocks=1 second_deadlock_stack=1")
        env.pop("AMEM_IPC", None)
        r = subprocess.run([exe, rccl], env=env, capture_output=True, text=True, timeout=600)
        report = (r.stdout + r.stderr)[-8000:]
        assert r.returncode == 0, report
        assert "hook race done: 0 errors" in r.stdout, report
        assert "WARNING: ThreadSanitizer" not in r.stderr, report
    finally:
        shutil.rmtree(outdir, ignore_errors=True)
