"""The allocator hook for an unpatched RCCL (libamem_rccl_hook.so): VMM allocations made by a
library whose file name starts with "librccl" appear in the registry by themselves, survive a
pause/resume cycle bit-exactly at the same addresses, and disappear from the registry when that
library frees them. The caller here is a stand-in that allocates the way NCCL's ncclCuMemAlloc
does; the RCCL build of this ROCm release keeps its own buffers in plain allocations."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r'''
import ctypes as C, os, sys
import numpy as np
root, standin = sys.argv[1], sys.argv[2]
sys.path.insert(0, root)
libdir = os.path.join(root, "asystem-amem_amd", "lib")
# order matters: the hook must precede the HIP runtime in the global symbol scope
hook = C.CDLL(os.path.join(libdir, "libamem_rccl_hook.so"), mode=C.RTLD_GLOBAL)
from asystem_amem_amd import binding as B, harness as H
lib = B.load()
rccl = C.CDLL(standin, mode=C.RTLD_GLOBAL)
rccl.standin_cumem_alloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
rccl.standin_cumem_free.argtypes = [C.c_void_p]
hook.amem_rccl_hook_registered.restype = C.c_int64
MiB = 1 << 20
rng = np.random.default_rng(31)
bufs = []
for k, n in enumerate([4 * MiB, 16 * MiB, 2 * MiB]):
    p = C.c_void_p()
    assert rccl.standin_cumem_alloc(C.byref(p), n) == 0
    data = rng.integers(0, 256, n, dtype=np.uint8)
    data[n // 4: n // 2] = 0
    assert lib.amem_copy_to_device(p.value, data.ctypes.data, n) == 0
    bufs.append((p.value, n, data))
# the application's own VMM allocation is none of the hook's business
va, h, asz = C.c_uint64(), C.c_uint64(), C.c_uint64()
assert lib.amem_vmm_alloc(2 * MiB, 0, C.byref(va), C.byref(h), C.byref(asz)) == 0
assert lib.amem_region_count(0) == 3 and hook.amem_rccl_hook_registered() == 3
tab = H.region_table(lib, 0)
assert sorted(tab) == sorted(b[0] for b in bufs)
for p, n, _ in bufs:
    assert tab[p]["alloc_sz"] == n and tab[p]["type"] == B.TYPE_LOCAL and tab[p]["state"] == B.STATE_ALLOC and tab[p]["handle"] != 0
lib.ncclPause(None); lib.ncclResume(None)                      # warm cycle
free0 = H.mem_free(lib)
assert lib.ncclPause(None) == 0 and lib.amem_check_paused(0) == 1
assert H.mem_free(lib) - free0 >= 22 * MiB - 4 * MiB
assert lib.ncclResume(None) == 0 and lib.amem_check_paused(0) == 0
for p, n, data in bufs:
    out = np.empty(n, dtype=np.uint8)
    assert lib.amem_copy_from_device(out.ctypes.data, p, n) == 0
    assert np.array_equal(out, data)
# the resumed handle is not the one the allocator created; freeing by address still works
for p, n, _ in bufs[:2]:
    assert rccl.standin_cumem_free(p) == 0
assert lib.amem_region_count(0) == 1 and hook.amem_rccl_hook_registered() == 1
assert lib.ncclPause(None) == 0 and lib.ncclResume(None) == 0
out = np.empty(bufs[2][1], dtype=np.uint8)
assert lib.amem_copy_from_device(out.ctypes.data, bufs[2][0], out.nbytes) == 0 and np.array_equal(out, bufs[2][2])
assert rccl.standin_cumem_free(bufs[2][0]) == 0
assert lib.amem_region_count(0) == 0 and lib.amem_handle_count(0) == 0
assert lib.amem_vmm_free(va.value, asz.value, h.value) == 0
print("rccl hook ok")
'''


def test_hook_registers_and_releases_rccl_style_allocations(gpu, tmp_path):
    standin = str(tmp_path / "librccl_standin.so")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    subprocess.run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__",
                    "-I" + os.path.join(rocm, "include"), os.path.join(ROOT, "tests", "rccl_standin", "librccl_standin.cpp"),
                    "-o", standin, "-L" + os.path.join(rocm, "lib"), "-lamdhip64"], check=True, capture_output=True, text=True)
    env = dict(os.environ, AMEM_ENABLE="1", GMM_LOG="1", AMEM_IPC="0")
    r = subprocess.run([sys.executable, "-c", CHILD, ROOT, standin], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0 and "rccl hook ok" in r.stdout, (r.returncode, r.stdout[-3000:], r.stderr[-3000:])


REAL_RCCL_CHILD = r'''
import ctypes as C, os, sys
import numpy as np
root = sys.argv[1]
sys.path.insert(0, root)
libdir = os.path.join(root, "asystem-amem_amd", "lib")
hook = C.CDLL(os.path.join(libdir, "libamem_rccl_hook.so"), mode=C.RTLD_GLOBAL)   # before the runtime and RCCL
from asystem_amem_amd import binding as B, harness as H
lib = B.load()
hip = C.CDLL("libamdhip64.so")
try:
    rccl = C.CDLL("librccl.so")
except OSError as e:
    print("no librccl.so:", e); print("rccl skipped"); sys.exit(0)
hook.amem_rccl_hook_registered.restype = C.c_int64
class UID(C.Structure):
    _fields_ = [("b", C.c_char * 128)]
rccl.ncclCommInitRank.argtypes = [C.POINTER(C.c_void_p), C.c_int, UID, C.c_int]
rccl.ncclAllReduce.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
rccl.ncclCommDestroy.argtypes = [C.c_void_p]
assert hip.hipSetDevice(0) == 0
uid, comm = UID(), C.c_void_p()
assert rccl.ncclGetUniqueId(C.byref(uid)) == 0
assert rccl.ncclCommInitRank(C.byref(comm), 1, uid, 0) == 0
# the buffers of the collective: tracked VMM memory, the way the reference's nccl-tests patch
# allocates them with ncclMemAlloc
MiB = 1 << 20
n = 4 * MiB // 4
bufs = []
for _ in range(2):
    va, h, asz = C.c_uint64(), C.c_uint64(), C.c_uint64()
    assert lib.amem_vmm_alloc(4 * MiB, 0, C.byref(va), C.byref(h), C.byref(asz)) == 0
    assert lib.amem_add_alloc_info(va.value, asz.value, B.TYPE_LOCAL, 0, h.value, -1, 0, None, B.CALLER_P2P) == 0
    bufs.append((va.value, asz.value))
send, recv = bufs[0][0], bufs[1][0]
rng = np.random.default_rng(5)

def allreduce_wrong():
    x = rng.standard_normal(n).astype(np.float32)
    assert lib.amem_copy_to_device(send, x.ctypes.data, x.nbytes) == 0
    junk = np.full(n, -1.0, dtype=np.float32)
    assert lib.amem_copy_to_device(recv, junk.ctypes.data, junk.nbytes) == 0
    assert rccl.ncclAllReduce(send, recv, n, 7, 0, comm, None) == 0            # ncclFloat32, ncclSum, null stream
    assert hip.hipDeviceSynchronize() == 0
    y = np.empty_like(x)
    assert lib.amem_copy_from_device(y.ctypes.data, recv, y.nbytes) == 0
    return int(np.count_nonzero(x != y))                                        # one rank: the sum is the input

assert allreduce_wrong() == 0
by_hook = hook.amem_rccl_hook_registered()
print("regions RCCL allocated through the VMM API:", by_hook)
assert lib.amem_region_count(0) == 2 + by_hook
for cycle in range(3):
    free0 = H.mem_free(lib)
    assert lib.ncclPause(None) == 0 and lib.amem_check_paused(0) == 1
    assert H.mem_free(lib) - free0 >= 6 * MiB
    assert lib.ncclResume(None) == 0 and lib.amem_check_paused(0) == 0
    assert allreduce_wrong() == 0, cycle                                       # same addresses, same communicator
assert rccl.ncclCommDestroy(comm) == 0
for va, asz in bufs:
    assert lib.amem_del_alloc_info(va, 0, 0) == 0 and lib.amem_vmm_free(va, asz, 0) == 0
assert lib.amem_region_count(0) == hook.amem_rccl_hook_registered()
print("rccl ok")
'''


def test_real_rccl_communicator_works_across_cycles(gpu):
    """The check the reference puts into nccl-tests (nccl_patch/nccl-tests.diff:24-50: pause and
    resume between iterations, then #wrong must be 0), on a one-rank communicator of the RCCL that
    ships with ROCm, with the hook library in place: an all-reduce between tracked buffers gives
    the right answer before a cycle and after each of three."""
    env = dict(os.environ, AMEM_ENABLE="1", GMM_LOG="1", AMEM_IPC="0", NCCL_CUMEM_ENABLE="1")
    r = subprocess.run([sys.executable, "-c", REAL_RCCL_CHILD, ROOT], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0 and ("rccl ok" in r.stdout or "rccl skipped" in r.stdout), \
        (r.returncode, r.stdout[-3000:], r.stderr[-3000:])
    if "rccl skipped" in r.stdout:
        pytest.skip("librccl.so is not loadable on this machine")


IMPORT_CHILD = r'''
import ctypes as C, os, sys
import numpy as np
root, standin = sys.argv[1], sys.argv[2]
sys.path.insert(0, root)
libdir = os.path.join(root, "asystem-amem_amd", "lib")
hook = C.CDLL(os.path.join(libdir, "libamem_rccl_hook.so"), mode=C.RTLD_GLOBAL)
from asystem_amem_amd import binding as B, harness as H
lib = B.load()
rccl = C.CDLL(standin, mode=C.RTLD_GLOBAL)
rccl.standin_cumem_alloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
rccl.standin_cumem_free.argtypes = [C.c_void_p]
rccl.standin_export.argtypes = [C.c_void_p, C.POINTER(C.c_int)]
rccl.standin_import_map.argtypes = [C.c_int, C.c_size_t, C.POINTER(C.c_void_p)]
hook.amem_rccl_hook_registered.restype = C.c_int64
MiB = 1 << 20
ipc_dir = os.environ["GMM_IPC_DIR"]
notes = lambda: sorted(f for f in os.listdir(ipc_dir) if f.startswith("amem_export_"))
rng = np.random.default_rng(41)
# rank A (the process's first slot) allocates the way ncclCuMemAlloc does
owned = []
for n in (4 * MiB, 8 * MiB, 2 * MiB):
    p = C.c_void_p()
    assert rccl.standin_cumem_alloc(C.byref(p), n) == 0
    data = rng.integers(1, 256, n, dtype=np.uint8)
    assert lib.amem_copy_to_device(p.value, data.ctypes.data, n) == 0
    owned.append((p.value, n, data))
slot_a = lib.amem_get_slot()
assert slot_a >= 0 and lib.amem_region_count(0) == 3
# without the loopback option two ranks of one process follow the reference's same-process rule:
# the import is mapped and works, but stays outside the registry (gmm_client_impl.cpp:482-484)
slot_b = lib.amem_ipc_claim_slot()
assert slot_b >= 0 and slot_b != slot_a and lib.amem_ipc_act_as(slot_b) == 0
fd, q = C.c_int(-1), C.c_void_p()
assert rccl.standin_export(owned[2][0], C.byref(fd)) == 0
assert rccl.standin_import_map(fd.value, owned[2][1], C.byref(q)) == 0
os.close(fd.value)
assert lib.amem_region_count(0) == 3 and hook.amem_rccl_hook_registered() == 3
assert rccl.standin_cumem_free(q.value) == 0
# with it, rank B registers what it imports with rank A through the socket service
assert lib.amem_set_option(b"peer_loopback", 1) == 0
imports = []
for p, n, data in owned:
    fd, q = C.c_int(-1), C.c_void_p()
    assert lib.amem_ipc_act_as(-1) == 0
    assert rccl.standin_export(p, C.byref(fd)) == 0              # rank A exports
    assert lib.amem_ipc_act_as(slot_b) == 0
    assert rccl.standin_import_map(fd.value, n, C.byref(q)) == 0  # rank B imports and maps
    os.close(fd.value)
    imports.append(q.value)
assert lib.amem_ipc_act_as(-1) == 0
assert len(notes()) == 3                                           # one note per exported buffer, for importers elsewhere
tab = H.region_table(lib, 0)
assert len(tab) == 6 and hook.amem_rccl_hook_registered() == 6
for (p, n, _), q in zip(owned, imports):
    assert tab[q]["type"] == B.TYPE_PEER_POSIX and tab[q]["alloc_sz"] == n and tab[q]["tags"] == B.CALLER_P2P_PEER
    assert tab[q]["mc_handle"] == p                                # the importer names the region by the owner's address, which no resume changes
    assert tab[p]["has_peer"] == 1 and tab[p]["peers"][slot_b] == q
lib.ncclPause(None); lib.ncclResume(None)                          # warm cycle
free0 = H.mem_free(lib)
assert lib.ncclPause(None) == 0
c = H.counters(lib)
assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"]) == (3, 3, 3)
assert H.mem_free(lib) - free0 >= 14 * MiB - 2 * MiB              # the importer let go first, so the memory really went
assert lib.ncclResume(None) == 0
c = H.counters(lib)
assert (c["offload_cnt"], c["release_shadow_cnt"], c["release_local_cnt"], c["paused"]) == (0, 0, 0, 0)
for (p, n, data), q in zip(owned, imports):
    for addr in (p, q):
        out = np.empty(n, dtype=np.uint8)
        assert lib.amem_copy_from_device(out.ctypes.data, addr, n) == 0 and np.array_equal(out, data)
# rank B drops its mappings, then rank A frees: the registry and the notes empty out
for q in imports:
    assert rccl.standin_cumem_free(q) == 0
assert lib.amem_region_count(0) == 3
for p, n, _ in owned:
    assert rccl.standin_cumem_free(p) == 0
assert lib.amem_region_count(0) == 0 and hook.amem_rccl_hook_registered() == 0 and notes() == []
print("rccl hook import side ok")
'''


@pytest.mark.parametrize("via", ["memory", "notes"])
def test_hook_registers_imported_mappings_with_their_owner(gpu, tmp_path, via):
    """The importer's half of the hook (the reference's site in ncclP2pImportShareableBuffer,
    nccl_patch/nccl_2.27.5-1.diff:572-579): a second rank, living in the same process under a slot of its
    own, imports the descriptors the first rank exports; the hook names the owner from the descriptor's
    identity and registers each mapping as PEER_POSIX, so a pause drops the importer's mappings before
    the owner's release and a resume maps the new memory back at the importer's addresses.
    "notes": the importer finds the owner through the note files under GMM_IPC_DIR, as an importer in
    another process has to, instead of through what its own process remembers of its exports."""
    standin = str(tmp_path / "librccl_standin.so")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    subprocess.run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__",
                    "-I" + os.path.join(rocm, "include"), os.path.join(ROOT, "tests", "rccl_standin", "librccl_standin.cpp"),
                    "-o", standin, "-L" + os.path.join(rocm, "lib"), "-lamdhip64"], check=True, capture_output=True, text=True)
    env = dict(os.environ, AMEM_ENABLE="1", GMM_LOG="1", GMM_IPC_DIR=str(tmp_path), AMEM_GROUPID=str(0x7400 + os.getpid() % 1024))
    env.pop("AMEM_IPC", None)
    if via == "notes":
        env["AMEM_HOOK_NOTES_ONLY"] = "1"
    r = subprocess.run([sys.executable, "-c", IMPORT_CHILD, ROOT, standin], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0 and "rccl hook import side ok" in r.stdout, (r.returncode, r.stdout[-3000:], r.stderr[-3000:])


PLAIN_ALLOC_CHILD = r'''
import ctypes as C, os, sys
import numpy as np
root = sys.argv[1]
sys.path.insert(0, root)
libdir = os.path.join(root, "asystem-amem_amd", "lib")
hook = C.CDLL(os.path.join(libdir, "libamem_rccl_hook.so"), mode=C.RTLD_GLOBAL)   # before the runtime and RCCL
from asystem_amem_amd import binding as B, harness as H
lib = B.load()
hip = C.CDLL("libamdhip64.so")
try:
    rccl = C.CDLL("librccl.so")
except OSError as e:
    print("no librccl.so:", e); print("rccl skipped"); sys.exit(0)
hook.amem_rccl_hook_registered.restype = C.c_int64
hook.amem_rccl_hook_served_bytes.restype = C.c_uint64
class UID(C.Structure):
    _fields_ = [("b", C.c_char * 128)]
rccl.ncclCommInitRank.argtypes = [C.POINTER(C.c_void_p), C.c_int, UID, C.c_int]
rccl.ncclAllReduce.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
rccl.ncclCommDestroy.argtypes = [C.c_void_p]
assert hip.hipSetDevice(0) == 0
uid, comm = UID(), C.c_void_p()
assert rccl.ncclGetUniqueId(C.byref(uid)) == 0
assert rccl.ncclCommInitRank(C.byref(comm), 1, uid, 0) == 0
served, regions = hook.amem_rccl_hook_served_bytes(), hook.amem_rccl_hook_registered()
hook.amem_rccl_hook_unserved_bytes.restype = C.c_uint64
hook.amem_rccl_hook_unserved_bytes.argtypes = [C.POINTER(C.c_uint64)] * 3
small, flagged, unservable = C.c_uint64(), C.c_uint64(), C.c_uint64()
left = hook.amem_rccl_hook_unserved_bytes(C.byref(small), C.byref(flagged), C.byref(unservable))
print("one-rank communicator of the real RCCL: %.1f MiB in %d regions served through the virtual-memory API; left alone %.1f MiB "
      "(%.1f below the 1 MiB threshold, %.1f uncached / fine-grained, %.1f not servable)" %
      (served / 2**20, regions, left / 2**20, small.value / 2**20, flagged.value / 2**20, unservable.value / 2**20))
if served == 0:
    print("this RCCL made no plain allocation of 1 MiB or more"); print("rccl skipped"); sys.exit(0)
assert lib.amem_region_count(0) == regions
tab = H.region_table(lib, 0)
assert sum(t["alloc_sz"] for t in tab.values()) == served and all(t["type"] == B.TYPE_LOCAL for t in tab.values())
MiB = 1 << 20
n = 4 * MiB // 4
bufs = []
for _ in range(2):
    p = C.c_void_p()
    assert hip.hipMalloc(C.byref(p), 4 * MiB) == 0     # the application's own buffers: ordinary memory, not the hook's business
    bufs.append(p.value)
send, recv = bufs
assert lib.amem_region_count(0) == regions
rng = np.random.default_rng(6)

def allreduce_wrong():
    x = rng.standard_normal(n).astype(np.float32)
    assert lib.amem_copy_to_device(send, x.ctypes.data, x.nbytes) == 0
    junk = np.full(n, -1.0, dtype=np.float32)
    assert lib.amem_copy_to_device(recv, junk.ctypes.data, junk.nbytes) == 0
    assert rccl.ncclAllReduce(send, recv, n, 7, 0, comm, None) == 0            # ncclFloat32, ncclSum, null stream
    assert hip.hipDeviceSynchronize() == 0
    y = np.empty_like(x)
    assert lib.amem_copy_from_device(y.ctypes.data, recv, y.nbytes) == 0
    return int(np.count_nonzero(x != y))

assert allreduce_wrong() == 0
lib.ncclPause(None); lib.ncclResume(None)                                      # warm cycle
for cycle in range(3):
    free0 = H.mem_free(lib)
    assert lib.ncclPause(None) == 0 and lib.amem_check_paused(0) == 1
    released = H.mem_free(lib) - free0
    assert released >= served - 2 * MiB, (released, served)                    # the communicator's own memory is gone
    assert lib.ncclResume(None) == 0 and lib.amem_check_paused(0) == 0
    assert allreduce_wrong() == 0, cycle                                       # the same communicator still works
assert rccl.ncclCommDestroy(comm) == 0                                         # RCCL frees what it was served
assert hook.amem_rccl_hook_served_bytes() == 0 and hook.amem_rccl_hook_registered() == 0 and lib.amem_region_count(0) == 0
print("released per pause: %.1f MiB" % (released / 2**20))
print("rccl plain ok")
'''


def test_real_rccl_buffers_served_through_the_vmm_api_are_released_and_restored(gpu, measured):
    """A real communicator's own memory in the registry (what the reference's hooks in ncclCuMemAlloc are
    for, nccl_patch/nccl_2.27.5-1.diff:278-280). The RCCL of this ROCm release keeps its buffers in plain
    allocations, which nothing can unmap; with AMEM_HOOK_PLAIN_ALLOC set, the hook serves RCCL's plain
    allocations of at least that size through the virtual-memory API and registers them. A one-rank
    communicator then really gives its memory back at ncclPause, gets it back at ncclResume at the same
    addresses, and an all-reduce through it is right after each of three cycles (the check of
    nccl_patch/nccl-tests.diff:24-50). Uncached and fine-grained allocations are left alone."""
    env = dict(os.environ, AMEM_ENABLE="1", GMM_LOG="1", AMEM_IPC="0", AMEM_HOOK_PLAIN_ALLOC=str(1 << 20))
    r = subprocess.run([sys.executable, "-c", PLAIN_ALLOC_CHILD, ROOT], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0 and ("rccl plain ok" in r.stdout or "rccl skipped" in r.stdout), \
        (r.returncode, r.stdout[-3000:], r.stderr[-3000:])
    for line in r.stdout.splitlines():
        if line.startswith("one-rank communicator") or line.startswith("released per pause"):
            measured(line)
    if "rccl skipped" in r.stdout:
        pytest.skip("librccl.so is not loadable here, or it made no plain allocation the hook serves")


GUARDS_CHILD = r'''
import ctypes as C, os, sys
import numpy as np
root, standin = sys.argv[1], sys.argv[2]
sys.path.insert(0, root)
libdir = os.path.join(root, "asystem-amem_amd", "lib")
hook = C.CDLL(os.path.join(libdir, "libamem_rccl_hook.so"), mode=C.RTLD_GLOBAL)
from asystem_amem_amd import binding as B, harness as H
lib = B.load()
rccl = C.CDLL(standin, mode=C.RTLD_GLOBAL)
rccl.standin_plain_alloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t, C.c_uint, C.c_int]
rccl.standin_plain_free.argtypes = [C.c_void_p]
rccl.standin_ipc_handle.argtypes = [C.c_void_p]
hook.amem_rccl_hook_registered.restype = C.c_int64
hook.amem_rccl_hook_served_bytes.restype = C.c_uint64
hook.amem_rccl_hook_unserved_bytes.restype = C.c_uint64
hook.amem_rccl_hook_unserved_bytes.argtypes = [C.POINTER(C.c_uint64)] * 3
hook.amem_rccl_hook_exclude.argtypes = [C.c_void_p]
MiB = 1 << 20
FINE_GRAINED = 1                                                   # hipDeviceMallocFinegrained
rng = np.random.default_rng(51)

def unserved():
    a, b, c = C.c_uint64(), C.c_uint64(), C.c_uint64()
    total = hook.amem_rccl_hook_unserved_bytes(C.byref(a), C.byref(b), C.byref(c))
    assert total == a.value + b.value + c.value
    return a.value, b.value, c.value

# what the threshold of 1 MiB does with five allocations made the way RCCL makes them
big, big2, small, fine, plain = [C.c_void_p() for _ in range(5)]
assert rccl.standin_plain_alloc(C.byref(big), 8 * MiB, 0, 1) == 0      # served and registered
assert rccl.standin_plain_alloc(C.byref(big2), 4 * MiB, 0, 0) == 0     # served and registered (hipMalloc)
assert rccl.standin_plain_alloc(C.byref(small), 256 << 10, 0, 1) == 0  # below the threshold
assert rccl.standin_plain_alloc(C.byref(fine), 2 * MiB, FINE_GRAINED, 1) == 0   # keeps its semantics
assert hook.amem_rccl_hook_served_bytes() == 12 * MiB and hook.amem_rccl_hook_registered() == 2
assert unserved() == (256 << 10, 2 * MiB, 0)
assert lib.amem_region_count(0) == 2
data = {}
for p, n in ((big, 8 * MiB), (big2, 4 * MiB)):
    d = rng.integers(1, 256, n, dtype=np.uint8)
    assert lib.amem_copy_to_device(p.value, d.ctypes.data, n) == 0
    data[p.value] = d

# (a) legacy IPC: refused for a served mapping with a line that says what to do, untouched for the rest
assert rccl.standin_ipc_handle(big.value) != 0
assert rccl.standin_ipc_handle(big.value + 4096) != 0              # any address inside it
assert rccl.standin_ipc_handle(small.value) == 0                   # an ordinary allocation still gets its handle
sys.stderr.flush()

# (c) a buffer the caller registers with a NIC is taken out of the registry by hand
lib.ncclPause(None); lib.ncclResume(None)                          # warm cycle
free0 = H.mem_free(lib)
assert lib.ncclPause(None) == 0
assert H.mem_free(lib) - free0 >= 12 * MiB - 2 * MiB              # both served buffers are released
assert hook.amem_rccl_hook_exclude(big2.value) == 2                # not while paused: its memory is gone
assert lib.ncclResume(None) == 0
assert hook.amem_rccl_hook_exclude(big2.value + 8192) == 0         # by any address inside the buffer
assert hook.amem_rccl_hook_exclude(big2.value) == 1                # it is no longer the hook's
assert hook.amem_rccl_hook_exclude(small.value) == 1               # never was
assert lib.amem_region_count(0) == 1 and hook.amem_rccl_hook_registered() == 1
assert hook.amem_rccl_hook_served_bytes() == 12 * MiB              # still a mapping the hook has to free one day
free1 = H.mem_free(lib)
assert lib.ncclPause(None) == 0
released = H.mem_free(lib) - free1
assert 8 * MiB - 2 * MiB <= released < 12 * MiB - MiB, released    # only the buffer still registered went
out = np.empty(4 * MiB, dtype=np.uint8)                            # the excluded one is readable while paused
assert lib.amem_copy_from_device(out.ctypes.data, big2.value, out.nbytes) == 0 and np.array_equal(out, data[big2.value])
assert lib.ncclResume(None) == 0
for p, d in data.items():
    out = np.empty(d.nbytes, dtype=np.uint8)
    assert lib.amem_copy_from_device(out.ctypes.data, p, d.nbytes) == 0 and np.array_equal(out, d)
for p in (big, big2, small, fine):
    assert rccl.standin_plain_free(p.value) == 0
assert hook.amem_rccl_hook_served_bytes() == 0 and hook.amem_rccl_hook_registered() == 0 and unserved() == (0, 0, 0)
assert lib.amem_region_count(0) == 0 and lib.amem_handle_count(0) == 0
print("rccl hook guards ok")
'''


def test_hook_guards_for_served_allocations(gpu, tmp_path):
    """The opt-in mode's guard rails, with a caller that allocates the way RCCL 2.27 does (a file named
    librccl_*.so calling hipExtMallocWithFlags / hipMalloc): what is served and what is left alone is
    counted by reason; hipIpcGetMemHandle on a served mapping fails with one line that names
    AMEM_HOOK_PLAIN_ALLOC and NCCL_P2P_DISABLE=1, and works as ever for ordinary memory; a buffer taken
    out by amem_rccl_hook_exclude (the manual form of the reference's removal before NIC registration,
    nccl_patch/nccl_2.27.5-1.diff:309-312, :364-367) keeps its memory through a pause; the line at exit
    says how much could be registered and how much not."""
    standin = str(tmp_path / "librccl_standin.so")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    subprocess.run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__",
                    "-I" + os.path.join(rocm, "include"), os.path.join(ROOT, "tests", "rccl_standin", "librccl_standin.cpp"),
                    "-o", standin, "-L" + os.path.join(rocm, "lib"), "-lamdhip64"], check=True, capture_output=True, text=True)
    env = dict(os.environ, AMEM_ENABLE="1", GMM_LOG="1", AMEM_IPC="0", AMEM_HOOK_PLAIN_ALLOC=str(1 << 20))
    r = subprocess.run([sys.executable, "-c", GUARDS_CHILD, ROOT, standin], env=env, capture_output=True, text=True, timeout=240)
    assert r.returncode == 0 and "rccl hook guards ok" in r.stdout, (r.returncode, r.stdout[-3000:], r.stderr[-3000:])
    errs = [l for l in r.stderr.splitlines() if "hipIpcGetMemHandle" in l and "[ERRO]" in l]
    assert len(errs) == 2 and all("AMEM_HOOK_PLAIN_ALLOC" in l and "NCCL_P2P_DISABLE=1" in l for l in errs), r.stderr[-3000:]
    summary = [l for l in r.stderr.splitlines() if "RCCL's plain allocations since load" in l]
    assert len(summary) == 1 and "12.0 MiB in 2 allocations served" in summary[0], r.stderr[-3000:]
    assert "2.2 MiB left alone (0.2 MiB below the threshold, 2.0 MiB uncached / fine-grained, 0.0 MiB not servable)" in summary[0], summary
