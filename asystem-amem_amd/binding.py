"""ctypes binding of libamem_nccl.so.1 — the Python caller's view of the C ABI in
include/amem.h. Python frameworks bind the reference the same way: its README has SGLang's
PyNCCL wrapper load `ncclPause`, `ncclResume` and `ncclSetGroupID` from the NCCL shared
library through ctypes (README.md:268-274 of the reference).

Loading never builds anything and never falls back: a missing library is an error.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libamem_nccl.so.1")

MAX_DEVS = 8
MAX_CALLER = 16
CHUNK = 65536
DESC_ZERO = (1 << 64) - 1
NOALLOC_MAX_EXTENTS = 8192
NOALLOC_MAX_CHUNKS = 262144

STATE_INVALID, STATE_ALLOC, STATE_OFFLOADING, STATE_HOLE, STATE_PRELOADING, STATE_REMAPPED = range(6)
TYPE_LOCAL, TYPE_LOCAL_FABRIC, TYPE_LOCAL_SYMM, TYPE_PEER_POSIX, TYPE_PEER_FABRIC, TYPE_PEER_SYMM = range(6)
CALLER_DEFAULT, CALLER_P2P, CALLER_FABRIC, CALLER_POSIX, CALLER_SYMM, CALLER_NVLS = range(6)
CALLER_P2P_PEER, CALLER_PROXY, CALLER_SYMM_PEER = 7, 9, 10


class RegionInfo(C.Structure):
    _fields_ = [
        ("va", C.c_uint64), ("handle", C.c_uint64), ("mc_handle", C.c_uint64),
        ("alloc_sz", C.c_uint64), ("tags", C.c_uint64), ("peers", C.c_uint64 * MAX_DEVS),
        ("cpu_addr", C.c_uint64), ("user_info", C.c_uint64), ("parked_bytes", C.c_uint64),
        ("handle_gen", C.c_uint64),
        ("dev", C.c_int32), ("pid", C.c_int32), ("refcount", C.c_int32), ("shared_fd", C.c_int32),
        ("type", C.c_int32), ("state", C.c_int32), ("has_peer", C.c_int32), ("oos_flag", C.c_int32),
    ]

    def as_dict(self):
        d = {k: getattr(self, k) for k, _ in self._fields_ if k != "peers"}
        d["peers"] = list(self.peers)
        return d


class Counters(C.Structure):
    _fields_ = [
        ("release_local_cnt", C.c_int64), ("release_shadow_cnt", C.c_int64), ("offload_cnt", C.c_int64),
        ("smoke_log", C.c_int64), ("alloc_bytes", C.c_uint64 * MAX_CALLER), ("del_bytes", C.c_uint64),
        ("pause_cnt", C.c_uint64), ("resume_cnt", C.c_uint64),
        ("paused", C.c_int32), ("group_id", C.c_int32), ("enabled", C.c_int32), ("slot", C.c_int32),
    ]


class CycleStats(C.Structure):
    _fields_ = [(n, C.c_double) for n in (
        "pause_ms", "resume_ms", "pause_scan_ms", "pause_plan_ms", "pause_copy_ms", "pause_unmap_ms",
        "resume_map_ms", "resume_copy_ms", "resume_peer_ms", "k1_ms", "k2_ms", "k3_ms")] + [
        (n, C.c_uint64) for n in (
        "k1_launches", "k2_launches", "k3_launches", "footprint_bytes", "parked_bytes", "zero_chunks",
        "total_chunks", "local_regions", "peer_regions", "dma_bytes", "kernel_bytes", "slab_bytes",
        "verify_mismatch")] + [(n, C.c_double) for n in (
        "pause_pool_ms", "pause_scratch_ms", "pause_sync_ms", "resume_scratch_ms")] + [("resume_dma_bytes", C.c_uint64), ("pause_narrow_launches", C.c_uint64),
                                                                         ("resume_plan_ms", C.c_double)]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_}


class Extent(C.Structure):
    _fields_ = [("va", C.c_uint64), ("bytes", C.c_uint64)]


class ChunkSum(C.Structure):
    _fields_ = [("sum64", C.c_uint64), ("xor64", C.c_uint64)]


class CopyDesc(C.Structure):
    _fields_ = [("va", C.c_uint64), ("off", C.c_uint64), ("bytes", C.c_uint64)]


_SIGNATURES = {
    # name: (restype, argtypes)
    "amem_add_alloc_info": (C.c_int, [C.c_uint64, C.c_uint64, C.c_int, C.c_int, C.c_uint64, C.c_int, C.c_uint64,
                                      C.c_void_p, C.c_int]),
    "amem_del_alloc_info": (C.c_int, [C.c_uint64, C.c_uint64, C.c_int]),
    "amem_add_refcount": (C.c_int, [C.c_void_p, C.c_int]),
    "amem_add_peer_info": (C.c_int, [C.c_uint64, C.c_uint64, C.c_int]),
    "amem_register_peer_info": (C.c_int, [C.c_uint64, C.c_uint64, C.c_int]),
    "amem_update_peer_info": (C.c_int, [C.c_uint64, C.c_int]),
    "amem_check_paused": (C.c_int, [C.c_int]),
    "amem_set_group_id": (C.c_int, [C.c_int]),
    "amem_get_group_id": (None, [C.POINTER(C.c_int)]),
    "amem_dump_alloc_stats": (None, [C.c_int]),
    "amem_mem_pause": (C.c_int, [C.c_int, C.c_uint64]),
    "amem_mem_resume": (C.c_int, [C.c_int, C.c_uint64]),
    "ncclPause": (C.c_int, [C.c_void_p]),
    "ncclResume": (C.c_int, [C.c_void_p]),
    "ncclMemStats": (C.c_int, []),
    "ncclSetGroupID": (C.c_int, [C.c_int]),
    "ncclGetGroupID": (C.c_int, [C.POINTER(C.c_int)]),
    "amem_vmm_alloc": (C.c_int, [C.c_uint64, C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64),
                                 C.POINTER(C.c_uint64)]),
    "amem_vmm_free": (C.c_int, [C.c_uint64, C.c_uint64, C.c_uint64]),
    "amem_vmm_export": (C.c_int, [C.c_uint64, C.POINTER(C.c_int)]),
    "amem_vmm_import": (C.c_int, [C.c_int, C.c_uint64, C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "amem_region_count": (C.c_int64, [C.c_int]),
    "amem_region_at": (C.c_int, [C.c_int, C.c_int64, C.POINTER(RegionInfo)]),
    "amem_region_find": (C.c_int, [C.c_int, C.c_uint64, C.POINTER(RegionInfo)]),
    "amem_handle_lookup": (C.c_uint64, [C.c_int, C.c_uint64]),
    "amem_handle_count": (C.c_int64, [C.c_int]),
    "amem_get_counters": (None, [C.POINTER(Counters)]),
    "amem_get_cycle_stats": (None, [C.POINTER(CycleStats)]),
    "amem_set_enabled": (C.c_int, [C.c_int]),
    "amem_set_option": (C.c_int, [C.c_char_p, C.c_int64]),
    "amem_get_option": (C.c_int64, [C.c_char_p]),
    "amem_pool_trim": (C.c_uint64, []),
    "amem_pool_reserve": (C.c_int, [C.c_uint64]),
    "amem_shutdown": (C.c_int, []),
    "amem_ipc_start": (C.c_int, []),
    "amem_get_slot": (C.c_int, []),
    "amem_ipc_claim_slot": (C.c_int, []),
    "amem_ipc_act_as": (C.c_int, [C.c_int]),
    "amem_ipc_served": (C.c_int, [C.c_int, C.POINTER(C.c_uint64)]),
    "amem_ipc_peer_alive": (C.c_int, [C.c_int]),
    "amem_chunk_count": (C.c_uint64, [C.POINTER(Extent), C.c_uint64]),
    "amem_zero_scan": (C.c_int, [C.POINTER(Extent), C.c_uint64, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "amem_zero_scan_noalloc": (C.c_int, [C.POINTER(Extent), C.c_uint64, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "amem_gather_pack": (C.c_int, [C.POINTER(CopyDesc), C.c_uint64, C.c_void_p, C.c_uint64, C.c_int,
                                   C.POINTER(C.c_float)]),
    "amem_scatter_unpack": (C.c_int, [C.POINTER(CopyDesc), C.c_uint64, C.c_void_p, C.c_uint64, C.c_int,
                                      C.POINTER(C.c_float)]),
}

# include/amem_testing.h: measurement and test helpers, same library
_TESTING_SIGNATURES = {
    "amem_probe_link": (C.c_int, [C.c_uint64, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "amem_probe_unmap": (C.c_int, [C.c_int, C.c_uint64, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "amem_calib_copy": (C.c_int, [C.c_uint64, C.c_int, C.POINTER(C.c_float)]),
    "amem_copy_to_device": (C.c_int, [C.c_uint64, C.c_void_p, C.c_uint64]),
    "amem_copy_from_device": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64]),
    "amem_device_mem_info": (C.c_int, [C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "amem_device_count": (C.c_int, []),
    "amem_device_pci_bus_id": (C.c_int, [C.c_char_p, C.c_int]),
}

# The reference's own C++-linkage names, as its library exports them.
MANGLED_REFERENCE_SYMBOLS = [
    "_Z17amem_addAllocInfoymiiyimPv16amem_caller_type", "_Z17amem_delAllocInfoyyi", "_Z13amem_memPauseim",
    "_Z14amem_memResumeim", "_Z16amem_checkPausedb", "_Z19amem_dumpAllocStatsb", "_Z15amem_setGroupIDi",
    "_Z15amem_getGroupIDPi", "_Z16amem_addRefcountPvi", "_Z16amem_addPeerInfoyyi",
    "_Z21amem_registerPeerInfoyyi", "_Z19amem_updatePeerInfoyi", "amem_groupID", "gmm_libP",
]

_lib = None


def load(path=None):
    """Load the library (once) and declare every entry point of include/amem.h and include/amem_testing.h."""
    global _lib
    if _lib is not None:
        return _lib
    path = path or LIB_PATH   # no environment override: the package only ever loads the library it ships
    if not os.path.exists(path):
        raise RuntimeError(
            "%s is missing: build it with `python asystem-amem_amd/build.py` "
            "(there is no Python or CPU fallback for the pause/resume path)" % path)
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (res, args) in list(_SIGNATURES.items()) + list(_TESTING_SIGNATURES.items()):
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def c_abi_names():
    return sorted(_SIGNATURES)


def testing_abi_names():
    return sorted(_TESTING_SIGNATURES)
