"""ctypes access to the CPU restatement of the reference's pause/resume path (liboracle.so).

TEST INFRASTRUCTURE: imported only by tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg. Nothing under asystem-amem_amd/ imports this package.
"""
import ctypes as C
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")
MAX_DEVS, MAX_CALLER, CHUNK = 8, 16, 65536
DESC_ZERO = (1 << 64) - 1


class RegionInfo(C.Structure):
    _fields_ = [("va", C.c_uint64), ("handle", C.c_uint64), ("mc_handle", C.c_uint64), ("alloc_sz", C.c_uint64),
                ("tags", C.c_uint64), ("peers", C.c_uint64 * MAX_DEVS), ("cpu_addr", C.c_uint64),
                ("user_info", C.c_uint64), ("dev", C.c_int32), ("pid", C.c_int32), ("refcount", C.c_int32),
                ("shared_fd", C.c_int32), ("type", C.c_int32), ("state", C.c_int32), ("has_peer", C.c_int32),
                ("oos_flag", C.c_int32)]

    def as_dict(self):
        d = {k: getattr(self, k) for k, _ in self._fields_ if k != "peers"}
        d["peers"] = list(self.peers)
        return d


class Counters(C.Structure):
    _fields_ = [("release_local_cnt", C.c_int64), ("release_shadow_cnt", C.c_int64), ("offload_cnt", C.c_int64),
                ("smoke_log", C.c_int64), ("alloc_bytes", C.c_uint64 * MAX_CALLER), ("del_bytes", C.c_uint64),
                ("pause_cnt", C.c_uint64), ("resume_cnt", C.c_uint64), ("paused", C.c_int32),
                ("group_id", C.c_int32), ("handle_count", C.c_int32), ("region_count", C.c_int32)]


class ChunkSum(C.Structure):
    _fields_ = [("sum64", C.c_uint64), ("xor64", C.c_uint64)]


class CopyDesc(C.Structure):
    _fields_ = [("va", C.c_uint64), ("off", C.c_uint64), ("bytes", C.c_uint64)]


def build():
    subprocess.run(["make", "-s", "-B", "-C", HERE, "liboracle.so"], check=True)
    return LIB_PATH


_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is missing: run __graft_entry__.build()" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    u64, i = C.c_uint64, C.c_int
    P = C.POINTER
    sig = {
        "oracle_vmm_alloc": (i, [u64, P(u64), P(u64), P(u64)]),
        "oracle_vmm_free": (i, [u64, u64, u64]),
        "oracle_vmm_export": (i, [u64, P(i)]),
        "oracle_vmm_import": (i, [i, u64, P(u64), P(u64)]),
        "oracle_vmm_live_bytes": (u64, []),
        "oracle_vmm_reset": (None, []),
        "oracle_vmm_handle_of": (u64, [u64]),
        "oracle_vmm_retain": (u64, [u64]),
        "oracle_reset": (None, []),
        "oracle_ctx_enable": (i, [i, i]),
        "oracle_add_alloc_info": (i, [i, u64, u64, i, i, u64, i, u64, u64, i]),
        "oracle_del_alloc_info": (i, [i, u64, u64, i]),
        "oracle_add_refcount": (i, [i, u64, i]),
        "oracle_add_peer_info": (i, [i, u64, u64, i]),
        "oracle_register_peer_info": (i, [i, u64, u64, i]),
        "oracle_update_peer_info": (i, [i, u64, i]),
        "oracle_check_paused": (i, [i]),
        "oracle_set_group_id": (i, [i, i]),
        "oracle_get_group_id": (i, [i]),
        "oracle_mem_stats_total": (u64, [i]),
        "oracle_mem_pause": (i, [i]),
        "oracle_mem_resume": (i, [i]),
        "oracle_mem_pause_mt": (i, [i, i]),
        "oracle_mem_resume_mt": (i, [i, i]),
        "oracle_region_count": (C.c_int64, [i, i]),
        "oracle_region_at": (i, [i, i, C.c_int64, P(RegionInfo)]),
        "oracle_region_find": (i, [i, i, u64, P(RegionInfo)]),
        "oracle_handle_lookup": (u64, [i, i, u64]),
        "oracle_get_counters": (None, [i, P(Counters)]),
        "oracle_zero_scan": (u64, [C.c_void_p, u64, C.c_void_p, C.c_void_p]),
        "oracle_gather_pack": (None, [P(CopyDesc), u64, C.c_void_p]),
        "oracle_scatter_unpack": (None, [P(CopyDesc), u64, C.c_void_p]),
    }
    for name, (res, args) in sig.items():
        f = getattr(L, name)
        f.restype, f.argtypes = res, args
    _lib = L
    return L


def region_table(L, ctx, dev=0):
    out = {}
    info = RegionInfo()
    for k in range(L.oracle_region_count(ctx, dev)):
        if L.oracle_region_at(ctx, dev, k, C.byref(info)) == 0:
            out[info.va] = info.as_dict()
    return out


def counters(L, ctx):
    c = Counters()
    L.oracle_get_counters(ctx, C.byref(c))
    d = {k: getattr(c, k) for k, _ in c._fields_ if k != "alloc_bytes"}
    d["alloc_bytes"] = list(c.alloc_bytes)
    return d
