// The exported surface of libamem_nccl.so.1: the C ABI of include/amem.h, the reference's
// C++-linkage names of include/amem_nccl.h, and the registry logic behind both.
// Registry behaviour follows amem_nccl_plugin/amem_nccl.cpp line by line where cited.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "../../include/amem.h"
#include "../../include/amem_nccl.h"
#include "../../include/amem_testing.h"
#include "ctx.h"
#include "engine.h"
#include "ipc.h"
#include "log.h"
#include "vmm.h"

// Data symbols of the reference library (amem_nccl.cpp:35-36).
void* gmm_libP = NULL;
int amem_groupID = 0;

namespace amem {

Globals& globals() {
  static Globals g;
  return g;
}

static int g_device_count = -1;
bool gpu_present() {
  if (g_device_count < 0) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); n = 0; }
    g_device_count = n;
  }
  return g_device_count > 0;
}

int current_device() {
  int dev = 0;
  if (!gpu_present()) return 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); dev = 0; }
  return (dev >= 0 && dev < AMEM_MAX_DEVS) ? dev : 0;
}

// InitClientCtx (amem_nccl.cpp:55-80): the context appears with the first tracked
// allocation; until then the group id may still change.
static Ctx* init_ctx(int dev) {
  Globals& g = globals();
  std::lock_guard<std::mutex> lk(g.init_mtx);
  if (!g.ctx) {
    LOGGER(DEBUG, "Init: init client on card %d", dev);
    g.ctx = new Ctx();
    const char* ipc = getenv("AMEM_IPC");
    if (!ipc || atoi(ipc) != 0) (void)ipc_start(dev);
    // Streams and device code are set up while there is still device memory to load them into.
    // (the current device: pause and resume act on it, and selecting it changes nothing for the caller)
    if (gpu_present()) (void)engine_for(current_device());
  }
  return g.ctx;
}

static Ctx* ctx_or_null() { return globals().ctx; }

static void fill_info(uint64_t va, const Region& r, amem_region_info* o) {
  memset(o, 0, sizeof(*o));
  o->va = va;
  o->handle = r.handle;
  o->mc_handle = r.mcHandle;
  o->alloc_sz = r.allocSz;
  o->tags = r.tags;
  memcpy(o->peers, r.peers, sizeof(o->peers));
  o->cpu_addr = (uint64_t)(uintptr_t)r.cpuAddr;
  o->user_info = (uint64_t)(uintptr_t)r.userInfo;
  o->parked_bytes = r.parkedBytes;
  o->handle_gen = r.handleGen;
  o->dev = r.dev;
  o->pid = r.pid;
  o->refcount = r.refcount;
  o->shared_fd = r.sharedFD;
  o->type = r.type;
  o->state = r.state;
  o->has_peer = r.hasPeer;
  o->oos_flag = r.oosFlag;
}

// Service-thread handler of GMM_OP_RELEASE_PEER_HANDLE (gmm_worker_impl.cpp:392-397).
int amem_release_peer_mapping(uint64_t va) {
  Ctx* c = ctx_or_null();
  if (!c || !gpu_present()) return 1;
  uint64_t handle = 0;
  size_t size = 0;
  {
    std::lock_guard<std::mutex> lk(c->fields);
    bool found = false;
    for (int dev = 0; dev < AMEM_MAX_DEVS && !found; ++dev) {  // the service thread's device need not be the region's
      auto it = c->allocTable[dev].find(va);
      if (it == c->allocTable[dev].end()) continue;
      handle = it->second.handle;
      size = it->second.allocSz;
      found = true;
    }
    if (!found) return 1;
  }
  if (!handle) handle = vmm_handle_of(va);
  return (int)vmm_unmap_release(va, size, handle, 0);
}

}  // namespace amem

using namespace amem;

extern "C" {

int amem_add_alloc_info(uint64_t va, uint64_t size, int type, int dev, uint64_t handle, int peer_dev,
                        uint64_t peer_handle, void* user_info, int caller) {
  LOGGER(DEBUG, "AllocInfo: localDev:%d", dev);
  Globals& g = globals();
  if (g.disabled > 0) return 0;
  if (dev < 0 || dev >= AMEM_MAX_DEVS) return 1;
  int ret = 0;
  const int peerFlag = from_peer(type) ? 1 : 0;
  int srcDevDetected = -1;
  // A mapping of somebody else's memory whose owner the caller cannot name (amem_nccl.cpp:119).
  const bool oosFlag = peerFlag && peer_dev == -1;
  Ctx* c = init_ctx(dev);
  {
    std::lock_guard<std::mutex> ls(c->structure);
    std::lock_guard<std::mutex> lf(c->fields);
    if (c->paused) {
      LOGGER(WARN, "Redundant pause: groupID:%d pid:%d NCCL is already paused! DO NOT issue any NCCL op "
             "including memory alloc!", amem_groupID, getpid());
      return 1;
    }
    auto& table = c->allocTable[dev];
    auto it = table.find(va);
    if (it == table.end()) {
      Region r;
      r.dev = dev;
      r.pid = getpid();
      r.allocSz = size;
      r.state = AMEM_STATE_ALLOC;
      r.type = type;
      r.userInfo = user_info;
      r.tags = (size_t)caller;
      r.handle = handle;
      r.mcHandle = peer_handle;  // the ctor's in_mcHandle slot receives peerHandle (amem_nccl.cpp:145)
      r.oosFlag = oosFlag;
      r.handleGen = 1;
      if (peerFlag) r.ownerSlot = peer_dev;
      table.emplace(va, r);
      if (caller >= 0 && caller < AMEM_MAX_CALLER) c->allocBytes[caller] += size;
      if (peerFlag && gpu_present()) srcDevDetected = vmm_handle_device(handle);
      // The first successful add is always printed, later ones only at DEBUG (amem_nccl.cpp:166-178).
      if (c->smokeLog != 0)
        LOGGER(DEBUG, "AllocInfo: add meminfo successfully, groupID:%d pid:%d allocSz:%ld curDev:%d peer:%d "
               "(detected:%d) dptr:%llx type:%s localHandle:%llx rmtHandle:%lx caller:%d", amem_groupID, getpid(),
               (long)size, dev, peer_dev, srcDevDetected, (unsigned long long)va, peerFlag ? "remote" : "local",
               (unsigned long long)handle, (unsigned long)peer_handle, caller);
      else
        LOGGER(INFO, "AllocInfo: add meminfo successfully, groupID:%d pid:%d allocSz:%ld curDev:%d peer:%d "
               "(detected:%d) dptr:%llx type:%s localHandle:%llx rmtHandle:%lx caller:%d", amem_groupID, getpid(),
               (long)size, dev, peer_dev, srcDevDetected, (unsigned long long)va, peerFlag ? "remote" : "local",
               (unsigned long long)handle, (unsigned long)peer_handle, caller);
    } else {
      // Re-registration of a known VA overwrites these fields only (amem_nccl.cpp:179-191).
      LOGGER(WARN, "AllocInfo: find meminfo successfully, groupID:%d pid:%d allocSz:%ld curDev:%d peer:%d "
             "dptr:%llx type:%s localHandle:%llx rmtHandle:%lx caller:%d already exists!", amem_groupID, getpid(),
             (long)size, dev, peer_dev, (unsigned long long)va, peerFlag ? "remote" : "local",
             (unsigned long long)handle, (unsigned long)peer_handle, caller);
      Region& r = it->second;
      r.type = type;
      r.state = AMEM_STATE_ALLOC;
      r.allocSz = size;
      r.handle = handle;
      r.userInfo = user_info;
      r.tags = (size_t)caller;
    }
  }

  auto erase_entry = [&] {
    std::lock_guard<std::mutex> ls(c->structure);
    std::lock_guard<std::mutex> lf(c->fields);
    c->allocTable[dev].erase(va);
  };
  if (peerFlag && peer_dev >= 0) {
    // Case 1: the caller names the owner (amem_nccl.cpp:195-220).
    ret = peer_register(peer_handle, va, peer_dev);
    if (ret != 0) {
      LOGGER(WARN, "ALLocInfo: communication failed. groupID:%d pid:%d allocSz:%ld curDev:%d dptr:%llx "
             "localHandle:%llx rmtHandle:%lx register peer:%d failed, remove metadata", amem_groupID, getpid(),
             (long)size, dev, (unsigned long long)va, (unsigned long long)handle, (unsigned long)peer_handle, peer_dev);
      erase_entry();
    }
  } else if (peerFlag && peer_dev == -1) {
    // Cases 2 and 3 (amem_nccl.cpp:222-256). The handle's properties name a device, which
    // identifies the owner only when every process of the group drives its own GPU and so
    // holds the slot equal to its device ordinal; with several processes on one GPU (the
    // owner's device is then this process's own device) the owner cannot be told apart.
    if (srcDevDetected >= 0 && srcDevDetected != dev) {
      {
        std::lock_guard<std::mutex> lf(c->fields);
        auto it = c->allocTable[dev].find(va);
        if (it != c->allocTable[dev].end()) it->second.ownerSlot = srcDevDetected;
      }
      ret = peer_register(peer_handle, va, srcDevDetected);
      if (ret != 0) {
        LOGGER(WARN, "ALLocInfo: communication failed. groupID:%d pid:%d allocSz:%ld curDev:%d dptr:%llx "
               "localHandle:%llx rmtHandle:%lx register peer:%d failed, remove metadata", amem_groupID, getpid(),
               (long)size, dev, (unsigned long long)va, (unsigned long long)handle, (unsigned long)peer_handle,
               srcDevDetected);
        erase_entry();
      }
    } else {
      LOGGER(ERROR, "ALLocInfo: info is invalid!! may cause inconsistent or hang. groupID:%d pid:%d allocSz:%ld "
             "curDev:%d dptr:%llx localHandle:%llx rmtHandle:%lx peer:%d", amem_groupID, getpid(), (long)size, dev,
             (unsigned long long)va, (unsigned long long)handle, (unsigned long)peer_handle, peer_dev);
      erase_entry();
      ret = 1;
    }
  } else if (!peerFlag) {
    // Case 4: local memory is indexed by handle (amem_nccl.cpp:258-265).
    std::lock_guard<std::mutex> ls(c->structure);
    std::lock_guard<std::mutex> lf(c->fields);   // the service thread looks handles up under `fields`
    c->handleTable[dev].emplace(handle, va);
  }
  {
    std::lock_guard<std::mutex> lf(c->fields);
    c->smokeLog++;
  }
  return ret;
}

int amem_del_alloc_info(uint64_t va, uint64_t handle, int caller) {
  (void)caller;
  Globals& g = globals();
  if (g.disabled > 0) return 0;
  if (va == 0) return 0;
  int curet = 0;
  if (handle == 0 && gpu_present()) handle = vmm_handle_of(va);  // amem_nccl.cpp:423-426
  Ctx* c = ctx_or_null();
  if (!c) return curet;
  const int dev = current_device();
  std::lock_guard<std::mutex> ls(c->structure);
  std::lock_guard<std::mutex> lf(c->fields);
  auto& table = c->allocTable[dev];
  auto it = table.find(va);
  if (it != table.end()) {
    Region& r = it->second;
    if (r.tags < AMEM_MAX_CALLER) c->allocBytes[r.tags] -= r.allocSz;
    else c->delBytes += r.allocSz;
    if (handle == 0) handle = r.handle;
    if (c->paused) {
      if (Engine* en = engine_if_exists(dev)) en->forget(va);  // its parked bytes are dropped
    }
    table.erase(it);
    LOGGER(DEBUG, "groupID:%d pid:%d curDev:%d erase dptr:%llx done", amem_groupID, getpid(), dev,
           (unsigned long long)va);
  }
  c->handleTable[dev].erase(handle);
  return curet;
}

int amem_add_refcount(void* va, int n) {
  if (globals().disabled > 0) return 0;
  Ctx* c = ctx_or_null();
  int ret = 1;
  if (c) {
    const int dev = current_device();
    std::lock_guard<std::mutex> lf(c->fields);
    auto it = c->allocTable[dev].find((uint64_t)(uintptr_t)va);
    if (it != c->allocTable[dev].end()) {
      it->second.refcount += n;
      ret = 0;
      LOGGER(DEBUG, "Add refcount: success. groupID:%d pid:%d dptr:%p add refcount:%d", amem_groupID, getpid(), va, n);
    }
  }
  if (ret)
    LOGGER(ERROR, "Add refcount: failed to find metadata. groupID:%d pid:%d dptr:%p when adding refcount:%d",
           amem_groupID, getpid(), va, n);
  return ret;
}

int amem_add_peer_info(uint64_t src_va, uint64_t peer_va, int peer_dev) {
  Ctx* c = ctx_or_null();
  int ret = 1;
  if (c && peer_dev >= 0 && peer_dev < AMEM_MAX_DEVS) {
    const int dev = current_device();
    std::lock_guard<std::mutex> lf(c->fields);
    auto it = c->allocTable[dev].find(src_va);
    if (it != c->allocTable[dev].end()) {
      it->second.peers[peer_dev] = peer_va;
      it->second.hasPeer = true;
      ret = 0;
    }
  }
  if (ret)
    LOGGER(ERROR, "Add peerInfo: failed to find localDptr. groupID:%d pid:%d failed to find for localDptr:%llx "
           "to register peer:%d peerPtr:%llx", amem_groupID, getpid(), (unsigned long long)src_va, peer_dev,
           (unsigned long long)peer_va);
  return ret;
}

// The two handlers below run on the service thread, whose current device is the one the service
// was started on; a process that drives several GPUs keeps one table per device, so the entry is
// looked for in all of them (addresses and handles are unique within a process).
int amem_register_peer_info(uint64_t src_handle, uint64_t peer_va, int peer_dev) {
  Ctx* c = ctx_or_null();
  int ret = 1;
  if (c && peer_dev >= 0 && peer_dev < AMEM_MAX_DEVS) {
    std::lock_guard<std::mutex> lf(c->fields);
    for (int dev = 0; dev < AMEM_MAX_DEVS && ret; ++dev) {
      auto ht = c->handleTable[dev].find(src_handle);
      auto it = c->allocTable[dev].end();
      if (ht != c->handleTable[dev].end()) {
        it = c->allocTable[dev].find(ht->second);
      } else {
        // Not a handle of this process: an importer that cannot know the current handle value (it changes
        // with every resume) may name the region by the owner's address instead, which never changes.
        it = c->allocTable[dev].find(src_handle);
        if (it != c->allocTable[dev].end() && from_peer(it->second.type)) it = c->allocTable[dev].end();
      }
      if (it == c->allocTable[dev].end()) continue;
      it->second.peers[peer_dev] = peer_va;
      it->second.hasPeer = true;
      ret = 0;
      LOGGER(DEBUG, "groupID:%d pid:%d localDptr:%llx localHandle:%llx register peer:%d peerPtr:%llx done",
             amem_groupID, getpid(), (unsigned long long)it->first, (unsigned long long)src_handle, peer_dev,
             (unsigned long long)peer_va);
    }
  }
  if (ret)
    LOGGER(ERROR, "groupID:%d pid:%d failed to find info for handle:%llx to register peer:%d peerPtr:%llx",
           amem_groupID, getpid(), (unsigned long long)src_handle, peer_dev, (unsigned long long)peer_va);
  return ret;
}

int amem_update_peer_info(uint64_t va, int shared_fd) {
  Ctx* c = ctx_or_null();
  if (!c) { if (shared_fd >= 0) close(shared_fd); return 1; }
  int dev = -1;
  size_t size = 0;
  int state = AMEM_STATE_INVALID;
  const bool gpu = gpu_present();
  {
    // Only an address that a pause has emptied can take new memory. The CUDA driver refuses to map
    // over an existing mapping; this HIP runtime accepts it (measured) and the old mapping would be
    // lost without being unmapped. So the hole is claimed here, under the lock: of two updates for one
    // address (a retried owner resume, two service threads of one process) the second finds it taken.
    std::lock_guard<std::mutex> lf(c->fields);
    for (int d = 0; d < AMEM_MAX_DEVS && dev < 0; ++d) {
      auto it = c->allocTable[d].find(va);
      if (it == c->allocTable[d].end()) continue;
      dev = d;
      size = it->second.allocSz;
      state = it->second.state;
      if (state == AMEM_STATE_HOLE && gpu) it->second.state = AMEM_STATE_PRELOADING;
    }
  }
  if (dev < 0) {
    LOGGER(ERROR, "groupID:%d pid:%d failed to find info for dptr:%llx to remap fd:%x", amem_groupID, getpid(),
           (unsigned long long)va, shared_fd);
    if (shared_fd >= 0) close(shared_fd);
    return 1;
  }
  if (state != AMEM_STATE_HOLE) {
    LOGGER(ERROR, "groupID:%d pid:%d dptr:%llx is not released (state %d): refusing to map fd:%d over it", amem_groupID,
           getpid(), (unsigned long long)va, state, shared_fd);
    if (shared_fd >= 0) close(shared_fd);
    return 1;
  }
  if (!gpu) {
    LOGGER(ERROR, "pid:%d no HIP device: cannot import fd:%d", getpid(), shared_fd);
    close(shared_fd);
    return 1;
  }
  uint64_t newh = 0;
  int ret = (int)vmm_import_map(dev, va, size, shared_fd, true, &newh);  // amem_importAndMap
  {
    std::lock_guard<std::mutex> lf(c->fields);
    auto it = c->allocTable[dev].find(va);
    if (it != c->allocTable[dev].end() && it->second.state == AMEM_STATE_PRELOADING) {
      if (ret == 0) {
        it->second.state = AMEM_STATE_ALLOC;
        it->second.handle = newh;
        it->second.handleGen++;
      } else {
        it->second.state = AMEM_STATE_HOLE;  // nothing is mapped: a later update may try again
      }
    }
    if (ret == 0) {
      c->releaseShadowCnt--;
      c->shadow_cv.notify_all();
    }
  }
  if (ret == 0)
    LOGGER(DEBUG, "groupID:%d pid:%d curDev:%d update ptr:%llx fd:%d done", amem_groupID, getpid(), dev,
           (unsigned long long)va, shared_fd);
  return ret;
}

int amem_check_paused(int warn) {
  if (globals().disabled > 0) return 0;
  Ctx* c = ctx_or_null();
  if (!c) return 0;
  std::lock_guard<std::mutex> lf(c->fields);
  if (warn && c->paused) {
    LOGGER(ERROR, "groupID:%d pid:%d NCCL of current process is already paused! DO NOT issue any NCCL op!",
           amem_groupID, getpid());
    log_backtrace();  // who issued it (amem_nccl.cpp:461)
  }
  return c->paused ? 1 : 0;
}

int amem_set_group_id(int id) {
  if (globals().disabled > 0) return 0;
  if (!ctx_or_null()) {
    LOGGER(INFO, "groupID:%d (old) pid:%d, set as new groupID:%d done", amem_groupID, getpid(), id);
    amem_groupID = id;
    return 0;
  }
  LOGGER(WARN, "groupID:%d pid:%d, trying to set to new groupID:%d, reject as to late", amem_groupID, getpid(), id);
  return 1;
}

void amem_get_group_id(int* id) {
  if (globals().disabled > 0) return;
  if (id) *id = amem_groupID;
}

void amem_dump_alloc_stats(int verbose) {
  if (globals().disabled > 0) return;
  Ctx* c = ctx_or_null();
  size_t total = 0, del = 0;
  size_t by_caller[AMEM_MAX_CALLER] = {0};
  if (c) {
    std::lock_guard<std::mutex> lf(c->fields);
    memcpy(by_caller, c->allocBytes, sizeof(by_caller));
    del = c->delBytes;
  }
  for (int i = 0; i < AMEM_MAX_CALLER; ++i) {
    if (by_caller[i] != 0 && verbose)
      LOGGER(DEBUG, "DumpStats: groupID:%d pid:%d caller_%d allocBytes:%ld", amem_groupID, getpid(), i, (long)by_caller[i]);
    total += by_caller[i];
  }
  total += del;
  LOGGER(DEBUG, "DumpStats in total: groupID:%d pid:%d total GPU alloc:%ld (%ld MB), note including those mapped "
         "from peer, and defensive skiped %ld MB", amem_groupID, getpid(), (long)total, (long)(total >> 20), (long)(del >> 20));
}

int amem_mem_pause(int pid, uint64_t tag) {
  (void)pid; (void)tag;
  LOGGER(DEBUG, "memPause: start here.");
  if (globals().disabled > 0) return 0;
  Ctx* c = ctx_or_null();
  if (!c) return 0;
  const int dev = current_device();
  std::lock_guard<std::mutex> ls(c->structure);
  {
    std::lock_guard<std::mutex> lf(c->fields);
    if (c->paused) return 0;  // idempotent (amem_nccl.cpp:481-488)
    c->paused = true;
  }
  if (c->allocTable[dev].empty()) return 0;
  Engine* en = engine_for(dev);
  if (!en) {
    std::lock_guard<std::mutex> lf(c->fields);
    c->paused = false;
    return (int)hipErrorNoDevice;
  }
  bool rolled_back = false;
  int ret = en->pause(*c, &rolled_back);
  if (rolled_back) {
    std::lock_guard<std::mutex> lf(c->fields);
    c->paused = false;
  }
  return ret;
}

int amem_mem_resume(int pid, uint64_t tag) {
  (void)pid; (void)tag;
  LOGGER(DEBUG, "memResume: start here.");
  if (globals().disabled > 0) return 0;
  Ctx* c = ctx_or_null();
  if (!c) return 0;
  const int dev = current_device();
  std::lock_guard<std::mutex> ls(c->structure);
  {
    std::lock_guard<std::mutex> lf(c->fields);
    if (!c->paused) return 0;  // idempotent (amem_nccl.cpp:589-594)
  }
  int ret = 0;
  if (!c->allocTable[dev].empty()) {
    Engine* en = engine_for(dev);
    if (!en) return (int)hipErrorNoDevice;
    bool incomplete = false;
    ret = en->resume(*c, &incomplete);
    if (incomplete) return ret;  // still paused: a later resume picks up the remaining regions
  }
  std::lock_guard<std::mutex> lf(c->fields);
  c->paused = false;
  c->resumeCnt++;
  return ret;
}

int ncclPause(void* comm) { (void)comm; (void)amem_mem_pause((int)getpid(), 0); return 0; }
int ncclResume(void* comm) { (void)comm; (void)amem_mem_resume((int)getpid(), 0); return 0; }
int ncclMemStats(void) { amem_dump_alloc_stats(1); return 0; }
int ncclSetGroupID(int id) { return amem_set_group_id(id); }
int ncclGetGroupID(int* id) { amem_get_group_id(id); return 0; }

// ---- VMM helpers ----

static int need_gpu(const char* what) {
  if (gpu_present()) return 0;
  LOGGER(ERROR, "pid:%d %s needs a HIP device and none is visible", getpid(), what);
  return (int)hipErrorNoDevice;
}

int amem_vmm_alloc(uint64_t bytes, int dev, uint64_t* va, uint64_t* handle, uint64_t* alloc_size) {
  if (int e = need_gpu("amem_vmm_alloc")) return e;
  size_t sz = 0;
  int e = (int)vmm_alloc(bytes, dev, va, handle, &sz);
  if (alloc_size) *alloc_size = sz;
  return e;
}
int amem_vmm_free(uint64_t va, uint64_t alloc_size, uint64_t handle) {
  if (int e = need_gpu("amem_vmm_free")) return e;
  return (int)vmm_free(va, alloc_size, handle);
}
int amem_vmm_export(uint64_t handle, int* fd) {
  if (int e = need_gpu("amem_vmm_export")) return e;
  return (int)vmm_export_fd(handle, fd);
}
int amem_vmm_import(int fd, uint64_t size, int dev, uint64_t* va, uint64_t* handle) {
  if (int e = need_gpu("amem_vmm_import")) return e;
  void* ptr = nullptr;
  hipError_t e = CHECK_HIP(hipMemAddressReserve(&ptr, size, kVmmAlign, nullptr, 0));
  if (e != hipSuccess) return (int)e;
  e = vmm_import_map(dev, (uint64_t)(uintptr_t)ptr, size, fd, false, handle);
  if (e != hipSuccess) { (void)hipMemAddressFree(ptr, size); return (int)e; }
  *va = (uint64_t)(uintptr_t)ptr;
  return 0;
}

// ---- inspection ----

int64_t amem_region_count(int dev) {
  Ctx* c = ctx_or_null();
  if (!c || dev < 0 || dev >= AMEM_MAX_DEVS) return 0;
  std::lock_guard<std::mutex> ls(c->structure);
  return (int64_t)c->allocTable[dev].size();
}
int amem_region_at(int dev, int64_t index, amem_region_info* out) {
  Ctx* c = ctx_or_null();
  if (!c || !out || dev < 0 || dev >= AMEM_MAX_DEVS || index < 0) return 1;
  std::lock_guard<std::mutex> ls(c->structure);
  std::lock_guard<std::mutex> lf(c->fields);
  auto& t = c->allocTable[dev];
  if ((size_t)index >= t.size()) return 1;
  auto it = t.begin();
  std::advance(it, index);
  fill_info(it->first, it->second, out);
  return 0;
}
int amem_region_find(int dev, uint64_t va, amem_region_info* out) {
  Ctx* c = ctx_or_null();
  if (!c || !out || dev < 0 || dev >= AMEM_MAX_DEVS) return 1;
  std::lock_guard<std::mutex> ls(c->structure);
  std::lock_guard<std::mutex> lf(c->fields);
  auto it = c->allocTable[dev].find(va);
  if (it == c->allocTable[dev].end()) return 1;
  fill_info(it->first, it->second, out);
  return 0;
}
uint64_t amem_handle_lookup(int dev, uint64_t handle) {
  Ctx* c = ctx_or_null();
  if (!c || dev < 0 || dev >= AMEM_MAX_DEVS) return 0;
  std::lock_guard<std::mutex> ls(c->structure);
  std::lock_guard<std::mutex> lf(c->fields);
  auto it = c->handleTable[dev].find(handle);
  return it == c->handleTable[dev].end() ? 0 : it->second;
}
int64_t amem_handle_count(int dev) {
  Ctx* c = ctx_or_null();
  if (!c || dev < 0 || dev >= AMEM_MAX_DEVS) return 0;
  std::lock_guard<std::mutex> ls(c->structure);
  return (int64_t)c->handleTable[dev].size();
}
void amem_get_counters(amem_counters* out) {
  if (!out) return;
  memset(out, 0, sizeof(*out));
  out->group_id = amem_groupID;
  out->enabled = globals().disabled > 0 ? 0 : 1;
  out->slot = ipc_slot();
  Ctx* c = ctx_or_null();
  if (!c) return;
  std::lock_guard<std::mutex> lf(c->fields);
  out->release_local_cnt = c->releaseLocalCnt;
  out->release_shadow_cnt = c->releaseShadowCnt;
  out->offload_cnt = c->offloadCnt;
  out->smoke_log = c->smokeLog;
  for (int i = 0; i < AMEM_MAX_CALLER; ++i) out->alloc_bytes[i] = c->allocBytes[i];
  out->del_bytes = c->delBytes;
  out->pause_cnt = c->pauseCnt;
  out->resume_cnt = c->resumeCnt;
  out->paused = c->paused;
}
void amem_get_cycle_stats(amem_cycle_stats* out) {
  if (!out) return;
  memset(out, 0, sizeof(*out));
  if (!gpu_present()) return;
  if (Engine* en = engine_if_exists(current_device())) *out = en->stats();
}

// ---- controls ----

int amem_set_enabled(int on) {
  Ctx* c = ctx_or_null();
  if (c) {
    std::lock_guard<std::mutex> ls(c->structure);
    for (int d = 0; d < AMEM_MAX_DEVS; ++d) if (!c->allocTable[d].empty()) return 1;
  }
  globals().disabled = on ? 0 : 1;
  return 0;
}

struct OptRef { const char* name; int64_t* p; int64_t lo, hi; };
static OptRef* opt_table(size_t* n) {
  Options& o = options();
  static OptRef t[] = {
      {"zero_elide", &o.zero_elide, 0, 1},
      {"verify", &o.verify, 0, 1},
      {"pause_path", &o.pause_path, 0, 4},
      {"interleave_bytes", &o.interleave_bytes, 1 << 16, (int64_t)1 << 40},
      {"pause_xcds", &o.pause_xcds, 0, 8},
      {"pause_wgs", &o.pause_wgs, 0, 65536},
      {"dma_min_bytes", &o.dma_min_bytes, 0, (int64_t)1 << 40},
      {"staging_bytes", &o.staging_bytes, 0, (int64_t)1 << 36},
      {"slab_bytes", &o.slab_bytes, 1 << 16, (int64_t)1 << 36},
      {"link_wgs", &o.link_wgs, 1, 65536},
      {"hbm_wgs", &o.hbm_wgs, 1, 1 << 20},
      {"hbm_move_wgs", &o.hbm_move_wgs, 1, (int64_t)1 << 30},
      {"resume_batch_bytes", &o.resume_batch_bytes, 1, (int64_t)1 << 40},
      {"resume_dma_min_bytes", &o.resume_dma_min_bytes, 0, (int64_t)1 << 40},
      {"peer_timeout_ms", &o.peer_timeout_ms, 0, (int64_t)1 << 40},
      {"peer_loopback", &o.peer_loopback, 0, 1},
      {"offload_free_tag", &o.offload_free_tag, -1, AMEM_MAX_CALLER - 1},
      {"pool_limit_bytes", &o.pool_limit_bytes, 0, (int64_t)1 << 46},
      {"scratch_on_host", &o.scratch_on_host, 0, 1},
      {"release_thread", &o.release_thread, 0, 1},
      {"pause_adaptive", &o.pause_adaptive, 0, 1},
  };
  *n = sizeof(t) / sizeof(t[0]);
  return t;
}
int amem_set_option(const char* name, int64_t value) {
  size_t n;
  OptRef* t = opt_table(&n);
  for (size_t i = 0; name && i < n; ++i) {
    if (strcmp(t[i].name, name) == 0) {
      if (value < t[i].lo || value > t[i].hi) return 1;
      if (strcmp(name, "slab_bytes") == 0 && (value & (value - 1))) return 1;
      Ctx* c = ctx_or_null();
      if (c) {
        std::lock_guard<std::mutex> lf(c->fields);
        if (c->paused) return 1;  // the layout of parked bytes depends on the options
      }
      *t[i].p = value;
      return 0;
    }
  }
  return 1;
}
int64_t amem_get_option(const char* name) {
  size_t n;
  OptRef* t = opt_table(&n);
  for (size_t i = 0; name && i < n; ++i)
    if (strcmp(t[i].name, name) == 0) return *t[i].p;
  return -1;
}

uint64_t amem_pool_trim(void) {
  if (!gpu_present()) return 0;
  Engine* en = engine_if_exists(current_device());
  if (!en) return 0;
  Ctx* c = ctx_or_null();
  if (!c) return en->trim_pool();
  std::lock_guard<std::mutex> ls(c->structure);  // not while a pause or resume is running
  {
    std::lock_guard<std::mutex> lf(c->fields);
    if (c->paused) return 0;  // the pool holds the parked bytes
  }
  return en->trim_pool();
}

int amem_pool_reserve(uint64_t bytes) {
  if (int e = need_gpu("amem_pool_reserve")) return e;
  Engine* en = engine_for(current_device());
  if (!en) return (int)hipErrorNoDevice;
  return (int)en->reserve_pool(bytes);
}

int amem_shutdown(void) {
  Globals& g = globals();
  std::lock_guard<std::mutex> lk(g.init_mtx);
  Ctx* c = g.ctx;
  if (c) {
    std::lock_guard<std::mutex> lf(c->fields);
    if (c->paused) return 1;
  }
  ipc_stop();
  destroy_engines();
  delete c;
  g.ctx = nullptr;
  return 0;
}

int amem_ipc_start(void) {
  return ipc_start(current_device());
}
int amem_get_slot(void) { return ipc_slot(); }
int amem_ipc_claim_slot(void) {
  if (ipc_slot() < 0 && ipc_start(current_device()) < 0) return -1;
  return ipc_claim_extra();
}
int amem_ipc_act_as(int slot) { return ipc_act_as(slot); }
int amem_ipc_served(int slot, uint64_t counts[3]) { return counts ? ipc_served(slot, counts) : 1; }
int amem_ipc_peer_alive(int slot) { return peer_alive(slot) ? 1 : 0; }

// ---- kernels on their own ----

uint64_t amem_chunk_count(const amem_extent* extents, uint64_t n) {
  uint64_t c = 0;
  for (uint64_t i = 0; i < n; ++i) c += (extents[i].bytes + AMEM_CHUNK_BYTES - 1) / AMEM_CHUNK_BYTES;
  return c;
}
int amem_zero_scan(const amem_extent* extents, uint64_t n, uint8_t* flags, amem_chunk_sum* sums, float* kernel_ms) {
  if (int e = need_gpu("amem_zero_scan")) return e;
  Engine* en = engine_for(current_device());
  if (!en) return (int)hipErrorNoDevice;
  return (int)en->zero_scan(extents, n, flags, sums, kernel_ms);
}
int amem_zero_scan_noalloc(const amem_extent* extents, uint64_t n, uint8_t* flags, amem_chunk_sum* sums,
                           float* kernel_ms) {
  if (int e = need_gpu("amem_zero_scan_noalloc")) return e;
  Engine* en = engine_for(current_device());  // creates the device's engine on the first call only
  if (!en) return (int)hipErrorNoDevice;
  return (int)en->zero_scan_noalloc(extents, n, flags, sums, kernel_ms);
}
int amem_gather_pack(const amem_copy_desc* descs, uint64_t n, void* staging, uint64_t staging_bytes, int host_side,
                     float* kernel_ms) {
  if (int e = need_gpu("amem_gather_pack")) return e;
  Engine* en = engine_for(current_device());
  if (!en) return (int)hipErrorNoDevice;
  return (int)en->move(false, descs, n, staging, staging_bytes, host_side != 0, kernel_ms);
}
int amem_scatter_unpack(const amem_copy_desc* descs, uint64_t n, const void* staging, uint64_t staging_bytes,
                        int host_side, float* kernel_ms) {
  if (int e = need_gpu("amem_scatter_unpack")) return e;
  Engine* en = engine_for(current_device());
  if (!en) return (int)hipErrorNoDevice;
  return (int)en->move(true, descs, n, (void*)staging, staging_bytes, host_side != 0, kernel_ms);
}
int amem_probe_link(uint64_t bytes, int reps, double* d2h_gbps, double* h2d_gbps) {
  if (int e = need_gpu("amem_probe_link")) return e;
  Engine* en = engine_for(current_device());
  if (!en) return (int)hipErrorNoDevice;
  return (int)en->probe_link(bytes, reps, d2h_gbps, h2d_gbps);
}
int amem_calib_copy(uint64_t bytes, int reps, float* kernel_ms) {
  if (int e = need_gpu("amem_calib_copy")) return e;
  Engine* en = engine_for(current_device());
  if (!en) return (int)hipErrorNoDevice;
  return (int)en->calib_copy(bytes, reps, kernel_ms);
}
int amem_copy_to_device(uint64_t va, const void* host, uint64_t bytes) {
  if (int e = need_gpu("amem_copy_to_device")) return e;
  return (int)CHECK_HIP(hipMemcpy((void*)(uintptr_t)va, host, bytes, hipMemcpyHostToDevice));
}
int amem_copy_from_device(void* host, uint64_t va, uint64_t bytes) {
  if (int e = need_gpu("amem_copy_from_device")) return e;
  return (int)CHECK_HIP(hipMemcpy(host, (const void*)(uintptr_t)va, bytes, hipMemcpyDeviceToHost));
}
int amem_device_mem_info(uint64_t* free_bytes, uint64_t* total_bytes) {
  if (int e = need_gpu("amem_device_mem_info")) return e;
  size_t f = 0, t = 0;
  int e = (int)CHECK_HIP(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return e;
}
int amem_device_count(void) { return gpu_present() ? g_device_count : 0; }
int amem_device_pci_bus_id(char* out, int len) {
  if (int e = need_gpu("amem_device_pci_bus_id")) return e;
  if (!out || len < 13) return 1;
  return (int)CHECK_HIP(hipDeviceGetPCIBusId(out, len, current_device()));
}
int amem_probe_unmap(int count, uint64_t bytes, double* unmap_us_p50, double* unmap_us_mean, double* map_us_mean) {
  if (int e = need_gpu("amem_probe_unmap")) return e;
  if (count < 1 || count > 4096 || bytes == 0) return 1;
  const int dev = current_device();
  struct M { uint64_t va, handle; size_t size; };
  std::vector<M> maps;
  hipError_t e = hipSuccess;
  // addresses first, so that the timed triple is what a resume does: create, map, grant access
  for (int i = 0; i < count && e == hipSuccess; ++i) {
    void* ptr = nullptr;
    const size_t size = (bytes + kVmmAlign - 1) / kVmmAlign * kVmmAlign;
    e = CHECK_HIP(hipMemAddressReserve(&ptr, size, kVmmAlign, nullptr, 0));
    if (e == hipSuccess) maps.push_back({(uint64_t)(uintptr_t)ptr, 0, size});
  }
  double map_us = 0;
  size_t mapped = 0;
  for (; mapped < maps.size() && e == hipSuccess; ++mapped) {
    const auto t0 = std::chrono::steady_clock::now();
    e = vmm_create_map(maps[mapped].va, dev, maps[mapped].size, &maps[mapped].handle);
    map_us += std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    if (e != hipSuccess) break;
  }
  (void)CHECK_HIP(hipDeviceSynchronize());
  std::vector<double> us;
  for (size_t i = 0; i < mapped; ++i) {
    const auto t0 = std::chrono::steady_clock::now();
    hipError_t e2 = vmm_unmap(maps[i].va, maps[i].size);
    us.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
    if (e == hipSuccess) e = e2;
  }
  for (size_t i = 0; i < mapped; ++i) (void)vmm_release(maps[i].handle, 0);
  for (const M& m : maps) (void)hipMemAddressFree((void*)(uintptr_t)m.va, m.size);
  if (!us.empty()) {
    double sum = 0;
    for (double v : us) sum += v;
    std::sort(us.begin(), us.end());
    if (unmap_us_p50) *unmap_us_p50 = us[us.size() / 2];
    if (unmap_us_mean) *unmap_us_mean = sum / us.size();
    if (map_us_mean) *map_us_mean = map_us / us.size();
  }
  return (int)e;
}

}  // extern "C"

// ---------------------------------------------------------------------------------------
// The reference's C++-linkage names (amem_nccl.h:330-367), forwarding to the C ABI.
// ---------------------------------------------------------------------------------------

int amem_registerPeerInfo(amem_handle_t srcHandle, amem_dptr_t peerPtr, int peerDev) {
  return amem_register_peer_info(srcHandle, peerPtr, peerDev);
}
int amem_addPeerInfo(amem_dptr_t srcPtr, amem_dptr_t peerPtr, int peerDev) {
  return amem_add_peer_info(srcPtr, peerPtr, peerDev);
}
int amem_updatePeerInfo(amem_dptr_t dptr, int sharedFD) { return amem_update_peer_info(dptr, sharedFD); }
int amem_addAllocInfo(amem_dptr_t localDptr, size_t allocSz, int type, int localDev, amem_handle_t localHandle,
                      int peerDev, uint64_t peerHandle, void* userInfo, amem_caller_type caller_type) {
  return amem_add_alloc_info(localDptr, allocSz, type, localDev, localHandle, peerDev, peerHandle, userInfo,
                             (int)caller_type);
}
int amem_delAllocInfo(amem_dptr_t dptr, amem_handle_t handle, int caller) {
  return amem_del_alloc_info(dptr, handle, caller);
}
int amem_memPause(pid_t pid, uint64_t tag) { return amem_mem_pause((int)pid, tag); }
int amem_memResume(pid_t pid, uint64_t tag) { return amem_mem_resume((int)pid, tag); }
void amem_dumpAllocStats(bool verbose) { amem_dump_alloc_stats(verbose ? 1 : 0); }
bool amem_checkPaused(bool warn) { return amem_check_paused(warn ? 1 : 0) != 0; }
int amem_addRefcount(void* dptr, int refcount) { return amem_add_refcount(dptr, refcount); }
int amem_setGroupID(int id) { return amem_set_group_id(id); }
void amem_getGroupID(int* id) { amem_get_group_id(id); }

// Library load / unload (x_init / x_fini, amem_nccl.cpp:706-729). Unlike the reference,
// loading does not delete other processes' rendezvous files.
static void __attribute__((constructor)) amem_lib_init(void) {
  set_log_level_from_env();
  Globals& g = globals();
  g.disabled = getenv("AMEM_ENABLE") ? !atoi(getenv("AMEM_ENABLE")) : 1;
  g.offload_free_tag = getenv("AMEM_NCCL_OFFLOAD_FREE_TAG") ? atoi(getenv("AMEM_NCCL_OFFLOAD_FREE_TAG")) : -1;
  amem_groupID = getenv("AMEM_GROUPID") ? atoi(getenv("AMEM_GROUPID")) : 0;
  int cuMemFlag = getenv("NCCL_CUMEM_ENABLE") ? atoi(getenv("NCCL_CUMEM_ENABLE")) : 1;
  if (cuMemFlag == 0) g.disabled = 1;
  // The reference parses the tag (amem_nccl.cpp:478, :587) and then compares against a macro, so the
  // variable never acts there and regions of every tag keep their bytes. By default this library
  // does the same. With AMEM_OFFLOAD_FREE_TAG_APPLY=1 the variable takes effect: it selects the
  // caller tag whose regions are released without being copied and come back zero-filled, which is
  // what the reference's README documents (README.md:224, run.sh:9-18).
  const bool apply_tag = getenv("AMEM_OFFLOAD_FREE_TAG_APPLY") && atoi(getenv("AMEM_OFFLOAD_FREE_TAG_APPLY")) != 0;
  if (g.offload_free_tag >= 0 && g.offload_free_tag < AMEM_MAX_CALLER) {
    if (apply_tag) {
      options().offload_free_tag = g.offload_free_tag;
      LOGGER(WARN, "groupID:%d pid:%d AMEM_NCCL_OFFLOAD_FREE_TAG=%d is applied: regions registered with caller tag %d "
             "are released without a copy and come back ZERO-FILLED after resume (the reference keeps their bytes)",
             amem_groupID, getpid(), g.offload_free_tag, g.offload_free_tag);
    } else if (!g.disabled) {
      LOGGER(INFO, "groupID:%d pid:%d AMEM_NCCL_OFFLOAD_FREE_TAG=%d is read but not applied, as in the reference "
             "(regions of every tag keep their bytes); set AMEM_OFFLOAD_FREE_TAG_APPLY=1 to release regions of that "
             "tag without a copy", amem_groupID, getpid(), g.offload_free_tag);
    }
  }
  LOGGER(INFO, "groupID:%d pid:%d build:%s %s NCCL plugin loaded. pause func:%s offload_free_tag:%d cuMemEnabled:%d",
         amem_groupID, getpid(), __DATE__, __TIME__, g.disabled ? "Off" : "On", g.offload_free_tag, cuMemFlag);
}

static void __attribute__((destructor)) amem_lib_fini(void) {
  ipc_stop();
  LOGGER(INFO, "groupID:%d pid:%d exit", amem_groupID, getpid());
}
