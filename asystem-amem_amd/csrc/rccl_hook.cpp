// libamem_rccl_hook.so — the allocator hook for an unpatched RCCL.
//
// The reference feeds its registry from call sites patched into NCCL's source
// (nccl_patch/nccl_2.27.5-1.diff: ncclCuMemAlloc :278-280, ncclMemAlloc :41-47,
// ncclCuMemFree :288-290, ...). RCCL is not patched here. Instead this small library is put
// in front of the HIP runtime in symbol lookup order (LD_PRELOAD, or loaded RTLD_GLOBAL before
// librccl.so) and defines the HIP virtual-memory calls RCCL makes. Every call is forwarded to
// the real runtime; those that come from librccl.so are also mirrored into the registry:
//
//   hipMemMap(ptr, size, handle)   remembers the pending mapping
//   hipMemSetAccess(ptr, size)     the mapping is now usable  -> amem_add_alloc_info(ptr, size, LOCAL, dev, handle)
//   hipMemUnmap(ptr, size)         the mapping is going away  -> amem_del_alloc_info(ptr) first
//   hipMemImportFromShareableHandle remembers imported handles: their mappings are another
//                                  process's memory and are not registered by this hook
//
// Calls made by anything else (the pause/resume engine itself, the application) pass through
// untouched. The module a call comes from is found from its return address.
#define _GNU_SOURCE 1
#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <unordered_map>
#include <unordered_set>

#include <hip/hip_runtime_api.h>

#include "../../include/amem.h"

#define HOOK_API extern "C" __attribute__((visibility("default")))

namespace {

struct Pending {
  size_t size;
  uint64_t handle;
};

std::mutex g_mtx;
std::unordered_map<uint64_t, Pending> g_mapped;      // RCCL mappings seen at hipMemMap
std::unordered_set<uint64_t> g_registered;           // those handed to the registry
std::unordered_set<uint64_t> g_imported_handles;     // handles RCCL imported from a peer
int g_verbose = -1;

bool verbose() {
  if (g_verbose < 0) g_verbose = getenv("AMEM_HOOK_LOG") ? atoi(getenv("AMEM_HOOK_LOG")) : 0;
  return g_verbose > 0;
}

template <typename F>
F real(const char* name) {
  void* p = dlsym(RTLD_NEXT, name);
  if (!p) {
    fprintf(stderr, "AMEM [FATAL] rccl_hook: the HIP runtime does not define %s\n", name);
    abort();
  }
  return (F)p;
}

// True when `ret` is an address inside librccl.so.
bool from_rccl(void* ret) {
  static thread_local uintptr_t lo = 0, hi = 0;   // last code range found to be RCCL's
  static thread_local uintptr_t nlo = 0, nhi = 0; // last code range found not to be
  const uintptr_t a = (uintptr_t)ret;
  if (a >= lo && a < hi) return true;
  if (a >= nlo && a < nhi) return false;
  Dl_info info;
  if (!dladdr(ret, &info) || !info.dli_fname) return false;
  const char* base = strrchr(info.dli_fname, '/');
  base = base ? base + 1 : info.dli_fname;
  const bool is_rccl = strncmp(base, "librccl", 7) == 0;
  // remember a 4 KiB window around the address; good enough to skip dladdr on hot call sites
  if (is_rccl) { lo = a & ~(uintptr_t)4095; hi = lo + 4096; }
  else { nlo = a & ~(uintptr_t)4095; nhi = nlo + 4096; }
  return is_rccl;
}

}  // namespace

HOOK_API hipError_t hipMemMap(void* ptr, size_t size, size_t offset, hipMemGenericAllocationHandle_t handle,
                              unsigned long long flags) {
  static auto fn = real<hipError_t (*)(void*, size_t, size_t, hipMemGenericAllocationHandle_t, unsigned long long)>("hipMemMap");
  hipError_t e = fn(ptr, size, offset, handle, flags);
  if (verbose() && g_verbose > 1) {
    Dl_info info;
    fprintf(stderr, "AMEM [VERB] rccl_hook: hipMemMap(%p, %zu) called from %s\n", ptr, size,
            dladdr(__builtin_return_address(0), &info) && info.dli_fname ? info.dli_fname : "?");
  }
  if (e == hipSuccess && from_rccl(__builtin_return_address(0))) {
    std::lock_guard<std::mutex> lk(g_mtx);
    g_mapped[(uint64_t)(uintptr_t)ptr] = {size, (uint64_t)(uintptr_t)handle};
    if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: map %p size %zu handle %p\n", ptr, size, (void*)handle);
  }
  return e;
}

HOOK_API hipError_t hipMemSetAccess(void* ptr, size_t size, const hipMemAccessDesc* desc, size_t count) {
  static auto fn = real<hipError_t (*)(void*, size_t, const hipMemAccessDesc*, size_t)>("hipMemSetAccess");
  hipError_t e = fn(ptr, size, desc, count);
  if (e != hipSuccess || !from_rccl(__builtin_return_address(0))) return e;
  Pending p = {0, 0};
  bool fresh = false;
  {
    std::lock_guard<std::mutex> lk(g_mtx);
    auto it = g_mapped.find((uint64_t)(uintptr_t)ptr);
    if (it != g_mapped.end() && !g_imported_handles.count(it->second.handle)) {
      p = it->second;
      fresh = g_registered.insert((uint64_t)(uintptr_t)ptr).second;
    }
  }
  if (fresh) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    // the shape of the reference's hook in ncclCuMemAlloc (nccl_patch/nccl_2.27.5-1.diff:278-280)
    int rc = amem_add_alloc_info((uint64_t)(uintptr_t)ptr, p.size, AMEM_TYPE_LOCAL, dev, p.handle, -1, 0, NULL,
                                 AMEM_CALLER_DEFAULT);
    if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: registered %p size %zu rc %d\n", ptr, p.size, rc);
    if (rc != 0) {
      std::lock_guard<std::mutex> lk(g_mtx);
      g_registered.erase((uint64_t)(uintptr_t)ptr);
    }
  }
  return e;
}

HOOK_API hipError_t hipMemUnmap(void* ptr, size_t size) {
  static auto fn = real<hipError_t (*)(void*, size_t)>("hipMemUnmap");
  if (from_rccl(__builtin_return_address(0))) {
    bool was_registered;
    {
      std::lock_guard<std::mutex> lk(g_mtx);
      was_registered = g_registered.erase((uint64_t)(uintptr_t)ptr) > 0;
      g_mapped.erase((uint64_t)(uintptr_t)ptr);
    }
    // the shape of the reference's hook in ncclCuMemFree (nccl_patch/nccl_2.27.5-1.diff:288-290)
    if (was_registered) (void)amem_del_alloc_info((uint64_t)(uintptr_t)ptr, 0, 0);
    if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: unmap %p size %zu registered %d\n", ptr, size, (int)was_registered);
  }
  return fn(ptr, size);
}

HOOK_API hipError_t hipMemImportFromShareableHandle(hipMemGenericAllocationHandle_t* handle, void* osHandle,
                                                    hipMemAllocationHandleType shHandleType) {
  static auto fn = real<hipError_t (*)(hipMemGenericAllocationHandle_t*, void*, hipMemAllocationHandleType)>(
      "hipMemImportFromShareableHandle");
  hipError_t e = fn(handle, osHandle, shHandleType);
  if (e == hipSuccess && handle && from_rccl(__builtin_return_address(0))) {
    std::lock_guard<std::mutex> lk(g_mtx);
    g_imported_handles.insert((uint64_t)(uintptr_t)*handle);
  }
  return e;
}

// Number of RCCL mappings currently mirrored into the registry (for tests and diagnostics).
HOOK_API int64_t amem_rccl_hook_registered(void) {
  std::lock_guard<std::mutex> lk(g_mtx);
  return (int64_t)g_registered.size();
}
