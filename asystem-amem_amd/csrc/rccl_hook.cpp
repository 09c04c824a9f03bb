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
//   hipMemExportToShareableHandle  the owner's side of an exchange: remembers which handle the exported
//                                  descriptor stands for, under the descriptor's identity (device and inode
//                                  numbers of the file behind it, which every duplicate of it shares), in
//                                  this process and as a small file under GMM_IPC_DIR for other processes
//   hipMemImportFromShareableHandle the importer's side: looks the descriptor's identity up and so learns
//                                  the owner's slot and the owner's handle value; a later hipMemSetAccess
//                                  on a mapping of the imported handle registers it as somebody else's
//                                  memory -> amem_add_alloc_info(ptr, size, PEER_POSIX, dev, handle,
//                                  owner slot, owner handle), the shape of the reference's hook in
//                                  ncclP2pImportShareableBuffer (nccl_patch/nccl_2.27.5-1.diff:572-579).
//                                  An import whose owner cannot be named stays unregistered.
//
// What interposition cannot see: the reference also takes buffers out of the registry just before
// they are registered with a NIC (diff:309-312, :364-367, :379-488). RCCL reaches the verbs library
// and the dma-buf export of the HSA runtime through dlopen + dlsym on explicit handles, which no
// library placed in front of them can intercept; a patched RCCL calls amem_delAllocInfo there itself.
//
//   hipMalloc / hipFree            only with AMEM_HOOK_PLAIN_ALLOC=<bytes> in the environment (off by default):
//                                  an RCCL build that keeps its buffers in plain allocations (the one ROCm 7.2
//                                  ships does, whatever NCCL_CUMEM_ENABLE says) gives the engine nothing it
//                                  could release. With the variable set, hipMalloc calls of at least that many
//                                  bytes coming from RCCL are served through the virtual-memory API instead
//                                  (reserve, create, map, grant access: what ncclCuMemAlloc would have done)
//                                  and registered, and hipFree of such an address undoes it. Memory served
//                                  this way cannot be shared through hipIpcGetMemHandle, so the switch is
//                                  for layouts in which RCCL does not hand these buffers to another process
//                                  over legacy IPC (one rank per node, or P2P over IPC disabled).
//
//   hipIpcGetMemHandle             a mapping served in place of a plain allocation cannot be shared that way:
//                                  for such an address the call is refused and one ERROR line says why and
//                                  what to set (NCCL_P2P_DISABLE=1, or no AMEM_HOOK_PLAIN_ALLOC); every other
//                                  address is forwarded
//
// amem_rccl_hook_exclude(ptr) takes one buffer back out of the registry by hand: the manual form of the
// reference's removals before NIC registration, for callers that know which buffers they register.
// amem_rccl_hook_unserved_bytes() and a line at process exit say how much RCCL allocated that the hook left
// alone (below the threshold; uncached, fine-grained or otherwise flagged; not servable).
//
// Calls made by anything else (the pause/resume engine itself, the application) pass through
// untouched. The module a call comes from is found from its return address.
//
// Locking: g_mtx guards this file's maps and nothing else. No call into the HIP runtime or into
// libamem_nccl is made while it is held (the engine calls hipFree, which lands here, while it holds
// its own locks; a hook that called into the engine under g_mtx would close a cycle).
#define _GNU_SOURCE 1
#include <dlfcn.h>
#include <errno.h>
#include <fcntl.h>
#include <signal.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <string>

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

// The maps below are never destroyed: hipFree and the other hooks may still be called by other
// libraries' clean-up code after this library's static objects would have been torn down.
std::mutex g_mtx;
std::unordered_map<uint64_t, Pending>& g_mapped = *new std::unordered_map<uint64_t, Pending>();      // RCCL mappings seen at hipMemMap
std::unordered_set<uint64_t>& g_registered = *new std::unordered_set<uint64_t>();           // those handed to the registry
struct Owner {
  int slot;         // slot of the owning process, -1 when unknown
  uint64_t handle;  // the owner's handle value when the descriptor was exported (it changes with every resume)
  uint64_t va;      // the owner's address of the region (it never changes); 0 when unknown
  // What the importer names the region by when it registers with the owner: the address where it is
  // known, because a handle value noted at export time is dead after the owner's next resume.
  uint64_t name() const { return va ? va : handle; }
};
std::unordered_map<uint64_t, Owner>& g_imported_handles = *new std::unordered_map<uint64_t, Owner>();   // handles RCCL imported from a peer -> who owns the memory
std::unordered_map<std::string, Owner>& g_exports = *new std::unordered_map<std::string, Owner>();         // descriptor identity -> this process's handle behind it
std::unordered_map<uint64_t, std::string>& g_export_of = *new std::unordered_map<uint64_t, std::string>();    // exported handle -> descriptor identity (to forget it again)
std::unordered_map<uint64_t, std::string>& g_export_at = *new std::unordered_map<uint64_t, std::string>();    // address the exported handle was mapped at -> identity; the
                                                          // handle value changes with every resume, the address never
int g_verbose = -1;

// What every duplicate of a descriptor has in common, in this and in any other process.
std::string identity_of(int fd) {
  struct stat st;
  if (fd < 0 || fstat(fd, &st) != 0) return std::string();
  char b[64];
  snprintf(b, sizeof(b), "%llx_%llx", (unsigned long long)st.st_dev, (unsigned long long)st.st_ino);
  return b;
}
std::string export_file(const std::string& id) {
  int gid = 0;
  amem_get_group_id(&gid);
  const char* d = getenv("GMM_IPC_DIR");
  char b[320];
  snprintf(b, sizeof(b), "%s/amem_export_%x_%s", d ? d : "/tmp", gid, id.c_str());
  return b;
}

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
  Owner owner = {-1, 0, 0};
  bool fresh = false, imported = false;
  {
    std::lock_guard<std::mutex> lk(g_mtx);
    auto it = g_mapped.find((uint64_t)(uintptr_t)ptr);
    if (it != g_mapped.end()) {
      auto im = g_imported_handles.find(it->second.handle);
      if (im != g_imported_handles.end()) { imported = true; owner = im->second; }
      if (!imported || owner.slot >= 0) {
        p = it->second;
        fresh = g_registered.insert((uint64_t)(uintptr_t)ptr).second;
      } else if (verbose()) {
        fprintf(stderr, "AMEM [DEBG] rccl_hook: %p maps an imported handle whose owner is unknown; not registered\n", ptr);
      }
    }
  }
  if (fresh) {
    int dev = 0;
    (void)hipGetDevice(&dev);
    int rc;
    if (imported)
      // the shape of the reference's hook in ncclP2pImportShareableBuffer (nccl_patch/nccl_2.27.5-1.diff:572-579)
      rc = amem_add_alloc_info((uint64_t)(uintptr_t)ptr, p.size, AMEM_TYPE_PEER_POSIX, dev, p.handle, owner.slot,
                               owner.name(), NULL, AMEM_CALLER_P2P_PEER);
    else
      // the shape of the reference's hook in ncclCuMemAlloc (nccl_patch/nccl_2.27.5-1.diff:278-280)
      rc = amem_add_alloc_info((uint64_t)(uintptr_t)ptr, p.size, AMEM_TYPE_LOCAL, dev, p.handle, -1, 0, NULL,
                               AMEM_CALLER_DEFAULT);
    if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: registered %p size %zu %s rc %d\n", ptr, p.size,
                           imported ? "imported" : "local", rc);
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
    std::string id;
    {
      std::lock_guard<std::mutex> lk(g_mtx);
      was_registered = g_registered.erase((uint64_t)(uintptr_t)ptr) > 0;
      g_mapped.erase((uint64_t)(uintptr_t)ptr);
      auto ex = g_export_at.find((uint64_t)(uintptr_t)ptr);
      if (ex != g_export_at.end()) {
        id = ex->second;
        auto ow = g_exports.find(id);
        if (ow != g_exports.end()) { g_export_of.erase(ow->second.handle); g_exports.erase(ow); }
        g_export_at.erase(ex);
      }
    }
    if (!id.empty()) unlink(export_file(id).c_str());   // the note for importers in other processes
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
    Owner owner = {-1, 0, 0};
    if (shHandleType == hipMemHandleTypePosixFileDescriptor) {
      const std::string id = identity_of((int)(uintptr_t)osHandle);
      bool found = false;
      // (AMEM_HOOK_NOTES_ONLY makes an importer look at the notes even for descriptors its own process
      // exported, the way an importer in another process has to: for tests of that path)
      static const bool notes_only = getenv("AMEM_HOOK_NOTES_ONLY") != nullptr;
      if (!id.empty() && !notes_only) {
        std::lock_guard<std::mutex> lk(g_mtx);
        auto it = g_exports.find(id);
        if (it != g_exports.end()) { owner = it->second; found = true; }
      }
      if (!found && !id.empty()) {
        // exported by another process: it left a note under the descriptor's identity
        // (only a note this user wrote counts, and a symbolic link in its place is not followed)
        const std::string path = export_file(id);
        const int nfd = open(path.c_str(), O_RDONLY | O_NOFOLLOW | O_CLOEXEC);
        struct stat st;
        if (nfd >= 0 && fstat(nfd, &st) == 0 && S_ISREG(st.st_mode) && st.st_uid == geteuid()) {
          char buf[128] = {0};
          const ssize_t n = read(nfd, buf, sizeof(buf) - 1);
          int slot = -1, pid = 0;
          unsigned long long h = 0, va = 0;
          const int fields = n > 0 ? sscanf(buf, "%d %llx %d %llx", &slot, &h, &pid, &va) : 0;
          if (fields >= 3 && slot >= 0 && slot < AMEM_MAX_DEVS) {
            // Identities are reused (the inode number of a descriptor's file is), so a note may be what a
            // process that has died left behind. It counts only while its writer is alive and somebody
            // holds the slot it names; a stale one is removed.
            const bool writer_alive = pid > 0 && (kill((pid_t)pid, 0) == 0 || errno == EPERM);
            if (writer_alive && amem_ipc_peer_alive(slot)) {
              owner = {slot, (uint64_t)h, fields >= 4 ? (uint64_t)va : 0};
            } else {
              if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: note %s is stale (pid %d %s, slot %d %s); ignored\n",
                                     path.c_str(), pid, writer_alive ? "alive" : "gone", slot,
                                     amem_ipc_peer_alive(slot) ? "held" : "free");
              unlink(path.c_str());
            }
          }
        }
        if (nfd >= 0) close(nfd);
      }
    }
    if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: imported handle %p, owner slot %d handle %llx\n", (void*)*handle,
                           owner.slot, (unsigned long long)owner.handle);
    std::lock_guard<std::mutex> lk(g_mtx);
    g_imported_handles[(uint64_t)(uintptr_t)*handle] = owner;
  }
  return e;
}

HOOK_API hipError_t hipMemExportToShareableHandle(void* shareableHandle, hipMemGenericAllocationHandle_t handle,
                                                  hipMemAllocationHandleType handleType, unsigned long long flags) {
  static auto fn = real<hipError_t (*)(void*, hipMemGenericAllocationHandle_t, hipMemAllocationHandleType, unsigned long long)>(
      "hipMemExportToShareableHandle");
  hipError_t e = fn(shareableHandle, handle, handleType, flags);
  if (e == hipSuccess && shareableHandle && handleType == hipMemHandleTypePosixFileDescriptor &&
      from_rccl(__builtin_return_address(0))) {
    const std::string id = identity_of(*(int*)shareableHandle);
    const int slot = amem_get_slot();
    if (!id.empty() && slot >= 0) {
      const uint64_t h = (uint64_t)(uintptr_t)handle;
      // (asked before the lock is taken: the look-up takes the registry's locks)
      int dev = 0;
      (void)hipGetDevice(&dev);
      const uint64_t va = amem_handle_lookup(dev, h);
      std::string stale;
      {
        std::lock_guard<std::mutex> lk(g_mtx);
        auto old = g_export_of.find(h);
        if (old != g_export_of.end() && old->second != id) stale = old->second;
        g_exports[id] = {slot, h, va};
        g_export_of[h] = id;
        if (va) g_export_at[va] = id;
      }
      if (!stale.empty()) unlink(export_file(stale).c_str());
      // the note is this user's alone, and is never written through a link somebody else left under its name
      const std::string note = export_file(id);
      unlink(note.c_str());
      const int nfd = open(note.c_str(), O_WRONLY | O_CREAT | O_EXCL | O_NOFOLLOW | O_CLOEXEC, 0600);
      if (nfd >= 0) {
        char buf[128];
        const int n = snprintf(buf, sizeof(buf), "%d %llx %d %llx\n", slot, (unsigned long long)h, (int)getpid(),
                               (unsigned long long)va);
        if (write(nfd, buf, (size_t)n) != n && verbose()) fprintf(stderr, "AMEM [WARN] rccl_hook: short write to %s\n", note.c_str());
        close(nfd);
      }
      if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: exported handle %p as %s (slot %d)\n", (void*)handle, id.c_str(), slot);
    }
  }
  return e;
}

// hipMemRelease from RCCL ends a handle's life as far as RCCL is concerned: forget what was noted about it.
HOOK_API hipError_t hipMemRelease(hipMemGenericAllocationHandle_t handle) {
  static auto fn = real<hipError_t (*)(hipMemGenericAllocationHandle_t)>("hipMemRelease");
  if (from_rccl(__builtin_return_address(0))) {
    std::string id;
    {
      std::lock_guard<std::mutex> lk(g_mtx);
      const uint64_t h = (uint64_t)(uintptr_t)handle;
      g_imported_handles.erase(h);
      auto it = g_export_of.find(h);
      if (it != g_export_of.end()) { id = it->second; g_exports.erase(id); g_export_of.erase(it); }
    }
    if (!id.empty()) unlink(export_file(id).c_str());
  }
  return fn(handle);
}

// ---- plain allocations served through the virtual-memory API (opt-in) ----

namespace {
std::unordered_map<uint64_t, uint64_t>& g_substituted = *new std::unordered_map<uint64_t, uint64_t>();  // address handed to RCCL -> mapped size
// RCCL's plain allocations that were left as they are, by reason (only kept while the opt-in mode is on)
enum LeftWhy { LEFT_SMALL = 0, LEFT_FLAGGED = 1, LEFT_UNSERVABLE = 2, LEFT_KINDS = 3 };
struct Left { uint64_t size; int why; };
std::unordered_map<uint64_t, Left>& g_left = *new std::unordered_map<uint64_t, Left>();
uint64_t g_left_bytes[LEFT_KINDS] = {0, 0, 0};        // held by RCCL right now
uint64_t g_left_total[LEFT_KINDS] = {0, 0, 0};        // allocated since load, for the line at exit
uint64_t g_served_total = 0, g_served_count = 0;        // since load, for the line at exit
// Entries in g_substituted plus g_left. hipFree is called by everybody, the engine included; while
// this is zero it goes straight through without touching g_mtx.
std::atomic<long> g_tracked{0};
long long g_plain_min = -2;
size_t plain_alloc_min() {
  if (g_plain_min == -2) {
    const char* e = getenv("AMEM_HOOK_PLAIN_ALLOC");
    g_plain_min = (e && atoll(e) > 0) ? atoll(e) : 0;
  }
  return (size_t)g_plain_min;
}

void note_left(void* ptr, size_t size, int why) {
  if (!ptr) return;
  std::lock_guard<std::mutex> lk(g_mtx);
  auto ins = g_left.emplace((uint64_t)(uintptr_t)ptr, Left{(uint64_t)size, why});
  if (ins.second) { g_left_bytes[why] += size; g_left_total[why] += size; g_tracked.fetch_add(1, std::memory_order_relaxed); }
}

// The served mapping that holds `addr`, or 0. (g_mtx held by the caller.)
uint64_t served_base_of(uint64_t addr) {
  for (auto& kv : g_substituted)
    if (addr >= kv.first && addr < kv.first + kv.second) return kv.first;
  return 0;
}
}  // namespace

// Serve one plain allocation of RCCL's through the virtual-memory API and register it. False when that
// is not possible, in which case the caller falls back to the ordinary allocation.
static bool serve_plain(void** ptr, size_t size) {
  int dev = 0;
  (void)hipGetDevice(&dev);
  uint64_t va = 0, handle = 0, asz = 0;
  if (amem_vmm_alloc(size, dev, &va, &handle, &asz) != 0) return false;  // no room that way: the plain way decides
  // the shape of the reference's hook in ncclCuMemAlloc (nccl_patch/nccl_2.27.5-1.diff:278-280)
  const int rc = amem_add_alloc_info(va, asz, AMEM_TYPE_LOCAL, dev, handle, -1, 0, NULL, AMEM_CALLER_DEFAULT);
  {
    std::lock_guard<std::mutex> lk(g_mtx);
    g_substituted[va] = asz;
    g_tracked.fetch_add(1, std::memory_order_relaxed);
    g_served_total += asz;
    g_served_count++;
    if (rc == 0) g_registered.insert(va);
  }
  if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: plain allocation of %zu bytes served as a mapping at %llx of %llu bytes, registered rc %d\n",
                         size, (unsigned long long)va, (unsigned long long)asz, rc);
  *ptr = (void*)(uintptr_t)va;
  return true;
}

HOOK_API hipError_t hipMalloc(void** ptr, size_t size) {
  static auto fn = real<hipError_t (*)(void**, size_t)>("hipMalloc");
  const size_t min = plain_alloc_min();
  const bool rccl = min && ptr && from_rccl(__builtin_return_address(0));
  if (rccl && size >= min && serve_plain(ptr, size)) return hipSuccess;
  hipError_t e = fn(ptr, size);
  if (rccl && e == hipSuccess) note_left(*ptr, size, size >= min ? LEFT_UNSERVABLE : LEFT_SMALL);
  return e;
}

HOOK_API hipError_t hipFree(void* ptr) {
  static auto fn = real<hipError_t (*)(void*)>("hipFree");
  if (!ptr || g_tracked.load(std::memory_order_relaxed) == 0) return fn(ptr);
  uint64_t asz = 0;
  bool was_registered = false;
  {
    std::lock_guard<std::mutex> lk(g_mtx);
    auto it = g_substituted.find((uint64_t)(uintptr_t)ptr);
    if (it != g_substituted.end()) {
      asz = it->second;
      g_substituted.erase(it);
      g_tracked.fetch_sub(1, std::memory_order_relaxed);
      was_registered = g_registered.erase((uint64_t)(uintptr_t)ptr) > 0;
    } else {
      auto lf = g_left.find((uint64_t)(uintptr_t)ptr);
      if (lf != g_left.end()) {
        g_left_bytes[lf->second.why] -= lf->second.size;
        g_left.erase(lf);
        g_tracked.fetch_sub(1, std::memory_order_relaxed);
      }
    }
  }
  if (!asz) return fn(ptr);
  (void)hipDeviceSynchronize();  // hipFree waits for the device; so does this
  if (was_registered) (void)amem_del_alloc_info((uint64_t)(uintptr_t)ptr, 0, 0);
  const int rc = amem_vmm_free((uint64_t)(uintptr_t)ptr, asz, 0);  // works for a paused (unmapped) address too
  if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: hipFree(%p) of a served mapping, %llu bytes, rc %d\n", ptr,
                         (unsigned long long)asz, rc);
  return rc == 0 ? hipSuccess : hipErrorInvalidValue;
}

HOOK_API hipError_t hipExtMallocWithFlags(void** ptr, size_t size, unsigned int flags) {
  static auto fn = real<hipError_t (*)(void**, size_t, unsigned int)>("hipExtMallocWithFlags");
  // flags 0 is an ordinary allocation under another name (this is how RCCL 2.27 allocates everything);
  // fine-grained, uncached and signal memory keep their own semantics and are never served differently
  const size_t min = plain_alloc_min();
  const bool rccl = (min || verbose()) && ptr && from_rccl(__builtin_return_address(0));
  if (rccl && min && flags == hipDeviceMallocDefault && size >= min && serve_plain(ptr, size)) return hipSuccess;
  if (rccl && verbose() && size >= (1u << 20))
    fprintf(stderr, "AMEM [DEBG] rccl_hook: hipExtMallocWithFlags(%zu, flags %x) left as it is\n", size, flags);
  hipError_t e = fn(ptr, size, flags);
  if (rccl && min && e == hipSuccess)
    note_left(*ptr, size, flags != hipDeviceMallocDefault ? LEFT_FLAGGED : size >= min ? LEFT_UNSERVABLE : LEFT_SMALL);
  return e;
}

// A mapping served in place of a plain allocation cannot become a legacy IPC handle, which is how a
// multi-rank RCCL shares its buffers between the processes of one node unless told otherwise. For such
// an address the call is refused here (what the runtime does with a virtual-memory mapping handed to
// this call is not relied upon) and one line says why; every other address goes through untouched.
HOOK_API hipError_t hipIpcGetMemHandle(hipIpcMemHandle_t* handle, void* devPtr) {
  static auto fn = real<hipError_t (*)(hipIpcMemHandle_t*, void*)>("hipIpcGetMemHandle");
  uint64_t base = 0;
  if (devPtr && g_tracked.load(std::memory_order_relaxed) != 0) {
    std::lock_guard<std::mutex> lk(g_mtx);
    base = served_base_of((uint64_t)(uintptr_t)devPtr);
  }
  if (!base) return fn(handle, devPtr);
  fprintf(stderr, "AMEM [ERRO] rccl_hook: hipIpcGetMemHandle(%p) refused: the buffer at %llx is a virtual-memory mapping the hook "
          "served in place of a plain allocation (AMEM_HOOK_PLAIN_ALLOC), and such a mapping cannot be shared over legacy IPC. "
          "Run RCCL with NCCL_P2P_DISABLE=1 (or one rank per node), or unset AMEM_HOOK_PLAIN_ALLOC.\n",
          devPtr, (unsigned long long)base);
  return hipErrorInvalidValue;
}

// Bytes currently served to RCCL through the virtual-memory API in place of plain allocations.
HOOK_API uint64_t amem_rccl_hook_served_bytes(void) {
  std::lock_guard<std::mutex> lk(g_mtx);
  uint64_t n = 0;
  for (auto& kv : g_substituted) n += kv.second;
  return n;
}

// Bytes RCCL currently holds in plain allocations that the hook left alone while AMEM_HOOK_PLAIN_ALLOC is
// set: `below_threshold` were smaller than the variable's value, `flagged` asked for uncached, fine-grained
// or otherwise special memory (which keeps its semantics), `unservable` could not be created through the
// virtual-memory API. Any pointer may be NULL. Returns the sum.
HOOK_API uint64_t amem_rccl_hook_unserved_bytes(uint64_t* below_threshold, uint64_t* flagged, uint64_t* unservable) {
  std::lock_guard<std::mutex> lk(g_mtx);
  if (below_threshold) *below_threshold = g_left_bytes[LEFT_SMALL];
  if (flagged) *flagged = g_left_bytes[LEFT_FLAGGED];
  if (unservable) *unservable = g_left_bytes[LEFT_UNSERVABLE];
  return g_left_bytes[LEFT_SMALL] + g_left_bytes[LEFT_FLAGGED] + g_left_bytes[LEFT_UNSERVABLE];
}

// Number of RCCL mappings currently mirrored into the registry (for tests and diagnostics).
HOOK_API int64_t amem_rccl_hook_registered(void) {
  std::lock_guard<std::mutex> lk(g_mtx);
  return (int64_t)g_registered.size();
}

// Take the buffer that holds `ptr` out of the registry: a pause no longer releases it and it keeps its
// memory. The manual form of what the reference does just before a buffer is registered with a NIC
// (nccl_patch/nccl_2.27.5-1.diff:309-312, :364-367), for callers that know which buffers they register;
// the hook cannot see those sites itself. 0 done; 1 the address belongs to nothing the hook registered;
// 2 refused while paused (the buffer's memory is already gone and only the registry can bring it back).
HOOK_API int amem_rccl_hook_exclude(void* ptr) {
  if (!ptr) return 1;
  if (amem_check_paused(0)) return 2;
  const uint64_t addr = (uint64_t)(uintptr_t)ptr;
  uint64_t base = 0;
  {
    std::lock_guard<std::mutex> lk(g_mtx);
    for (uint64_t va : g_registered) {
      uint64_t size = 0;
      auto m = g_mapped.find(va);
      if (m != g_mapped.end()) size = m->second.size;
      auto sub = g_substituted.find(va);
      if (sub != g_substituted.end()) size = sub->second;
      if (addr >= va && addr < va + (size ? size : 1)) { base = va; break; }
    }
    if (base) g_registered.erase(base);
  }
  if (!base) return 1;
  (void)amem_del_alloc_info(base, 0, 0);
  if (verbose()) fprintf(stderr, "AMEM [DEBG] rccl_hook: %llx taken out of the registry on request\n", (unsigned long long)base);
  return 0;
}

// What the opt-in mode did for this process, once, when it ends: how much of what RCCL allocated could be
// put into the registry, and how much could not and why.
static void __attribute__((destructor)) amem_rccl_hook_summary(void) {
  if (plain_alloc_min() == 0) return;
  uint64_t total, count, left[LEFT_KINDS];
  {
    std::lock_guard<std::mutex> lk(g_mtx);
    total = g_served_total; count = g_served_count;
    for (int k = 0; k < LEFT_KINDS; ++k) left[k] = g_left_total[k];
  }
  fprintf(stderr, "AMEM [INFO] rccl_hook: AMEM_HOOK_PLAIN_ALLOC=%zu, RCCL's plain allocations since load: %.1f MiB in %llu "
          "allocations served through the virtual-memory API and registered; %.1f MiB left alone (%.1f MiB below the "
          "threshold, %.1f MiB uncached / fine-grained, %.1f MiB not servable)\n", plain_alloc_min(), total / 1048576.0,
          (unsigned long long)count, (left[0] + left[1] + left[2]) / 1048576.0, left[LEFT_SMALL] / 1048576.0,
          left[LEFT_FLAGGED] / 1048576.0, left[LEFT_UNSERVABLE] / 1048576.0);
}
