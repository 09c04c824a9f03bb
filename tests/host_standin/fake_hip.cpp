// TEST INFRASTRUCTURE, never part of the shipped library.
//
// A stand-in for the part of the HIP runtime the engine calls, on host memory, so that the library's
// own unchanged sources (capi, engine, ipc, vmm, slab_pool, log) can be linked into a second, test-only
// shared object and driven through real pause/resume cycles by several real processes on a machine
// without a GPU. "Device memory" of the virtual-memory API is a memfd mapped with MAP_FIXED inside a
// PROT_NONE reservation, which reproduces what the engine relies on: reserve / create / map / set
// access / unmap / release, identical addresses after a remap, export as a file descriptor that another
// process can import, and memory that lives until its last handle and mapping are gone. Streams are
// synchronous, events are timestamps. The shipped library is never built this way and never loads this.
//
// Knobs (environment, read once): AMEM_FAKE_HIP_MEM_MIB caps the "device memory" (default 1 TiB) so that
// out-of-memory paths can be forced from the host.
#ifndef _GNU_SOURCE
#define _GNU_SOURCE 1
#endif
#include <hip/hip_runtime_api.h>

#include <errno.h>
#include <fcntl.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <map>
#include <mutex>
#include <set>

namespace {

struct Phys {
  int fd;
  size_t size;
  int refs;  // creator or importer 1, +1 per mapping
};
struct Mapping {
  size_t size;
  Phys* phys;
  bool access;
};
struct FakeEvent {
  std::chrono::steady_clock::time_point t;
};

std::mutex g_mtx;
std::map<uintptr_t, Mapping> g_maps;      // by first address
std::map<uintptr_t, size_t> g_reserved;   // address reservations
std::map<uintptr_t, size_t> g_blocks;     // hipMalloc and hipHostMalloc blocks
std::set<Phys*> g_phys;
size_t g_live = 0;
thread_local hipError_t t_last = hipSuccess;
thread_local int t_dev = 0;

size_t capacity() {
  static size_t cap = [] {
    const char* e = getenv("AMEM_FAKE_HIP_MEM_MIB");
    return e ? (size_t)atoll(e) << 20 : (size_t)1 << 40;
  }();
  return cap;
}

hipError_t fail(hipError_t e) {
  t_last = e;
  return e;
}

void unref(Phys* p) {
  if (--p->refs > 0) return;
  close(p->fd);
  g_live -= p->size;
  g_phys.erase(p);
  delete p;
}

// the mapping that contains `a`, or end()
std::map<uintptr_t, Mapping>::iterator mapping_of(uintptr_t a) {
  auto it = g_maps.upper_bound(a);
  if (it == g_maps.begin()) return g_maps.end();
  --it;
  return (a < it->first + it->second.size) ? it : g_maps.end();
}

bool inside(const std::map<uintptr_t, size_t>& m, uintptr_t a, size_t n, uintptr_t* base, size_t* size) {
  auto it = m.upper_bound(a);
  if (it == m.begin()) return false;
  --it;
  if (a + n > it->first + it->second) return false;
  if (base) *base = it->first;
  if (size) *size = it->second;
  return true;
}

}  // namespace

extern "C" {

hipError_t hipGetDeviceCount(int* n) { *n = 1; return hipSuccess; }
hipError_t hipGetDevice(int* d) { *d = t_dev; return hipSuccess; }
hipError_t hipSetDevice(int d) { if (d != 0) return fail(hipErrorInvalidDevice); t_dev = d; return hipSuccess; }
hipError_t hipGetLastError(void) { hipError_t e = t_last; t_last = hipSuccess; return e; }
const char* hipGetErrorString(hipError_t e) {
  switch (e) {
    case hipSuccess: return "no error";
    case hipErrorInvalidValue: return "invalid argument";
    case hipErrorOutOfMemory: return "out of memory";
    case hipErrorInvalidDevice: return "invalid device ordinal";
    default: return "error (host stand-in)";
  }
}
hipError_t hipDeviceSynchronize(void) { return hipSuccess; }
hipError_t hipDeviceGetPCIBusId(char* out, int len, int) { snprintf(out, (size_t)len, "0000:00:00.0"); return hipSuccess; }

hipError_t hipMemGetInfo(size_t* free_b, size_t* total) {
  std::lock_guard<std::mutex> lk(g_mtx);
  if (total) *total = capacity();
  if (free_b) *free_b = capacity() - g_live;
  return hipSuccess;
}

// ---- ordinary and pinned allocations ----
static hipError_t block_alloc(void** p, size_t n, bool counted) {
  if (!p || n == 0) return fail(hipErrorInvalidValue);
  std::lock_guard<std::mutex> lk(g_mtx);
  if (counted && g_live + n > capacity()) return fail(hipErrorOutOfMemory);
  void* q = nullptr;
  if (posix_memalign(&q, 4096, n) != 0) return fail(hipErrorOutOfMemory);
  g_blocks[(uintptr_t)q] = n;
  if (counted) g_live += n;
  *p = q;
  return hipSuccess;
}
static std::set<uintptr_t>& counted_blocks() { static std::set<uintptr_t> s; return s; }
hipError_t hipMalloc(void** p, size_t n) {
  hipError_t e = block_alloc(p, n, true);
  if (e == hipSuccess) { std::lock_guard<std::mutex> lk(g_mtx); counted_blocks().insert((uintptr_t)*p); }
  return e;
}
hipError_t hipFree(void* p) {
  if (!p) return hipSuccess;
  std::lock_guard<std::mutex> lk(g_mtx);
  auto it = g_blocks.find((uintptr_t)p);
  if (it == g_blocks.end()) return fail(hipErrorInvalidValue);
  if (counted_blocks().erase((uintptr_t)p)) g_live -= it->second;
  g_blocks.erase(it);
  free(p);
  return hipSuccess;
}
hipError_t hipExtMallocWithFlags(void** p, size_t n, unsigned int) { return hipMalloc(p, n); }
hipError_t hipIpcGetMemHandle(hipIpcMemHandle_t* h, void* p) {
  std::lock_guard<std::mutex> lk(g_mtx);
  if (!h || g_blocks.find((uintptr_t)p) == g_blocks.end()) return fail(hipErrorInvalidValue);
  memset(h, 0, sizeof(*h));
  return hipSuccess;
}
hipError_t hipMemGetAllocationGranularity(size_t* g, const hipMemAllocationProp*, hipMemAllocationGranularity_flags) {
  *g = 4096;
  return hipSuccess;
}
hipError_t hipHostMalloc(void** p, size_t n, unsigned int) { return block_alloc(p, n, false); }
hipError_t hipHostFree(void* p) { return hipFree(p); }
hipError_t hipHostGetDevicePointer(void** dp, void* hp, unsigned int) { *dp = hp; return hipSuccess; }

hipError_t hipMemcpy(void* dst, const void* src, size_t n, hipMemcpyKind) { memcpy(dst, src, n); return hipSuccess; }
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t n, hipMemcpyKind, hipStream_t) { memcpy(dst, src, n); return hipSuccess; }
hipError_t hipMemset(void* dst, int v, size_t n) { memset(dst, v, n); return hipSuccess; }

// ---- streams and events: everything has completed by the time a call returns ----
hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned int) { *s = (hipStream_t) new int(0); return hipSuccess; }
hipError_t hipStreamDestroy(hipStream_t s) { delete (int*)s; return hipSuccess; }
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t* e) { *e = (hipEvent_t) new FakeEvent(); return hipSuccess; }
hipError_t hipEventDestroy(hipEvent_t e) { delete (FakeEvent*)e; return hipSuccess; }
hipError_t hipEventRecord(hipEvent_t e, hipStream_t) { ((FakeEvent*)e)->t = std::chrono::steady_clock::now(); return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b) {
  *ms = std::chrono::duration<float, std::milli>(((FakeEvent*)b)->t - ((FakeEvent*)a)->t).count();
  return hipSuccess;
}

// ---- virtual memory management ----
hipError_t hipMemAddressReserve(void** ptr, size_t size, size_t align, void*, unsigned long long) {
  if (!ptr || size == 0) return fail(hipErrorInvalidValue);
  if (align < 4096) align = 4096;
  char* raw = (char*)mmap(nullptr, size + align, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
  if (raw == MAP_FAILED) return fail(hipErrorOutOfMemory);
  char* base = (char*)(((uintptr_t)raw + align - 1) / align * align);
  if (base > raw) munmap(raw, base - raw);
  const size_t tail = (raw + size + align) - (base + size);
  if (tail) munmap(base + size, tail);
  std::lock_guard<std::mutex> lk(g_mtx);
  g_reserved[(uintptr_t)base] = size;
  *ptr = base;
  return hipSuccess;
}
hipError_t hipMemAddressFree(void* ptr, size_t size) {
  std::lock_guard<std::mutex> lk(g_mtx);
  auto it = g_reserved.find((uintptr_t)ptr);
  if (it == g_reserved.end() || it->second != size) return fail(hipErrorInvalidValue);
  if (mapping_of((uintptr_t)ptr) != g_maps.end()) return fail(hipErrorInvalidValue);  // still mapped
  munmap(ptr, size);
  g_reserved.erase(it);
  return hipSuccess;
}
hipError_t hipMemCreate(hipMemGenericAllocationHandle_t* h, size_t size, const hipMemAllocationProp* prop, unsigned long long) {
  if (!h || size == 0 || !prop) return fail(hipErrorInvalidValue);
  if (prop->location.type != hipMemLocationTypeDevice || prop->location.id != 0) return fail(hipErrorInvalidDevice);
  std::lock_guard<std::mutex> lk(g_mtx);
  if (g_live + size > capacity()) return fail(hipErrorOutOfMemory);
  int fd = memfd_create("amem_fake_hip", MFD_CLOEXEC);
  if (fd < 0) return fail(hipErrorOutOfMemory);
  if (ftruncate(fd, (off_t)size) != 0) { close(fd); return fail(hipErrorOutOfMemory); }
  Phys* p = new Phys{fd, size, 1};
  g_phys.insert(p);
  g_live += size;
  *h = (hipMemGenericAllocationHandle_t)p;
  return hipSuccess;
}
hipError_t hipMemRelease(hipMemGenericAllocationHandle_t h) {
  std::lock_guard<std::mutex> lk(g_mtx);
  Phys* p = (Phys*)h;
  if (!g_phys.count(p)) return fail(hipErrorInvalidValue);  // the real runtime would touch freed memory here
  unref(p);
  return hipSuccess;
}
hipError_t hipMemMap(void* ptr, size_t size, size_t offset, hipMemGenericAllocationHandle_t h, unsigned long long) {
  std::lock_guard<std::mutex> lk(g_mtx);
  Phys* p = (Phys*)h;
  if (!g_phys.count(p) || offset + size > p->size) return fail(hipErrorInvalidValue);
  if (!inside(g_reserved, (uintptr_t)ptr, size, nullptr, nullptr)) return fail(hipErrorInvalidValue);
  for (uintptr_t a : {(uintptr_t)ptr, (uintptr_t)ptr + size - 1})
    if (mapping_of(a) != g_maps.end()) return fail(hipErrorInvalidValue);  // already mapped
  auto nx = g_maps.lower_bound((uintptr_t)ptr);
  if (nx != g_maps.end() && nx->first < (uintptr_t)ptr + size) return fail(hipErrorInvalidValue);
  if (mmap(ptr, size, PROT_NONE, MAP_SHARED | MAP_FIXED, p->fd, (off_t)offset) == MAP_FAILED) return fail(hipErrorOutOfMemory);
  p->refs++;
  g_maps[(uintptr_t)ptr] = Mapping{size, p, false};
  return hipSuccess;
}
hipError_t hipMemSetAccess(void* ptr, size_t size, const hipMemAccessDesc* desc, size_t count) {
  if (!desc || count == 0) return fail(hipErrorInvalidValue);
  std::lock_guard<std::mutex> lk(g_mtx);
  auto it = mapping_of((uintptr_t)ptr);
  if (it == g_maps.end() || (uintptr_t)ptr + size > it->first + it->second.size) return fail(hipErrorInvalidValue);
  const bool rw = desc[0].flags == hipMemAccessFlagsProtReadWrite;
  if (mprotect(ptr, size, rw ? (PROT_READ | PROT_WRITE) : PROT_NONE) != 0) return fail(hipErrorInvalidValue);
  it->second.access = rw;
  return hipSuccess;
}
hipError_t hipMemUnmap(void* ptr, size_t size) {
  std::lock_guard<std::mutex> lk(g_mtx);
  auto it = g_maps.find((uintptr_t)ptr);
  if (it == g_maps.end() || it->second.size > size) return fail(hipErrorInvalidValue);
  // every mapping that lies inside [ptr, ptr + size) goes, as on the real runtime
  uintptr_t end = (uintptr_t)ptr + size;
  while (it != g_maps.end() && it->first + it->second.size <= end) {
    if (mmap((void*)it->first, it->second.size, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE | MAP_FIXED, -1, 0) == MAP_FAILED)
      return fail(hipErrorUnknown);
    unref(it->second.phys);
    it = g_maps.erase(it);
  }
  return hipSuccess;
}
// As measured on the real runtime: the handle comes back without a reference being taken.
hipError_t hipMemRetainAllocationHandle(hipMemGenericAllocationHandle_t* h, void* addr) {
  std::lock_guard<std::mutex> lk(g_mtx);
  auto it = mapping_of((uintptr_t)addr);
  if (it == g_maps.end()) return fail(hipErrorInvalidValue);
  *h = (hipMemGenericAllocationHandle_t)it->second.phys;
  return hipSuccess;
}
hipError_t hipMemGetAddressRange(hipDeviceptr_t* base, size_t* size, hipDeviceptr_t ptr) {
  std::lock_guard<std::mutex> lk(g_mtx);
  auto it = mapping_of((uintptr_t)ptr);
  if (it != g_maps.end()) {
    if (base) *base = (hipDeviceptr_t)it->first;
    if (size) *size = it->second.size;
    return hipSuccess;
  }
  uintptr_t b = 0;
  size_t s = 0;
  if (inside(g_blocks, (uintptr_t)ptr, 1, &b, &s)) {
    if (base) *base = (hipDeviceptr_t)b;
    if (size) *size = s;
    return hipSuccess;
  }
  return fail(hipErrorInvalidValue);
}
hipError_t hipMemGetAccess(unsigned long long* flags, const hipMemLocation*, void* ptr) {
  std::lock_guard<std::mutex> lk(g_mtx);
  auto it = mapping_of((uintptr_t)ptr);
  if (it == g_maps.end()) return fail(hipErrorInvalidValue);
  *flags = it->second.access ? (unsigned long long)hipMemAccessFlagsProtReadWrite : 0ull;
  return hipSuccess;
}
hipError_t hipMemExportToShareableHandle(void* out, hipMemGenericAllocationHandle_t h, hipMemAllocationHandleType type, unsigned long long) {
  std::lock_guard<std::mutex> lk(g_mtx);
  Phys* p = (Phys*)h;
  if (!out || !g_phys.count(p) || type != hipMemHandleTypePosixFileDescriptor) return fail(hipErrorInvalidValue);
  int fd = fcntl(p->fd, F_DUPFD_CLOEXEC, 0);
  if (fd < 0) return fail(hipErrorUnknown);
  *(int*)out = fd;
  return hipSuccess;
}
hipError_t hipMemImportFromShareableHandle(hipMemGenericAllocationHandle_t* h, void* os_handle, hipMemAllocationHandleType type) {
  if (!h || type != hipMemHandleTypePosixFileDescriptor) return fail(hipErrorInvalidValue);
  const int fd = (int)(uintptr_t)os_handle;
  struct stat st;
  if (fd < 0 || fstat(fd, &st) != 0 || st.st_size <= 0) return fail(hipErrorInvalidValue);
  int mine = fcntl(fd, F_DUPFD_CLOEXEC, 0);
  if (mine < 0) return fail(hipErrorInvalidValue);
  std::lock_guard<std::mutex> lk(g_mtx);
  Phys* p = new Phys{mine, (size_t)st.st_size, 1};
  g_phys.insert(p);
  g_live += p->size;  // an import keeps the memory alive, and a release of it is what frees this process's share
  *h = (hipMemGenericAllocationHandle_t)p;
  return hipSuccess;
}
hipError_t hipMemGetAllocationPropertiesFromHandle(hipMemAllocationProp* prop, hipMemGenericAllocationHandle_t h) {
  std::lock_guard<std::mutex> lk(g_mtx);
  if (!prop || !g_phys.count((Phys*)h)) return fail(hipErrorInvalidValue);
  memset(prop, 0, sizeof(*prop));
  prop->type = hipMemAllocationTypePinned;
  prop->location.type = hipMemLocationTypeDevice;
  prop->location.id = 0;
  prop->requestedHandleTypes = hipMemHandleTypePosixFileDescriptor;
  return hipSuccess;
}

}  // extern "C"
