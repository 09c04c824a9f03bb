#include "vmm.h"

#include <stdio.h>
#include <unistd.h>

#include <mutex>

#include "log.h"

namespace amem {

hipError_t check_hip(hipError_t e, const char* expr, const char* file, int line) {
  if (e != hipSuccess) {
    int dev = -1;
    (void)hipGetDevice(&dev);
    printf("%s:%d func:%s gpu:%d error:%d str:%s\n", file, line, expr, dev, (int)e,
           hipGetErrorString(e));
    fflush(stdout);
  }
  return e;
}

static hipMemAllocationProp device_prop(int dev) {
  hipMemAllocationProp p = {};
  p.type = hipMemAllocationTypePinned;
  p.location.type = hipMemLocationTypeDevice;
  p.location.id = dev;
  p.requestedHandleTypes = hipMemHandleTypePosixFileDescriptor;  // amem_nccl.h:36
  return p;
}

static hipError_t set_rw(uint64_t va, size_t size, int dev) {
  hipMemAccessDesc acc = {};
  acc.location.type = hipMemLocationTypeDevice;
  acc.location.id = dev;
  acc.flags = hipMemAccessFlagsProtReadWrite;
  return hipMemSetAccess((void*)(uintptr_t)va, size, &acc, 1);
}

hipError_t vmm_alloc(size_t bytes, int dev, uint64_t* va, uint64_t* handle, size_t* alloc_size) {
  if (!va || !handle || bytes == 0) return hipErrorInvalidValue;
  const size_t size = (bytes + kVmmAlign - 1) / kVmmAlign * kVmmAlign;
  hipMemAllocationProp prop = device_prop(dev);
  void* ptr = nullptr;
  hipMemGenericAllocationHandle_t h = nullptr;
  bool mapped = false;
  hipError_t e = CHECK_HIP(hipMemAddressReserve(&ptr, size, kVmmAlign, nullptr, 0));
  if (e == hipSuccess) e = CHECK_HIP(hipMemCreate(&h, size, &prop, 0));
  if (e == hipSuccess) {
    e = CHECK_HIP(hipMemMap(ptr, size, 0, h, 0));
    mapped = (e == hipSuccess);
  }
  if (e == hipSuccess) e = CHECK_HIP(set_rw((uint64_t)(uintptr_t)ptr, size, dev));
  if (e != hipSuccess) {
    if (mapped) (void)hipMemUnmap(ptr, size);
    if (h) (void)hipMemRelease(h);
    if (ptr) (void)hipMemAddressFree(ptr, size);
    return e;
  }
  *va = (uint64_t)(uintptr_t)ptr;
  *handle = handle_bits(h);
  if (alloc_size) *alloc_size = size;
  return hipSuccess;
}

// The reference learns a handle with cuMemRetainAllocationHandle + cuMemRelease
// (amem_nccl.h:147-148). On this HIP runtime hipMemRetainAllocationHandle returns the
// handle without taking a reference (measured: memory is freed by the first release after
// an unmap even when a retain came before), so the matching release must NOT be issued: it
// would drop the creator's reference.
// hipMemRetainAllocationHandle must only see addresses mapped through the virtual-memory API:
// given ordinary hipMalloc memory it crashes inside the runtime (measured on ROCm 7.2), while
// hipMemGetAccess answers with an error for such memory and for reserved-but-unmapped
// addresses alike. So the access query goes first.
bool vmm_is_mapped(uint64_t va) {
  if (va == 0) return false;
  int dev = 0;
  (void)hipGetDevice(&dev);
  hipMemLocation loc;
  loc.type = hipMemLocationTypeDevice;
  loc.id = dev;
  unsigned long long flags = 0;
  if (hipMemGetAccess(&flags, &loc, (void*)(uintptr_t)va) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return true;
}

uint64_t vmm_handle_of(uint64_t va) {
  if (!vmm_is_mapped(va)) return 0;
  hipMemGenericAllocationHandle_t h = nullptr;
  if (hipMemRetainAllocationHandle(&h, (void*)(uintptr_t)va) != hipSuccess || !h) {
    (void)hipGetLastError();
    return 0;
  }
  return handle_bits(h);
}

bool vmm_range_of(uint64_t addr, uint64_t* base, uint64_t* size) {
  hipDeviceptr_t b = nullptr;
  size_t s = 0;
  if (hipMemGetAddressRange(&b, &s, (hipDeviceptr_t)(uintptr_t)addr) != hipSuccess || s == 0) {
    (void)hipGetLastError();
    return false;
  }
  *base = (uint64_t)(uintptr_t)b;
  *size = s;
  return true;
}

// Size of the mapping that starts at `va` (cuMemGetAddressRange in amem_cuMemReleaseHandle,
// amem_nccl.h:150), or `fallback` when the runtime cannot tell.
static size_t mapped_size(uint64_t va, size_t fallback) {
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)(uintptr_t)va) != hipSuccess || size == 0 ||
      (uint64_t)(uintptr_t)base != va) {
    (void)hipGetLastError();
    return fallback;
  }
  return size;
}

hipError_t vmm_free(uint64_t va, size_t alloc_size, uint64_t handle) {
  if (va == 0) return hipErrorInvalidValue;
  hipError_t e = hipSuccess;
  const uint64_t mapped = vmm_handle_of(va);
  if (mapped != 0) {
    if (handle == 0) handle = mapped;
    e = CHECK_HIP(hipMemUnmap((void*)(uintptr_t)va, mapped_size(va, alloc_size)));
    hipError_t e2 = CHECK_HIP(hipMemRelease(as_handle(handle)));
    if (e == hipSuccess) e = e2;
  }
  hipError_t e3 = CHECK_HIP(hipMemAddressFree((void*)(uintptr_t)va, alloc_size));
  return e == hipSuccess ? e3 : e;
}

hipError_t vmm_unmap_release(uint64_t va, size_t size, uint64_t handle, int extra) {
  if (va == 0) return hipSuccess;
  hipError_t e = CHECK_HIP(hipMemUnmap((void*)(uintptr_t)va, mapped_size(va, size)));
  if (handle != 0) {
    hipError_t e2 = CHECK_HIP(hipMemRelease(as_handle(handle)));
    if (e == hipSuccess) e = e2;
    while (extra-- > 0) {
      e2 = CHECK_HIP(hipMemRelease(as_handle(handle)));
      if (e == hipSuccess) e = e2;
    }
  }
  return e;
}

hipError_t vmm_unmap(uint64_t va, size_t size) {
  if (va == 0) return hipSuccess;
  return CHECK_HIP(hipMemUnmap((void*)(uintptr_t)va, mapped_size(va, size)));
}

hipError_t vmm_release(uint64_t handle, int extra) {
  hipError_t e = hipSuccess;
  if (handle == 0) return e;
  for (int k = 0; k <= (extra > 0 ? extra : 0); ++k) {
    hipError_t e2 = CHECK_HIP(hipMemRelease(as_handle(handle)));
    if (e == hipSuccess) e = e2;
  }
  return e;
}

hipError_t vmm_create_map(uint64_t va, int dev, size_t size, uint64_t* new_handle) {
  hipMemAllocationProp prop = device_prop(dev);
  hipMemGenericAllocationHandle_t h = nullptr;
  hipError_t e = CHECK_HIP(hipMemCreate(&h, size, &prop, 0));
  if (e != hipSuccess) return e;
  e = CHECK_HIP(hipMemMap((void*)(uintptr_t)va, size, 0, h, 0));
  if (e == hipSuccess) {
    e = CHECK_HIP(set_rw(va, size, dev));
    if (e != hipSuccess) (void)hipMemUnmap((void*)(uintptr_t)va, size);
  }
  if (e != hipSuccess) {
    // leave the address as it was found: reserved, nothing mapped, no memory held
    (void)hipMemRelease(h);
    (void)hipGetLastError();
    *new_handle = 0;
    return e;
  }
  *new_handle = handle_bits(h);
  return e;
}

hipError_t vmm_export_fd(uint64_t handle, int* fd) {
  int out = -1;
  hipError_t e = CHECK_HIP(hipMemExportToShareableHandle((void*)&out, as_handle(handle),
                                                         hipMemHandleTypePosixFileDescriptor, 0));
  *fd = out;
  return e;
}

hipError_t vmm_import_map(int dev, uint64_t va, size_t size, int fd, bool close_fd,
                          uint64_t* new_handle) {
  // One import at a time per process. Several service threads of one process (one per rank it hosts)
  // may be asked to map descriptors at the same moment; the runtime runs these calls one after the
  // other anyway, and importing, mapping and granting access from three threads at once has failed
  // here now and then (hipMemSetAccess on the fresh mapping: invalid argument) in a process that
  // held several hundred other descriptors open. Importers in different processes are not affected.
  static std::mutex one_at_a_time;
  std::lock_guard<std::mutex> serial(one_at_a_time);
  hipMemGenericAllocationHandle_t h = nullptr;
  // hipMemMap accepts an address that already holds a mapping (measured on ROCm 7.2) and the old
  // mapping is then lost without having been unmapped: refuse here what the runtime does not.
  if (vmm_is_mapped(va)) {
    LOGGER(ERROR, "pid:%d curDev:%d dptr:%llx still holds a mapping; not importing inFD:%d over it", getpid(), dev,
           (unsigned long long)va, fd);
    if (close_fd) close(fd);
    if (new_handle) *new_handle = 0;
    return hipErrorInvalidValue;
  }
  hipError_t e = CHECK_HIP(hipMemImportFromShareableHandle(&h, (void*)(uintptr_t)fd,
                                                           hipMemHandleTypePosixFileDescriptor));
  if (e == hipSuccess) {
    e = CHECK_HIP(hipMemMap((void*)(uintptr_t)va, size, 0, h, 0));
    if (e == hipSuccess) {
      e = CHECK_HIP(set_rw(va, size, dev));
      if (e != hipSuccess) (void)hipMemUnmap((void*)(uintptr_t)va, size);
    } else {
      LOGGER(ERROR, "pid:%d newMap ret:%d", getpid(), (int)e);
    }
    if (e != hipSuccess) {
      LOGGER(ERROR, "pid:%d curDev:%d newHandle:%llx inFD:%d ret:%d", getpid(), dev,
             (unsigned long long)handle_bits(h), fd, (int)e);
      (void)hipMemRelease(h);  // the import's reference; nothing is mapped
      (void)hipGetLastError();
      h = nullptr;
    }
  } else {
    LOGGER(ERROR, "pid:%d curDev:%d import of inFD:%d ret:%d", getpid(), dev, fd, (int)e);
    h = nullptr;
  }
  if (close_fd) close(fd);
  if (new_handle) *new_handle = handle_bits(h);
  return e;
}

int vmm_handle_device(uint64_t handle) {
  if (handle == 0) return -1;
  hipMemAllocationProp prop = {};
  if (hipMemGetAllocationPropertiesFromHandle(&prop, as_handle(handle)) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  return prop.location.id;
}

}  // namespace amem
