// A stand-in for the part of RCCL that allocates communication buffers through the HIP
// virtual-memory API, built by tests/test_gpu_rccl_hook.py into a file named librccl_standin.so
// so that the allocator hook treats its calls as RCCL's. It follows the call order of NCCL's
// ncclCuMemAlloc / ncclCuMemFree as the reference's patch shows them
// (nccl_patch/nccl_2.27.5-1.diff:272-296): create, reserve, map, set access; and on free:
// look the handle up from the address, unmap, release, free the reservation.
// The RCCL 2.27.7 shipped with ROCm 7.2 never takes this path on its own (its buffers come from
// plain allocations even with NCCL_CUMEM_ENABLE=1), which is why a stand-in is needed.
#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

extern "C" __attribute__((visibility("default"))) int standin_cumem_alloc(void** ptr, size_t size) {
  hipMemAllocationProp prop = {};
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.requestedHandleTypes = hipMemHandleTypePosixFileDescriptor;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 1;
  prop.location.id = dev;
  size_t gran = 0;
  if (hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityMinimum) != hipSuccess) return 2;
  if (gran < (2u << 20)) gran = 2u << 20;
  size = (size + gran - 1) / gran * gran;
  hipMemGenericAllocationHandle_t handle;
  if (hipMemCreate(&handle, size, &prop, 0) != hipSuccess) return 3;
  if (hipMemAddressReserve(ptr, size, gran, nullptr, 0) != hipSuccess) return 4;
  if (hipMemMap(*ptr, size, 0, handle, 0) != hipSuccess) return 5;
  hipMemAccessDesc acc = {};
  acc.location.type = hipMemLocationTypeDevice;
  acc.location.id = dev;
  acc.flags = hipMemAccessFlagsProtReadWrite;
  if (hipMemSetAccess(*ptr, size, &acc, 1) != hipSuccess) return 6;
  return 0;
}

extern "C" __attribute__((visibility("default"))) int standin_cumem_free(void* ptr) {
  hipMemGenericAllocationHandle_t handle = nullptr;
  // this HIP runtime's retain takes no reference, so there is no release to pair with it
  if (hipMemRetainAllocationHandle(&handle, ptr) != hipSuccess) return 1;
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)ptr) != hipSuccess) return 2;
  if (hipMemUnmap(ptr, size) != hipSuccess) return 3;
  if (hipMemRelease(handle) != hipSuccess) return 4;
  if (hipMemAddressFree(ptr, size) != hipSuccess) return 5;
  return 0;
}

// The owner's half of a buffer exchange, as ncclP2pAllocateShareableBuffer does it: the handle is
// looked up from the address and exported as a POSIX file descriptor.
extern "C" __attribute__((visibility("default"))) int standin_export(void* ptr, int* fd) {
  hipMemGenericAllocationHandle_t handle = nullptr;
  if (hipMemRetainAllocationHandle(&handle, ptr) != hipSuccess) return 1;
  if (hipMemExportToShareableHandle((void*)fd, handle, hipMemHandleTypePosixFileDescriptor, 0) != hipSuccess) return 2;
  return 0;
}

// The importer's half, in the call order of ncclP2pImportShareableBuffer
// (nccl_patch/nccl_2.27.5-1.diff:560-590): import, reserve, map, allow access by the local GPU.
extern "C" __attribute__((visibility("default"))) int standin_import_map(int fd, size_t size, void** ptr) {
  hipMemGenericAllocationHandle_t handle = nullptr;
  if (hipMemImportFromShareableHandle(&handle, (void*)(uintptr_t)fd, hipMemHandleTypePosixFileDescriptor) != hipSuccess) return 1;
  if (hipMemAddressReserve(ptr, size, 0, nullptr, 0) != hipSuccess) return 2;
  if (hipMemMap(*ptr, size, 0, handle, 0) != hipSuccess) return 3;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 4;
  hipMemAccessDesc acc = {};
  acc.location.type = hipMemLocationTypeDevice;
  acc.location.id = dev;
  acc.flags = hipMemAccessFlagsProtReadWrite;
  if (hipMemSetAccess(*ptr, size, &acc, 1) != hipSuccess) return 5;
  return 0;
}

// RCCL 2.27 keeps its own buffers in plain allocations (hipExtMallocWithFlags with flags 0, fine-grained
// memory for what the host polls). These three make the same calls from a file named librccl_*.so.
// (Each call is followed by more code on purpose: the hook tells RCCL's calls by their return address,
// and a call compiled into a jump would return straight into this function's caller.)
extern "C" __attribute__((visibility("default"))) int standin_plain_alloc(void** ptr, size_t size, unsigned int flags, int use_ext) {
  const hipError_t e = use_ext ? hipExtMallocWithFlags(ptr, size, flags) : hipMalloc(ptr, size);
  if (e != hipSuccess) (void)hipGetLastError();
  return (int)e;
}
extern "C" __attribute__((visibility("default"))) int standin_plain_free(void* ptr) {
  const hipError_t e = hipFree(ptr);
  if (e != hipSuccess) (void)hipGetLastError();
  return (int)e;
}
// What a multi-rank RCCL does with a buffer it wants a neighbour process to reach over legacy IPC.
extern "C" __attribute__((visibility("default"))) int standin_ipc_handle(void* ptr) {
  hipIpcMemHandle_t h;
  hipError_t e = hipIpcGetMemHandle(&h, ptr);
  (void)hipGetLastError();
  return (int)e;
}
