// HIP virtual-memory-management wrappers: the call sequences of the reference's static
// helpers (amem_nccl_plugin/amem_nccl.h:141-234) and of its VMM allocator
// (amem_nccl_plugin/gmm_cuda_mem_impl.cpp:84-283), on hipMem*.
#ifndef AMEM_VMM_H_
#define AMEM_VMM_H_

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

namespace amem {

// Print-and-continue error check, the reference's CHECK_DRV convention
// (gmm_cuda_common.h:38-55): the code is returned so the caller can accumulate it.
hipError_t check_hip(hipError_t e, const char* expr, const char* file, int line);
#define CHECK_HIP(x) amem::check_hip((x), #x, __FILE__, __LINE__)

static inline hipMemGenericAllocationHandle_t as_handle(uint64_t h) {
  return (hipMemGenericAllocationHandle_t)(uintptr_t)h;
}
static inline uint64_t handle_bits(hipMemGenericAllocationHandle_t h) {
  return (uint64_t)(uintptr_t)h;
}

static constexpr size_t kVmmAlign = 2ull << 20;  // gmm_cuda_mem_impl.cpp:242

// reserve -> create -> map -> setAccess, unwinding on failure.
hipError_t vmm_alloc(size_t bytes, int dev, uint64_t* va, uint64_t* handle, size_t* alloc_size);
// unmap -> release -> addressFree; the first two are skipped for a VA with no mapping.
hipError_t vmm_free(uint64_t va, size_t alloc_size, uint64_t handle);

// Drop the mapping at `va` and the references held on `handle`: one for the mapping's
// creator plus `extra` more (amem_cuMemReleaseHandle, amem_nccl.h:141-161, without its
// retain/release pair: the registry already knows the handle).
hipError_t vmm_unmap_release(uint64_t va, size_t size, uint64_t handle, int extra);
// The two halves of vmm_unmap_release, for callers that run them on different threads.
hipError_t vmm_unmap(uint64_t va, size_t size);
hipError_t vmm_release(uint64_t handle, int extra);

// New physical memory at an existing reservation (amem_cuAllocAndExport, amem_nccl.h:164-193).
hipError_t vmm_create_map(uint64_t va, int dev, size_t size, uint64_t* new_handle);
hipError_t vmm_export_fd(uint64_t handle, int* fd);
// Import an fd and map it at `va` (amem_importAndMap, amem_nccl.h:216-234). Closes `fd`
// when `close_fd`.
hipError_t vmm_import_map(int dev, uint64_t va, size_t size, int fd, bool close_fd,
                          uint64_t* new_handle);
// Allocation or mapping that contains `addr`: its base and size. False when the runtime knows none.
bool vmm_range_of(uint64_t addr, uint64_t* base, uint64_t* size);
// True when `va` is mapped through the virtual-memory API (safe to ask about any address).
bool vmm_is_mapped(uint64_t va);
// Handle currently mapped at `va`; 0 if none or if `va` is not virtual-memory-API memory. Takes no reference.
uint64_t vmm_handle_of(uint64_t va);
// Device that owns the physical memory behind `handle`, -1 if unknown.
int vmm_handle_device(uint64_t handle);

}  // namespace amem
#endif
