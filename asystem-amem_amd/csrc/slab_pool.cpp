#include "slab_pool.h"

#include "log.h"
#include "vmm.h"

namespace amem {

SlabPool::SlabPool(uint64_t slab_bytes) {
  shift_ = 16;
  while ((1ull << shift_) < slab_bytes && shift_ < 40) ++shift_;
  slab_bytes_ = 1ull << shift_;
}

SlabPool::~SlabPool() { trim(); }

hipError_t SlabPool::ensure(uint64_t bytes) {
  while (capacity() < bytes) {
    void* p = nullptr;
    // Default flags. Without hipHostMallocNumaUser the runtime places pinned memory on the NUMA
    // node closest to the current device, which is the placement the reference asks for by hand
    // (amem_allocHost, amem_nccl.h:251-267: the GPU's node, else node 0); the caller's current
    // device is the engine's device here. Coherent / non-coherent / portable variants measured
    // the same for both the copy engine and kernels that read or write the slab.
    // The benchmark prints where a slab ended up beside the GPU's node (host.slab_numa_node,
    // host.gpu_numa_node, host.nodes_online). The machines this was measured on expose a single
    // node (nodes_online "0", the GPU's numa_node -1), so placement cannot be wrong there and the
    // claim about the runtime's choice stays unmeasured on a multi-node host; what is measured is
    // that slabs made this way carry 0.95-0.98 of the host link in both directions.
    hipError_t e = CHECK_HIP(hipHostMalloc(&p, slab_bytes_, hipHostMallocDefault));
    if (e != hipSuccess) return e;
    slabs_.push_back((uint8_t*)p);
    LOGGER(DEBUG, "slab pool: +1 slab of %llu MiB, %zu slabs", (unsigned long long)(slab_bytes_ >> 20),
           slabs_.size());
  }
  return hipSuccess;
}

uint64_t SlabPool::trim() {
  uint64_t freed = capacity();
  for (uint8_t* p : slabs_) (void)CHECK_HIP(hipHostFree(p));
  slabs_.clear();
  return freed;
}

}  // namespace amem
