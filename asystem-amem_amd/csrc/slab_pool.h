// Pinned host slab pool: where paused bytes live. Replaces the reference's one private
// pinned buffer per region, created on first pause and never freed (amem_allocHost,
// amem_nccl_plugin/amem_nccl.h:237-283; call site amem_nccl.cpp:505-508) and the host-memory
// records of gmm_host_mem.h:37-65. Slabs are equally sized hipHostMalloc blocks, reused by
// every later cycle; the parked bytes of a cycle occupy logical offsets [0, used) laid
// across the slabs in order.
#ifndef AMEM_SLAB_POOL_H_
#define AMEM_SLAB_POOL_H_

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <vector>

namespace amem {

class SlabPool {
 public:
  explicit SlabPool(uint64_t slab_bytes);
  ~SlabPool();
  // Make logical offsets [0, bytes) addressable. Allocates slabs as needed.
  hipError_t ensure(uint64_t bytes);
  uint64_t slab_bytes() const { return slab_bytes_; }
  uint32_t shift() const { return shift_; }
  uint64_t capacity() const { return (uint64_t)slabs_.size() * slab_bytes_; }
  size_t slab_count() const { return slabs_.size(); }
  // Host address of a logical offset.
  uint8_t* host_addr(uint64_t off) const { return slabs_[off >> shift_] + (off & (slab_bytes_ - 1)); }
  const std::vector<uint8_t*>& slabs() const { return slabs_; }
  // Bytes from `off` to the end of its slab.
  uint64_t room(uint64_t off) const { return slab_bytes_ - (off & (slab_bytes_ - 1)); }
  uint64_t trim();

 private:
  uint64_t slab_bytes_;
  uint32_t shift_;
  std::vector<uint8_t*> slabs_;
};

}  // namespace amem
#endif
