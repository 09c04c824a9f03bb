// A native caller on the GPU, written the way a patched RCCL would use the plugin: memory comes
// from the HIP virtual-memory API in the order of the reference's allocator hook site
// (nccl_patch/nccl_2.27.5-1.diff:262-280: create, reserve, map, set access, then amem_addAllocInfo),
// pause and resume go through the reference's own C++ names, and the free path looks the handle up
// from the address because the one kept from allocation time is stale after a resume
// (diff:286-296). No Python, no test harness: only this file, the two headers and the library.
#include <hip/hip_runtime_api.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include <vector>

#include "amem_nccl.h"

#define HIP_OK(x)                                                                       \
  do {                                                                                  \
    hipError_t e_ = (x);                                                                \
    if (e_ != hipSuccess) {                                                             \
      printf("%s:%d %s -> %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_));        \
      return 100;                                                                       \
    }                                                                                   \
  } while (0)

struct Buf {
  void* ptr;
  size_t size;
  hipMemGenericAllocationHandle_t handle;
  std::vector<unsigned char> expect;
};

static unsigned long long xorshift(unsigned long long& s) {
  s ^= s << 13; s ^= s >> 7; s ^= s << 17;
  return s;
}

int main() {
  int dev = 0;
  HIP_OK(hipSetDevice(dev));
  hipMemAllocationProp prop;
  memset(&prop, 0, sizeof(prop));
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.location.id = dev;
  prop.requestedHandleTypes = hipMemHandleTypePosixFileDescriptor;
  size_t gran = 0;
  HIP_OK(hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityRecommended));
  if (gran < (2u << 20)) gran = 2u << 20;

  if (amem_setGroupID(170) != 0) return 1;
  const size_t want[] = {3u << 20, 8u << 20, (2u << 20) + 4096, 24u << 20};
  std::vector<Buf> bufs;
  unsigned long long seed = 0x9E3779B97F4A7C15ull;
  for (size_t w : want) {
    Buf b;
    b.size = (w + gran - 1) / gran * gran;
    HIP_OK(hipMemCreate(&b.handle, b.size, &prop, 0));
    HIP_OK(hipMemAddressReserve(&b.ptr, b.size, gran, NULL, 0));
    HIP_OK(hipMemMap(b.ptr, b.size, 0, b.handle, 0));
    hipMemAccessDesc acc;
    memset(&acc, 0, sizeof(acc));
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = dev;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    HIP_OK(hipMemSetAccess(b.ptr, b.size, &acc, 1));
    if (amem_addAllocInfo((amem_dptr_t)(uintptr_t)b.ptr, b.size, AMEM_TYPE_LOCAL, dev,
                          (amem_handle_t)(uintptr_t)b.handle, -1, 0, NULL, AMEM_CALLER_NCCL_P2P) != 0)
      return 2;
    b.expect.assign(b.size, 0);
    for (size_t i = 0; i < b.size; i += 8) {           // every third 64 KiB chunk stays zero
      if ((i >> 16) % 3 == 2) continue;
      unsigned long long v = xorshift(seed);
      memcpy(&b.expect[i], &v, 8);
    }
    HIP_OK(hipMemcpy(b.ptr, b.expect.data(), b.size, hipMemcpyHostToDevice));
    bufs.push_back(b);
  }
  amem_dumpAllocStats();

  size_t total = 0;
  for (const Buf& b : bufs) total += b.size;
  for (int cycle = 0; cycle < 3; ++cycle) {
    size_t free0 = 0, free1 = 0, free2 = 0, all = 0;
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemGetInfo(&free0, &all));
    if (amem_memPause(getpid()) != 0) return 3;
    if (!amem_checkPaused(false)) return 4;
    HIP_OK(hipMemGetInfo(&free1, &all));
    if (cycle > 0 && free1 < free0 + total - (4u << 20)) {       // cycle 0 also allocates the engine's tables
      printf("pause released %zu of %zu bytes\n", free1 - free0, total);
      return 5;
    }
    // registering while paused is refused, as in the reference (amem_nccl.cpp:133-137)
    if (amem_addAllocInfo(0x7f0000000000ull, 2u << 20, AMEM_TYPE_LOCAL, dev, 0x1234ull) != 1) return 6;
    if (amem_memResume(getpid()) != 0) return 7;
    if (amem_checkPaused(false)) return 8;
    HIP_OK(hipMemGetInfo(&free2, &all));
    for (Buf& b : bufs) {
      std::vector<unsigned char> got(b.size);
      HIP_OK(hipMemcpy(got.data(), b.ptr, b.size, hipMemcpyDeviceToHost));   // the pointer kept from before the pause
      if (memcmp(got.data(), b.expect.data(), b.size) != 0) {
        printf("cycle %d: bytes at %p differ after resume\n", cycle, b.ptr);
        return 9;
      }
      unsigned long long v = xorshift(seed);                                  // and the memory is writable again
      size_t at = (size_t)(v % (b.size / 8)) * 8;
      memcpy(&b.expect[at], &v, 8);
      HIP_OK(hipMemcpy((char*)b.ptr + at, &v, 8, hipMemcpyHostToDevice));
    }
  }

  for (Buf& b : bufs) {
    hipMemGenericAllocationHandle_t now = NULL;
    HIP_OK(hipMemRetainAllocationHandle(&now, b.ptr));     // the allocation-time handle is stale by now
    if (now == NULL) return 10;
    if (amem_delAllocInfo((amem_dptr_t)(uintptr_t)b.ptr, (amem_handle_t)(uintptr_t)now, 0) != 0) return 11;
    HIP_OK(hipMemUnmap(b.ptr, b.size));
    HIP_OK(hipMemRelease(now));
    HIP_OK(hipMemAddressFree(b.ptr, b.size));
  }
  if (amem_memPause(getpid()) != 0 || amem_memResume(getpid()) != 0) return 12;   // nothing tracked any more
  printf("c++ cycle on the gpu ok\n");
  return 0;
}
