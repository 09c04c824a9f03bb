// A C++ caller written against the reference's own API (names, default arguments and the
// amem_caller_type enum of amem_nccl_plugin/amem_nccl.h:330-367), as a patched NCCL would call it.
#include <stdio.h>
#include <unistd.h>

#include "amem_nccl.h"

int main() {
  amem_dptr_t ptr = 0x7f0000000000ull;
  amem_handle_t handle = 0x1234ull;
  if (amem_setGroupID(170) != 0) return 1;
  // the shape of the hook in ncclCuMemAlloc (nccl_patch/nccl_2.27.5-1.diff:278-280)
  if (amem_addAllocInfo(ptr, 4u << 20, 0, 0, handle, -1, 0, NULL, AMEM_CALLER_NCCL_P2P) != 0) return 2;
  // defaults: peerDev = -1, peerHandle = 0, userInfo = NULL, caller = AMEM_CALLER_NCCL_DEFAULT
  if (amem_addAllocInfo(ptr + (1ull << 30), 2u << 20, 0, 0, handle + 1) != 0) return 3;
  if (amem_addRefcount((void*)ptr, 1) != 0) return 4;
  if (amem_addPeerInfo(ptr, 0x5000, 3) != 0) return 5;
  if (amem_registerPeerInfo(handle, 0x6000, 4) != 0) return 6;
  if (amem_checkPaused() != false) return 7;
  int id = 0;
  amem_getGroupID(&id);
  if (id != 170 || amem_groupID != 170 || gmm_libP != NULL) return 8;
  amem_dumpAllocStats();
  if (amem_delAllocInfo(ptr, handle) != 0) return 9;           // default caller = -1
  if (amem_delAllocInfo(ptr + (1ull << 30), handle + 1, 0) != 0) return 10;
  if (amem_memPause(getpid()) != 0 || amem_memResume(getpid()) != 0) return 11;  // nothing tracked: no-ops
  printf("c++ reference caller ok\n");
  return 0;
}
