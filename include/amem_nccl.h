/*
 * amem_nccl.h — the reference plugin's own C++-linkage API, exported by libamem_nccl.so.1
 * beside the C ABI of amem.h, so that a caller compiled against the reference header
 * (amem_nccl_plugin/amem_nccl.h:330-367) links unchanged: same names, same parameter types
 * (hence the same mangled symbols), same default arguments, same return values.
 *
 * A virtual address and a physical handle are `unsigned long long` here exactly as
 * CUdeviceptr and CUmemGenericAllocationHandle are in the reference; no CUDA or HIP type
 * appears in a signature. Each function forwards to its C twin in amem.h.
 */
#ifndef AMEM_NCCL_H_
#define AMEM_NCCL_H_

#include <stddef.h>
#include <stdint.h>
#include <sys/types.h>

#include "amem.h"

#pragma GCC visibility push(default)

typedef unsigned long long amem_dptr_t;   /* CUdeviceptr in the reference */
typedef unsigned long long amem_handle_t; /* CUmemGenericAllocationHandle in the reference */

/* amem_nccl_plugin/amem_nccl.h:39-49: AMEM_STATE_INVALID, _ALLOC, _OFFLOADING, _HOLE, _PRELOADING,
 * _REMAPPED, _MAX with the reference's values; the enumerators live in amem.h. */
typedef enum amem_alloc_state amem_allocState;

/* amem_nccl_plugin/amem_nccl.h:52-64: AMEM_TYPE_CUMEM_LOCAL (= _LOCAL_POSIX = 0), _LOCAL_FABRIC 1,
 * _LOCAL_SYMM 2, _PEER_POSIX 3, _PEER_FABRIC 4, _PEER_SYMM 5, _MAX 6; the enumerators live in
 * amem.h, which is why the hook sites of the patched NCCL compile against this header as written. */
typedef enum amem_alloc_type amem_allocType;

/* amem_nccl_plugin/amem_nccl.h:82-84 */
static inline int amem_fromPeer(amem_allocType type) {
  return (type <= AMEM_TYPE_CUMEM_LOCAL_SYMM) ? 0 : 1;
}

/* amem_nccl_plugin/amem_nccl.h:67-80; values equal enum amem_caller of amem.h, which also holds
 * AMEM_CALLER_MAX. */
typedef enum {
  AMEM_CALLER_NCCL_DEFAULT = 0,
  AMEM_CALLER_NCCL_P2P = 1,
  AMEM_CALLER_NCCL_FABRIC = 2,
  AMEM_CALLER_NCCL_POSIX = 3,
  AMEM_CALLER_NCCL_SYMM = 4,
  AMEM_CALLER_NCCL_NVLS = 5,
  AMEM_CALLER_NCCL_RESERVED = 6,
  AMEM_CALLER_NCCL_P2P_PEER = 7,
  AMEM_CALLER_NCCL_RESERVED2 = 8,
  AMEM_CALLER_NCCL_PROXY = 9,
  AMEM_CALLER_NCCL_SYMM_PEER = 10
} amem_caller_type;

/* amem_nccl_plugin/amem_nccl.h:330 */
int amem_registerPeerInfo(amem_handle_t srcHandle, amem_dptr_t peerPtr, int peerDev);
/* amem_nccl_plugin/amem_nccl.h:333 */
int amem_addPeerInfo(amem_dptr_t srcPtr, amem_dptr_t peerPtr, int peerDev);
/* amem_nccl_plugin/amem_nccl.h:336 */
int amem_updatePeerInfo(amem_dptr_t dptr, int sharedFD);
/* amem_nccl_plugin/amem_nccl.h:344-346 */
int amem_addAllocInfo(amem_dptr_t localDptr, size_t allocSz, int type, int localDev,
                      amem_handle_t localHandle, int peerDev = -1, uint64_t peerHandle = 0ULL,
                      void* userInfo = NULL,
                      amem_caller_type caller_type = AMEM_CALLER_NCCL_DEFAULT);
/* amem_nccl_plugin/amem_nccl.h:348 */
int amem_delAllocInfo(amem_dptr_t dptr, amem_handle_t handle, int caller = -1);
/* amem_nccl_plugin/amem_nccl.h:351 */
int amem_memPause(pid_t pid, uint64_t tag = 0);
/* amem_nccl_plugin/amem_nccl.h:354 */
int amem_memResume(pid_t pid, uint64_t tag = 0);
/* amem_nccl_plugin/amem_nccl.h:356 */
void amem_dumpAllocStats(bool verbose = true);
/* amem_nccl_plugin/amem_nccl.h:359 */
bool amem_checkPaused(bool warn = true);
/* amem_nccl_plugin/amem_nccl.h:362 */
int amem_addRefcount(void* dptr, int refcount);
/* amem_nccl_plugin/amem_nccl.h:366-367 */
int amem_setGroupID(int id);
void amem_getGroupID(int* id);

/* Data symbols the reference library exports (amem_nccl.cpp:35-36). gmm_libP is the
 * reference's dlopen handle of the CUDA driver; it stays NULL here and exists only so
 * that the symbol resolves. */
extern void* gmm_libP;
extern int amem_groupID;

#pragma GCC visibility pop

#endif /* AMEM_NCCL_H_ */
