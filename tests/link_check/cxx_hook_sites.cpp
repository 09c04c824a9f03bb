// The hook sites of the reference's NCCL patch, compiled against this repository's amem_nccl.h.
//
// Every statement between a "diff:<line>" comment and the next blank line is the text of that line
// of nccl_patch/nccl_2.27.5-1.diff (leading '+' and indentation removed): the calls a patched NCCL
// makes into the plugin. What NCCL and the CUDA driver would supply around them (CUdeviceptr,
// CUmemGenericAllocationHandle, the comm / proxy / IPC structures, ncclResult_t) is declared here
// with just the members those lines touch. The file is built with -Wall -Wextra -Werror; main()
// walks through the sites on a registry without a GPU and checks what the calls return.
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <unistd.h>

#include "amem_nccl.h"

typedef unsigned long long CUdeviceptr;
typedef unsigned long long CUmemGenericAllocationHandle;
typedef enum { ncclSuccess = 0 } ncclResult_t;
enum { CU_MEM_HANDLE_TYPE_POSIX_FILE_DESCRIPTOR = 1, CU_MEM_HANDLE_TYPE_FABRIC = 8 };
struct ncclComm { int cudaDev; int rank; void* baseUCSymPtr; };
typedef struct ncclComm* ncclComm_t;
struct ncclProxyState { int cudaDev; };
struct ncclProxyConnection { int sameProcess; };
struct ncclIpcImpInfo { size_t size; size_t offset; int impFd; };
struct ncclReg { uintptr_t begAddr; };
typedef struct { char data[64]; } CUmemFabricHandle;
typedef union { uint64_t data; CUmemFabricHandle handle; } ncclCuDesc;

static int g_ret[32];
static int g_n = 0;
#define NOTE(call) (g_ret[g_n++] = (call))

// src/allocator.cc, ncclMemAlloc
static void site_ncclMemAlloc(void** ptr, size_t handleSize, int currentDev, CUmemGenericAllocationHandle handle,
                              int requestedHandleTypes) {
  // diff:42-46
  if (requestedHandleTypes == CU_MEM_HANDLE_TYPE_FABRIC) {
  NOTE(
  amem_addAllocInfo((CUdeviceptr)*ptr, handleSize, AMEM_TYPE_CUMEM_LOCAL_FABRIC, currentDev, handle, -1, 0, NULL, AMEM_CALLER_NCCL_FABRIC)
  );
  } else {
  NOTE(
  amem_addAllocInfo((CUdeviceptr)*ptr, handleSize, AMEM_TYPE_CUMEM_LOCAL_POSIX, currentDev, handle, -1, 0, NULL, AMEM_CALLER_NCCL_POSIX)
  );
  }
}

// src/allocator.cc, ncclCommSymmetricAllocInternal
static void site_symmetricAlloc(struct ncclComm* comm, void* regSymAddr, size_t allocSize, int cuDev,
                                CUmemGenericAllocationHandle memHandle) {
  // diff:57
  NOTE(
  amem_addAllocInfo((CUdeviceptr)regSymAddr, allocSize, AMEM_TYPE_CUMEM_LOCAL_SYMM, cuDev, memHandle, -1, 0, comm, AMEM_CALLER_NCCL_SYMM)
  );
}

// src/include/alloc.h, ncclCuMemAllocAddr / ncclCuMemFreeAddr / ncclCuMemAlloc / ncclCuMemFree
static void site_ncclCuMemAllocAddr(void** ptr, CUmemGenericAllocationHandle* handleIn, size_t size, int cudaDev) {
  // diff:259
  NOTE(
  amem_addAllocInfo((CUdeviceptr)ptr, size, AMEM_TYPE_CUMEM_LOCAL, cudaDev, *handleIn, -1, 0, NULL, AMEM_CALLER_NCCL_DEFAULT)
  );
}
static void site_ncclCuMemFreeAddr(void* ptr) {
  // diff:269
  NOTE(
  amem_delAllocInfo((CUdeviceptr) ptr, 0, 0)
  );
}
static void site_ncclCuMemAlloc(void** ptr, size_t size, int currentDev, CUmemGenericAllocationHandle handle) {
  // diff:279
  NOTE(
  amem_addAllocInfo((CUdeviceptr)*ptr, size, AMEM_TYPE_CUMEM_LOCAL, currentDev, handle, -1, 0, NULL, AMEM_CALLER_NCCL_P2P)
  );
}
static void site_ncclCuMemFree(void* ptr, CUmemGenericAllocationHandle handle) {
  // diff:289
  NOTE(
  amem_delAllocInfo((CUdeviceptr) ptr, handle, 0)
  );
}

// src/include/alloc.h and src/transport/net.cc, the "defensive remove" of buffers registered with a NIC
static void site_defensiveRemove(void* devMem) {
  // diff:311
  NOTE(
  amem_delAllocInfo((CUdeviceptr)devMem, 0, 0)
  );
}

// src/transport/nvls.cc, nvlsAllocateMem
static void site_nvls(struct ncclComm* comm, void** ucptr, size_t ucsize, CUmemGenericAllocationHandle* ucHandle,
                      CUmemGenericAllocationHandle* mcHandle) {
  // diff:532
  NOTE(
  amem_addAllocInfo((CUdeviceptr)*ucptr, ucsize, AMEM_TYPE_CUMEM_LOCAL_SYMM, comm->cudaDev, (uint64_t)*ucHandle, -1, (uint64_t)*mcHandle, comm, AMEM_CALLER_NCCL_NVLS)
  );
}

// src/transport/p2p.cc, ncclP2pAllocateShareableBuffer (behind a misspelt guard in the patch, so never built there)
static void site_addRefcount(void** ptr, int refcount) {
  // diff:546
  NOTE(
  amem_addRefcount(*ptr, refcount)
  );
}

// src/transport/p2p.cc, ncclP2pImportShareableBuffer
static void site_import(struct ncclComm* comm, CUdeviceptr dptr, size_t size, CUmemGenericAllocationHandle handle,
                        int peerDev, ncclCuDesc* cuDesc, int type) {
  // diff:574-578
  if (type == CU_MEM_HANDLE_TYPE_POSIX_FILE_DESCRIPTOR) {
  NOTE(
  amem_addAllocInfo(dptr, size, AMEM_TYPE_CUMEM_PEER_POSIX, comm->cudaDev, handle, peerDev, (uint64_t)cuDesc->data, comm, AMEM_CALLER_NCCL_P2P_PEER)
  );
  } else {
  NOTE(
  amem_addAllocInfo(dptr, size, AMEM_TYPE_CUMEM_PEER_FABRIC, comm->cudaDev, handle, peerDev, (uint64_t)cuDesc, comm, AMEM_CALLER_NCCL_P2P_PEER)
  );
  }
}

// src/transport/p2p.cc, ncclIpcLocalRegisterBuffer
static void site_addPeerInfo(struct ncclReg* regRecord, void* rmtRegAddr, int peerRank) {
  // diff:631
  NOTE(
  amem_addPeerInfo(regRecord->begAddr, (CUdeviceptr)rmtRegAddr, peerRank)
  );
}

// src/transport/p2p.cc, p2pProxyRegister and its failure path
static void site_proxyRegister(struct ncclProxyConnection* connection, struct ncclProxyState* proxyState, void* regAddr,
                               struct ncclIpcImpInfo* ipcExpInfo, CUmemGenericAllocationHandle handle,
                               int ncclCuMemHandleType) {
  // diff:641-643
  if (ncclCuMemHandleType == CU_MEM_HANDLE_TYPE_POSIX_FILE_DESCRIPTOR) { // No peer info available!!
  NOTE(
  amem_addAllocInfo((CUdeviceptr)regAddr, ipcExpInfo->size, AMEM_TYPE_CUMEM_PEER_POSIX, proxyState->cudaDev, handle, -1, ipcExpInfo->impFd, connection, AMEM_CALLER_NCCL_PROXY)
  );
  }
  // diff:653
  NOTE(
  amem_delAllocInfo((CUdeviceptr) regAddr, 0, 0)
  );
}

// src/transport/p2p.cc, ncclIpcSymmetricFinalize
static void site_symmetricFinalize(struct ncclComm* comm) {
  // diff:663
  NOTE(
  amem_delAllocInfo((CUdeviceptr) comm->baseUCSymPtr, 0, 0)
  );
}

// src/init.cc: the five public entry points (diff:70-111), without NCCL's tracing macros
static ncclResult_t site_ncclPause(ncclComm_t* comm) {
  (void)comm;
  ncclResult_t ret = ncclSuccess;
  // diff:74
  amem_memPause(getpid(), 0);

  return ret;
}
static ncclResult_t site_ncclResume(ncclComm_t* comm) {
  (void)comm;
  ncclResult_t ret = ncclSuccess;
  // diff:84
  amem_memResume(getpid(), 0);

  return ret;
}
static ncclResult_t site_ncclMemStats() {
  ncclResult_t ret = ncclSuccess;
  // diff:95
  amem_dumpAllocStats();

  return ret;
}
static ncclResult_t site_ncclSetGroupID(int id) {
  // diff:103-104
  int ret_ = amem_setGroupID(id);
  return (ncclResult_t) ret_;
}
static ncclResult_t site_ncclGetGroupID(int *id) {
  // diff:109-110
  amem_getGroupID(id);
  return ncclSuccess;
}

// every public collective (diff:121-229)
static bool site_gate() {
  // diff:121
  return
  amem_checkPaused()
  ;
}

int main() {
  // the reference's enumerators carry the reference's values (amem_nccl.h:39-64 of the plugin)
  static_assert(AMEM_TYPE_CUMEM_LOCAL == 0 && AMEM_TYPE_CUMEM_LOCAL_POSIX == 0 && AMEM_TYPE_CUMEM_LOCAL_FABRIC == 1 &&
                AMEM_TYPE_CUMEM_LOCAL_SYMM == 2 && AMEM_TYPE_CUMEM_PEER_POSIX == 3 && AMEM_TYPE_CUMEM_PEER_FABRIC == 4 &&
                AMEM_TYPE_CUMEM_PEER_SYMM == 5 && AMEM_TYPE_CUMEM_MAX == 6, "amem_allocType");
  static_assert(AMEM_STATE_INVALID == 0 && AMEM_STATE_ALLOC == 1 && AMEM_STATE_OFFLOADING == 2 && AMEM_STATE_HOLE == 3 &&
                AMEM_STATE_PRELOADING == 4 && AMEM_STATE_REMAPPED == 5 && AMEM_STATE_MAX == 6, "amem_allocState");
  static_assert(AMEM_CALLER_NCCL_SYMM_PEER == 10 && AMEM_CALLER_MAX == AMEM_MAX_CALLER && AMEM_MAX_DEVS == 8, "callers");
  amem_allocState st = AMEM_STATE_HOLE;
  amem_allocType ty = AMEM_TYPE_CUMEM_PEER_SYMM;
  if (amem_fromPeer(AMEM_TYPE_CUMEM_LOCAL_SYMM) != 0 || amem_fromPeer(AMEM_TYPE_CUMEM_PEER_POSIX) != 1 ||
      amem_fromPeer(ty) != 1 || st != 3) return 1;

  struct ncclComm comm = {0, 0, (void*)0x7f3000000000ull};
  struct ncclProxyState proxy = {0};
  struct ncclProxyConnection conn = {0};
  struct ncclIpcImpInfo imp = {2u << 20, 0, 42};
  struct ncclReg reg = {0x7f1000000000ull};
  ncclCuDesc desc;
  memset(&desc, 0, sizeof(desc));
  desc.data = 0x1111;
  void* p1 = (void*)0x7f1000000000ull;
  void* p2 = (void*)0x7f1100000000ull;
  void* p3 = (void*)0x7f1200000000ull;
  void* p4 = (void*)0x7f1300000000ull;
  void* p5 = (void*)0x7f1400000000ull;
  CUmemGenericAllocationHandle h = 0x1111, mc = 0x9999;
  int id = -1;
  if (site_ncclSetGroupID(171) != ncclSuccess || site_ncclGetGroupID(&id) != ncclSuccess || id != 171) return 2;
  site_ncclMemAlloc(&p1, 4u << 20, 0, h, CU_MEM_HANDLE_TYPE_POSIX_FILE_DESCRIPTOR);   // [0]
  site_ncclMemAlloc(&p2, 4u << 20, 0, h + 1, CU_MEM_HANDLE_TYPE_FABRIC);               // [1]
  site_symmetricAlloc(&comm, p3, 2u << 20, 0, h + 2);                                  // [2]
  site_ncclCuMemAlloc(&p4, 8u << 20, 0, h + 3);                                        // [3]
  site_nvls(&comm, &p5, 2u << 20, &h, &mc);                                            // [4] a known handle again: accepted
  void* holder = p4;
  CUmemGenericAllocationHandle hin = h + 5;
  site_ncclCuMemAllocAddr(&holder, &hin, 2u << 20, 0);                                 // [5] registers the address of `holder`, as the patch does
  site_addRefcount(&p4, 2);                                                            // [6]
  site_addPeerInfo(&reg, (void*)0x7f2000000000ull, 3);                                 // [7]
  if (site_gate()) return 3;
  if (site_ncclMemStats() != ncclSuccess) return 4;
  for (int i = 0; i < g_n; ++i)
    if (g_ret[i] != 0) { printf("hook site %d returned %d\n", i, g_ret[i]); return 5; }
  const int local_sites = g_n;
  // importer-side sites: without a peer service to register with, the entry is dropped again and the
  // call reports it (amem_nccl.cpp:209-220, :245-256 of the plugin)
  site_import(&comm, 0x7f4000000000ull, 2u << 20, h + 6, 1, &desc, CU_MEM_HANDLE_TYPE_POSIX_FILE_DESCRIPTOR);
  site_import(&comm, 0x7f4100000000ull, 2u << 20, h + 7, 1, &desc, CU_MEM_HANDLE_TYPE_FABRIC);
  site_proxyRegister(&conn, &proxy, (void*)0x7f4200000000ull, &imp, h + 8, CU_MEM_HANDLE_TYPE_POSIX_FILE_DESCRIPTOR);
  for (int i = local_sites; i < local_sites + 3; ++i)
    if (g_ret[i] == 0) { printf("importer site %d was accepted without an owner\n", i); return 6; }
  if (g_ret[local_sites + 3] != 0) return 7;   // the delete on the failure path always returns 0
  site_ncclCuMemFree(p4, h + 3);
  site_ncclCuMemFreeAddr((void*)&holder);
  site_defensiveRemove(p1);
  comm.baseUCSymPtr = p3;
  site_symmetricFinalize(&comm);
  if (site_ncclPause(NULL) != ncclSuccess || site_ncclResume(NULL) != ncclSuccess) return 8;
  printf("hook sites ok: %d calls\n", g_n);
  return 0;
}
