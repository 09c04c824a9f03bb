// Per-process state: the region registry, its counters and the engine resources.
// Mirrors the live members of the reference's gmm_client_ctx
// (amem_nccl_plugin/gmm_client.h:136-152) and its amem_allocMdata record
// (amem_nccl_plugin/amem_nccl.h:87-138).
#ifndef AMEM_CTX_H_
#define AMEM_CTX_H_

#include <stdint.h>
#include <sys/types.h>

#include <condition_variable>
#include <map>
#include <mutex>
#include <unordered_map>

#include "../../include/amem.h"

namespace amem {


// One tracked region, keyed by its virtual address. Field names follow the reference.
struct Region {
  int dev = 0;
  pid_t pid = 0;
  int refcount = 0;
  int sharedFD = 0;
  uint64_t handle = 0;
  uint64_t mcHandle = 0;
  size_t allocSz = 0;
  size_t tags = 0;
  int type = 0;
  int state = AMEM_STATE_INVALID;
  uint64_t peers[AMEM_MAX_DEVS] = {0};
  bool hasPeer = false;
  bool oosFlag = false;
  void* cpuAddr = nullptr;
  void* userInfo = nullptr;
  // engine bookkeeping (no reference counterpart)
  uint64_t parkedBytes = 0;
  uint64_t handleGen = 0;
  int ownerSlot = -1;  // imported regions: slot of the owning process, when known
};

static inline bool from_peer(int type) { return type > AMEM_TYPE_LOCAL_SYMM; }  // amem_nccl.h:82-84

struct Ctx {
  // `structure` guards insertion and erasure in the tables and is held for the whole of a
  // pause or resume, so the engine may keep pointers to map nodes. `fields` guards region
  // fields, counters and the handle index, which the IPC service thread also touches (peers[],
  // hasPeer, state of imported regions, releaseShadowCnt, handleTable lookups): readers hold
  // `fields`, writers of the tables hold both. Lock order: structure, then fields.
  std::mutex structure;
  std::mutex fields;
  std::condition_variable shadow_cv;  // signalled when releaseShadowCnt drops

  std::map<uint64_t, Region> allocTable[AMEM_MAX_DEVS];            // ascending VA
  std::unordered_map<uint64_t, uint64_t> handleTable[AMEM_MAX_DEVS];  // handle -> VA, local only

  int releaseLocalCnt = 0;
  int releaseShadowCnt = 0;
  int offloadCnt = 0;
  int smokeLog = 0;
  size_t allocBytes[AMEM_MAX_CALLER] = {0};
  size_t delBytes = 0;
  bool paused = false;
  size_t pauseCnt = 0;
  size_t resumeCnt = 0;

};

// Global switches set at load (amem_nccl.cpp:706-723) or through the C ABI.
struct Globals {
  int disabled = 1;  // AMEM_DISABLE_DEFAULT, amem_nccl.cpp:43
  int offload_free_tag = -1;
  Ctx* ctx = nullptr;
  std::mutex init_mtx;
};
Globals& globals();

// Current HIP device; 0 when HIP reports none (the reference ignores cudaGetDevice's
// status with curDev preset to 0, amem_nccl.cpp:300-301).
int current_device();
bool gpu_present();

}  // namespace amem
#endif
