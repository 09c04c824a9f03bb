/*
 * amem_oracle.h — CPU restatement of the reference's pause/resume path. TEST INFRASTRUCTURE:
 * only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this; the
 * shipped library never does.
 *
 * It restates, in plain C and on host memory, what the reference does through the CUDA
 * driver (all citations are into /root/reference/amem_nccl_plugin/):
 *   - the region registry and its counters          amem_nccl.cpp:102-464, 679-703; amem_nccl.h:39-138
 *   - amem_memPause / amem_memResume                 amem_nccl.cpp:467-677
 *   - the VMM call order of the static helpers       amem_nccl.h:141-327
 *   - the peer bookkeeping across processes          gmm_client_impl.cpp:479-532, gmm_worker_impl.cpp:375-397
 * "Device memory" is host memory behind a VMM stand-in: reserve = mmap(PROT_NONE),
 * create = memfd, map = mmap(MAP_FIXED|MAP_SHARED) of the memfd at the reserved address,
 * export = dup of the memfd. Several simulated processes ("contexts", one per slot) live in
 * one real process; a peer RPC is a direct call into the other context.
 *
 * The reference cannot be built here (it needs the CUDA driver and runtime libraries and
 * nccl.h, none of which exist in this image), so there is no oracle/_ref. It holds no
 * golden vectors or unit tests for this path either. What pins each function:
 *   registry return codes / counters   closed forms read off the cited lines (tests/test_oracle_registry.py)
 *   ncclMemStats totals                the sample in the reference's README.md:206-211 (tests/golden/memstats_readme.json)
 *   pause counters                     the published log line in docs/images/run_result.webp
 *                                      (offload:549 releaseLocal:448 releasePeer:448; tests/golden/run_result_counters.json)
 *   restored bytes, same VA            identity: bytes before pause == bytes after resume, pointer equality
 *   zero flags / checksums             special cases with known answers and an independent numpy computation
 *   pack / unpack                      independent numpy slicing on small cases
 * Deliberate deviation from the reference text, shared with the engine: deleting a region
 * decrements the per-caller byte counter that its registration incremented (the reference
 * indexes that array with the delete call's `caller` argument, default -1, amem_nccl.cpp:437).
 */
#ifndef AMEM_ORACLE_H_
#define AMEM_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#define ORACLE_MAX_DEVS 8
#define ORACLE_MAX_CALLER 16
#define ORACLE_MAX_CTX 8
#define ORACLE_CHUNK 65536u

typedef struct oracle_region_info {
  uint64_t va, handle, mc_handle, alloc_sz, tags;
  uint64_t peers[ORACLE_MAX_DEVS];
  uint64_t cpu_addr, user_info;
  int32_t dev, pid, refcount, shared_fd, type, state, has_peer, oos_flag;
} oracle_region_info;

typedef struct oracle_counters {
  int64_t release_local_cnt, release_shadow_cnt, offload_cnt, smoke_log;
  uint64_t alloc_bytes[ORACLE_MAX_CALLER];
  uint64_t del_bytes, pause_cnt, resume_cnt;
  int32_t paused, group_id, handle_count, region_count;
} oracle_counters;

/* ---- VMM stand-in (gmm_cuda_mem_impl.cpp:237-283 call order; amem_nccl.h:141-234) ---- */
int oracle_vmm_alloc(uint64_t bytes, uint64_t* va, uint64_t* handle, uint64_t* alloc_size);
int oracle_vmm_free(uint64_t va, uint64_t alloc_size, uint64_t handle);
int oracle_vmm_export(uint64_t handle, int* fd);
int oracle_vmm_import(int fd, uint64_t size, uint64_t* va, uint64_t* handle);
uint64_t oracle_vmm_live_bytes(void);   /* bytes of physical memory (memfds) still referenced */
void oracle_vmm_reset(void);            /* test hygiene: unmap and close everything the stand-in still holds */
uint64_t oracle_vmm_handle_of(uint64_t va);
uint64_t oracle_vmm_retain(uint64_t va);   /* one more reference, as cuMemRetainAllocationHandle takes */

/* ---- contexts: one simulated process per slot ---- */
void oracle_reset(void);                /* drop every context, keep VMM objects */
int oracle_ctx_enable(int slot, int on); /* AMEM_ENABLE for that simulated process */

/* ---- registry (same argument meaning as the C ABI in include/amem.h) ---- */
int oracle_add_alloc_info(int ctx, uint64_t va, uint64_t size, int type, int dev, uint64_t handle, int peer_dev,
                          uint64_t peer_handle, uint64_t user_info, int caller);
int oracle_del_alloc_info(int ctx, uint64_t va, uint64_t handle, int caller);
int oracle_add_refcount(int ctx, uint64_t va, int n);
int oracle_add_peer_info(int ctx, uint64_t src_va, uint64_t peer_va, int peer_dev);
int oracle_register_peer_info(int ctx, uint64_t src_handle, uint64_t peer_va, int peer_dev);
int oracle_update_peer_info(int ctx, uint64_t va, int shared_fd);
int oracle_check_paused(int ctx);
int oracle_set_group_id(int ctx, int id);
int oracle_get_group_id(int ctx);
uint64_t oracle_mem_stats_total(int ctx);

/* ---- pause / resume ---- */
int oracle_mem_pause(int ctx);
/* Returns 0 when complete; 2 when this context still waits for owners to re-export
 * (the reference spins there, amem_nccl.cpp:659-662): call again after the owners resumed. */
int oracle_mem_resume(int ctx);
/* Same data path with regions sharded over `threads` host threads (the all-cores baseline). */
int oracle_mem_pause_mt(int ctx, int threads);
int oracle_mem_resume_mt(int ctx, int threads);

/* ---- inspection ---- */
int64_t oracle_region_count(int ctx, int dev);
int oracle_region_at(int ctx, int dev, int64_t index, oracle_region_info* out); /* ascending VA */
int oracle_region_find(int ctx, int dev, uint64_t va, oracle_region_info* out);
uint64_t oracle_handle_lookup(int ctx, int dev, uint64_t handle);
void oracle_get_counters(int ctx, oracle_counters* out);

/* ---- CPU twins of the device kernels ---- */
typedef struct oracle_chunk_sum { uint64_t sum64, xor64; } oracle_chunk_sum;
typedef struct oracle_copy_desc { uint64_t va, off, bytes; } oracle_copy_desc;
#define ORACLE_DESC_ZERO (~(uint64_t)0)
/* flags[c] = 1 iff chunk c of [ptr, ptr+bytes) is all zero; sums may be NULL. Returns chunk count. */
uint64_t oracle_zero_scan(const void* ptr, uint64_t bytes, uint8_t* flags, oracle_chunk_sum* sums);
void oracle_gather_pack(const oracle_copy_desc* descs, uint64_t n, void* staging);
void oracle_scatter_unpack(const oracle_copy_desc* descs, uint64_t n, const void* staging);

#endif
