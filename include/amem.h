/*
 * amem.h — C ABI of the MI355X AMem pause/resume engine (libamem_nccl.so.1).
 *
 * Plain C: fixed-width integers, pointers and sizes only. Device virtual addresses and
 * physical-allocation handles cross this boundary as opaque uint64_t (the reference's
 * CUdeviceptr / CUmemGenericAllocationHandle are both `unsigned long long`); inside the
 * library they are cast to hipDeviceptr_t / hipMemGenericAllocationHandle_t.
 *
 * Every entry point that replaces a function of the reference cites it as
 * `amem_nccl_plugin/<file>:<line>`. The same library also exports the reference's
 * C++-linkage names with identical signatures (see amem_nccl.h) so that code compiled
 * against the reference header links unchanged.
 *
 * Error convention (reference: gmm_cuda_common.h:38-55, amem_nccl.cpp return paths):
 * int 0 = success, non-zero = failure or rejection. While the engine is disabled
 * (AMEM_ENABLE unset or 0, or NCCL_CUMEM_ENABLE=0; amem_nccl.cpp:711-718) every
 * reference-mirroring entry point returns 0 and does nothing.
 */
#ifndef AMEM_H_
#define AMEM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
/* The library is built with hidden visibility; everything declared here is exported. */
#pragma GCC visibility push(default)

#define AMEM_MAX_DEVS 8    /* amem_nccl.h:32; also the length of peers[] */
#define AMEM_MAX_CALLER 16 /* amem_nccl.h:33 */
#define AMEM_CHUNK_BYTES 65536u /* zero-detect / checksum chunk */

/* amem_nccl.h:39-49 */
enum amem_alloc_state {
  AMEM_STATE_INVALID = 0,
  AMEM_STATE_ALLOC = 1,
  AMEM_STATE_OFFLOADING = 2,
  AMEM_STATE_HOLE = 3,
  AMEM_STATE_PRELOADING = 4,
  AMEM_STATE_REMAPPED = 5,
  AMEM_STATE_MAX = 6
};

/* amem_nccl.h:52-64. type <= LOCAL_SYMM means the region owns its bytes. Every value has two
 * spellings: the reference's own (AMEM_TYPE_CUMEM_*, which its hook sites use) and a shorter
 * one without the CUDA driver's prefix. */
enum amem_alloc_type {
  AMEM_TYPE_CUMEM_LOCAL = 0,
  AMEM_TYPE_CUMEM_LOCAL_POSIX = 0,
  AMEM_TYPE_CUMEM_LOCAL_FABRIC = 1,
  AMEM_TYPE_CUMEM_LOCAL_SYMM = 2,
  AMEM_TYPE_CUMEM_PEER_POSIX = 3,
  AMEM_TYPE_CUMEM_PEER_FABRIC = 4,
  AMEM_TYPE_CUMEM_PEER_SYMM = 5,
  AMEM_TYPE_CUMEM_MAX = 6,
  AMEM_TYPE_LOCAL = AMEM_TYPE_CUMEM_LOCAL,
  AMEM_TYPE_LOCAL_POSIX = AMEM_TYPE_CUMEM_LOCAL_POSIX,
  AMEM_TYPE_LOCAL_FABRIC = AMEM_TYPE_CUMEM_LOCAL_FABRIC,
  AMEM_TYPE_LOCAL_SYMM = AMEM_TYPE_CUMEM_LOCAL_SYMM,
  AMEM_TYPE_PEER_POSIX = AMEM_TYPE_CUMEM_PEER_POSIX,
  AMEM_TYPE_PEER_FABRIC = AMEM_TYPE_CUMEM_PEER_FABRIC,
  AMEM_TYPE_PEER_SYMM = AMEM_TYPE_CUMEM_PEER_SYMM,
  AMEM_TYPE_MAX = AMEM_TYPE_CUMEM_MAX
};

/* amem_nccl.h:67-80 */
enum amem_caller {
  AMEM_CALLER_DEFAULT = 0,
  AMEM_CALLER_P2P = 1,
  AMEM_CALLER_FABRIC = 2,
  AMEM_CALLER_POSIX = 3,
  AMEM_CALLER_SYMM = 4,
  AMEM_CALLER_NVLS = 5,
  AMEM_CALLER_RESERVED = 6,
  AMEM_CALLER_P2P_PEER = 7,
  AMEM_CALLER_RESERVED2 = 8,
  AMEM_CALLER_PROXY = 9,
  AMEM_CALLER_SYMM_PEER = 10,
  AMEM_CALLER_MAX = AMEM_MAX_CALLER
};

/* ---------------------------------------------------------------------------------------
 * 1. The allocator hook and the per-process region registry
 * ------------------------------------------------------------------------------------- */

/* Record one VMM allocation (local) or one imported mapping (peer).
 * Replaces amem_addAllocInfo, amem_nccl.cpp:102-269 (declared amem_nccl.h:344-346).
 * Returns 0; 1 when called while paused (:133-137) or when a peer mapping's owner cannot
 * be determined (:245-256); the RPC status when registering with the owner fails, in which
 * case the entry is erased again (:209-220).
 * For peer types `peer_dev` names the owner: the owner's slot (see amem_get_slot) when
 * several processes share one GPU, which is the only multi-process layout this library
 * runs; -1 asks the library to detect it from the handle. */
int amem_add_alloc_info(uint64_t va, uint64_t size, int type, int dev, uint64_t handle,
                        int peer_dev, uint64_t peer_handle, void* user_info, int caller);

/* Forget a region before its VA is freed. Replaces amem_delAllocInfo,
 * amem_nccl.cpp:414-448. handle == 0 asks the library to look the handle up from the
 * mapping. Always returns 0. The per-caller byte counter that the add incremented is the
 * one decremented (the reference indexes by this call's `caller` argument instead, which
 * its hooks hard-code to 0; the argument is accepted and ignored here). */
int amem_del_alloc_info(uint64_t va, uint64_t handle, int caller);

/* Add `n` extra physical-handle references that pause must also drop.
 * Replaces amem_addRefcount, amem_nccl.cpp:332-356. 0 ok, 1 region not found. */
int amem_add_refcount(void* va, int n);

/* Same-process peer record: peers[peer_dev] = peer_va, hasPeer = true.
 * Replaces amem_addPeerInfo, amem_nccl.cpp:359-381. 0 ok, 1 not found. */
int amem_add_peer_info(uint64_t src_va, uint64_t peer_va, int peer_dev);

/* Owner-side half of an import: find the local region that `src_handle` backs and
 * record the importer's VA. Replaces amem_registerPeerInfo, amem_nccl.cpp:297-329.
 * Runs on the IPC service thread when an importer registers. 0 ok, 1 not found.
 * Extension: a value that is no handle of this process is also looked up as the address of a
 * local region. An importer that cannot know the owner's current handle value (it changes with
 * every resume) may name the region by the owner's address, which never changes; the allocator
 * hook for an unpatched RCCL does. */
int amem_register_peer_info(uint64_t src_handle, uint64_t peer_va, int peer_dev);

/* Importer-side half of a resume: import `shared_fd`, map it at the region's original VA,
 * close the fd. Replaces amem_updatePeerInfo, amem_nccl.cpp:385-409. 0 ok. */
int amem_update_peer_info(uint64_t va, int shared_fd);

/* Paused gate. Replaces amem_checkPaused, amem_nccl.cpp:452-464. Returns 1 when paused. */
int amem_check_paused(int warn);

/* Group id, settable only before the first tracked allocation.
 * Replace amem_setGroupID / amem_getGroupID, amem_nccl.cpp:679-703. set: 0 ok, 1 too late. */
int amem_set_group_id(int id);
void amem_get_group_id(int* id);

/* Per-caller byte statistics to stdout. Replaces amem_dumpAllocStats, amem_nccl.cpp:82-99. */
void amem_dump_alloc_stats(int verbose);

/* ---------------------------------------------------------------------------------------
 * 2. Pause / resume
 * ------------------------------------------------------------------------------------- */

/* Park the bytes of every local region of the current device in pinned host memory,
 * then unmap and release all physical memory behind every tracked VA (imported mappings
 * first). VAs stay reserved. Replaces amem_memPause, amem_nccl.cpp:467-574.
 * Idempotent; returns 0, or non-zero when a HIP call failed (the reference always
 * returns 0 and only prints driver errors). */
int amem_mem_pause(int pid, uint64_t tag);

/* Re-create physical memory at the identical VAs, restore the bytes, re-export to every
 * recorded importer and wait until every mapping this process imports is back.
 * Replaces amem_memResume, amem_nccl.cpp:577-677. Idempotent. */
int amem_mem_resume(int pid, uint64_t tag);

/* The five public names the patched NCCL exports (nccl_patch/nccl_2.27.5-1.diff:68-112,
 * :337-351). `comm` is ignored. ncclPause/ncclResume report 0 whatever the inner call
 * returned, as the reference does (:70-88); ncclSetGroupID returns the inner int (:102-105). */
int ncclPause(void* comm);
int ncclResume(void* comm);
int ncclMemStats(void);
int ncclSetGroupID(int id);
int ncclGetGroupID(int* id);

/* ---------------------------------------------------------------------------------------
 * 3. VMM allocation helpers
 * ------------------------------------------------------------------------------------- */

/* Reserve a VA range, create device memory exportable as a POSIX fd, map it and grant
 * read/write to `dev`; unwinds on failure. `bytes` is rounded up to 2 MiB.
 * Replaces gmm_cuda_vmm_alloc, gmm_cuda_mem_impl.cpp:237-273 (call order and unwind of
 * gpu_vmm_alloc, :84-194). Does not register the region. */
int amem_vmm_alloc(uint64_t bytes, int dev, uint64_t* va, uint64_t* handle,
                   uint64_t* alloc_size);

/* Unmap, release and free the VA range. Works for a region in any state: a region the
 * engine has paused (no physical memory) only has its reservation freed.
 * Replaces gmm_cuda_vmm_free / gpu_vmm_free, gmm_cuda_mem_impl.cpp:196-222, :275-283.
 * `handle` may be 0: the current handle is then looked up from the mapping, which is what
 * a caller must do after a resume replaced the handle it created. */
int amem_vmm_free(uint64_t va, uint64_t alloc_size, uint64_t handle);

/* Export a handle as a POSIX fd / import one and map it at a fresh VA.
 * Counterparts of the export in amem_cuAllocAndExport (amem_nccl.h:186-190) and of
 * amem_importAndMap (amem_nccl.h:216-234) for the initial, caller-side exchange that the
 * reference leaves to NCCL. amem_vmm_import does not close `fd`. */
int amem_vmm_export(uint64_t handle, int* fd);
int amem_vmm_import(int fd, uint64_t size, int dev, uint64_t* va, uint64_t* handle);

/* ---------------------------------------------------------------------------------------
 * 4. Registry inspection (the reference exposes these as public data members of
 *    gmm_client_ctx, gmm_client.h:136-152, and fields of amem_allocMdata, amem_nccl.h:87-138)
 * ------------------------------------------------------------------------------------- */

typedef struct amem_region_info {
  uint64_t va;
  uint64_t handle;
  uint64_t mc_handle;
  uint64_t alloc_sz;
  uint64_t tags;
  uint64_t peers[AMEM_MAX_DEVS];
  uint64_t cpu_addr;     /* host address of the first parked byte; 0 before the first pause */
  uint64_t user_info;
  uint64_t parked_bytes; /* bytes of this region held in host memory by the last pause */
  uint64_t handle_gen;   /* number of physical handles this VA has had (1 after add) */
  int32_t dev;
  int32_t pid;
  int32_t refcount;
  int32_t shared_fd;
  int32_t type;
  int32_t state;
  int32_t has_peer;
  int32_t oos_flag;
} amem_region_info;

typedef struct amem_counters {
  int64_t release_local_cnt;
  int64_t release_shadow_cnt;
  int64_t offload_cnt;
  int64_t smoke_log;
  uint64_t alloc_bytes[AMEM_MAX_CALLER];
  uint64_t del_bytes;
  uint64_t pause_cnt;
  uint64_t resume_cnt;
  int32_t paused;
  int32_t group_id;
  int32_t enabled;
  int32_t slot;
} amem_counters;

/* Number of regions tracked for `dev`; entries are ordered by ascending VA. */
int64_t amem_region_count(int dev);
/* Copy the `index`-th region (ascending VA) of `dev`. 0 ok, 1 out of range. */
int amem_region_at(int dev, int64_t index, amem_region_info* out);
/* Copy the region whose key is `va`. 0 ok, 1 not found. */
int amem_region_find(int dev, uint64_t va, amem_region_info* out);
/* handleTable lookup: VA that `handle` backs (local regions only), 0 if absent. */
uint64_t amem_handle_lookup(int dev, uint64_t handle);
int64_t amem_handle_count(int dev);
void amem_get_counters(amem_counters* out);

/* Per-phase timing of the most recent pause and resume, in milliseconds unless named. */
typedef struct amem_cycle_stats {
  double pause_ms, resume_ms;
  double pause_scan_ms;     /* K1 launch -> flags on host */
  double pause_plan_ms;     /* host: runs, staging layout, descriptor upload */
  double pause_copy_ms;     /* first copy enqueued -> last byte in host memory */
  double pause_unmap_ms;    /* host time inside hipMemUnmap + hipMemRelease */
  double resume_map_ms;     /* host time inside hipMemCreate + hipMemMap + hipMemSetAccess */
  double resume_copy_ms;    /* first copy enqueued -> last byte in device memory */
  double resume_peer_ms;    /* export + notify importers + wait for owners */
  double k1_ms;             /* device time of the zero/checksum scan (HIP events) */
  double k2_ms;             /* device time of gather-pack launches (sum) */
  double k3_ms;             /* device time of scatter-unpack launches (sum) */
  uint64_t k1_launches, k2_launches, k3_launches;
  uint64_t footprint_bytes; /* sum of allocSz over local regions */
  uint64_t parked_bytes;    /* bytes that crossed the host link per leg */
  uint64_t zero_chunks, total_chunks;
  uint64_t local_regions, peer_regions;
  uint64_t dma_bytes;       /* of parked_bytes, how much the pause moved by hipMemcpyAsync */
  uint64_t kernel_bytes;    /* of parked_bytes, how much moved by the pack/unpack kernels */
  uint64_t slab_bytes;      /* pinned host memory held by the pool */
  uint64_t verify_mismatch; /* chunks whose checksum differed after resume (verify mode) */
  double pause_pool_ms;     /* of pause_ms: growing the pinned host pool (non-zero when slabs were added) */
  double pause_scratch_ms;  /* of pause_ms: allocating or growing the engine's own tables, staging and events */
  double pause_sync_ms;     /* of pause_ms: the device synchronisation and memory queries before the scan */
  double resume_scratch_ms; /* of resume_ms: allocating or growing the engine's own tables and events */
  uint64_t resume_dma_bytes; /* of parked_bytes, how much the resume brought back by hipMemcpyAsync */
  uint64_t pause_narrow_launches; /* of k2_launches, how many "pause_adaptive" issued with fewer workgroups */
  double resume_plan_ms;    /* of resume_ms: host work before the first region is mapped (scatter list, table upload) */
} amem_cycle_stats;
void amem_get_cycle_stats(amem_cycle_stats* out);

/* ---------------------------------------------------------------------------------------
 * 5. Engine controls without a reference counterpart
 * ------------------------------------------------------------------------------------- */

/* Turn the engine on or off at run time (the reference reads AMEM_ENABLE once at load,
 * amem_nccl.cpp:711). Only allowed while nothing is tracked. 0 ok, 1 rejected. */
int amem_set_enabled(int on);

/* Tunables. Unknown name or bad value returns 1. Names:
 *   "zero_elide"      0/1   skip all-zero 64 KiB chunks (default 1)
 *   "verify"          0/1   re-scan after resume and compare checksums (default 0)
 *   "pause_path"      how pause moves bytes and overlaps the unmaps:
 *                     0 = one pack kernel writes pinned host memory, then regions are unmapped
 *                     1 = pack into device staging, large hipMemcpyAsync, unmap meanwhile
 *                     3 = many short pack launches into pinned host memory, confined to
 *                         "pause_xcds" XCDs and "pause_wgs" workgroups, while a second host
 *                         thread unmaps each group of regions as soon as its launch is done
 *                         (and a third releases their handles, see "release_thread")
 *                     2 = the default, currently 3
 *                     4 = measurement aid: the reference's own structure in HIP calls (one waited-for
 *                         whole-region hipMemcpyAsync per region each way, no scan, no elision)
 *   "interleave_bytes" parked bytes per launch of path 3 (default 4 MiB)
 *   "pause_wgs"       workgroups of path 3's pack kernel; 0 (default) = 8
 *   "pause_xcds"      XCDs those workgroups are confined to (1-8); 0 (default) = 1
 *   "dma_min_bytes"   extents at least this long use hipMemcpyAsync in the direct path
 *   "staging_bytes"   size of each of the two device staging buffers
 *   "slab_bytes"      size of one pinned host slab (power of two, default 256 MiB); read when the
 *                     device's engine is created, i.e. set it before the first tracked allocation
 *   "link_wgs"        workgroups of a kernel that reads or writes host memory (default 96)
 *   "hbm_wgs"         most workgroups of the scan kernel (default 65536)
 *   "hbm_move_wgs"    most workgroups of the pack/unpack kernel when both sides are device memory
 *                     (default 4194304: one workgroup per 4 KiB piece up to 16 GiB, striding beyond)
 *   "resume_batch_bytes" resume maps regions in batches of about this many bytes and follows each
 *                     batch with one unpack launch (default 64 MiB)
 *   "resume_dma_min_bytes" resume brings runs of parked bytes at least this long back with
 *                     hipMemcpyAsync on a second stream while the unpack kernel handles the shorter ones
 *                     and the zero fill on the first (default 0: everything goes through the kernel,
 *                     which measured 2 % below the copy engine's rate and needs no second stream)
 *   "peer_timeout_ms" how long resume waits for owners before failing (0 = forever)
 *   "offload_free_tag" caller tag (0-15, -1 = none) whose regions hold scratch data: pause releases
 *                     them without copying and resume hands them back zero-filled. This is what
 *                     AMEM_NCCL_OFFLOAD_FREE_TAG is documented to do in the reference, where the
 *                     variable is parsed but never takes effect (amem_nccl.cpp:40, :503, :620) and
 *                     regions of every tag keep their bytes. The variable alone changes nothing
 *                     here either; together with AMEM_OFFLOAD_FREE_TAG_APPLY=1 it becomes this
 *                     option's initial value when the library is loaded (a WARN line says so)
 *   "release_thread"  0/1 (default 1): the default pause path releases handles on a thread of their own
 *                     instead of on the one that unmaps
 *   "pause_adaptive"  0/1 (default 1): the default pause path keeps only a few launches queued and issues
 *                     them with 6 or 4 workgroups instead of "pause_wgs" while finished groups pile up
 *                     in front of the unmapping thread: an unmap costs less beside a narrower kernel, and
 *                     the copy has time to spare when there are many regions. 0 = every launch "pause_wgs" wide
 *   "scratch_on_host" 0/1: keep the engine's own tables in pinned host memory. That is where they go
 *                     anyway when the device has no room for them at pause time; 1 forces it
 *   "pool_limit_bytes" most pinned host memory one pause may need (0 = no limit). A pause that
 *                     would need more fails with an out-of-memory error before it has released
 *                     anything, and the process stays un-paused
 *   "peer_loopback"   0/1   treat this process's own slot like any other peer: registration and
 *                     re-export go through the socket service of the same process (default 0:
 *                     a process never registers with itself, gmm_client_impl.cpp:482-484, :512-514) */
int amem_set_option(const char* name, int64_t value);
int64_t amem_get_option(const char* name);

/* Release the pinned host pool (only while not paused). Returns bytes freed. */
uint64_t amem_pool_trim(void);
/* Grow the pinned host pool of the current device to at least `bytes` ahead of time, so that the
 * first pause does not pay for pinning host memory (the reference creates its host buffers inside
 * the first pause, amem_nccl.cpp:505-508). 0 ok, else a HIP error. No reference counterpart. */
int amem_pool_reserve(uint64_t bytes);

/* Tear the per-process context down to the state before the first tracked allocation:
 * registry emptied (nothing is unmapped or freed), pool released, IPC service stopped,
 * counters zeroed. Rejected (1) while paused. The reference has only x_fini (:726-729). */
int amem_shutdown(void);

/* Slot of this process within its group on this node: index into peers[] that importers
 * pass as `peer_dev`. Taken from AMEM_SLOT or claimed first-free when the IPC service
 * starts. Returns -1 before that. amem_ipc_start starts the service explicitly (it is
 * otherwise started together with the context, by the first tracked allocation, unless
 * AMEM_IPC=0) and returns the slot. */
int amem_ipc_start(void);
int amem_get_slot(void);
/* A process that hosts several ranks gives each of them a slot of its own: amem_ipc_claim_slot
 * claims one more slot for this process (lock file, socket and service thread like the first one)
 * and returns it, or -1 when none is free. amem_ipc_act_as(slot) makes the calling thread register
 * the imported regions it adds from then on as that slot (-1: as the process's first slot again);
 * 0 ok, 1 when this process does not hold `slot`. With "peer_loopback" on, the ranks of one process
 * register with and update each other over their sockets exactly as ranks in different processes
 * do; with it off (default) they follow the reference's same-process rule and stay out of each
 * other's pause scope (gmm_client_impl.cpp:482-484). No reference counterpart: the reference has
 * one worker per (process, GPU). */
int amem_ipc_claim_slot(void);
int amem_ipc_act_as(int slot);
/* What the service of this process's `slot` has answered with success since it started:
 * counts[0] registrations of an importer (gmm_worker_impl.cpp:375-382), counts[1] re-exported
 * descriptors mapped at an importer's address (:384-390), counts[2] release requests (:392-397).
 * 0 ok, 1 when this process does not hold `slot`. Inspection only. */
int amem_ipc_served(int slot, uint64_t counts[3]);
/* 1 while some process holds `slot` of this group on this node (its lock dies with it), else 0. */
int amem_ipc_peer_alive(int slot);

/* ---------------------------------------------------------------------------------------
 * 6. The device kernels, callable on their own (no reference counterpart: the reference
 *    moves bytes only with cuMemcpyDtoHAsync / cuMemcpyHtoDAsync, amem_nccl.h:304-327)
 * ------------------------------------------------------------------------------------- */

typedef struct amem_extent {
  uint64_t va;    /* device address, 16-byte aligned */
  uint64_t bytes; /* multiple of 16 */
} amem_extent;

typedef struct amem_chunk_sum {
  uint64_t sum64; /* sum of all little-endian uint32 words, mod 2^64 */
  uint64_t xor64; /* xor of all little-endian uint64 words */
} amem_chunk_sum;

/* Zero-chunk detector + checksum. Every extent is cut into 64 KiB chunks (the last one
 * of an extent may be shorter); chunks are numbered extent by extent. Writes one flag
 * byte (1 = all bytes zero) and one checksum pair per chunk to host arrays of
 * amem_chunk_count(extents, n) entries. `sums` may be NULL. Returns 0, or a HIP error. */
uint64_t amem_chunk_count(const amem_extent* extents, uint64_t n);
int amem_zero_scan(const amem_extent* extents, uint64_t n, uint8_t* flags,
                   amem_chunk_sum* sums, float* kernel_ms);

/* amem_zero_scan for callers that cannot allocate device memory (tight serving loops, harnesses
 * that forbid hipMalloc). No counterpart in the reference. Same arguments and bit-identical
 * results; the tables the scan kernel needs beyond its inputs and outputs (segment table, chunk
 * prefix, flags and checksums before they reach the host) live in one fixed device array of about
 * 4.4 MiB that every GPU the library runs on holds until the process ends, and the host side of
 * every transfer is pinned memory made when the device's engine is set up (by the first tracked
 * allocation, or by the first call of any entry point of this section on that device: make one
 * warm-up call first). After that set-up a call allocates and frees nothing, on the device or the
 * host. It is serialised with every other engine call on the engine's lock, enqueues its copies and
 * its kernel on the engine's own stream and synchronises that stream before it returns: call it
 * outside any stream capture.
 * Limits: at most AMEM_NOALLOC_MAX_EXTENTS extents and AMEM_NOALLOC_MAX_CHUNKS chunks (16 GiB)
 * per call; beyond them the call logs the limit and returns hipErrorInvalidValue (1) without
 * touching the GPU. All calls on one GPU share the fixed array, which keeps the last call's
 * contents; a call never reads what it has not just written, and calls that overlap on one GPU
 * are queued on the engine's lock rather than racing. */
#define AMEM_NOALLOC_MAX_EXTENTS 8192u
#define AMEM_NOALLOC_MAX_CHUNKS 262144u
int amem_zero_scan_noalloc(const amem_extent* extents, uint64_t n, uint8_t* flags,
                           amem_chunk_sum* sums, float* kernel_ms);

typedef struct amem_copy_desc {
  uint64_t va;      /* scattered side: device address, 16-byte aligned */
  uint64_t off;     /* contiguous side: byte offset into the staging buffer, 16-byte aligned;
                       AMEM_DESC_ZERO on unpack means "write zeros to va" */
  uint64_t bytes;   /* multiple of 16 */
} amem_copy_desc;
#define AMEM_DESC_ZERO (~(uint64_t)0)

/* Gather-pack: staging[off .. off+bytes) = device[va .. va+bytes) for every descriptor.
 * Scatter-unpack: the reverse, plus zero fill for AMEM_DESC_ZERO descriptors.
 * `staging` is a device pointer or a hipHostMalloc pointer; `host_side` non-zero selects
 * the launch shape tuned for the host link. Descriptor arrays are host memory.
 * Synchronous. Returns 0, or a HIP error. */
int amem_gather_pack(const amem_copy_desc* descs, uint64_t n, void* staging,
                     uint64_t staging_bytes, int host_side, float* kernel_ms);
int amem_scatter_unpack(const amem_copy_desc* descs, uint64_t n, const void* staging,
                        uint64_t staging_bytes, int host_side, float* kernel_ms);

#pragma GCC visibility pop
#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* AMEM_H_ */
