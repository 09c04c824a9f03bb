/* CPU restatement of the reference's pause/resume path — test infrastructure, see amem_oracle.h. */
#define _GNU_SOURCE
#include "amem_oracle.h"

#include <errno.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <unistd.h>

#define API __attribute__((visibility("default")))

/* amem_nccl.h:39-49 */
enum { ST_INVALID = 0, ST_ALLOC, ST_OFFLOADING, ST_HOLE, ST_PRELOADING, ST_REMAPPED };
/* amem_nccl.h:52-64, :82-84 */
enum { TY_LOCAL = 0, TY_LOCAL_FABRIC = 1, TY_LOCAL_SYMM = 2, TY_PEER_POSIX = 3 };
static int from_peer(int type) { return type <= TY_LOCAL_SYMM ? 0 : 1; }

/* ------------------------------------------------------------------------------------
 * VMM stand-in
 * ---------------------------------------------------------------------------------- */

typedef struct phys {
  uint64_t id; /* the "handle": never reused, never zero */
  int fd;
  uint64_t size;
  int refs; /* creation reference + one per mapping, as the driver counts them */
  int live;
} phys;

typedef struct mapping {
  uint64_t va, size, handle;
} mapping;

static phys* g_phys;
static size_t g_nphys, g_cap_phys;
static mapping* g_maps;
static size_t g_nmaps, g_cap_maps;
static uint64_t g_next_handle = 0x1000;
static pthread_mutex_t g_vmm_mtx = PTHREAD_MUTEX_INITIALIZER;

static phys* phys_find(uint64_t id) {
  for (size_t i = 0; i < g_nphys; ++i)
    if (g_phys[i].live && g_phys[i].id == id) return &g_phys[i];
  return NULL;
}

static phys* phys_new(int fd, uint64_t size) {
  if (g_nphys == g_cap_phys) {
    g_cap_phys = g_cap_phys ? g_cap_phys * 2 : 256;
    g_phys = (phys*)realloc(g_phys, g_cap_phys * sizeof(phys));
  }
  /* reuse a dead slot (the id is still fresh) */
  phys* p = NULL;
  for (size_t i = 0; i < g_nphys; ++i)
    if (!g_phys[i].live) { p = &g_phys[i]; break; }
  if (!p) p = &g_phys[g_nphys++];
  p->id = g_next_handle++;
  p->fd = fd;
  p->size = size;
  p->refs = 1;
  p->live = 1;
  return p;
}

static void phys_unref(phys* p) {
  if (--p->refs == 0) {
    close(p->fd);
    p->live = 0;
  }
}

static mapping* map_find(uint64_t va) {
  for (size_t i = 0; i < g_nmaps; ++i)
    if (g_maps[i].va == va) return &g_maps[i];
  return NULL;
}

static uint64_t v_reserve(uint64_t size) {
  void* p = mmap(NULL, size, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
  return p == MAP_FAILED ? 0 : (uint64_t)(uintptr_t)p;
}

static uint64_t v_create(uint64_t size) {
  int fd = memfd_create("amem_oracle", MFD_CLOEXEC);
  if (fd < 0) return 0;
  if (ftruncate(fd, (off_t)size) != 0) { close(fd); return 0; }
  pthread_mutex_lock(&g_vmm_mtx);
  uint64_t id = phys_new(fd, size)->id;
  pthread_mutex_unlock(&g_vmm_mtx);
  return id;
}

static int v_map(uint64_t va, uint64_t size, uint64_t handle) {
  pthread_mutex_lock(&g_vmm_mtx);
  phys* p = phys_find(handle);
  int rc = 1;
  if (p && size <= p->size) {
    void* q = mmap((void*)(uintptr_t)va, size, PROT_READ | PROT_WRITE, MAP_FIXED | MAP_SHARED, p->fd, 0);
    if (q != MAP_FAILED) {
      p->refs++;
      if (g_nmaps == g_cap_maps) {
        g_cap_maps = g_cap_maps ? g_cap_maps * 2 : 256;
        g_maps = (mapping*)realloc(g_maps, g_cap_maps * sizeof(mapping));
      }
      g_maps[g_nmaps++] = (mapping){va, size, handle};
      rc = 0;
    }
  }
  pthread_mutex_unlock(&g_vmm_mtx);
  return rc;
}

static int v_unmap(uint64_t va, uint64_t size) {
  pthread_mutex_lock(&g_vmm_mtx);
  mapping* m = map_find(va);
  int rc = 1;
  if (m) {
    /* back to an inaccessible reservation at the same address */
    void* q = mmap((void*)(uintptr_t)va, size, PROT_NONE, MAP_FIXED | MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    phys* p = phys_find(m->handle);
    if (p) phys_unref(p);
    *m = g_maps[--g_nmaps];
    rc = q == MAP_FAILED;
  }
  pthread_mutex_unlock(&g_vmm_mtx);
  return rc;
}

static int v_release(uint64_t handle) {
  pthread_mutex_lock(&g_vmm_mtx);
  phys* p = phys_find(handle);
  int rc = 1;
  if (p) { phys_unref(p); rc = 0; }
  pthread_mutex_unlock(&g_vmm_mtx);
  return rc;
}

/* cuMemRetainAllocationHandle as the CUDA driver counts it: one more reference on the
   physical memory mapped at `va`. Used by tests to model callers that retain a handle. */
API uint64_t oracle_vmm_retain(uint64_t va) {
  pthread_mutex_lock(&g_vmm_mtx);
  mapping* m = map_find(va);
  phys* p = m ? phys_find(m->handle) : NULL;
  uint64_t h = 0;
  if (p) { p->refs++; h = p->id; }
  pthread_mutex_unlock(&g_vmm_mtx);
  return h;
}

API uint64_t oracle_vmm_handle_of(uint64_t va) {
  pthread_mutex_lock(&g_vmm_mtx);
  mapping* m = map_find(va);
  uint64_t h = m ? m->handle : 0;
  pthread_mutex_unlock(&g_vmm_mtx);
  return h;
}

/* Test hygiene: drop everything the host-memory stand-in still holds (mappings go back to nothing,
   physical objects are closed), so that a test that did not free its regions one by one leaves no
   descriptors or memory behind for the next one. Reservations of regions that were paused at that
   moment (address space only, no memory) are left to the process's end. */
API void oracle_vmm_reset(void) {
  pthread_mutex_lock(&g_vmm_mtx);
  for (size_t i = 0; i < g_nmaps; ++i) munmap((void*)(uintptr_t)g_maps[i].va, g_maps[i].size);
  g_nmaps = 0;
  for (size_t i = 0; i < g_nphys; ++i)
    if (g_phys[i].live) { close(g_phys[i].fd); g_phys[i].live = 0; }
  pthread_mutex_unlock(&g_vmm_mtx);
}

API uint64_t oracle_vmm_live_bytes(void) {
  uint64_t n = 0;
  pthread_mutex_lock(&g_vmm_mtx);
  for (size_t i = 0; i < g_nphys; ++i)
    if (g_phys[i].live) n += g_phys[i].size;
  pthread_mutex_unlock(&g_vmm_mtx);
  return n;
}

/* gmm_cuda_vmm_alloc, gmm_cuda_mem_impl.cpp:237-273: round to 2 MiB, create, reserve, map, access. */
API int oracle_vmm_alloc(uint64_t bytes, uint64_t* va, uint64_t* handle, uint64_t* alloc_size) {
  const uint64_t al = 2ull << 20;
  uint64_t size = (bytes + al - 1) / al * al;
  uint64_t h = v_create(size);
  if (!h) return 1;
  uint64_t a = v_reserve(size);
  if (!a) { v_release(h); return 1; }
  if (v_map(a, size, h)) { v_release(h); munmap((void*)(uintptr_t)a, size); return 1; }
  *va = a;
  *handle = h;
  if (alloc_size) *alloc_size = size;
  return 0;
}

/* gmm_cuda_vmm_free, gmm_cuda_mem_impl.cpp:275-283 (unmap, address free, release). */
API int oracle_vmm_free(uint64_t va, uint64_t alloc_size, uint64_t handle) {
  uint64_t mapped = oracle_vmm_handle_of(va);
  if (mapped) {
    if (!handle) handle = mapped;
    v_unmap(va, alloc_size);
    v_release(handle);
  }
  return munmap((void*)(uintptr_t)va, alloc_size);
}

API int oracle_vmm_export(uint64_t handle, int* fd) {
  pthread_mutex_lock(&g_vmm_mtx);
  phys* p = phys_find(handle);
  int rc = 1;
  if (p) { *fd = dup(p->fd); rc = *fd < 0; }
  pthread_mutex_unlock(&g_vmm_mtx);
  return rc;
}

static uint64_t v_import(int fd, uint64_t size) {
  int mine = dup(fd);
  if (mine < 0) return 0;
  pthread_mutex_lock(&g_vmm_mtx);
  uint64_t id = phys_new(mine, size)->id;
  pthread_mutex_unlock(&g_vmm_mtx);
  return id;
}

API int oracle_vmm_import(int fd, uint64_t size, uint64_t* va, uint64_t* handle) {
  uint64_t h = v_import(fd, size);
  if (!h) return 1;
  uint64_t a = v_reserve(size);
  if (!a || v_map(a, size, h)) { v_release(h); return 1; }
  *va = a;
  *handle = h;
  return 0;
}

/* ------------------------------------------------------------------------------------
 * Registry: amem_allocMdata (amem_nccl.h:87-138) and the live members of gmm_client_ctx
 * (gmm_client.h:136-152), one set per simulated process.
 * ---------------------------------------------------------------------------------- */

typedef struct mdata {
  uint64_t va;
  int dev, pid, refcount, sharedFD;
  uint64_t handle, mcHandle;
  uint64_t allocSz, tags;
  int type, state;
  uint64_t peers[ORACLE_MAX_DEVS];
  int hasPeer, oosFlag;
  void* cpuAddr;
  uint64_t userInfo;
} mdata;

typedef struct hentry { uint64_t handle, va; } hentry;

typedef struct octx {
  int exists, disabled, groupID;
  mdata* tab[ORACLE_MAX_DEVS];
  size_t n[ORACLE_MAX_DEVS], cap[ORACLE_MAX_DEVS];
  hentry* htab[ORACLE_MAX_DEVS];
  size_t hn[ORACLE_MAX_DEVS], hcap[ORACLE_MAX_DEVS];
  int releaseLocalCnt, releaseShadowCnt, offloadCnt, smokeLog;
  uint64_t allocBytes[ORACLE_MAX_CALLER], delBytes;
  int paused;
  uint64_t pauseCnt, resumeCnt;
  int has_ctx; /* gmm_ctx_p != NULL: created by the first add (amem_nccl.cpp:55-80) */
} octx;

static octx g_ctx[ORACLE_MAX_CTX];

static octx* C(int i) {
  if (i < 0 || i >= ORACLE_MAX_CTX) return NULL;
  if (!g_ctx[i].exists) {
    memset(&g_ctx[i], 0, sizeof(octx));
    g_ctx[i].exists = 1;
    g_ctx[i].disabled = 0;
  }
  return &g_ctx[i];
}

API void oracle_reset(void) {
  for (int i = 0; i < ORACLE_MAX_CTX; ++i) {
    if (!g_ctx[i].exists) continue;
    for (int d = 0; d < ORACLE_MAX_DEVS; ++d) {
      for (size_t k = 0; k < g_ctx[i].n[d]; ++k) free(g_ctx[i].tab[d][k].cpuAddr);
      free(g_ctx[i].tab[d]);
      free(g_ctx[i].htab[d]);
    }
    memset(&g_ctx[i], 0, sizeof(octx));
  }
}

API int oracle_ctx_enable(int slot, int on) {
  octx* c = C(slot);
  if (!c) return 1;
  c->disabled = !on;
  return 0;
}

static mdata* find(octx* c, int dev, uint64_t va) {
  for (size_t k = 0; k < c->n[dev]; ++k)
    if (c->tab[dev][k].va == va) return &c->tab[dev][k];
  return NULL;
}

static void erase(octx* c, int dev, uint64_t va) {
  for (size_t k = 0; k < c->n[dev]; ++k)
    if (c->tab[dev][k].va == va) {
      /* the reference drops the entry without freeing cpuAddr (amem_nccl.cpp:441); the host
         buffer is freed here only to keep the test process small */
      free(c->tab[dev][k].cpuAddr);
      memmove(&c->tab[dev][k], &c->tab[dev][k + 1], (c->n[dev] - k - 1) * sizeof(mdata));
      c->n[dev]--;
      return;
    }
}

/* entries are kept in ascending VA order so that iteration is deterministic */
static mdata* insert(octx* c, int dev, uint64_t va) {
  if (c->n[dev] == c->cap[dev]) {
    c->cap[dev] = c->cap[dev] ? c->cap[dev] * 2 : 64;
    c->tab[dev] = (mdata*)realloc(c->tab[dev], c->cap[dev] * sizeof(mdata));
  }
  size_t k = c->n[dev];
  while (k > 0 && c->tab[dev][k - 1].va > va) { c->tab[dev][k] = c->tab[dev][k - 1]; --k; }
  c->n[dev]++;
  memset(&c->tab[dev][k], 0, sizeof(mdata));
  c->tab[dev][k].va = va;
  return &c->tab[dev][k];
}

static uint64_t hlookup(octx* c, int dev, uint64_t handle) {
  for (size_t k = 0; k < c->hn[dev]; ++k)
    if (c->htab[dev][k].handle == handle) return c->htab[dev][k].va;
  return 0;
}
static int hhas(octx* c, int dev, uint64_t handle) {
  for (size_t k = 0; k < c->hn[dev]; ++k)
    if (c->htab[dev][k].handle == handle) return 1;
  return 0;
}
/* unordered_map::emplace keeps an existing key (amem_nccl.cpp:264, :630) */
static void hemplace(octx* c, int dev, uint64_t handle, uint64_t va) {
  if (hhas(c, dev, handle)) return;
  if (c->hn[dev] == c->hcap[dev]) {
    c->hcap[dev] = c->hcap[dev] ? c->hcap[dev] * 2 : 64;
    c->htab[dev] = (hentry*)realloc(c->htab[dev], c->hcap[dev] * sizeof(hentry));
  }
  c->htab[dev][c->hn[dev]++] = (hentry){handle, va};
}
static void herase(octx* c, int dev, uint64_t handle) {
  for (size_t k = 0; k < c->hn[dev]; ++k)
    if (c->htab[dev][k].handle == handle) { c->htab[dev][k] = c->htab[dev][--c->hn[dev]]; return; }
}

/* gmm_client_ctx::register_peer (gmm_client_impl.cpp:479-505): refuses when the owner is the
   calling process, otherwise the owner's worker runs amem_registerPeerInfo. */
static int rpc_register_peer(int me, uint64_t srcHandle, uint64_t dptr, int peer_slot) {
  if (peer_slot == me) return 1;
  if (peer_slot < 0 || peer_slot >= ORACLE_MAX_CTX || !g_ctx[peer_slot].exists || !g_ctx[peer_slot].has_ctx) return 1;
  return oracle_register_peer_info(peer_slot, srcHandle, dptr, me);
}

/* gmm_client_ctx::update_peer (gmm_client_impl.cpp:509-532) */
static int rpc_update_peer(int me, uint64_t peerDptr, int fd, int peer_slot) {
  if (peer_slot == me) return 0;
  if (peer_slot < 0 || peer_slot >= ORACLE_MAX_CTX || !g_ctx[peer_slot].exists) return 1;
  /* SCM_RIGHTS hands the receiver its own descriptor */
  int theirs = dup(fd);
  return oracle_update_peer_info(peer_slot, peerDptr, theirs);
}

/* amem_addAllocInfo, amem_nccl.cpp:102-269. In this model a context's slot doubles as its
   device-independent identity: peer_dev names the owner's slot. */
API int oracle_add_alloc_info(int ctx, uint64_t va, uint64_t size, int type, int dev, uint64_t handle, int peer_dev,
                              uint64_t peer_handle, uint64_t user_info, int caller) {
  octx* c = C(ctx);
  if (!c || c->disabled) return 0;                              /* :107-109 */
  int ret = 0;
  int peerFlag = from_peer(type);                               /* :113 */
  int oosFlag = (peerFlag && peer_dev == -1) ? 1 : 0;           /* :119 */
  c->has_ctx = 1;                                               /* :129 InitClientCtx */
  if (c->paused) return 1;                                      /* :133-137 */
  mdata* m = find(c, dev, va);
  if (!m) {                                                     /* :142-148 */
    m = insert(c, dev, va);
    m->dev = dev;
    m->pid = (int)getpid();
    m->allocSz = size;
    m->state = ST_ALLOC;
    m->type = type;
    m->userInfo = user_info;
    m->tags = (uint64_t)(int64_t)caller;
    m->handle = handle;
    m->mcHandle = peer_handle;
    m->oosFlag = oosFlag;
    if (caller >= 0 && caller < ORACLE_MAX_CALLER) c->allocBytes[caller] += size;
  } else {                                                      /* :179-191 */
    m->type = type;
    m->state = ST_ALLOC;
    m->allocSz = size;
    m->handle = handle;
    m->userInfo = user_info;
    m->tags = (uint64_t)(int64_t)caller;
  }
  if (peerFlag && peer_dev >= 0) {                              /* :195-220 */
    ret = rpc_register_peer(ctx, peer_handle, va, peer_dev);
    if (ret != 0) erase(c, dev, va);
  } else if (peerFlag && peer_dev == -1) {                      /* :222-256; owner not detectable here */
    erase(c, dev, va);
    ret = 1;
  } else {                                                      /* :258-265 */
    hemplace(c, dev, handle, va);
  }
  c->smokeLog++;                                                /* :267 */
  return ret;
}

/* amem_delAllocInfo, amem_nccl.cpp:414-448 */
API int oracle_del_alloc_info(int ctx, uint64_t va, uint64_t handle, int caller) {
  (void)caller;
  octx* c = C(ctx);
  if (!c || c->disabled) return 0;
  if (va == 0) return 0;
  if (!c->has_ctx) return 0;
  if (handle == 0) handle = oracle_vmm_handle_of(va);           /* :423-426 */
  int dev = 0;
  mdata* m = find(c, dev, va);
  if (m) {
    if (m->tags < ORACLE_MAX_CALLER) c->allocBytes[m->tags] -= m->allocSz;  /* intent of :436-440 */
    else c->delBytes += m->allocSz;
    if (handle == 0) handle = m->handle;
    erase(c, dev, va);
  }
  herase(c, dev, handle);                                       /* :445 */
  return 0;
}

/* amem_addRefcount, amem_nccl.cpp:332-356 */
API int oracle_add_refcount(int ctx, uint64_t va, int n) {
  octx* c = C(ctx);
  if (!c || c->disabled) return 0;
  mdata* m = c->has_ctx ? find(c, 0, va) : NULL;
  if (!m) return 1;
  m->refcount += n;
  return 0;
}

/* amem_addPeerInfo, amem_nccl.cpp:359-381 */
API int oracle_add_peer_info(int ctx, uint64_t src_va, uint64_t peer_va, int peer_dev) {
  octx* c = C(ctx);
  if (!c || peer_dev < 0 || peer_dev >= ORACLE_MAX_DEVS) return 1;
  mdata* m = c->has_ctx ? find(c, 0, src_va) : NULL;
  if (!m) return 1;
  m->peers[peer_dev] = peer_va;
  m->hasPeer = 1;
  return 0;
}

/* amem_registerPeerInfo, amem_nccl.cpp:297-329 */
API int oracle_register_peer_info(int ctx, uint64_t src_handle, uint64_t peer_va, int peer_dev) {
  octx* c = C(ctx);
  if (!c || !c->has_ctx || peer_dev < 0 || peer_dev >= ORACLE_MAX_DEVS) return 1;
  if (!hhas(c, 0, src_handle)) return 1;
  mdata* m = find(c, 0, hlookup(c, 0, src_handle));
  if (!m) return 1;
  m->peers[peer_dev] = peer_va;
  m->hasPeer = 1;
  return 0;
}

/* amem_updatePeerInfo, amem_nccl.cpp:385-409, with amem_importAndMap, amem_nccl.h:216-234 */
API int oracle_update_peer_info(int ctx, uint64_t va, int shared_fd) {
  octx* c = C(ctx);
  mdata* m = (c && c->has_ctx) ? find(c, 0, va) : NULL;
  if (!m) { close(shared_fd); return 1; }
  uint64_t h = v_import(shared_fd, m->allocSz);
  int ret = h ? v_map(va, m->allocSz, h) : 1;
  close(shared_fd);
  if (ret == 0) {
    m->state = ST_ALLOC;
    m->handle = h; /* the engine records the new import handle; the reference leaves the stale one */
    c->releaseShadowCnt--;
  }
  return ret;
}

/* amem_checkPaused, amem_nccl.cpp:452-464 */
API int oracle_check_paused(int ctx) {
  octx* c = C(ctx);
  if (!c || c->disabled || !c->has_ctx) return 0;
  return c->paused;
}

/* amem_setGroupID / amem_getGroupID, amem_nccl.cpp:679-703 */
API int oracle_set_group_id(int ctx, int id) {
  octx* c = C(ctx);
  if (!c || c->disabled) return 0;
  if (!c->has_ctx) { c->groupID = id; return 0; }
  return 1;
}
API int oracle_get_group_id(int ctx) { octx* c = C(ctx); return c ? c->groupID : 0; }

/* the total that amem_dumpAllocStats prints, amem_nccl.cpp:88-98 */
API uint64_t oracle_mem_stats_total(int ctx) {
  octx* c = C(ctx);
  uint64_t t = 0;
  if (!c) return 0;
  for (int i = 0; i < ORACLE_MAX_CALLER; ++i) t += c->allocBytes[i];
  return t + c->delBytes;
}

/* ------------------------------------------------------------------------------------
 * pause / resume
 * ---------------------------------------------------------------------------------- */

/* amem_cuMemReleaseHandle, amem_nccl.h:141-161 (its retain/release pair nets to nothing) */
static void release_handle(uint64_t va, uint64_t size, uint64_t handle, int refcount) {
  v_unmap(va, size);
  v_release(handle);
  while (refcount-- > 0) v_release(handle);
}

typedef struct job { octx* c; int tid, nthreads, resume; } job;

/* step 1 of pause / step 2 of resume for the regions of one thread: whole-region memcpy
   (amem_launchOffload / amem_lauchPreload, amem_nccl.h:304-327, each followed by a sync) */
static void* copy_worker(void* arg) {
  job* j = (job*)arg;
  octx* c = j->c;
  size_t k0 = 0;
  for (size_t k = 0; k < c->n[0]; ++k) {
    mdata* m = &c->tab[0][k];
    if (from_peer(m->type)) continue;
    if (!j->resume) {
      if (m->state != ST_OFFLOADING) continue;
    } else if (m->state != ST_PRELOADING) continue;
    if ((int)(k0++ % (size_t)j->nthreads) != j->tid) continue;
    if (!j->resume) {
      if (!m->cpuAddr) {                                         /* amem_nccl.cpp:505-508 */
        if (posix_memalign(&m->cpuAddr, 4096, m->allocSz)) m->cpuAddr = NULL;
      }
      memcpy(m->cpuAddr, (void*)(uintptr_t)m->va, m->allocSz);
    } else {
      memcpy((void*)(uintptr_t)m->va, m->cpuAddr, m->allocSz);
    }
  }
  return NULL;
}

static void run_copy(octx* c, int resume, int threads) {
  if (threads < 1) threads = 1;
  if (threads > 64) threads = 64;
  job jobs[64];
  pthread_t th[64];
  for (int t = 0; t < threads; ++t) {
    jobs[t] = (job){c, t, threads, resume};
    if (t) pthread_create(&th[t], NULL, copy_worker, &jobs[t]);
  }
  copy_worker(&jobs[0]);
  for (int t = 1; t < threads; ++t) pthread_join(th[t], NULL);
}

/* amem_memPause, amem_nccl.cpp:467-574 */
API int oracle_mem_pause_mt(int ctx, int threads) {
  octx* c = C(ctx);
  if (!c || c->disabled) return 0;
  if (!c->has_ctx) return 0;
  if (c->paused) return 0;                                       /* :481-488 */
  c->paused = 1;
  if (c->n[0] == 0) return 0;                                    /* :491 */
  /* 1. offload local memory (:502-513) */
  for (size_t k = 0; k < c->n[0]; ++k) {
    mdata* m = &c->tab[0][k];
    if (m->state == ST_ALLOC && !from_peer(m->type)) {
      m->state = ST_OFFLOADING;
      c->offloadCnt++;
    }
  }
  run_copy(c, 0, threads);
  /* 2. release handles mapped from peers (:517-526) */
  for (size_t k = 0; k < c->n[0]; ++k) {
    mdata* m = &c->tab[0][k];
    if (m->state == ST_ALLOC && from_peer(m->type)) {
      release_handle(m->va, m->allocSz, m->handle ? m->handle : oracle_vmm_handle_of(m->va), 0);
      m->state = ST_HOLE;
      c->releaseShadowCnt++;
    }
  }
  /* 3. release local handles (:529-558) */
  for (size_t k = 0; k < c->n[0]; ++k) {
    mdata* m = &c->tab[0][k];
    if (from_peer(m->type)) continue;
    uint64_t old = oracle_vmm_handle_of(m->va);                  /* :539-540 */
    release_handle(m->va, m->allocSz, old, m->refcount);         /* :546 */
    for (int i = 0; i < ORACLE_MAX_DEVS; ++i)
      if (m->peers[i] != 0) c->releaseLocalCnt++;                /* :547-550 */
    m->state = ST_HOLE;
    m->handle = 0;
    herase(c, 0, old);                                           /* :556 */
  }
  c->pauseCnt++;                                                 /* :561 */
  return 0;
}
API int oracle_mem_pause(int ctx) { return oracle_mem_pause_mt(ctx, 1); }

/* amem_memResume, amem_nccl.cpp:577-677 */
API int oracle_mem_resume_mt(int ctx, int threads) {
  octx* c = C(ctx);
  if (!c || c->disabled) return 0;
  if (!c->has_ctx) return 0;
  if (!c->paused) return 0;                                      /* :589-594 */
  int ret = 0;
  /* 1. new physical memory at the same address (:604-616) */
  for (size_t k = 0; k < c->n[0]; ++k) {
    mdata* m = &c->tab[0][k];
    if (m->state != ST_HOLE || from_peer(m->type)) continue;
    uint64_t h = v_create(m->allocSz);                           /* amem_cuAllocAndExport, amem_nccl.h:164-193 */
    if (!h || v_map(m->va, m->allocSz, h)) { ret = 1; continue; }
    m->handle = h;
    m->state = ST_PRELOADING;                                    /* :621 */
  }
  /* 2. bytes back (:620-624) */
  run_copy(c, 1, threads);
  /* 3./4. table update and peer notification (:627-649) */
  for (size_t k = 0; k < c->n[0]; ++k) {
    mdata* m = &c->tab[0][k];
    if (m->state != ST_PRELOADING) continue;
    c->offloadCnt--;
    m->state = ST_ALLOC;
    hemplace(c, 0, m->handle, m->va);
    if (m->hasPeer) {
      int fd = -1;
      oracle_vmm_export(m->handle, &fd);
      for (int i = 0; i < ORACLE_MAX_DEVS; ++i) {
        if (m->peers[i] == 0) continue;
        int r = rpc_update_peer(ctx, m->peers[i], fd, i);
        if (r != 0) ret = r; else c->releaseLocalCnt--;
      }
      close(fd);                                                 /* :648 */
    }
  }
  if (c->releaseShadowCnt > 0) return 2;                         /* :659-662 would spin here */
  c->paused = 0;                                                 /* :664-665 */
  c->resumeCnt++;
  return ret;
}
API int oracle_mem_resume(int ctx) { return oracle_mem_resume_mt(ctx, 1); }

/* ------------------------------------------------------------------------------------
 * inspection
 * ---------------------------------------------------------------------------------- */

static void fill_info(const mdata* m, oracle_region_info* o) {
  memset(o, 0, sizeof(*o));
  o->va = m->va; o->handle = m->handle; o->mc_handle = m->mcHandle; o->alloc_sz = m->allocSz; o->tags = m->tags;
  memcpy(o->peers, m->peers, sizeof(o->peers));
  o->cpu_addr = (uint64_t)(uintptr_t)m->cpuAddr; o->user_info = m->userInfo;
  o->dev = m->dev; o->pid = m->pid; o->refcount = m->refcount; o->shared_fd = m->sharedFD;
  o->type = m->type; o->state = m->state; o->has_peer = m->hasPeer; o->oos_flag = m->oosFlag;
}

API int64_t oracle_region_count(int ctx, int dev) { octx* c = C(ctx); return c ? (int64_t)c->n[dev] : 0; }
API int oracle_region_at(int ctx, int dev, int64_t index, oracle_region_info* out) {
  octx* c = C(ctx);
  if (!c || index < 0 || (size_t)index >= c->n[dev]) return 1;
  fill_info(&c->tab[dev][index], out);
  return 0;
}
API int oracle_region_find(int ctx, int dev, uint64_t va, oracle_region_info* out) {
  octx* c = C(ctx);
  mdata* m = c ? find(c, dev, va) : NULL;
  if (!m) return 1;
  fill_info(m, out);
  return 0;
}
API uint64_t oracle_handle_lookup(int ctx, int dev, uint64_t handle) { octx* c = C(ctx); return c ? hlookup(c, dev, handle) : 0; }
API void oracle_get_counters(int ctx, oracle_counters* o) {
  octx* c = C(ctx);
  memset(o, 0, sizeof(*o));
  if (!c) return;
  o->release_local_cnt = c->releaseLocalCnt; o->release_shadow_cnt = c->releaseShadowCnt;
  o->offload_cnt = c->offloadCnt; o->smoke_log = c->smokeLog;
  memcpy(o->alloc_bytes, c->allocBytes, sizeof(o->alloc_bytes));
  o->del_bytes = c->delBytes; o->pause_cnt = c->pauseCnt; o->resume_cnt = c->resumeCnt;
  o->paused = c->paused; o->group_id = c->groupID; o->handle_count = (int32_t)c->hn[0]; o->region_count = (int32_t)c->n[0];
}

/* ------------------------------------------------------------------------------------
 * CPU twins of the device kernels (no reference counterpart; definitions only):
 *   sum64 = sum of all little-endian uint32 words mod 2^64
 *   xor64 = xor of all little-endian uint64 words
 *   zero  = every byte of the chunk is 0
 * ---------------------------------------------------------------------------------- */

API uint64_t oracle_zero_scan(const void* ptr, uint64_t bytes, uint8_t* flags, oracle_chunk_sum* sums) {
  const uint8_t* p = (const uint8_t*)ptr;
  uint64_t nchunks = (bytes + ORACLE_CHUNK - 1) / ORACLE_CHUNK;
  for (uint64_t c = 0; c < nchunks; ++c) {
    uint64_t off = c * ORACLE_CHUNK;
    uint64_t len = bytes - off < ORACLE_CHUNK ? bytes - off : ORACLE_CHUNK;
    uint64_t sum = 0, x = 0;
    int zero = 1;
    for (uint64_t i = 0; i + 4 <= len; i += 4) {
      uint32_t w;
      memcpy(&w, p + off + i, 4);
      sum += w;
    }
    for (uint64_t i = 0; i + 8 <= len; i += 8) {
      uint64_t w;
      memcpy(&w, p + off + i, 8);
      x ^= w;
    }
    for (uint64_t i = 0; i < len; ++i)
      if (p[off + i]) { zero = 0; break; }
    flags[c] = (uint8_t)zero;
    if (sums) { sums[c].sum64 = sum; sums[c].xor64 = x; }
  }
  return nchunks;
}

API void oracle_gather_pack(const oracle_copy_desc* d, uint64_t n, void* staging) {
  for (uint64_t i = 0; i < n; ++i)
    memcpy((uint8_t*)staging + d[i].off, (const void*)(uintptr_t)d[i].va, d[i].bytes);
}

API void oracle_scatter_unpack(const oracle_copy_desc* d, uint64_t n, const void* staging) {
  for (uint64_t i = 0; i < n; ++i) {
    if (d[i].off == ORACLE_DESC_ZERO) memset((void*)(uintptr_t)d[i].va, 0, d[i].bytes);
    else memcpy((void*)(uintptr_t)d[i].va, (const uint8_t*)staging + d[i].off, d[i].bytes);
  }
}
