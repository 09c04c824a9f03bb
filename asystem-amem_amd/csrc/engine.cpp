#include "engine.h"

#include <string.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <thread>
#include <unordered_set>

#include "ipc.h"
#include "log.h"
#include "vmm.h"

namespace amem {

using Clock = std::chrono::steady_clock;
static inline double ms_since(Clock::time_point t0) {
  return std::chrono::duration<double, std::milli>(Clock::now() - t0).count();
}

Options& options() {
  static Options o;
  return o;
}

// Host time spent allocating engine scratch (tables, staging, events) since the counter was last
// read; pause and resume report it as a phase of their own. Only touched under Engine::busy_.
static double g_scratch_alloc_ms = 0;
static double take_scratch_alloc_ms() {
  const double v = g_scratch_alloc_ms;
  g_scratch_alloc_ms = 0;
  return v;
}
struct ScratchTimer {
  Clock::time_point t0 = Clock::now();
  ~ScratchTimer() { g_scratch_alloc_ms += ms_since(t0); }
};

// Pause is called when device memory is short, possibly gone. Scratch that does not fit on
// the device goes to pinned host memory, which the kernels reach over the link: slower
// table lookups, same results.
hipError_t DevBuf::ensure(size_t bytes, bool grow_on_host) {
  const bool forced = options().scratch_on_host != 0;
  if (bytes <= cap && (!forced || host)) return hipSuccess;
  const bool want_host = forced || grow_on_host;
  ScratchTimer timed;
  release();
  size_t want = std::max<size_t>(bytes + bytes / 4, 4096);
  if (!want_host) {
    if (hipMalloc(&p, want) == hipSuccess) { cap = want; return hipSuccess; }
    (void)hipGetLastError();
    p = nullptr;
    LOGGER(WARN, "no device memory for %zu KiB of engine scratch, placing it in pinned host memory", want >> 10);
  }
  hipError_t e = CHECK_HIP(hipHostMalloc(&host, want, hipHostMallocDefault));
  if (e != hipSuccess) { host = nullptr; return e; }
  e = CHECK_HIP(hipHostGetDevicePointer(&p, host, 0));
  if (e != hipSuccess) { (void)hipHostFree(host); host = p = nullptr; return e; }
  cap = want;
  return hipSuccess;
}
void DevBuf::release() {
  if (host) (void)CHECK_HIP(hipHostFree(host));
  else if (p) (void)CHECK_HIP(hipFree(p));
  p = host = nullptr;
  cap = 0;
}
hipError_t PinBuf::ensure(size_t bytes) {
  if (bytes <= cap) return hipSuccess;
  ScratchTimer timed;
  release();
  size_t want = std::max<size_t>(bytes + bytes / 4, 4096);
  hipError_t e = CHECK_HIP(hipHostMalloc(&p, want, hipHostMallocDefault));
  if (e != hipSuccess) { p = nullptr; return e; }
  cap = want;
  return hipSuccess;
}
void PinBuf::release() {
  if (p) (void)CHECK_HIP(hipHostFree(p));
  p = nullptr;
  cap = 0;
}

// Pinned host staging of the allocation-free scan: segment table + chunk prefix in, flags + checksums out.
static constexpr size_t kNaInBytes = kNoAllocMaxExtents * sizeof(ScanSeg) + (kNoAllocMaxExtents + 1) * sizeof(uint64_t);
static constexpr size_t kNaOutBytes = kNoAllocMaxChunks * (sizeof(ChunkSum) + 1);

Engine::Engine(int dev) : dev_(dev) {}

Engine::~Engine() {
  for (hipEvent_t e : events_) (void)hipEventDestroy(e);
  DevBuf* db[] = {&d_segs_, &d_prefix_, &d_flags_, &d_sums_, &d_descs_, &d_tiles_, &d_slabtab_,
                  &d_staging_[0], &d_staging_[1]};
  for (DevBuf* b : db) b->release();
  PinBuf* pb[] = {&h_segs_, &h_prefix_, &h_flags_, &h_sums_, &h_descs_, &h_tiles_, &h_slabtab_,
                  &h_sums_verify_, &na_in_, &na_out_};
  for (PinBuf* b : pb) b->release();
  for (hipEvent_t e : na_ev_) if (e) (void)hipEventDestroy(e);
  delete pool_;
  if (kstream_) (void)hipStreamDestroy(kstream_);
  if (dstream_) (void)hipStreamDestroy(dstream_);
}

hipError_t Engine::init() {
  if (inited_) return hipSuccess;
  hipError_t e = CHECK_HIP(hipSetDevice(dev_));
  if (e != hipSuccess) return e;
  // Non-blocking streams at the default priority: the null stream (on which the runtime
  // runs map/unmap commands) must not wait for copies in flight.
  // (a failed attempt may have left one of the streams behind: each is created once)
  if (!kstream_) {
    e = CHECK_HIP(hipStreamCreateWithFlags(&kstream_, hipStreamNonBlocking));
    if (e != hipSuccess) { kstream_ = nullptr; return e; }
  }
  if (!dstream_) {
    e = CHECK_HIP(hipStreamCreateWithFlags(&dstream_, hipStreamNonBlocking));
    if (e != hipSuccess) { dstream_ = nullptr; return e; }
  }
  // Load the kernels' code now: at the first pause there may be no device memory left for it.
  e = CHECK_HIP(preload_kernels());
  if (e != hipSuccess) return e;
  if (!pool_) pool_ = new SlabPool((uint64_t)options().slab_bytes);
  // Everything the allocation-free scan will ever need is made here, once per device: the device
  // address of its fixed table array, pinned host staging for tables and results, two events.
  if (!na_ready_) {
    hipError_t en = CHECK_HIP(noalloc_setup(dev_));
    if (en == hipSuccess) en = na_in_.ensure(kNaInBytes);
    if (en == hipSuccess) en = na_out_.ensure(kNaOutBytes);
    for (int k = 0; k < 2 && en == hipSuccess; ++k)
      if (!na_ev_[k]) en = CHECK_HIP(hipEventCreate(&na_ev_[k]));
    na_ready_ = (en == hipSuccess);
    if (!na_ready_) LOGGER(WARN, "pid:%d GPU:%d set-up of the allocation-free scan failed (%d); amem_zero_scan_noalloc "
                           "will report it", getpid(), dev_, (int)en);
  }
  inited_ = true;
  return hipSuccess;
}

hipEvent_t Engine::event_at(size_t i) {
  while (events_.size() <= i) {
    ScratchTimer timed;
    hipEvent_t ev = nullptr;
    (void)CHECK_HIP(hipEventCreate(&ev));
    events_.push_back(ev);
  }
  return events_[i];
}

hipError_t Engine::reserve_pool(uint64_t bytes) {
  std::lock_guard<std::mutex> busy(busy_);
  hipError_t e = init();
  if (e != hipSuccess) return e;
  const uint64_t limit = (uint64_t)options().pool_limit_bytes;
  if (limit && bytes > limit) return hipErrorOutOfMemory;
  e = pool_->ensure(bytes);
  stats_.slab_bytes = pool_->capacity();
  publish_stats();
  return e;
}

uint64_t Engine::trim_pool() {
  std::lock_guard<std::mutex> busy(busy_);
  if (!pool_) return 0;
  slab_table_count_ = 0;
  return pool_->trim();
}

// ---------------------------------------------------------------------------------------
// scan
// ---------------------------------------------------------------------------------------

static uint64_t chunks_of(uint64_t bytes) { return (bytes + kChunkBytes - 1) / kChunkBytes; }

hipError_t Engine::run_scan(const std::vector<ScanSeg>& segs, uint64_t* nchunks_out, bool want_sums,
                            float* ms) {
  const size_t n = segs.size();
  hipError_t e;
  if ((e = h_segs_.ensure(n * sizeof(ScanSeg))) != hipSuccess) return e;
  if ((e = h_prefix_.ensure((n + 1) * sizeof(uint64_t))) != hipSuccess) return e;
  uint64_t* prefix = (uint64_t*)h_prefix_.p;
  uint64_t total = 0;
  for (size_t i = 0; i < n; ++i) {
    ((ScanSeg*)h_segs_.p)[i] = segs[i];
    prefix[i] = total;
    total += chunks_of(segs[i].bytes);
  }
  prefix[n] = total;
  *nchunks_out = total;
  if (total == 0) { if (ms) *ms = 0; return hipSuccess; }
  if ((e = d_segs_.ensure(n * sizeof(ScanSeg), grow_on_host_)) != hipSuccess) return e;
  if ((e = d_prefix_.ensure((n + 1) * sizeof(uint64_t), grow_on_host_)) != hipSuccess) return e;
  if ((e = d_flags_.ensure(total, grow_on_host_)) != hipSuccess) return e;
  if ((e = h_flags_.ensure(total)) != hipSuccess) return e;
  if (want_sums) {
    if ((e = d_sums_.ensure(total * sizeof(ChunkSum), grow_on_host_)) != hipSuccess) return e;
  }
  e = CHECK_HIP(hipMemcpyAsync(d_segs_.p, h_segs_.p, n * sizeof(ScanSeg), hipMemcpyDefault, kstream_));
  if (e != hipSuccess) return e;
  e = CHECK_HIP(hipMemcpyAsync(d_prefix_.p, h_prefix_.p, (n + 1) * sizeof(uint64_t), hipMemcpyDefault, kstream_));
  if (e != hipSuccess) return e;
  hipEvent_t e0 = event_at(0), e1 = event_at(1);
  (void)CHECK_HIP(hipEventRecord(e0, kstream_));
  e = CHECK_HIP(launch_scan((const ScanSeg*)d_segs_.p, (const uint64_t*)d_prefix_.p, (uint32_t)n, total,
                            (uint8_t*)d_flags_.p, want_sums ? (ChunkSum*)d_sums_.p : nullptr,
                            (uint32_t)options().hbm_wgs, kstream_));
  if (e != hipSuccess) return e;
  (void)CHECK_HIP(hipEventRecord(e1, kstream_));
  e = CHECK_HIP(hipMemcpyAsync(h_flags_.p, d_flags_.p, total, hipMemcpyDefault, kstream_));
  if (e != hipSuccess) return e;
  e = CHECK_HIP(hipStreamSynchronize(kstream_));
  if (e != hipSuccess) return e;
  if (ms) {
    *ms = 0;
    (void)CHECK_HIP(hipEventElapsedTime(ms, e0, e1));
  }
  return hipSuccess;
}

// True when [va, va + bytes) lies inside one allocation or mapping known to the runtime.
// `hint` caches the last range found, since callers pass extents in address order.
static bool inside_known_memory(uint64_t va, uint64_t bytes, uint64_t hint[2]) {
  if (bytes == 0) return true;
  if (va >= hint[0] && va + bytes <= hint[0] + hint[1]) return true;
  uint64_t base = 0, size = 0;
  if (!vmm_range_of(va, &base, &size)) return false;
  hint[0] = base;
  hint[1] = size;
  return va >= base && va + bytes <= base + size;
}

hipError_t Engine::zero_scan(const amem_extent* ext, uint64_t n, uint8_t* flags, amem_chunk_sum* sums,
                             float* ms) {
  std::lock_guard<std::mutex> busy(busy_);
  hipError_t e = init();
  if (e != hipSuccess) return e;
  std::vector<ScanSeg> segs(n);
  uint64_t hint[2] = {0, 0};
  for (uint64_t i = 0; i < n; ++i) {
    if ((ext[i].va & 15) || (ext[i].bytes & 15) || ext[i].va == 0) return hipErrorInvalidValue;
    if (!inside_known_memory(ext[i].va, ext[i].bytes, hint)) return hipErrorInvalidValue;
    segs[i] = {ext[i].va, ext[i].bytes};
  }
  uint64_t total = 0;
  e = run_scan(segs, &total, sums != nullptr, ms);
  if (e != hipSuccess || total == 0) return e;
  memcpy(flags, h_flags_.p, total);
  if (sums) {
    e = CHECK_HIP(hipMemcpy(sums, d_sums_.p, total * sizeof(ChunkSum), hipMemcpyDefault));
  }
  return e;
}

// Same contract and results as zero_scan. After init() has run once on this device, a call makes
// no allocation of any kind: the tables the kernel reads and writes are the fixed device array of
// kernels.hip, the host side of every transfer is pinned memory made by init(), the events exist.
// Calls on one GPU share that array and the staging; busy_ is held from the first write to the last
// read, so overlapping calls queue up instead of racing.
hipError_t Engine::zero_scan_noalloc(const amem_extent* ext, uint64_t n, uint8_t* flags, amem_chunk_sum* sums,
                                     float* ms) {
  std::lock_guard<std::mutex> busy(busy_);
  hipError_t e = init();
  if (e != hipSuccess) return e;
  if (!na_ready_) return hipErrorNotInitialized;
  if (ms) *ms = 0;
  if (n > kNoAllocMaxExtents) {
    LOGGER(ERROR, "amem_zero_scan_noalloc: %llu extents, the fixed tables hold at most %u (use amem_zero_scan)",
           (unsigned long long)n, kNoAllocMaxExtents);
    return hipErrorInvalidValue;
  }
  ScanSeg* segs = (ScanSeg*)na_in_.p;
  uint64_t* prefix = (uint64_t*)((uint8_t*)na_in_.p + kNoAllocMaxExtents * sizeof(ScanSeg));
  uint64_t hint[2] = {0, 0};
  uint64_t total = 0;
  for (uint64_t i = 0; i < n; ++i) {
    if ((ext[i].va & 15) || (ext[i].bytes & 15) || ext[i].va == 0) return hipErrorInvalidValue;
    if (!inside_known_memory(ext[i].va, ext[i].bytes, hint)) return hipErrorInvalidValue;
    segs[i] = {ext[i].va, ext[i].bytes};
    prefix[i] = total;
    total += chunks_of(ext[i].bytes);
  }
  prefix[n] = total;
  if (total > kNoAllocMaxChunks) {
    LOGGER(ERROR, "amem_zero_scan_noalloc: %llu chunks of 64 KiB, the fixed tables hold at most %llu (use amem_zero_scan)",
           (unsigned long long)total, (unsigned long long)kNoAllocMaxChunks);
    return hipErrorInvalidValue;
  }
  if (total == 0) return hipSuccess;
  uint8_t* h_flags = (uint8_t*)na_out_.p + kNoAllocMaxChunks * sizeof(ChunkSum);
  ChunkSum* h_sums = (ChunkSum*)na_out_.p;
  e = CHECK_HIP(noalloc_scan(dev_, segs, prefix, (uint32_t)n, total, h_flags, sums ? h_sums : nullptr,
                             (uint32_t)options().hbm_wgs, kstream_, na_ev_[0], na_ev_[1]));
  hipError_t es = CHECK_HIP(hipStreamSynchronize(kstream_));  // also after a failed enqueue: the staging must be quiet
  if (e != hipSuccess) return e;
  if (es != hipSuccess) return es;
  memcpy(flags, h_flags, total);
  if (sums) memcpy(sums, h_sums, total * sizeof(ChunkSum));
  if (ms) (void)CHECK_HIP(hipEventElapsedTime(ms, na_ev_[0], na_ev_[1]));
  return hipSuccess;
}

// ---------------------------------------------------------------------------------------
// descriptor plumbing
// ---------------------------------------------------------------------------------------

hipError_t Engine::reserve_descs(size_t n) {
  hipError_t e;
  if ((e = h_descs_.ensure(std::max<size_t>(n, 1) * sizeof(CopyDesc))) != hipSuccess) return e;
  if ((e = h_tiles_.ensure((n + 1) * sizeof(uint64_t))) != hipSuccess) return e;
  if ((e = d_descs_.ensure(std::max<size_t>(n, 1) * sizeof(CopyDesc), grow_on_host_)) != hipSuccess) return e;
  return d_tiles_.ensure((n + 1) * sizeof(uint64_t), grow_on_host_);
}

hipError_t Engine::upload_descs(const CopyDesc* descs, size_t n, uint64_t* ntiles_out) {
  hipError_t e;
  if ((e = h_descs_.ensure(std::max<size_t>(n, 1) * sizeof(CopyDesc))) != hipSuccess) return e;
  if ((e = h_tiles_.ensure((n + 1) * sizeof(uint64_t))) != hipSuccess) return e;
  if ((e = d_descs_.ensure(std::max<size_t>(n, 1) * sizeof(CopyDesc), grow_on_host_)) != hipSuccess) return e;
  if ((e = d_tiles_.ensure((n + 1) * sizeof(uint64_t), grow_on_host_)) != hipSuccess) return e;
  uint64_t* tp = (uint64_t*)h_tiles_.p;
  uint64_t tiles = 0;
  for (size_t i = 0; i < n; ++i) {
    tp[i] = tiles;
    tiles += (descs[i].bytes + kTileBytes - 1) / kTileBytes;
  }
  tp[n] = tiles;
  *ntiles_out = tiles;
  if (n) memcpy(h_descs_.p, descs, n * sizeof(CopyDesc));
  if (n) {
    e = CHECK_HIP(hipMemcpyAsync(d_descs_.p, h_descs_.p, n * sizeof(CopyDesc), hipMemcpyDefault, kstream_));
    if (e != hipSuccess) return e;
  }
  return CHECK_HIP(hipMemcpyAsync(d_tiles_.p, h_tiles_.p, (n + 1) * sizeof(uint64_t), hipMemcpyDefault, kstream_));
}

// Device-side table of contiguous-side base addresses: pool slabs first, then the two
// staging buffers, then one spare entry for the standalone entry points.
hipError_t Engine::upload_slab_table() {
  const size_t ns = pool_->slab_count();
  const size_t entries = ns + 3;
  hipError_t e;
  if ((e = h_slabtab_.ensure(entries * sizeof(void*))) != hipSuccess) return e;
  if ((e = d_slabtab_.ensure(entries * sizeof(void*), grow_on_host_)) != hipSuccess) return e;
  uint8_t** tab = (uint8_t**)h_slabtab_.p;
  for (size_t i = 0; i < ns; ++i) {
    void* dp = nullptr;
    e = CHECK_HIP(hipHostGetDevicePointer(&dp, pool_->slabs()[i], 0));
    if (e != hipSuccess) return e;
    tab[i] = (uint8_t*)dp;
  }
  tab[ns] = (uint8_t*)d_staging_[0].p;
  tab[ns + 1] = (uint8_t*)d_staging_[1].p;
  tab[ns + 2] = nullptr;
  slab_table_count_ = ns;
  return CHECK_HIP(hipMemcpyAsync(d_slabtab_.p, h_slabtab_.p, entries * sizeof(void*), hipMemcpyDefault, kstream_));
}

// Append `d`, cut where its contiguous side would cross a slab boundary.
static void push_split(std::vector<CopyDesc>& out, CopyDesc d, uint64_t slab_bytes) {
  while (d.bytes) {
    const uint64_t room = slab_bytes - (d.off & (slab_bytes - 1));
    const uint64_t take = std::min(room, d.bytes);
    out.push_back({d.va, d.off, take});
    d.va += take; d.off += take; d.bytes -= take;
  }
}

// Walk the chunks of one region and emit its runs. Non-zero runs take consecutive logical
// offsets from *cursor; zero runs are emitted only when `zero_out` is given.
static void emit_runs(const uint8_t* flags, uint64_t va, uint64_t size, bool elide, uint64_t* cursor,
                      uint64_t slab_bytes, std::vector<CopyDesc>* data_out,
                      std::vector<CopyDesc>* zero_out, uint64_t* zero_chunks, uint64_t* zero_runs = nullptr) {
  const uint64_t n = chunks_of(size);
  uint64_t k = 0;
  while (k < n) {
    const bool z = elide && flags[k];
    uint64_t j = k + 1;
    while (j < n && (elide && flags[j]) == z) ++j;
    const uint64_t start = k * kChunkBytes;
    const uint64_t end = std::min(size, j * kChunkBytes);
    if (z) {
      if (zero_chunks) *zero_chunks += j - k;
      if (zero_runs) ++*zero_runs;
      if (zero_out) zero_out->push_back({va + start, kDescZero, end - start});
    } else {
      if (data_out) push_split(*data_out, {va + start, *cursor, end - start}, slab_bytes);
      *cursor += end - start;
    }
    k = j;
  }
}

hipError_t Engine::move(bool scatter, const amem_copy_desc* descs, uint64_t n, void* staging,
                        uint64_t staging_bytes, bool host_side, float* ms) {
  std::lock_guard<std::mutex> busy(busy_);
  hipError_t e = init();
  if (e != hipSuccess) return e;
  if (ms) *ms = 0;
  if (n == 0) return hipSuccess;
  if (!staging || ((uintptr_t)staging & 15)) return hipErrorInvalidValue;
  std::vector<CopyDesc> v(n);
  uint64_t hint[2] = {0, 0};
  if (!inside_known_memory((uint64_t)(uintptr_t)staging, staging_bytes, hint)) return hipErrorInvalidValue;
  hint[0] = hint[1] = 0;
  for (uint64_t i = 0; i < n; ++i) {
    const amem_copy_desc& d = descs[i];
    if (d.va == 0 || (d.va & 15) || (d.bytes & 15)) return hipErrorInvalidValue;
    if (!inside_known_memory(d.va, d.bytes, hint)) return hipErrorInvalidValue;
    if (d.off == kDescZero) {
      if (!scatter) return hipErrorInvalidValue;
    } else if ((d.off & 15) || d.off > staging_bytes || d.bytes > staging_bytes - d.off) {
      return hipErrorInvalidValue;
    }
    v[i] = {d.va, d.off, d.bytes};
  }
  uint64_t ntiles = 0;
  if ((e = upload_descs(v.data(), v.size(), &ntiles)) != hipSuccess) return e;
  if (slab_table_count_ != pool_->slab_count() || !d_slabtab_.p) {
    if ((e = upload_slab_table()) != hipSuccess) return e;
  }
  void* dp = staging;
  if (host_side) {
    e = CHECK_HIP(hipHostGetDevicePointer(&dp, staging, 0));
    if (e != hipSuccess) return e;
  }
  const size_t spare = pool_->slab_count() + 2;
  ((uint8_t**)h_slabtab_.p)[spare] = (uint8_t*)dp;
  e = CHECK_HIP(hipMemcpyAsync((uint8_t**)d_slabtab_.p + spare, (uint8_t**)h_slabtab_.p + spare,
                               sizeof(void*), hipMemcpyDefault, kstream_));
  if (e != hipSuccess) return e;
  SlabTable st = {(uint8_t* const*)d_slabtab_.p + spare, 63, ~(uint64_t)0 >> 1};
  hipEvent_t e0 = event_at(0), e1 = event_at(1);
  (void)CHECK_HIP(hipEventRecord(e0, kstream_));
  e = CHECK_HIP(launch_move(scatter, (const CopyDesc*)d_descs_.p, (const uint64_t*)d_tiles_.p,
                            (uint32_t)n, 0, ntiles, st, 0,
                            (uint32_t)(host_side ? options().link_wgs : options().hbm_move_wgs),
                            host_side ? 8 : kXcdsHbmShape, kstream_));
  if (e != hipSuccess) return e;
  (void)CHECK_HIP(hipEventRecord(e1, kstream_));
  e = CHECK_HIP(hipStreamSynchronize(kstream_));
  if (e == hipSuccess && ms) (void)CHECK_HIP(hipEventElapsedTime(ms, e0, e1));
  return e;
}

// ---------------------------------------------------------------------------------------
// pause
// ---------------------------------------------------------------------------------------

static int popcount_peers(const Region& r) {
  int n = 0;
  for (int i = 0; i < AMEM_MAX_DEVS; ++i) n += (r.peers[i] != 0);
  return n;
}

// Reference step 3 for one region (amem_nccl.cpp:529-557): drop the mapping and every
// reference, mark HOLE, forget the handle.
hipError_t Engine::release_local(Ctx& c, Region* r, uint64_t va, std::pair<uint64_t, int>* deferred) {
  auto t0 = Clock::now();
  uint64_t old = r->handle ? r->handle : vmm_handle_of(va);
  if (r->type == AMEM_TYPE_LOCAL_SYMM)
    LOGGER(DEBUG, "memPause: dptr:%llx is symmetric memory; no multicast object to unbind on this platform",
           (unsigned long long)va);
  // The reference drops `refcount` extra references here, one per retain its callers reported
  // (amem_nccl.cpp:541-549). On this runtime a retain takes no reference, so there are none to
  // drop, and a release beyond the creator's would touch a handle that is already freed. The
  // count is kept in the record and reported; no extra release is issued.
  if (r->refcount > 0)
    LOGGER(DEBUG, "memPause: groupID:%d pid:%d dptr:%llx refcount:%d (no extra releases on this runtime)",
           amem_groupID_value(), getpid(), (unsigned long long)va, r->refcount);
  hipError_t e;
  if (deferred) {
    e = vmm_unmap(va, r->allocSz);
    *deferred = {old, 0};
  } else {
    e = vmm_unmap_release(va, r->allocSz, old, 0);
  }
  {
    std::lock_guard<std::mutex> lk(c.fields);
    c.releaseLocalCnt += popcount_peers(*r);
    r->state = AMEM_STATE_HOLE;
    r->handle = 0;
    c.handleTable[dev_].erase(old);
  }
  stats_.pause_unmap_ms += ms_since(t0);
  return e;
}

// Reference structure, kept for A/B measurement only (pause_path 4): what amem_memPause does
// (amem_nccl.cpp:502-513, :529-558) expressed in HIP calls — per region one whole-region
// hipMemcpyAsync that is waited for before the next one starts, no scan, no elision; then per
// region the handle is looked up from the mapping, unmapped and released.
hipError_t Engine::pause_copy_reference(Ctx& c, std::vector<Region*>& regs) {
  hipError_t e = hipSuccess;
  auto tc = Clock::now();
  for (size_t i = 0; i < regs.size(); ++i) {
    for (uint32_t d = parked_[i].desc_begin; d < parked_[i].desc_end; ++d) {
      const CopyDesc& cd = gather_descs_[d];
      e = CHECK_HIP(hipMemcpyAsync(pool_->host_addr(cd.off), (const void*)(uintptr_t)cd.va, cd.bytes,
                                   hipMemcpyDeviceToHost, dstream_));
      if (e != hipSuccess) return e;
      stats_.dma_bytes += cd.bytes;
    }
    e = CHECK_HIP(hipStreamSynchronize(dstream_));
    if (e != hipSuccess) return e;
  }
  stats_.pause_copy_ms = ms_since(tc);
  for (size_t i = 0; i < regs.size(); ++i) {
    (void)vmm_handle_of(parked_[i].va);  // the reference's retain-to-discover (amem_nccl.cpp:539)
    hipError_t e2 = release_local(c, regs[i], parked_[i].va);
    if (e == hipSuccess) e = e2;
  }
  return e;
}

// Direct path: one gather kernel writes pinned host memory; runs of at least
// dma_min_bytes go by hipMemcpyAsync on the second stream at the same time.
hipError_t Engine::pause_copy_direct(Ctx& c, std::vector<Region*>& regs) {
  hipError_t e = hipSuccess;
  const uint64_t dma_min = (uint64_t)options().dma_min_bytes;
  std::vector<CopyDesc> kdescs;
  kdescs.reserve(gather_descs_.size());
  auto tc = Clock::now();
  for (const CopyDesc& d : gather_descs_) {
    if (dma_min && d.bytes >= dma_min) {
      e = CHECK_HIP(hipMemcpyAsync(pool_->host_addr(d.off), (const void*)(uintptr_t)d.va, d.bytes,
                                   hipMemcpyDeviceToHost, dstream_));
      if (e != hipSuccess) return e;
      stats_.dma_bytes += d.bytes;
    } else {
      kdescs.push_back(d);
      stats_.kernel_bytes += d.bytes;
    }
  }
  uint64_t ntiles = 0;
  if ((e = upload_descs(kdescs.data(), kdescs.size(), &ntiles)) != hipSuccess) return e;
  SlabTable st = {(uint8_t* const*)d_slabtab_.p, pool_->shift(), pool_->slab_bytes() - 1};
  hipEvent_t e0 = event_at(4), e1 = event_at(5);
  (void)CHECK_HIP(hipEventRecord(e0, kstream_));
  e = CHECK_HIP(launch_move(false, (const CopyDesc*)d_descs_.p, (const uint64_t*)d_tiles_.p,
                            (uint32_t)kdescs.size(), 0, ntiles, st, 0, (uint32_t)options().link_wgs, 8, kstream_));
  if (e != hipSuccess) return e;
  (void)CHECK_HIP(hipEventRecord(e1, kstream_));
  if (ntiles) stats_.k2_launches++;
  e = CHECK_HIP(hipStreamSynchronize(kstream_));
  if (e != hipSuccess) return e;
  e = CHECK_HIP(hipStreamSynchronize(dstream_));
  if (e != hipSuccess) return e;
  stats_.pause_copy_ms = ms_since(tc);
  float ms = 0;
  if (ntiles && hipEventElapsedTime(&ms, e0, e1) == hipSuccess) stats_.k2_ms += ms;
  for (size_t i = 0; i < regs.size(); ++i) {
    hipError_t e2 = release_local(c, regs[i], parked_[i].va);
    if (e == hipSuccess) e = e2;
  }
  return e;
}

// Launch shape of the interleaved path's gather kernel: 8 workgroups, all on one XCD. Measured on
// an MI355X, that shape alone moves 8 regions of 1 GiB at 54.7 GB/s (96 workgroups on all eight
// XCDs: the same), and with hundreds of regions to unmap beside it it still copies at 51 GB/s
// while an unmap costs 0.28 ms instead of the 2 ms it costs beside a kernel on every XCD
// (512 regions of 16 MiB: 175 ms against 260 ms). 4 workgroups copy at 44 GB/s, which is too
// slow to stay ahead of the unmaps; more than 8 gain nothing.
static constexpr uint32_t kPauseWgs = 8, kPauseXcds = 1;

// Interleaved path: the gather kernel writes pinned host memory itself, in many short
// launches (one per group of regions holding about interleave_bytes of parked data), with an
// event after each. A second host thread unmaps a group's regions as soon as that group's
// event has fired, and a third releases the handles behind it: the unmaps are what the pause
// waits for at the end, so nothing else rides on their thread (release_thread = 0 puts the
// releases back on it). An unmap issued while kernels are queued waits for roughly
// one kernel boundary, and the kernels keep running at link rate meanwhile, so short
// launches let most of the unmap time hide behind the transfer; a copy-engine transfer
// would instead stall for the whole of every unmap.
hipError_t Engine::pause_copy_interleaved(Ctx& c, std::vector<Region*>& regs) {
  hipError_t e;
  uint64_t ntiles_all = 0;
  if ((e = upload_descs(gather_descs_.data(), gather_descs_.size(), &ntiles_all)) != hipSuccess) return e;
  const uint64_t* tp = (const uint64_t*)h_tiles_.p;
  SlabTable pool_tab = {(uint8_t* const*)d_slabtab_.p, pool_->shift(), pool_->slab_bytes() - 1};
  const uint64_t want = (uint64_t)std::max<int64_t>(options().interleave_bytes, (int64_t)kChunkBytes);
  struct { uint32_t wgs, xcds; } shape = {kPauseWgs, kPauseXcds};
  if (options().pause_wgs > 0) shape.wgs = (uint32_t)options().pause_wgs;
  if (options().pause_xcds > 0) shape.xcds = (uint32_t)options().pause_xcds;
  LOGGER(DEBUG, "memPause: gather kernel on %u workgroups over %u XCD(s) for %llu MiB in %zu regions", shape.wgs,
         shape.xcds, (unsigned long long)(parked_total_ >> 20), parked_.size());
  struct Group { size_t r0, r1; uint32_t d0, d1; uint64_t bytes; };
  std::vector<Group> groups;
  const size_t n = parked_.size();
  for (size_t i = 0; i < n;) {
    size_t j = i;
    uint64_t bytes = 0;
    while (j < n && (bytes < want || j == i)) bytes += parked_[j++].parked_bytes;
    groups.push_back({i, j, parked_[i].desc_begin, parked_[j - 1].desc_end, bytes});
    i = j;
  }
  const size_t ev0 = 8;
  hipEvent_t start = event_at(ev0 + groups.size());  // creates every event before the thread starts
  std::atomic<size_t> launched{0};
  std::atomic<int> failed{0};
  const bool split = options().release_thread != 0;
  std::vector<std::pair<uint64_t, int>> to_release(split ? n : 0);
  std::atomic<size_t> unmapped{0};
  std::atomic<size_t> groups_unmapped{0};
  std::atomic<bool> unmapper_done{false};
  auto tc = Clock::now();
  std::thread unmapper([&] {
    (void)hipSetDevice(dev_);
    for (size_t g = 0; g < groups.size(); ++g) {
      while (launched.load(std::memory_order_acquire) <= g) {
        if (failed.load()) { unmapper_done.store(true); return; }
        std::this_thread::yield();
      }
      hipError_t es2 = CHECK_HIP(hipEventSynchronize(events_[ev0 + g]));
      if (es2 != hipSuccess) { failed.store((int)es2); break; }
      for (size_t r = groups[g].r0; r < groups[g].r1; ++r) {
        hipError_t e2 = release_local(c, regs[r], parked_[r].va, split ? &to_release[r] : nullptr);
        if (split) unmapped.store(r + 1, std::memory_order_release);
        if (e2 != hipSuccess) { failed.store((int)e2); break; }
      }
      if (failed.load()) break;
      groups_unmapped.store(g + 1, std::memory_order_release);
    }
    unmapper_done.store(true, std::memory_order_release);
  });
  std::thread releaser;
  if (split) releaser = std::thread([&] {
    (void)hipSetDevice(dev_);
    size_t done = 0;
    for (;;) {
      const bool last = unmapper_done.load(std::memory_order_acquire);
      const size_t avail = unmapped.load(std::memory_order_acquire);
      for (; done < avail; ++done) {
        hipError_t e2 = vmm_release(to_release[done].first, to_release[done].second);
        if (e2 != hipSuccess && !failed.load()) failed.store((int)e2);
      }
      if (last && done == unmapped.load(std::memory_order_acquire)) break;
      std::this_thread::yield();
    }
  });
  (void)CHECK_HIP(hipEventRecord(start, kstream_));
  e = hipSuccess;
  // Adaptive width (option pause_adaptive, on by default). The copy needs less time than the unmaps
  // (146 ms against 160-175 ms for the 10 GiB training-rank footprint), and an unmap costs less beside a
  // narrower kernel (measured in one process, cycle by cycle: 295 us beside 8 workgroups, 292 beside 5-7,
  // 279 beside 4, 235-245 with nothing running; 5 workgroups already saturate the link, 4 copy at 44 GB/s).
  // So the launcher keeps only a few launches queued, looks at how many finished groups still wait to be
  // unmapped, and gives up copy rate it does not need: 6 workgroups when the copy is more than 8 groups
  // ahead, 4 beyond 16, the full width again once the lead is under 4 groups. Where the copy is the
  // longer of the two (few large regions) the lead never builds up and nothing changes. Measured on two
  // machines: pause 172.5 -> 164.7 ms and 174.1 -> 165.7 ms; fixed widths of 5, 6, 7 and 12 workgroups
  // 170-174 ms, a fixed 4 169-172 ms (then the copy is the longer one), and limiting the queue depth
  // without narrowing changes nothing (173 ms).
  const bool adaptive = options().pause_adaptive != 0 && shape.xcds == 1 && shape.wgs > 4;
  constexpr size_t kDepth = 4;
  uint32_t wgs = shape.wgs;
  for (size_t g = 0; g < groups.size(); ++g) {
    const Group& G = groups[g];
    if (adaptive && g >= kDepth) {
      e = CHECK_HIP(hipEventSynchronize(events_[ev0 + g - kDepth]));
      if (e != hipSuccess) break;
      const size_t copied = g - kDepth + 1, gone = groups_unmapped.load(std::memory_order_acquire);
      const size_t lead = copied > gone ? copied - gone : 0;
      if (lead > 16) wgs = 4;
      else if (lead > 8) wgs = std::min<uint32_t>(shape.wgs, 6);
      else if (lead < 4) wgs = shape.wgs;
      if (wgs != shape.wgs) stats_.pause_narrow_launches++;
    }
    if (G.d1 > G.d0 && tp[G.d1] > tp[G.d0]) {
      e = CHECK_HIP(launch_move(false, (const CopyDesc*)d_descs_.p + G.d0, (const uint64_t*)d_tiles_.p + G.d0,
                                G.d1 - G.d0, tp[G.d0], tp[G.d1] - tp[G.d0], pool_tab, 0,
                                wgs, shape.xcds, kstream_));
      if (e != hipSuccess) break;
      stats_.k2_launches++;
      stats_.kernel_bytes += G.bytes;
    }
    e = CHECK_HIP(hipEventRecord(events_[ev0 + g], kstream_));
    if (e != hipSuccess) break;
    launched.store(g + 1, std::memory_order_release);
  }
  if (e != hipSuccess) failed.store((int)e);
  unmapper.join();
  if (releaser.joinable()) releaser.join();
  hipError_t es = CHECK_HIP(hipStreamSynchronize(kstream_));
  stats_.pause_copy_ms = ms_since(tc);
  if (!groups.empty()) {
    float ms = 0;
    if (hipEventElapsedTime(&ms, start, events_[ev0 + groups.size() - 1]) == hipSuccess) stats_.k2_ms += ms;
  }
  if (failed.load()) return (hipError_t)failed.load();
  return es;
}

// Staged path: regions are taken in rounds that fit one device staging buffer. A round is
// packed by a gather kernel at HBM rate, then leaves as a few large hipMemcpyAsync calls
// while the host unmaps and releases that round's regions. No kernel is in flight while
// the host unmaps: an unmap issued under a running kernel stalls for milliseconds, one
// issued under a copy-engine transfer does not.
hipError_t Engine::pause_copy_staged(Ctx& c, std::vector<Region*>& regs, bool* used) {
  *used = false;
  const uint64_t cap = (uint64_t)options().staging_bytes;
  if (cap < kChunkBytes) return hipSuccess;
  const uint64_t need = std::min<uint64_t>(cap, std::max<uint64_t>(parked_total_, kChunkBytes));
  for (int b = 0; b < 2; ++b) {
    if (d_staging_[b].cap >= need) continue;
    d_staging_[b].release();
    void* p = nullptr;
    if (hipMalloc(&p, need) != hipSuccess) {
      (void)hipGetLastError();
      LOGGER(INFO, "memPause: no room for %llu MiB of device staging, using the interleaved path",
             (unsigned long long)(need >> 20));
      d_staging_[0].release();
      d_staging_[1].release();
      return hipSuccess;
    }
    d_staging_[b].p = p;
    d_staging_[b].cap = need;
  }
  *used = true;
  hipError_t e;
  uint64_t ntiles_all = 0;
  if ((e = upload_descs(gather_descs_.data(), gather_descs_.size(), &ntiles_all)) != hipSuccess) return e;
  if ((e = upload_slab_table()) != hipSuccess) return e;
  const uint64_t* tp = (const uint64_t*)h_tiles_.p;
  const size_t ns = pool_->slab_count();
  SlabTable pool_tab = {(uint8_t* const*)d_slabtab_.p, pool_->shift(), pool_->slab_bytes() - 1};
  auto tc = Clock::now();
  size_t ev = 8;  // events 8.. are per-launch timing pairs
  std::vector<std::pair<hipEvent_t, hipEvent_t>> timed;
  hipEvent_t dma_done[2] = {event_at(2), event_at(3)};
  bool dma_pending[2] = {false, false};
  size_t i = 0;
  int round = 0;
  const size_t n = parked_.size();
  const uint64_t room = d_staging_[0].cap;
  while (i < n) {
    // a round: regions [i, j), descriptors [d0, d1), logical offsets [base, base + bytes)
    size_t j = i;
    uint64_t bytes = 0;
    const bool big = parked_[i].parked_bytes > room;
    if (big) { bytes = parked_[i].parked_bytes; j = i + 1; }
    else while (j < n && bytes + parked_[j].parked_bytes <= room) bytes += parked_[j++].parked_bytes;
    const uint32_t d0 = parked_[i].desc_begin, d1 = parked_[j - 1].desc_end;
    const uint64_t base = parked_[i].parked_off;
    const int buf = round & 1;
    if (bytes) {
      hipEvent_t s0 = event_at(ev++), s1 = event_at(ev++);
      if (big) {
        // larger than a staging buffer: straight to host memory
        (void)CHECK_HIP(hipEventRecord(s0, kstream_));
        e = CHECK_HIP(launch_move(false, (const CopyDesc*)d_descs_.p + d0, (const uint64_t*)d_tiles_.p + d0,
                                  d1 - d0, tp[d0], tp[d1] - tp[d0], pool_tab, 0,
                                  (uint32_t)options().link_wgs, 8, kstream_));
        if (e != hipSuccess) return e;
        (void)CHECK_HIP(hipEventRecord(s1, kstream_));
        e = CHECK_HIP(hipEventSynchronize(s1));
        if (e != hipSuccess) return e;
        stats_.kernel_bytes += bytes;
      } else {
        if (dma_pending[buf]) {
          e = CHECK_HIP(hipEventSynchronize(dma_done[buf]));
          if (e != hipSuccess) return e;
          dma_pending[buf] = false;
        }
        SlabTable stg = {(uint8_t* const*)d_slabtab_.p + ns + buf, 63, ~(uint64_t)0 >> 1};
        (void)CHECK_HIP(hipEventRecord(s0, kstream_));
        e = CHECK_HIP(launch_move(false, (const CopyDesc*)d_descs_.p + d0, (const uint64_t*)d_tiles_.p + d0,
                                  d1 - d0, tp[d0], tp[d1] - tp[d0], stg, base,
                                  (uint32_t)options().hbm_move_wgs, kXcdsHbmShape, kstream_));
        if (e != hipSuccess) return e;
        (void)CHECK_HIP(hipEventRecord(s1, kstream_));
        e = CHECK_HIP(hipEventSynchronize(s1));
        if (e != hipSuccess) return e;
        uint64_t x = 0;
        while (x < bytes) {
          const uint64_t take = std::min(bytes - x, pool_->room(base + x));
          e = CHECK_HIP(hipMemcpyAsync(pool_->host_addr(base + x), (uint8_t*)d_staging_[buf].p + x, take,
                                       hipMemcpyDeviceToHost, dstream_));
          if (e != hipSuccess) return e;
          x += take;
        }
        (void)CHECK_HIP(hipEventRecord(dma_done[buf], dstream_));
        dma_pending[buf] = true;
        stats_.dma_bytes += bytes;
      }
      timed.push_back({s0, s1});
      stats_.k2_launches++;
      ++round;
    }
    for (size_t r = i; r < j; ++r) {
      hipError_t e2 = release_local(c, regs[r], parked_[r].va);
      if (e2 != hipSuccess) return e2;
    }
    i = j;
  }
  e = CHECK_HIP(hipStreamSynchronize(dstream_));
  if (e != hipSuccess) return e;
  stats_.pause_copy_ms = ms_since(tc);
  for (auto& pr : timed) {
    float ms = 0;
    if (hipEventElapsedTime(&ms, pr.first, pr.second) == hipSuccess) stats_.k2_ms += ms;
  }
  // Device staging is given back: a paused process should hold no device memory for this.
  d_staging_[0].release();
  d_staging_[1].release();
  return hipSuccess;
}

int Engine::pause(Ctx& c, bool* rolled_back) {
  std::lock_guard<std::mutex> busy(busy_);
  struct Publish { Engine* e; ~Publish() { e->publish_stats(); } } publish_on_return{this};
  auto t0 = Clock::now();
  if (rolled_back) *rolled_back = false;
  hipError_t e = init();
  if (e != hipSuccess) return (int)e;
  int rc = 0;
  auto note = [&](hipError_t x) { if (x != hipSuccess && rc == 0) rc = (int)x; };
  // Tables that an earlier cycle had to place in host memory get another chance on the device.
  if (!options().scratch_on_host) {
    DevBuf* db[] = {&d_segs_, &d_prefix_, &d_flags_, &d_sums_, &d_descs_, &d_tiles_, &d_slabtab_};
    for (DevBuf* b : db) if (b->host) b->release();
  }
  grow_on_host_ = false;
  const int64_t path = options().pause_path;
  ref_mode_ = (path == 4);
  const bool elide = options().zero_elide != 0 && !ref_mode_;
  elide_used_ = elide;
  amem_cycle_stats fresh = {};
  fresh.slab_bytes = stats_.slab_bytes;
  stats_ = fresh;

  auto& table = c.allocTable[dev_];
  (void)take_scratch_alloc_ms();
  note(CHECK_HIP(hipDeviceSynchronize()));
  size_t free_sz = 0, total = 0;
  (void)CHECK_HIP(hipMemGetInfo(&free_sz, &total));
  LOGGER(INFO, "memPause: groupID:%d pid:%d GPU:%d memUsed: %ld MB before paused", amem_groupID_value(),
         getpid(), dev_, (long)((total - free_sz) >> 20));
  stats_.pause_sync_ms = ms_since(t0);

  std::vector<Region*> locals, invalid;
  std::vector<std::pair<uint64_t, Region*>> imported;
  parked_.clear();
  gather_descs_.clear();
  segs_.clear();
  for (auto& kv : table) {
    Region& r = kv.second;
    if (r.state != AMEM_STATE_ALLOC) continue;
    if (from_peer(r.type)) imported.push_back({kv.first, &r});
    else {
      // A kernel must never be pointed at memory that is not there: a region whose VA is not
      // (or no longer) mapped over its whole registered size is reported and not read.
      uint64_t base = 0, msize = 0;
      if ((kv.first & 15) || (r.allocSz & 15) || r.allocSz == 0 || !vmm_range_of(kv.first, &base, &msize) ||
          base != kv.first || msize < r.allocSz) {
        LOGGER(ERROR, "memPause: groupID:%d pid:%d dptr:%llx allocSz:%ld is not a mapped, 16-byte aligned range "
               "(mapping base:%llx size:%ld); its bytes are not saved", amem_groupID_value(), getpid(),
               (unsigned long long)kv.first, (long)r.allocSz, (unsigned long long)base, (long)msize);
        if (rc == 0) rc = (int)hipErrorInvalidValue;
        invalid.push_back(&r);
        continue;
      }
      // The handle is read off the mapping, as the reference does at this point
      // (amem_nccl.cpp:539-540): the one given at registration is only as good as the caller's
      // bookkeeping, and releasing a stale one would touch freed memory.
      const uint64_t mapped = vmm_handle_of(kv.first);
      if (mapped == 0) {
        LOGGER(ERROR, "memPause: groupID:%d pid:%d dptr:%llx allocSz:%ld is not memory of the virtual-memory API; "
               "it cannot be released and is left alone", amem_groupID_value(), getpid(),
               (unsigned long long)kv.first, (long)r.allocSz);
        if (rc == 0) rc = (int)hipErrorInvalidValue;
        invalid.push_back(&r);
        continue;
      }
      if (mapped != r.handle) {
        LOGGER(WARN, "memPause: groupID:%d pid:%d dptr:%llx was registered with handle %llx but is mapped to %llx; "
               "using the mapping's", amem_groupID_value(), getpid(), (unsigned long long)kv.first,
               (unsigned long long)r.handle, (unsigned long long)mapped);
        std::lock_guard<std::mutex> lk(c.fields);
        c.handleTable[dev_].erase(r.handle);
        r.handle = mapped;
        c.handleTable[dev_].emplace(mapped, kv.first);
      }
      locals.push_back(&r);
      segs_.push_back({kv.first, (uint64_t)r.allocSz});
    }
  }
  int rc_soft = rc;  // errors that concern single regions: the others are still paused, the error is returned at the end
  rc = 0;

  stats_.peer_regions = imported.size();
  stats_.local_regions = locals.size();

  // Reference step 1 (amem_nccl.cpp:502-513): save the bytes of every local region.
  {
    std::lock_guard<std::mutex> lk(c.fields);
    for (Region* r : locals) { r->state = AMEM_STATE_OFFLOADING; c.offloadCnt++; }
  }
  // Until the copy starts nothing has been copied, unmapped or released: a failure undoes the
  // bookkeeping and reports, and the caller is not paused.
  auto undo = [&]() {
    std::lock_guard<std::mutex> lk(c.fields);
    for (Region* r : locals) { r->state = AMEM_STATE_ALLOC; c.offloadCnt--; }
    parked_.clear();
    gather_descs_.clear();
    LOGGER(ERROR, "memPause: groupID:%d pid:%d GPU:%d failed with HIP error %d before anything was released; "
           "the process is not paused", amem_groupID_value(), getpid(), dev_, rc);
    if (rolled_back) *rolled_back = true;
    return rc;
  };
  auto ts = Clock::now();
  float k1ms = 0;
  have_sums_ = !ref_mode_;
  if (ref_mode_) {
    // reference structure: no scan, every byte of every region is copied
    nchunks_ = 0;
    for (const ScanSeg& sg : segs_) nchunks_ += chunks_of(sg.bytes);
    e = hipSuccess;
  } else {
    e = run_scan(segs_, &nchunks_, true, &k1ms);
  }
  note(e);
  if (e == hipSuccess && nchunks_ && !ref_mode_) {
    note(h_sums_.ensure(nchunks_ * sizeof(ChunkSum)));
    note(CHECK_HIP(hipMemcpyAsync(h_sums_.p, d_sums_.p, nchunks_ * sizeof(ChunkSum), hipMemcpyDefault, kstream_)));
  }
  if (rc != 0) return undo();
  stats_.k1_ms = k1ms;
  stats_.k1_launches = (nchunks_ && !ref_mode_) ? 1 : 0;
  stats_.pause_scan_ms = ms_since(ts);
  // the flags drive resume; keep them where no later scan can overwrite them
  if (ref_mode_) parked_flags_.assign(nchunks_, 0);
  else parked_flags_.assign((const uint8_t*)h_flags_.p, (const uint8_t*)h_flags_.p + nchunks_);
  stats_.total_chunks = nchunks_;

  auto tp = Clock::now();
  uint64_t cursor = 0, chunk0 = 0, zero_chunks = 0, zero_runs = 0;
  const uint8_t* flags = parked_flags_.data();
  uint64_t slab_bytes = pool_->slab_bytes();
  for (size_t i = 0; i < locals.size(); ++i) {
    ParkedRegion p = {};
    p.va = segs_[i].va;
    p.size = segs_[i].bytes;
    p.first_chunk = chunk0;
    p.nchunks = chunks_of(p.size);
    p.parked_off = cursor;
    p.desc_begin = (uint32_t)gather_descs_.size();
    // Regions registered under the offload-free caller tag are scratch: released without being
    // copied and handed back zero-filled (README.md:224 of the reference describes the intent;
    // its own comparison against the tag never takes effect, amem_nccl.cpp:40, :503, :620).
    p.skip = !ref_mode_ && options().offload_free_tag >= 0 && (int64_t)locals[i]->tags == options().offload_free_tag;
    if (p.skip) std::fill(parked_flags_.begin() + chunk0, parked_flags_.begin() + chunk0 + p.nchunks, (uint8_t)1);
    emit_runs(flags + chunk0, p.va, p.size, elide || p.skip, &cursor, slab_bytes, &gather_descs_, nullptr,
              p.skip ? nullptr : &zero_chunks, &zero_runs);
    p.desc_end = (uint32_t)gather_descs_.size();
    p.parked_bytes = cursor - p.parked_off;
    chunk0 += p.nchunks;
    stats_.footprint_bytes += p.size;
    parked_.push_back(p);
  }
  parked_total_ = cursor;
  stats_.parked_bytes = cursor;
  stats_.zero_chunks = zero_chunks;
  const uint64_t limit = (uint64_t)options().pool_limit_bytes;
  if (limit && cursor > limit) {
    LOGGER(ERROR, "memPause: groupID:%d pid:%d GPU:%d needs %llu MiB of pinned host memory, the limit is %llu MiB",
           amem_groupID_value(), getpid(), dev_, (unsigned long long)(cursor >> 20), (unsigned long long)(limit >> 20));
    e = hipErrorOutOfMemory;
  } else {
    auto tpool = Clock::now();
    e = pool_->ensure(cursor);
    stats_.pause_pool_ms = ms_since(tpool);
  }
  note(e);
  // Resume's scatter list is the gather list plus the zero runs (plus one entry per region that
  // was never saved). Its tables are sized now: what resume has to allocate must not come out of
  // the device memory the regions are about to give up.
  note(reserve_descs(gather_descs_.size() + zero_runs + table.size()));
  stats_.slab_bytes = pool_->capacity();
  if (rc != 0) return undo();

  // Imported mappings go before the local ones (reference step 2, amem_nccl.cpp:517-526): no
  // data to save, and the owner's release only frees memory once importers have let go.
  for (auto& pr : imported) {
    auto tu = Clock::now();
    Region* r = pr.second;
    LOGGER(DEBUG, "memPause: release peer handle %llx.", (unsigned long long)pr.first);
    const uint64_t h = vmm_handle_of(pr.first);  // the mapping's own, as for local regions
    if (h == 0) {
      LOGGER(ERROR, "memPause: groupID:%d pid:%d imported dptr:%llx is not mapped; left alone", amem_groupID_value(),
             getpid(), (unsigned long long)pr.first);
      if (rc_soft == 0) rc_soft = (int)hipErrorInvalidValue;
      continue;
    }
    note(vmm_unmap_release(pr.first, r->allocSz, h, 0));
    std::lock_guard<std::mutex> lk(c.fields);
    r->state = AMEM_STATE_HOLE;
    r->handle = 0;
    c.releaseShadowCnt++;
    stats_.pause_unmap_ms += ms_since(tu);
  }
  for (size_t i = 0; i < locals.size(); ++i) {
    locals[i]->parkedBytes = parked_[i].parked_bytes;
    locals[i]->cpuAddr = (parked_[i].parked_bytes && e == hipSuccess) ? pool_->host_addr(parked_[i].parked_off) : nullptr;
  }
  stats_.pause_plan_ms = ms_since(tp);

  if (rc == 0) {
    bool staged = false;
    if (ref_mode_) {
      note(pause_copy_reference(c, locals));
      staged = true;
    } else if ((path == 3 || path == 2) && !locals.empty()) {
      note(upload_slab_table());
      note(pause_copy_interleaved(c, locals));
      staged = true;
    } else if (path == 1 && !locals.empty()) {
      note(pause_copy_staged(c, locals, &staged));
    }
    if (!staged && rc == 0) {
      // no room for device staging (or path 0 asked for): write host memory from the kernel
      note(upload_slab_table());
      if (path == 0) note(pause_copy_direct(c, locals));
      else note(pause_copy_interleaved(c, locals));
    }
  }
  // The sums copy above rode kstream_; make sure it landed before the scratch is reused.
  note(CHECK_HIP(hipStreamSynchronize(kstream_)));

  // Reference step 3 also releases local regions that were not in ALLOC state and so were
  // not saved (amem_nccl.cpp:529-557 has no state test).
  if (rc == 0) {
    for (auto& kv : table) {
      Region& r = kv.second;
      if (from_peer(r.type) || r.state == AMEM_STATE_HOLE) continue;
      if (std::find(invalid.begin(), invalid.end(), &r) != invalid.end()) continue;  // reported above, left as found
      note(release_local(c, &r, kv.first));
    }
  } else {
    LOGGER(ERROR, "memPause: groupID:%d pid:%d GPU:%d failed with HIP error %d; physical memory of "
           "regions not yet released stays mapped", amem_groupID_value(), getpid(), dev_, rc);
  }
  note(CHECK_HIP(hipStreamSynchronize(dstream_)));
  long n_pause;
  int n_offload, n_local, n_shadow;
  {
    std::lock_guard<std::mutex> lk(c.fields);
    n_pause = (long)++c.pauseCnt;
    n_offload = c.offloadCnt; n_local = c.releaseLocalCnt; n_shadow = c.releaseShadowCnt;
  }
  stats_.pause_ms = ms_since(t0);
  stats_.pause_scratch_ms = take_scratch_alloc_ms();
  (void)CHECK_HIP(hipMemGetInfo(&free_sz, &total));
  LOGGER(INFO, "memPause: pause results. groupID:%d pid:%d GPU:%d pauseCnt:%ld memUsed:%ld MB after paused, "
         "released:%ld MB, duration:%ld ms offload:%d releaseLocal:%d releasePeer:%d",
         amem_groupID_value(), getpid(), dev_, n_pause, (long)((total - free_sz) >> 20),
         (long)(stats_.footprint_bytes >> 20), (long)stats_.pause_ms, n_offload, n_local, n_shadow);
  return rc ? rc : rc_soft;
}

void Engine::forget(uint64_t va) {
  for (ParkedRegion& p : parked_) {
    if (p.va == va) { p.va = 0; break; }
  }
}

// ---------------------------------------------------------------------------------------
// resume
// ---------------------------------------------------------------------------------------

int Engine::resume(Ctx& c, bool* incomplete) {
  std::lock_guard<std::mutex> busy(busy_);
  struct Publish { Engine* e; ~Publish() { e->publish_stats(); } } publish_on_return{this};
  if (incomplete) *incomplete = false;
  hipError_t e = init();
  if (e != hipSuccess) return (int)e;
  int rc = 0;
  auto note = [&](hipError_t x) { if (x != hipSuccess && rc == 0) rc = (int)x; };
  const bool elide = elide_used_;
  // Device memory is spoken for while paused: the regions need back exactly what they gave up.
  // Anything the engine still has to allocate goes to host memory.
  grow_on_host_ = true;
  struct Restore { bool& b; ~Restore() { b = false; } } restore_growth{grow_on_host_};
  size_t free_sz = 0, total = 0;
  (void)CHECK_HIP(hipMemGetInfo(&free_sz, &total));
  LOGGER(INFO, "groupID:%d pid:%d GPU:%d memUsed:%ld MB before resumed", amem_groupID_value(), getpid(), dev_,
         (long)((total - free_sz) >> 20));
  auto t0 = Clock::now();
  stats_.resume_ms = stats_.resume_map_ms = stats_.resume_copy_ms = stats_.resume_peer_ms = 0;
  stats_.k3_ms = 0; stats_.k3_launches = 0; stats_.verify_mismatch = 0; stats_.resume_dma_bytes = 0;
  stats_.resume_plan_ms = 0;
  (void)take_scratch_alloc_ms();
  auto& table = c.allocTable[dev_];

  // A pause that failed half-way leaves regions it never released in OFFLOADING: they still
  // have their memory and their bytes.
  {
    std::lock_guard<std::mutex> lk(c.fields);
    for (auto& kv : table) {
      Region& r = kv.second;
      if (!from_peer(r.type) && r.state == AMEM_STATE_OFFLOADING) { r.state = AMEM_STATE_ALLOC; c.offloadCnt--; }
    }
  }

  // Scatter list: per region, its parked runs and its zero runs.
  struct Item { Region* r; uint64_t va; uint32_t d0, d1; uint64_t bytes; uint32_t m0, m1; };
  std::vector<Item> items;
  items.reserve(table.size());
  // The lists are members so that their memory is kept from cycle to cycle: tens of thousands of
  // descriptors built into fresh vectors cost the resume 2 ms of allocation and first touches.
  std::vector<CopyDesc>& scatter = scatter_descs_;
  scatter.clear();
  // Runs at least resume_dma_min_bytes long (0 = none) come back by hipMemcpyAsync on the second
  // stream, next to the scatter kernel on the first; `dma` holds them, an item's are [m0, m1).
  std::vector<CopyDesc>& dma = dma_descs_;
  dma.clear();
  std::vector<CopyDesc>& zeros = zero_descs_;
  const uint64_t dma_min = ref_mode_ ? 0 : (uint64_t)options().resume_dma_min_bytes;
  const uint8_t* flags = parked_flags_.data();
  const uint64_t slab_bytes = pool_->slab_bytes();
  std::vector<ScanSeg> verify_segs;
  std::vector<uint64_t> verify_first_chunk;
  for (const ParkedRegion& p : parked_) {
    if (p.va == 0) continue;
    auto it = table.find(p.va);
    if (it == table.end()) continue;
    Region& r = it->second;
    if (r.state != AMEM_STATE_HOLE || from_peer(r.type)) continue;
    Item im = {&r, p.va, (uint32_t)scatter.size(), 0, p.size, (uint32_t)dma.size(), 0};
    uint64_t cursor = p.parked_off;
    zeros.clear();
    emit_runs(flags + p.first_chunk, p.va, p.size, elide || p.skip, &cursor, slab_bytes, &scatter, &zeros, nullptr);
    if (dma_min) {
      size_t keep = im.d0;
      for (size_t d = im.d0; d < scatter.size(); ++d) {
        if (scatter[d].bytes >= dma_min) dma.push_back(scatter[d]);
        else scatter[keep++] = scatter[d];
      }
      scatter.resize(keep);
    }
    scatter.insert(scatter.end(), zeros.begin(), zeros.end());
    im.d1 = (uint32_t)scatter.size();
    im.m1 = (uint32_t)dma.size();
    items.push_back(im);
    if (p.skip) continue;  // scratch regions come back as zeros by design: nothing to compare against
    verify_segs.push_back({p.va, p.size});
    verify_first_chunk.push_back(p.first_chunk);
  }
  // Local holes that were never saved come back as zeros.
  std::unordered_set<uint64_t> item_vas;
  for (const Item& im : items) item_vas.insert(im.va);
  for (auto& kv : table) {
    Region& r = kv.second;
    if (r.state != AMEM_STATE_HOLE || from_peer(r.type)) continue;
    if (item_vas.count(kv.first)) continue;
    Item im = {&r, kv.first, (uint32_t)scatter.size(), 0, (uint64_t)r.allocSz, (uint32_t)dma.size(), (uint32_t)dma.size()};
    scatter.push_back({kv.first, kDescZero, (uint64_t)r.allocSz & ~(uint64_t)15});
    im.d1 = (uint32_t)scatter.size();
    items.push_back(im);
  }
  uint64_t ntiles_all = 0;
  note(upload_descs(scatter.data(), scatter.size(), &ntiles_all));
  note(upload_slab_table());
  const uint64_t* tp = (const uint64_t*)h_tiles_.p;
  SlabTable pool_tab = {(uint8_t* const*)d_slabtab_.p, pool_->shift(), pool_->slab_bytes() - 1};

  // Regions whose new memory has importers. Each is exported only when its importers are told
  // (below), so that one descriptor is open at a time, as in the reference's loop
  // (amem_nccl.cpp:613, :646), however many regions there are.
  struct Export { Region* r; uint64_t va; uint64_t handle; };
  std::vector<Export> exports;
  uint64_t exportSz = 0;
  size_t ev = 8;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> timed;
  stats_.resume_plan_ms = ms_since(t0);
  auto tc = Clock::now();
  const uint64_t batch_bytes = (uint64_t)std::max<int64_t>(options().resume_batch_bytes, 1);
  size_t i = 0;
  while (i < items.size() && rc == 0) {
    size_t j = i;
    uint64_t bytes = 0;
    auto tm = Clock::now();
    while (j < items.size() && (bytes < batch_bytes || j == i)) {
      Item& im = items[j];
      uint64_t newh = 0;
      // amem_cuAllocAndExport (amem_nccl.h:164-193): create, map at the same VA, grant access.
      e = vmm_create_map(im.va, dev_, im.r->allocSz, &newh);
      note(e);
      if (e != hipSuccess) break;
      if (im.r->type == AMEM_TYPE_LOCAL_SYMM)
        LOGGER(DEBUG, "memResume: dptr:%llx is symmetric memory; no multicast object to bind on this platform",
               (unsigned long long)im.va);
      bool has_peer;
      {
        std::lock_guard<std::mutex> lk(c.fields);
        im.r->state = AMEM_STATE_PRELOADING;
        im.r->handle = newh;  // amem_updateAllocInfo, amem_nccl.cpp:272-291
        im.r->handleGen++;
        has_peer = im.r->hasPeer;
        c.handleTable[dev_].emplace(newh, im.va);
      }
      if (has_peer) {
        exports.push_back({im.r, im.va, newh});
        exportSz += im.r->allocSz;
      }
      if (ref_mode_) {
        // amem_lauchPreload with async=false (amem_nccl.h:316-327, call site amem_nccl.cpp:622):
        // one copy per region, waited for before the next region is touched
        for (uint32_t d = im.d0; d < im.d1; ++d) {
          if (scatter[d].off == kDescZero) continue;
          note(CHECK_HIP(hipMemcpyAsync((void*)(uintptr_t)scatter[d].va, pool_->host_addr(scatter[d].off), scatter[d].bytes,
                                        hipMemcpyHostToDevice, dstream_)));
        }
        note(CHECK_HIP(hipStreamSynchronize(dstream_)));
      }
      for (uint32_t m = im.m0; m < im.m1 && rc == 0; ++m) {
        note(CHECK_HIP(hipMemcpyAsync((void*)(uintptr_t)dma[m].va, pool_->host_addr(dma[m].off), dma[m].bytes,
                                      hipMemcpyHostToDevice, dstream_)));
        stats_.resume_dma_bytes += dma[m].bytes;
      }
      bytes += im.bytes;
      ++j;
    }
    stats_.resume_map_ms += ms_since(tm);
    if (j == i) break;
    const uint32_t d0 = items[i].d0, d1 = items[j - 1].d1;
    if (!ref_mode_ && d1 > d0 && tp[d1] > tp[d0]) {
      hipEvent_t s0 = event_at(ev++), s1 = event_at(ev++);
      (void)CHECK_HIP(hipEventRecord(s0, kstream_));
      note(CHECK_HIP(launch_move(true, (const CopyDesc*)d_descs_.p + d0, (const uint64_t*)d_tiles_.p + d0,
                                 d1 - d0, tp[d0], tp[d1] - tp[d0], pool_tab, 0,
                                 (uint32_t)options().link_wgs, 8, kstream_)));
      (void)CHECK_HIP(hipEventRecord(s1, kstream_));
      timed.push_back({s0, s1});
      stats_.k3_launches++;
    }
    {
      std::lock_guard<std::mutex> lk(c.fields);
      for (size_t k = i; k < j; ++k) { items[k].r->state = AMEM_STATE_ALLOC; c.offloadCnt--; }
    }
    i = j;
  }
  note(CHECK_HIP(hipStreamSynchronize(kstream_)));
  if (!dma.empty()) note(CHECK_HIP(hipStreamSynchronize(dstream_)));
  stats_.resume_copy_ms = ms_since(tc);
  for (auto& pr : timed) {
    float ms = 0;
    if (hipEventElapsedTime(&ms, pr.first, pr.second) == hipSuccess) stats_.k3_ms += ms;
  }

  if (options().verify && have_sums_ && rc == 0 && !verify_segs.empty()) {
    uint64_t nch = 0;
    float ms = 0;
    e = run_scan(verify_segs, &nch, true, &ms);
    note(e);
    if (e == hipSuccess) {
      note(h_sums_verify_.ensure(nch * sizeof(ChunkSum)));
      note(CHECK_HIP(hipMemcpy(h_sums_verify_.p, d_sums_.p, nch * sizeof(ChunkSum), hipMemcpyDefault)));
      const ChunkSum* before = (const ChunkSum*)h_sums_.p;
      const ChunkSum* after = (const ChunkSum*)h_sums_verify_.p;
      uint64_t a = 0;
      for (size_t s = 0; s < verify_segs.size(); ++s) {
        const uint64_t n = chunks_of(verify_segs[s].bytes);
        for (uint64_t k = 0; k < n; ++k, ++a) {
          const ChunkSum& b = before[verify_first_chunk[s] + k];
          if (b.sum64 != after[a].sum64 || b.xor64 != after[a].xor64) stats_.verify_mismatch++;
        }
      }
      if (stats_.verify_mismatch) {
        LOGGER(ERROR, "memResume: %llu chunks differ from their pre-pause checksum",
               (unsigned long long)stats_.verify_mismatch);
        if (rc == 0) rc = (int)hipErrorUnknown;
      }
    }
  }

  // Tell every importer where the new memory is (amem_nccl.cpp:633-649), after the bytes
  // are back so that an importer never maps memory still being filled.
  auto tpeer = Clock::now();
  for (Export& x : exports) {
    uint64_t peers[AMEM_MAX_DEVS];
    {
      std::lock_guard<std::mutex> lk(c.fields);
      memcpy(peers, x.r->peers, sizeof(peers));
    }
    int fd = -1;
    e = vmm_export_fd(x.handle, &fd);
    note(e);
    if (e != hipSuccess) continue;
    // every importer of the region is told at once (the reference tells them one after the other,
    // amem_nccl.cpp:636-645): they import and map side by side
    int slots[AMEM_MAX_DEVS], rets[AMEM_MAX_DEVS], nslots = 0;
    uint64_t vas[AMEM_MAX_DEVS];
    for (int s = 0; s < AMEM_MAX_DEVS; ++s) {
      if (peers[s] == 0) continue;
      slots[nslots] = s;
      vas[nslots++] = peers[s];
    }
    peer_update_many(slots, vas, nslots, fd, rets);
    for (int k = 0; k < nslots; ++k) {
      const int s = slots[k], ret = rets[k];
      if (ret != 0 && !peer_alive(s)) {
        // The importer's process is gone and its mapping with it: nothing to update, now or later.
        LOGGER(WARN, "groupID:%d pid:%d localDptr:%llx the importer in slot %d is gone, forgetting its mapping %llx",
               amem_groupID_value(), getpid(), (unsigned long long)x.va, s, (unsigned long long)peers[s]);
        std::lock_guard<std::mutex> lk(c.fields);
        x.r->peers[s] = 0;
        x.r->hasPeer = false;
        for (int j = 0; j < AMEM_MAX_DEVS; ++j) x.r->hasPeer |= x.r->peers[j] != 0;
        c.releaseLocalCnt--;
      } else if (ret != 0) {
        LOGGER(ERROR, "groupID:%d pid:%d localDptr:%llx newHandle:%llx fd:%d notify peer %d to remap dptr:%llx ret:%d",
               amem_groupID_value(), getpid(), (unsigned long long)x.va, (unsigned long long)x.handle, fd,
               s, (unsigned long long)peers[s], ret);
        if (rc == 0) rc = ret;
      } else {
        std::lock_guard<std::mutex> lk(c.fields);
        c.releaseLocalCnt--;
      }
    }
    if (fd >= 0) close(fd);
  }

  // Wait until every mapping this process imports has been re-established by its owner
  // (amem_nccl.cpp:659-662 polls every 500 ms; here the service thread signals).
  {
    std::unique_lock<std::mutex> lk(c.fields);
    const int64_t tmo = options().peer_timeout_ms;
    auto done = [&] { return c.releaseShadowCnt <= 0; };
    // True when every import still waiting belongs to a process that no longer exists.
    auto owners_gone = [&] {
      bool any = false;
      for (auto& kv : table) {
        const Region& r = kv.second;
        if (!from_peer(r.type) || r.state != AMEM_STATE_HOLE) continue;
        any = true;
        if (r.ownerSlot < 0 || peer_alive(r.ownerSlot)) return false;
      }
      return any;
    };
    const auto t_wait = Clock::now();
    while (!done()) {
      c.shadow_cv.wait_for(lk, std::chrono::milliseconds(200), done);
      if (done()) break;
      if (owners_gone()) {
        LOGGER(ERROR, "groupID:%d pid:%d GPU:%d peerLeft:%d and their owners are gone, giving up",
               amem_groupID_value(), getpid(), dev_, c.releaseShadowCnt);
        if (rc == 0) rc = 1;
        break;
      }
      if (tmo > 0 && ms_since(t_wait) >= (double)tmo) {
        LOGGER(ERROR, "groupID:%d pid:%d GPU:%d peerLeft:%d after %lld ms, giving up", amem_groupID_value(),
               getpid(), dev_, c.releaseShadowCnt, (long long)tmo);
        if (rc == 0) rc = 1;
        break;
      }
    }
  }
  stats_.resume_peer_ms = ms_since(tpeer);
  if (rc != 0) {
    // Regions still without memory keep their parked bytes: the caller stays paused and may
    // call resume again, e.g. once device memory another process held has been given back.
    size_t holes = 0;
    std::lock_guard<std::mutex> lk(c.fields);
    for (auto& kv : table) holes += kv.second.state == AMEM_STATE_HOLE && !from_peer(kv.second.type);
    // (an import still waiting for its owner is remapped by the service thread whenever the owner re-exports)
    if (holes) {
      LOGGER(ERROR, "memResume: groupID:%d pid:%d GPU:%d failed with error %d, %zu local regions are still released; "
             "the process stays paused and resume can be called again", amem_groupID_value(), getpid(), dev_, rc, holes);
      if (incomplete) *incomplete = true;
    }
  }
  stats_.resume_ms = ms_since(t0);
  stats_.resume_scratch_ms = take_scratch_alloc_ms();
  (void)CHECK_HIP(hipMemGetInfo(&free_sz, &total));
  long n_resume;
  int n_offload, n_local, n_shadow;
  {
    std::lock_guard<std::mutex> lk(c.fields);
    n_resume = (long)(c.resumeCnt + 1);
    n_offload = c.offloadCnt; n_local = c.releaseLocalCnt; n_shadow = c.releaseShadowCnt;
  }
  LOGGER(INFO, "groupID:%d pid:%d GPU:%d resumeCnt:%ld memUsed:%ld MB after resumed, duration:%ld ms "
         "offloadLeft:%d releaseLocalLeft:%d releasePeerLeft:%d exportSz:%ld",
         amem_groupID_value(), getpid(), dev_, n_resume, (long)((total - free_sz) >> 20),
         (long)stats_.resume_ms, n_offload, n_local, n_shadow, (long)(exportSz >> 20));
  return rc;
}

// ---------------------------------------------------------------------------------------
// measurement helpers
// ---------------------------------------------------------------------------------------

hipError_t Engine::probe_link(uint64_t bytes, int reps, double* d2h, double* h2d) {
  std::lock_guard<std::mutex> busy(busy_);
  hipError_t e = init();
  if (e != hipSuccess) return e;
  void *hp = nullptr, *dp = nullptr;
  if ((e = CHECK_HIP(hipHostMalloc(&hp, bytes, hipHostMallocDefault))) != hipSuccess) return e;
  if ((e = CHECK_HIP(hipMalloc(&dp, bytes))) != hipSuccess) { (void)hipHostFree(hp); return e; }
  memset(hp, 0x5a, bytes);
  (void)CHECK_HIP(hipMemset(dp, 0xa5, bytes));
  double best_d2h = 0, best_h2d = 0;
  for (int r = 0; r < reps + 1 && e == hipSuccess; ++r) {
    (void)CHECK_HIP(hipDeviceSynchronize());
    auto t0 = Clock::now();
    e = CHECK_HIP(hipMemcpy(hp, dp, bytes, hipMemcpyDeviceToHost));
    double a = ms_since(t0);
    t0 = Clock::now();
    if (e == hipSuccess) e = CHECK_HIP(hipMemcpy(dp, hp, bytes, hipMemcpyHostToDevice));
    double b = ms_since(t0);
    if (r == 0) continue;  // first pass touches the pinned pages
    best_d2h = std::max(best_d2h, bytes / a / 1e6);
    best_h2d = std::max(best_h2d, bytes / b / 1e6);
  }
  (void)CHECK_HIP(hipFree(dp));
  (void)CHECK_HIP(hipHostFree(hp));
  if (d2h) *d2h = best_d2h;
  if (h2d) *h2d = best_h2d;
  return e;
}

hipError_t Engine::calib_copy(uint64_t bytes, int reps, float* ms) {
  std::lock_guard<std::mutex> busy(busy_);
  hipError_t e = init();
  if (e != hipSuccess) return e;
  bytes &= ~(uint64_t)15;
  void *a = nullptr, *b = nullptr;
  if ((e = CHECK_HIP(hipMalloc(&a, bytes))) != hipSuccess) return e;
  if ((e = CHECK_HIP(hipMalloc(&b, bytes))) != hipSuccess) { (void)hipFree(a); return e; }
  (void)CHECK_HIP(hipMemset(a, 0x11, bytes));
  (void)CHECK_HIP(hipDeviceSynchronize());
  hipEvent_t e0 = event_at(0), e1 = event_at(1);
  float best = 0;
  for (int r = 0; r < reps && e == hipSuccess; ++r) {
    (void)CHECK_HIP(hipEventRecord(e0, kstream_));
    e = CHECK_HIP(launch_calib_copy(a, b, bytes, kstream_));
    (void)CHECK_HIP(hipEventRecord(e1, kstream_));
    if (e == hipSuccess) e = CHECK_HIP(hipStreamSynchronize(kstream_));
    float t = 0;
    if (e == hipSuccess && hipEventElapsedTime(&t, e0, e1) == hipSuccess && (best == 0 || t < best)) best = t;
  }
  (void)CHECK_HIP(hipFree(a));
  (void)CHECK_HIP(hipFree(b));
  if (ms) *ms = best;
  return e;
}

// ---------------------------------------------------------------------------------------
// per-device singletons
// ---------------------------------------------------------------------------------------

static Engine* g_engines[AMEM_MAX_DEVS] = {nullptr};
static std::mutex g_engines_mtx;

Engine* engine_for(int dev) {
  if (dev < 0 || dev >= AMEM_MAX_DEVS) return nullptr;
  std::lock_guard<std::mutex> lk(g_engines_mtx);
  if (g_engines[dev]) return g_engines[dev];
  if (!gpu_present()) {
    LOGGER(ERROR, "pid:%d no HIP device is visible: the pause/resume data path has no host fallback", getpid());
    return nullptr;
  }
  Engine* en = new Engine(dev);
  if (en->init() != hipSuccess) { delete en; return nullptr; }
  g_engines[dev] = en;
  return en;
}

Engine* engine_if_exists(int dev) {
  if (dev < 0 || dev >= AMEM_MAX_DEVS) return nullptr;
  std::lock_guard<std::mutex> lk(g_engines_mtx);
  return g_engines[dev];
}

void destroy_engines() {
  std::lock_guard<std::mutex> lk(g_engines_mtx);
  for (int i = 0; i < AMEM_MAX_DEVS; ++i) { delete g_engines[i]; g_engines[i] = nullptr; }
}

}  // namespace amem
