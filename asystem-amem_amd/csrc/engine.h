// The pause/resume data path on one GPU: zero/checksum scan, packing into pinned host
// memory, physical release, and the reverse. Replaces the bodies of amem_memPause /
// amem_memResume (amem_nccl_plugin/amem_nccl.cpp:467-677), whose data path is one
// synchronous cuMemcpy per region.
#ifndef AMEM_ENGINE_H_
#define AMEM_ENGINE_H_

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include <mutex>
#include <utility>
#include <vector>

#include "ctx.h"
#include "kernels.h"
#include "slab_pool.h"

namespace amem {

struct Options {
  int64_t zero_elide = 1;
  int64_t verify = 0;
  int64_t pause_path = 2;                 // 0 direct, 1 staged, 2 default (= 3), 3 interleaved, 4 reference structure (A/B only)
  int64_t pause_wgs = 0;                  // interleaved path: workgroups of the gather kernel, 0 = the default (8)
  int64_t pause_xcds = 0;                 // interleaved path: XCDs the gather kernel may occupy, 0 = the default (1)
  int64_t interleave_bytes = 4ll << 20;   // interleaved path: parked bytes per gather launch
  int64_t dma_min_bytes = 16ll << 20;     // direct path: runs this long go by hipMemcpyAsync
  int64_t staging_bytes = 256ll << 20;    // each of two device staging buffers
  int64_t slab_bytes = 256ll << 20;
  int64_t link_wgs = 96;                  // workgroups of a kernel touching host memory
  int64_t hbm_wgs = 65536;                // workgroup cap of the scan kernel
  int64_t hbm_move_wgs = 1 << 22;         // workgroup cap of the mover when both sides are device memory
  int64_t resume_batch_bytes = 64ll << 20;
  int64_t resume_dma_min_bytes = 0;       // resume: runs this long come back by hipMemcpyAsync on the second stream (0 = none)
  int64_t peer_timeout_ms = 60000;
  int64_t release_thread = 1;             // interleaved path: handles are released on a third thread
  int64_t pause_adaptive = 1;             // interleaved path: narrow the gather kernel while the copy runs ahead of the unmaps
  int64_t scratch_on_host = 0;            // 1: engine tables live in pinned host memory even if the device has room
  int64_t pool_limit_bytes = 0;           // cap on pinned host memory a pause may need, 0 = none
  int64_t offload_free_tag = -1;          // caller tag whose regions are released without being copied
  int64_t peer_loopback = 0;              // let a process register with / update its own service (tests)
};
Options& options();

// Growable device / pinned-host scratch.
struct DevBuf {
  void* p = nullptr;     // address the GPU uses
  void* host = nullptr;  // set when the buffer lives in pinned host memory
  size_t cap = 0;
  // grow_on_host: if the buffer has to grow, put it in pinned host memory without trying the device
  hipError_t ensure(size_t bytes, bool grow_on_host = false);
  void release();
};
struct PinBuf {
  void* p = nullptr;
  size_t cap = 0;
  hipError_t ensure(size_t bytes);
  void release();
};

struct ParkedRegion {
  uint64_t va;
  uint64_t size;
  uint64_t first_chunk;
  uint64_t nchunks;
  uint64_t parked_off;    // logical pool offset of the first parked byte
  uint64_t parked_bytes;
  uint32_t desc_begin, desc_end;  // range in gather_descs_
  bool skip;              // registered under the offload-free tag: nothing parked, zeros restored
};

class Engine {
 public:
  explicit Engine(int dev);
  ~Engine();
  hipError_t init();

  // Both are called with Ctx::structure held.
  // *rolled_back is set when the pause failed before releasing anything and undid itself.
  int pause(Ctx& c, bool* rolled_back);
  // *incomplete is set when regions are still released after a failed resume (retry possible).
  int resume(Ctx& c, bool* incomplete);
  // A region was deleted while paused: drop its parked bytes.
  void forget(uint64_t va);

  // Figures of the last finished pause and resume. Another thread may ask while a cycle runs: it
  // gets the snapshot published when the previous phase ended, never the record being filled in.
  amem_cycle_stats stats() const {
    std::lock_guard<std::mutex> lk(stats_mtx_);
    return published_;
  }
  uint64_t trim_pool();
  hipError_t reserve_pool(uint64_t bytes);

  // Standalone kernel entry points (synchronous).
  hipError_t zero_scan(const amem_extent* ext, uint64_t n, uint8_t* flags, amem_chunk_sum* sums,
                       float* ms);
  // zero_scan with every table in the fixed device array of kernels.hip and in pinned host
  // buffers made by init(): allocates nothing. Rejects more than kNoAllocMaxExtents extents or
  // kNoAllocMaxChunks chunks.
  hipError_t zero_scan_noalloc(const amem_extent* ext, uint64_t n, uint8_t* flags, amem_chunk_sum* sums,
                               float* ms);
  hipError_t move(bool scatter, const amem_copy_desc* descs, uint64_t n, void* staging,
                  uint64_t staging_bytes, bool host_side, float* ms);
  hipError_t probe_link(uint64_t bytes, int reps, double* d2h, double* h2d);
  hipError_t calib_copy(uint64_t bytes, int reps, float* ms);

 private:
  hipError_t run_scan(const std::vector<ScanSeg>& segs, uint64_t* nchunks_out, bool want_sums,
                      float* ms);
  hipError_t reserve_descs(size_t n);
  hipError_t upload_descs(const CopyDesc* descs, size_t n, uint64_t* ntiles_out);
  hipError_t upload_slab_table();
  hipError_t pause_copy_direct(Ctx& c, std::vector<Region*>& regs);
  hipError_t pause_copy_staged(Ctx& c, std::vector<Region*>& regs, bool* used);
  hipError_t pause_copy_interleaved(Ctx& c, std::vector<Region*>& regs);
  hipError_t pause_copy_reference(Ctx& c, std::vector<Region*>& regs);
  // With `deferred`, the mapping is removed but the handle is handed back to be released later.
  hipError_t release_local(Ctx& c, Region* r, uint64_t va, std::pair<uint64_t, int>* deferred = nullptr);
  hipEvent_t event_at(size_t i);

  int dev_;
  // One caller at a time: every entry point uses the same scratch tables and streams.
  // Taken after Ctx::structure where both are held.
  std::mutex busy_;
  bool inited_ = false;
  hipStream_t kstream_ = nullptr;  // kernels
  hipStream_t dstream_ = nullptr;  // hipMemcpyAsync
  SlabPool* pool_ = nullptr;
  size_t slab_table_count_ = 0;
  bool grow_on_host_ = false;  // set for the length of a resume

  DevBuf d_segs_, d_prefix_, d_flags_, d_sums_, d_descs_, d_tiles_, d_slabtab_;
  DevBuf d_staging_[2];
  PinBuf h_segs_, h_prefix_, h_flags_, h_sums_, h_descs_, h_tiles_, h_slabtab_, h_sums_verify_;
  std::vector<hipEvent_t> events_;
  // zero_scan_noalloc: host-side staging of the tables and results, and its own event pair
  PinBuf na_in_, na_out_;
  hipEvent_t na_ev_[2] = {nullptr, nullptr};
  bool na_ready_ = false;

  // state carried from pause to resume
  std::vector<ParkedRegion> parked_;
  std::vector<CopyDesc> gather_descs_;
  std::vector<CopyDesc> scatter_descs_, dma_descs_, zero_descs_;  // resume's lists; kept for their capacity
  std::vector<ScanSeg> segs_;
  uint64_t nchunks_ = 0;
  uint64_t parked_total_ = 0;
  bool have_sums_ = false;
  bool elide_used_ = true;   // zero_elide as it was when the parked layout was made
  bool ref_mode_ = false;    // the parked layout was made by the reference-structure path
  std::vector<uint8_t> parked_flags_;  // per-chunk zero flags of the last pause

  amem_cycle_stats stats_ = {};      // working record: written by the threads of the running cycle only
  amem_cycle_stats published_ = {};  // what stats() hands out
  mutable std::mutex stats_mtx_;
  void publish_stats() {
    std::lock_guard<std::mutex> lk(stats_mtx_);
    published_ = stats_;
  }
};

// Engine of a device, created on first use. Returns nullptr (after an ERROR log) when no
// GPU is present: there is no host fallback for the data path.
Engine* engine_for(int dev);
// The engine of a device if one has been created, else nullptr.
Engine* engine_if_exists(int dev);
void destroy_engines();

}  // namespace amem
#endif
