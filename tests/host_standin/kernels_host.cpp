// TEST INFRASTRUCTURE, never part of the shipped library.
//
// Host twins of the launchers declared in asystem-amem_amd/csrc/kernels.h, for the test-only build in
// which "device memory" is host memory (see fake_hip.cpp): the same argument records, the same results,
// computed by plain loops at the time of the call. They exist so that the engine's host logic around the
// kernels (planning, batching, threads, peer traffic) can run in several real processes without a GPU.
#include <stdlib.h>
#include <string.h>

#include "../../asystem-amem_amd/csrc/kernels.h"

namespace amem {

static uint32_t find_segment(const uint64_t* prefix, uint32_t n, uint64_t x) {
  uint32_t lo = 0, hi = n;
  while (hi - lo > 1) {
    uint32_t mid = (lo + hi) >> 1;
    if (prefix[mid] <= x) lo = mid; else hi = mid;
  }
  return lo;
}

hipError_t launch_scan(const ScanSeg* segs, const uint64_t* chunk_prefix, uint32_t nsegs, uint64_t nchunks,
                       uint8_t* flags, ChunkSum* sums, uint32_t, hipStream_t) {
  if (nchunks == 0 || nsegs == 0) return hipSuccess;
  for (uint64_t c = 0; c < nchunks; ++c) {
    const uint32_t s = find_segment(chunk_prefix, nsegs, c);
    const uint64_t off = (c - chunk_prefix[s]) * kChunkBytes;
    const uint64_t len = segs[s].bytes - off < kChunkBytes ? segs[s].bytes - off : kChunkBytes;
    const uint8_t* p = (const uint8_t*)(uintptr_t)(segs[s].va + off);
    uint64_t sum = 0, x = 0;
    for (uint64_t i = 0; i + 16 <= len; i += 16) {
      uint32_t w[4];
      memcpy(w, p + i, 16);
      sum += (uint64_t)w[0] + w[1] + w[2] + w[3];
      x ^= ((uint64_t)w[1] << 32 | w[0]) ^ ((uint64_t)w[3] << 32 | w[2]);
    }
    flags[c] = sum == 0;
    if (sums) { sums[c].sum64 = sum; sums[c].xor64 = x; }
  }
  return hipSuccess;
}

hipError_t launch_move(bool scatter, const CopyDesc* descs, const uint64_t* tile_prefix, uint32_t ndescs,
                       uint64_t first_tile, uint64_t ntiles, const SlabTable& slabs, uint64_t off_base, uint32_t,
                       uint32_t, hipStream_t) {
  if (ntiles == 0 || ndescs == 0) return hipSuccess;
  for (uint64_t t = first_tile; t < first_tile + ntiles; ++t) {
    const uint32_t d = find_segment(tile_prefix, ndescs, t);
    const uint64_t o = (t - tile_prefix[d]) * kTileBytes;
    const uint64_t rem = descs[d].bytes - o;
    const uint64_t len = rem < kTileBytes ? rem : kTileBytes;
    uint8_t* dev = (uint8_t*)(uintptr_t)(descs[d].va + o);
    if (scatter && descs[d].off == kDescZero) { memset(dev, 0, len); continue; }
    const uint64_t off = descs[d].off - off_base + o;
    uint8_t* stg = slabs.base[off >> slabs.shift] + (off & slabs.mask);
    if (scatter) memcpy(dev, stg, len); else memcpy(stg, dev, len);
  }
  return hipSuccess;
}

hipError_t preload_kernels() { return hipSuccess; }

hipError_t launch_calib_copy(const void* src, void* dst, uint64_t bytes, hipStream_t) {
  memcpy(dst, src, bytes);
  return hipSuccess;
}

static uint8_t* g_scratch = nullptr;
hipError_t noalloc_setup(int dev) {
  if (dev != 0) return hipErrorInvalidDevice;
  if (!g_scratch) g_scratch = (uint8_t*)malloc(kNoAllocScratchBytes);
  return g_scratch ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t noalloc_scan(int, const ScanSeg* h_segs, const uint64_t* h_prefix, uint32_t nsegs, uint64_t nchunks,
                        uint8_t* h_flags, ChunkSum* h_sums, uint32_t, hipStream_t, hipEvent_t before, hipEvent_t after) {
  if (nsegs > kNoAllocMaxExtents || nchunks > kNoAllocMaxChunks) return hipErrorInvalidValue;
  if (before) (void)hipEventRecord(before, nullptr);
  hipError_t e = launch_scan(h_segs, h_prefix, nsegs, nchunks, h_flags, h_sums, 0, nullptr);
  if (after) (void)hipEventRecord(after, nullptr);
  return e;
}

}  // namespace amem
