// Host-visible declarations of the device kernels' argument records and launchers.
#ifndef AMEM_KERNELS_H_
#define AMEM_KERNELS_H_

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

namespace amem {

static constexpr uint64_t kChunkBytes = 65536;  // zero-detect / checksum granule
static constexpr uint64_t kTileBytes = 16384;   // unit of work of the tile mover
static constexpr uint64_t kDescZero = ~(uint64_t)0;

// One scanned address range; chunk numbering runs range by range.
struct ScanSeg {
  uint64_t va;
  uint64_t bytes;
};

struct ChunkSum {
  uint64_t sum64;  // sum of all little-endian uint32 words mod 2^64
  uint64_t xor64;  // xor of all little-endian uint64 words
};

// One contiguous copy between a scattered device range and the contiguous side.
struct CopyDesc {
  uint64_t va;
  uint64_t off;    // byte offset on the contiguous side, or kDescZero (scatter: fill zeros)
  uint64_t bytes;
};

// The contiguous side: equally sized slabs, slab i covering offsets [i << shift, (i+1) << shift).
// `base` is an array in device-readable memory.
struct SlabTable {
  uint8_t* const* base;
  uint32_t shift;
  uint64_t mask;
};

hipError_t launch_scan(const ScanSeg* d_segs, const uint64_t* d_chunk_prefix, uint32_t nsegs,
                       uint64_t nchunks, uint8_t* d_flags, ChunkSum* d_sums, uint32_t max_blocks,
                       hipStream_t stream);

// `xcds` = 1..8 confines the link-shaped mover to that many XCDs; kXcdsHbmShape selects the mover
// shaped for device memory on both sides (`max_blocks` then caps its grid of 4 KiB pieces).
static constexpr uint32_t kXcdsHbmShape = 0xffffffffu;
hipError_t launch_move(bool scatter, const CopyDesc* d_descs, const uint64_t* d_tile_prefix,
                       uint32_t ndescs, uint64_t first_tile, uint64_t ntiles,
                       const SlabTable& slabs, uint64_t off_base, uint32_t max_blocks, uint32_t xcds,
                       hipStream_t stream);

// Limits of the scan that allocates nothing: its tables live in one fixed device array.
static constexpr uint32_t kNoAllocMaxExtents = 8192;
static constexpr uint64_t kNoAllocMaxChunks = 262144;  // 16 GiB of 64 KiB chunks
static constexpr size_t kNoAllocScratchBytes = 131072 + 65792 + 262144 + 4194304;  // tables, each rounded to 256 B
// Look up the device address of the fixed array for `dev`, which must be the current device. Once per device.
hipError_t noalloc_setup(int dev);
// Enqueue table upload, scan and result download on `stream`, using only the fixed array and the
// caller's pinned host buffers. hipErrorInvalidValue beyond the limits above.
hipError_t noalloc_scan(int dev, const ScanSeg* h_segs, const uint64_t* h_prefix, uint32_t nsegs,
                        uint64_t nchunks, uint8_t* h_flags, ChunkSum* h_sums, uint32_t max_blocks,
                        hipStream_t stream, hipEvent_t before, hipEvent_t after);

// Makes the runtime load this library's device code now rather than at the first launch.
hipError_t preload_kernels();
hipError_t launch_calib_copy(const void* d_src, void* d_dst, uint64_t bytes, hipStream_t stream);

}  // namespace amem
#endif
