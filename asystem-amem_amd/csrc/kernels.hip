// Device kernels of the pause/resume data path, written for gfx950 (CDNA4, wave64).
//
// The reference has no device code: its only data movers are cuMemcpyDtoHAsync /
// cuMemcpyHtoDAsync, one call per region (amem_nccl_plugin/amem_nccl.h:304-327). These
// kernels exist so that thousands of scattered regions and 64 KiB chunks move at link or
// HBM rate instead of at per-call rate:
//
//   scan_chunks    one wavefront per 64 KiB chunk: is-all-zero flag + (sum64, xor64)
//   move_tiles     gather-pack / scatter-unpack / zero-fill over a descriptor list
//   calib_copy     plain copy used to calibrate hardware traffic counters
//
// All of it is integer/byte work bound by HBM or by the host link; nothing here is shaped
// for the matrix cores.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels.h"

namespace amem {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

static constexpr int kWave = 64;
static constexpr int kBlock = 256;
static constexpr int kWavesPerBlock = kBlock / kWave;
static constexpr uint32_t kXcds = 8;  // accelerator complex dies of the MI355X
static constexpr int kRounds = (int)(kTileBytes / (kBlock * 16));  // 16-byte loads a lane keeps in flight per tile

// Largest index i in [0, n) with prefix[i] <= x, for a non-decreasing prefix[0..n] with
// prefix[0] <= x < prefix[n].
__device__ __forceinline__ uint32_t find_segment(const uint64_t* __restrict__ prefix,
                                                 uint32_t n, uint64_t x) {
  uint32_t lo = 0, hi = n;
  while (hi - lo > 1) {
    uint32_t mid = (lo + hi) >> 1;
    if (prefix[mid] <= x) lo = mid; else hi = mid;
  }
  return lo;
}

__device__ __forceinline__ uint64_t wave_reduce_add(uint64_t v) {
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) {
    uint32_t lo = __shfl_xor((uint32_t)v, m, kWave);
    uint32_t hi = __shfl_xor((uint32_t)(v >> 32), m, kWave);
    v += ((uint64_t)hi << 32) | lo;
  }
  return v;
}

__device__ __forceinline__ uint64_t wave_reduce_xor(uint64_t v) {
#pragma unroll
  for (int m = kWave / 2; m >= 1; m >>= 1) {
    uint32_t lo = __shfl_xor((uint32_t)v, m, kWave);
    uint32_t hi = __shfl_xor((uint32_t)(v >> 32), m, kWave);
    v ^= ((uint64_t)hi << 32) | lo;
  }
  return v;
}

__device__ __forceinline__ void accumulate(const u32x4& v, uint64_t& sum, uint64_t& x) {
  sum += (uint64_t)v.x + (uint64_t)v.y + (uint64_t)v.z + (uint64_t)v.w;
  x ^= ((uint64_t)v.y << 32 | v.x) ^ ((uint64_t)v.w << 32 | v.z);
}

// One wavefront per chunk. A full chunk is 64 KiB = 64 lanes x 16 B x 64 rounds; every
// load instruction of the wave covers 1 KiB of consecutive addresses. Eight loads are
// issued before the first is consumed so each lane keeps 128 B in flight.
// A chunk is all-zero exactly when sum64 == 0: the words are unsigned and a chunk holds
// at most 2^14 of them, so the 64-bit sum cannot wrap.
__global__ __launch_bounds__(kBlock) void scan_chunks(const ScanSeg* __restrict__ segs,
                                                      const uint64_t* __restrict__ chunk_prefix,
                                                      uint32_t nsegs, uint64_t nchunks,
                                                      uint8_t* __restrict__ flags,
                                                      ChunkSum* __restrict__ sums) {
  const int lane = threadIdx.x & (kWave - 1);
  const uint64_t wave0 = (uint64_t)blockIdx.x * kWavesPerBlock + (threadIdx.x / kWave);
  const uint64_t nwaves = (uint64_t)gridDim.x * kWavesPerBlock;
  for (uint64_t c = wave0; c < nchunks; c += nwaves) {
    const uint32_t s = find_segment(chunk_prefix, nsegs, c);
    const uint64_t k = c - chunk_prefix[s];
    const uint64_t seg_bytes = segs[s].bytes;
    const uint64_t off = k * kChunkBytes;
    const uint32_t len = (uint32_t)((seg_bytes - off < kChunkBytes) ? (seg_bytes - off) : kChunkBytes);
    const u32x4* __restrict__ p = (const u32x4*)(segs[s].va + off) + lane;
    const uint32_t nvec = len >> 4;  // 16-byte vectors in this chunk
    uint64_t sum = 0, x = 0;
    uint32_t i = lane;
    // full rounds of 8 x 1 KiB
    for (; i + 7 * kWave < nvec; i += 8 * kWave, p += 8 * kWave) {
      u32x4 v0 = __builtin_nontemporal_load(p);
      u32x4 v1 = __builtin_nontemporal_load(p + kWave);
      u32x4 v2 = __builtin_nontemporal_load(p + 2 * kWave);
      u32x4 v3 = __builtin_nontemporal_load(p + 3 * kWave);
      u32x4 v4 = __builtin_nontemporal_load(p + 4 * kWave);
      u32x4 v5 = __builtin_nontemporal_load(p + 5 * kWave);
      u32x4 v6 = __builtin_nontemporal_load(p + 6 * kWave);
      u32x4 v7 = __builtin_nontemporal_load(p + 7 * kWave);
      accumulate(v0, sum, x); accumulate(v1, sum, x);
      accumulate(v2, sum, x); accumulate(v3, sum, x);
      accumulate(v4, sum, x); accumulate(v5, sum, x);
      accumulate(v6, sum, x); accumulate(v7, sum, x);
    }
    for (; i < nvec; i += kWave, p += kWave) {
      u32x4 v = __builtin_nontemporal_load(p);
      accumulate(v, sum, x);
    }
    sum = wave_reduce_add(sum);
    x = wave_reduce_xor(x);
    if (lane == 0) {
      flags[c] = (sum == 0) ? 1 : 0;
      if (sums) { sums[c].sum64 = sum; sums[c].xor64 = x; }
    }
  }
}

// Resolve a byte offset of the contiguous side to an address. The contiguous side is a
// list of equally sized slabs (power-of-two bytes); a single buffer is one slab with
// shift 63.
__device__ __forceinline__ uint8_t* slab_addr(const SlabTable& t, uint64_t off) {
  return t.base[off >> t.shift] + (off & t.mask);
}

// Tile mover. Descriptor d covers tiles [tile_prefix[d], tile_prefix[d+1]) of kTileBytes
// each (the last tile of a descriptor may be shorter); a launch handles the `ndescs`
// descriptors whose tiles are [first_tile, first_tile + ntiles). A workgroup takes tiles
// grid-stride; within a tile, 256 lanes x 16 B = 4 KiB per round, all rounds of the tile
// loaded before any store. `off_base` is subtracted from every descriptor offset, so a sub-range
// of a long descriptor list can be packed into a buffer that starts at that offset.
//   MODE 0  gather : staging[off + o] = device[va + o]
//   MODE 1  scatter: device[va + o] = staging[off + o], or zeros when off == kDescZero
// `xcds` confines the work to the first `xcds` of the chip's 8 XCDs: workgroups are dealt to
// XCDs round-robin by workgroup id, so a workgroup whose id modulo 8 is >= xcds retires at
// once and the others renumber themselves densely. A host-side hipMemUnmap issued while a
// kernel runs has to wait for a TLB shoot-down on every XCD that has waves in flight
// (measured: 0.43 ms with one XCD busy, 0.55 ms with two, 2.2 ms with all eight), while one
// XCD alone already drives the host link at 52 of its 57 GB/s.
template <int MODE>
__global__ __launch_bounds__(kBlock) void move_tiles(const CopyDesc* __restrict__ descs,
                                                     const uint64_t* __restrict__ tile_prefix,
                                                     uint32_t ndescs, uint64_t first_tile,
                                                     uint64_t ntiles, SlabTable slabs,
                                                     uint64_t off_base, uint32_t xcds) {
  const uint32_t tid = threadIdx.x;
  if ((blockIdx.x & (kXcds - 1)) >= xcds) return;
  const uint64_t wg = (uint64_t)(blockIdx.x / kXcds) * xcds + (blockIdx.x & (kXcds - 1));
  const uint64_t nwg = (uint64_t)(gridDim.x / kXcds) * xcds;
  for (uint64_t tt = wg; tt < ntiles; tt += nwg) {
    const uint64_t t = first_tile + tt;
    const uint32_t d = find_segment(tile_prefix, ndescs, t);
    const uint64_t o = (t - tile_prefix[d]) * kTileBytes;
    const uint64_t rem = descs[d].bytes - o;
    const uint32_t len = (uint32_t)(rem < kTileBytes ? rem : kTileBytes);
    const uint32_t nvec = len >> 4;
    const uint64_t off = descs[d].off;
    u32x4* dev = (u32x4*)(descs[d].va + o);
    if (MODE == 1 && off == kDescZero) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (uint32_t i = tid; i < nvec; i += kBlock) __builtin_nontemporal_store(z, dev + i);
      continue;
    }
    u32x4* stg = (u32x4*)slab_addr(slabs, off - off_base + o);
    const u32x4* __restrict__ src = (MODE == 0) ? dev : stg;
    u32x4* __restrict__ dst = (MODE == 0) ? stg : dev;
    uint32_t i = tid;
    for (; i + (kRounds - 1) * kBlock < nvec; i += kRounds * kBlock) {
      u32x4 v[kRounds];
#pragma unroll
      for (int r = 0; r < kRounds; ++r) v[r] = __builtin_nontemporal_load(src + i + r * kBlock);
#pragma unroll
      for (int r = 0; r < kRounds; ++r) __builtin_nontemporal_store(v[r], dst + i + r * kBlock);
    }
    for (; i < nvec; i += kBlock) {
      u32x4 a = __builtin_nontemporal_load(src + i);
      __builtin_nontemporal_store(a, dst + i);
    }
  }
}

// The same mover shaped for the case where both sides are device memory, which is bound by HBM
// rather than by the host link. Measured on an MI355X with the benchmark footprint's 33,600 runs
// (6.9 GiB, read + written counted): the link shape above (16 KiB per 256 lanes, 4 loads in flight
// per lane, 65,536 workgroups striding) 5.7 TB/s; the same without striding 5.8; 8 KiB per 256
// lanes 6.1; 4 KiB per 64 lanes 6.1; 2 KiB per 64 lanes 6.2; any shape with a single load per lane
// 4.6; this one — 4 KiB per workgroup of two wavefronts, two 16-byte loads in flight per lane,
// non-temporal, one workgroup per piece with no stride loop up to the grid cap — 6.4 TB/s, 80 % of
// the HBM peak (plain loads and stores instead of non-temporal ones: 5.8). The descriptor of a
// piece is found in the same 16 KiB tile prefix (a piece is a quarter of a tile); a direct
// piece-to-descriptor table measured the same as the search.
static constexpr int kHbmBlock = 128;
static constexpr uint32_t kHbmPiece = 4096;
static constexpr uint32_t kPiecesPerTile = (uint32_t)(kTileBytes / kHbmPiece);
static_assert(kHbmPiece == kHbmBlock * 16 * 2, "two 16-byte loads per lane");

template <int MODE>
__global__ __launch_bounds__(kHbmBlock) void move_pieces_hbm(const CopyDesc* __restrict__ descs,
                                                             const uint64_t* __restrict__ tile_prefix,
                                                             uint32_t ndescs, uint64_t first_tile,
                                                             uint64_t ntiles, SlabTable slabs,
                                                             uint64_t off_base) {
  const uint32_t tid = threadIdx.x;
  const uint64_t npieces = ntiles * kPiecesPerTile;
  for (uint64_t w = blockIdx.x; w < npieces; w += gridDim.x) {
    const uint64_t t = first_tile + w / kPiecesPerTile;
    const uint32_t d = find_segment(tile_prefix, ndescs, t);
    const uint64_t o = (t - tile_prefix[d]) * kTileBytes + (w % kPiecesPerTile) * kHbmPiece;
    const uint64_t bytes = descs[d].bytes;
    if (o >= bytes) continue;  // the last tile of a descriptor may have fewer pieces
    const uint64_t rem = bytes - o;
    const uint32_t nvec = (uint32_t)(rem < kHbmPiece ? rem : kHbmPiece) >> 4;
    const uint64_t off = descs[d].off;
    u32x4* dev = (u32x4*)(descs[d].va + o);
    if (MODE == 1 && off == kDescZero) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (uint32_t i = tid; i < nvec; i += kHbmBlock) __builtin_nontemporal_store(z, dev + i);
      continue;
    }
    u32x4* stg = (u32x4*)slab_addr(slabs, off - off_base + o);
    const u32x4* __restrict__ src = (MODE == 0) ? dev : stg;
    u32x4* __restrict__ dst = (MODE == 0) ? stg : dev;
    if (nvec == kHbmPiece / 16) {
      u32x4 a = __builtin_nontemporal_load(src + tid);
      u32x4 b = __builtin_nontemporal_load(src + tid + kHbmBlock);
      __builtin_nontemporal_store(a, dst + tid);
      __builtin_nontemporal_store(b, dst + tid + kHbmBlock);
    } else {
      for (uint32_t i = tid; i < nvec; i += kHbmBlock) {
        u32x4 a = __builtin_nontemporal_load(src + i);
        __builtin_nontemporal_store(a, dst + i);
      }
    }
  }
}

__global__ __launch_bounds__(kBlock) void calib_copy(const u32x4* __restrict__ src,
                                                     u32x4* __restrict__ dst, uint64_t nvec) {
  uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  const uint64_t stride = (uint64_t)gridDim.x * kBlock;
  for (; i < nvec; i += stride) dst[i] = src[i];
}

// ------------------------------------------------------------------------------------
// Launchers. Callers have validated: addresses 16-byte aligned, byte counts multiples of
// 16, prefix arrays consistent with the segment / descriptor arrays, every slab index a
// descriptor can reach present in the table.
// ------------------------------------------------------------------------------------

static uint32_t clamp_grid(uint64_t want, uint32_t cap) {
  if (want < 1) want = 1;
  return (uint32_t)(want < cap ? want : cap);
}

hipError_t launch_scan(const ScanSeg* d_segs, const uint64_t* d_chunk_prefix, uint32_t nsegs,
                       uint64_t nchunks, uint8_t* d_flags, ChunkSum* d_sums, uint32_t max_blocks,
                       hipStream_t stream) {
  if (nchunks == 0 || nsegs == 0) return hipSuccess;
  const uint32_t grid = clamp_grid((nchunks + kWavesPerBlock - 1) / kWavesPerBlock, max_blocks);
  (void)hipGetLastError();  // an earlier call's sticky error is not this launch's
  hipLaunchKernelGGL(scan_chunks, dim3(grid), dim3(kBlock), 0, stream, d_segs, d_chunk_prefix,
                     nsegs, nchunks, d_flags, d_sums);
  return hipGetLastError();
}

hipError_t launch_move(bool scatter, const CopyDesc* d_descs, const uint64_t* d_tile_prefix,
                       uint32_t ndescs, uint64_t first_tile, uint64_t ntiles,
                       const SlabTable& slabs, uint64_t off_base, uint32_t max_blocks, uint32_t xcds,
                       hipStream_t stream) {
  if (ntiles == 0 || ndescs == 0) return hipSuccess;
  if (xcds == kXcdsHbmShape) {
    // both sides in device memory: one small workgroup per 4 KiB piece
    const uint64_t npieces = ntiles * kPiecesPerTile;
    const uint32_t grid = (uint32_t)(npieces < max_blocks ? npieces : max_blocks);
    (void)hipGetLastError();
    if (scatter)
      hipLaunchKernelGGL(move_pieces_hbm<1>, dim3(grid), dim3(kHbmBlock), 0, stream, d_descs, d_tile_prefix,
                         ndescs, first_tile, ntiles, slabs, off_base);
    else
      hipLaunchKernelGGL(move_pieces_hbm<0>, dim3(grid), dim3(kHbmBlock), 0, stream, d_descs, d_tile_prefix,
                         ndescs, first_tile, ntiles, slabs, off_base);
    return hipGetLastError();
  }
  if (xcds < 1 || xcds > kXcds) xcds = kXcds;
  // the grid is a multiple of 8 so that every XCD is dealt the same number of workgroups;
  // `max_blocks` counts the workgroups that actually work
  const uint32_t per_xcd = (clamp_grid(ntiles, max_blocks) + xcds - 1) / xcds;
  const uint32_t grid = per_xcd * kXcds;
  (void)hipGetLastError();
  if (scatter)
    hipLaunchKernelGGL(move_tiles<1>, dim3(grid), dim3(kBlock), 0, stream, d_descs, d_tile_prefix,
                       ndescs, first_tile, ntiles, slabs, off_base, xcds);
  else
    hipLaunchKernelGGL(move_tiles<0>, dim3(grid), dim3(kBlock), 0, stream, d_descs, d_tile_prefix,
                       ndescs, first_tile, ntiles, slabs, off_base, xcds);
  return hipGetLastError();
}

// ------------------------------------------------------------------------------------
// Scan without allocation. The scan needs device memory beyond its inputs and outputs: the
// segment table, the chunk prefix, and the flag and checksum arrays the kernel writes before
// they are copied to the host. The ordinary path keeps those in growable hipMalloc buffers;
// callers that may not allocate (tight serving loops, harnesses that forbid it) use this fixed
// array instead; the call synchronises its stream, so it belongs outside any stream capture.
// Every GPU the library runs on holds its own copy of
// the array, at its own address, until the process ends.
// ------------------------------------------------------------------------------------

static constexpr size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
static constexpr size_t kNaSegsOff = 0;
static constexpr size_t kNaPrefixOff = kNaSegsOff + align256(kNoAllocMaxExtents * sizeof(ScanSeg));
static constexpr size_t kNaFlagsOff = kNaPrefixOff + align256((kNoAllocMaxExtents + 1) * sizeof(uint64_t));
static constexpr size_t kNaSumsOff = kNaFlagsOff + align256(kNoAllocMaxChunks);
static constexpr size_t kNaBytes = kNaSumsOff + align256(kNoAllocMaxChunks * sizeof(ChunkSum));
static_assert(kNaBytes == kNoAllocScratchBytes, "kernels.h states the size of the fixed scratch array");

static __device__ __align__(256) uint8_t scratch[kNaBytes];

// Device address of `scratch` on each GPU. In host code the array's name is only a stand-in for
// the symbol, not an address the GPU can use: the address comes from hipGetSymbolAddress, once per
// device, and everything below uses that pointer.
static uint8_t* g_scratch_ptr[8] = {nullptr};

hipError_t noalloc_setup(int dev) {
  if (dev < 0 || dev >= 8) return hipErrorInvalidDevice;
  if (g_scratch_ptr[dev]) return hipSuccess;
  uint8_t* ptr = nullptr;
  hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));  // the current device's copy
  if (e != hipSuccess) return e;
  if (!ptr) return hipErrorInvalidSymbol;
  g_scratch_ptr[dev] = ptr;
  return hipSuccess;
}

// Segment table and chunk prefix come from `h_segs` / `h_prefix` (pinned host memory), the flags
// and checksums go to `h_flags` / `h_sums` (pinned host memory; h_sums may be null). Everything is
// enqueued on `stream`; the caller synchronises. The kernel writes entry c of both arrays for every
// c < nchunks and only those are copied back, so nothing of an earlier call's contents is read and
// nothing has to be cleared.
hipError_t noalloc_scan(int dev, const ScanSeg* h_segs, const uint64_t* h_prefix, uint32_t nsegs,
                        uint64_t nchunks, uint8_t* h_flags, ChunkSum* h_sums, uint32_t max_blocks,
                        hipStream_t stream, hipEvent_t before, hipEvent_t after) {
  if (dev < 0 || dev >= 8 || !g_scratch_ptr[dev]) return hipErrorNotInitialized;
  if (nsegs == 0 || nchunks == 0) return hipSuccess;
  if (nsegs > kNoAllocMaxExtents || nchunks > kNoAllocMaxChunks) return hipErrorInvalidValue;
  uint8_t* ptr = g_scratch_ptr[dev];
  ScanSeg* d_segs = (ScanSeg*)(ptr + kNaSegsOff);
  uint64_t* d_prefix = (uint64_t*)(ptr + kNaPrefixOff);
  uint8_t* d_flags = ptr + kNaFlagsOff;
  ChunkSum* d_sums = (ChunkSum*)(ptr + kNaSumsOff);
  hipError_t e = hipMemcpyAsync(d_segs, h_segs, nsegs * sizeof(ScanSeg), hipMemcpyHostToDevice, stream);
  if (e != hipSuccess) return e;
  e = hipMemcpyAsync(d_prefix, h_prefix, (nsegs + 1) * sizeof(uint64_t), hipMemcpyHostToDevice, stream);
  if (e != hipSuccess) return e;
  if (before && (e = hipEventRecord(before, stream)) != hipSuccess) return e;
  e = launch_scan(d_segs, d_prefix, nsegs, nchunks, d_flags, h_sums ? d_sums : nullptr, max_blocks, stream);
  if (e != hipSuccess) return e;
  if (after && (e = hipEventRecord(after, stream)) != hipSuccess) return e;
  e = hipMemcpyAsync(h_flags, d_flags, nchunks, hipMemcpyDeviceToHost, stream);
  if (e != hipSuccess) return e;
  if (h_sums) e = hipMemcpyAsync(h_sums, d_sums, nchunks * sizeof(ChunkSum), hipMemcpyDeviceToHost, stream);
  return e;
}

hipError_t preload_kernels() {
  const void* fns[] = {(const void*)scan_chunks, (const void*)move_tiles<0>, (const void*)move_tiles<1>,
                       (const void*)move_pieces_hbm<0>, (const void*)move_pieces_hbm<1>, (const void*)calib_copy};
  for (const void* f : fns) {
    hipFuncAttributes attr;
    hipError_t e = hipFuncGetAttributes(&attr, f);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t launch_calib_copy(const void* d_src, void* d_dst, uint64_t bytes, hipStream_t stream) {
  const uint64_t nvec = bytes >> 4;
  if (nvec == 0) return hipSuccess;
  const uint32_t grid = clamp_grid((nvec + kBlock - 1) / kBlock, 8192);
  (void)hipGetLastError();
  hipLaunchKernelGGL(calib_copy, dim3(grid), dim3(kBlock), 0, stream, (const u32x4*)d_src,
                     (u32x4*)d_dst, nvec);
  return hipGetLastError();
}

}  // namespace amem
