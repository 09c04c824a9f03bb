/*
 * Synthetic footprint generator: region sizes, zero-chunk masks and chunk contents of the
 * benchmark configurations, integer arithmetic only so that every machine produces the
 * same bytes. This is workload synthesis for tests and benchmarks (host code, plain C);
 * it is not part of the pause/resume engine.
 *
 * RNG: state = splitmix64(seed * 4 + stream), forced non-zero, then Marsaglia's
 * xorshift64 (x ^= x << 13; x ^= x >> 7; x ^= x << 17). A 32-bit draw is the high word.
 * Streams: 0 sizes, 1 zero mask, 2 contents, 3 writes between cycles.
 * Contents are defined per 64 KiB chunk so that they can be produced and checked in
 * parallel and without keeping a copy: chunk number c of generation g holds the
 * little-endian 64-bit outputs of a xorshift64 stream whose state is
 * splitmix64(splitmix64(seed * 4 + 2) + c * 0x9E3779B97F4A7C15 + g), forced non-zero.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define FP_CHUNK 65536ull
#define FP_API __attribute__((visibility("default")))

FP_API uint64_t amem_fp_splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

FP_API void amem_fp_rng_init(uint64_t* state, uint64_t seed, uint64_t stream) {
  uint64_t s = amem_fp_splitmix64(seed * 4 + stream);
  *state = s ? s : 1;
}

FP_API uint64_t amem_fp_next64(uint64_t* state) {
  uint64_t x = *state;
  x ^= x << 13;
  x ^= x >> 7;
  x ^= x << 17;
  *state = x;
  return x;
}

FP_API uint32_t amem_fp_next32(uint64_t* state) { return (uint32_t)(amem_fp_next64(state) >> 32); }

/* Log-uniform size: octave k uniform in [0, octaves), then a uniform multiple of `unit`
 * inside [lo << k, lo << (k + 1)). */
static uint64_t log_uniform(uint64_t* st, uint64_t lo, uint32_t octaves, uint64_t unit) {
  uint32_t k = amem_fp_next32(st) % octaves;
  uint64_t base = lo << k;
  uint64_t steps = base / unit; /* multiples of unit inside the octave */
  return base + unit * (amem_fp_next32(st) % steps);
}

/* Region (or sub-allocation) sizes of configuration `cfg`, written to out[0..max_n).
 * Stops after `max_n` sizes, or as soon as the running total reaches `byte_budget`
 * (0 = no budget). Returns the count.
 *   cfg 1: 64 draws of 2 MiB x U{1..16}
 *   cfg 2: 128 x 4 MiB, 96 x 2 MiB, 32 x 16 MiB, in that order (no randomness)
 *   cfg 3: 2560 draws log-uniform in [2, 64) MiB, 2 MiB steps
 *   cfg 4: 100000 draws log-uniform in [4, 64) KiB, 4 KiB steps */
FP_API uint64_t amem_fp_sizes(int cfg, uint64_t seed, uint64_t* out, uint64_t max_n, uint64_t byte_budget) {
  uint64_t st, n = 0, total = 0, want = 0;
  const uint64_t MiB = 1ull << 20, KiB = 1ull << 10;
  amem_fp_rng_init(&st, seed, 0);
  switch (cfg) {
    case 1: want = 64; break;
    case 2: want = 256; break;
    case 3: want = 2560; break;
    case 4: want = 100000; break;
    default: return 0;
  }
  if (want > max_n) want = max_n;
  for (uint64_t i = 0; i < want; ++i) {
    uint64_t sz;
    if (cfg == 1) sz = 2 * MiB * (1 + amem_fp_next32(&st) % 16);
    else if (cfg == 2) sz = i < 128 ? 4 * MiB : (i < 224 ? 2 * MiB : 16 * MiB);
    else if (cfg == 3) sz = log_uniform(&st, 2 * MiB, 5, 2 * MiB);
    else sz = log_uniform(&st, 4 * KiB, 4, 4 * KiB);
    out[n++] = sz;
    total += sz;
    if (byte_budget && total >= byte_budget) break;
  }
  return n;
}

/* mask[c] = 1 for a chunk that is all zero; `pct` percent of chunks on average. */
FP_API void amem_fp_zero_mask(uint64_t seed, uint64_t nchunks, int pct, uint8_t* mask) {
  uint64_t st;
  amem_fp_rng_init(&st, seed, 1);
  for (uint64_t c = 0; c < nchunks; ++c) mask[c] = (int)(amem_fp_next32(&st) % 100) < pct;
}

static void fill_chunk(uint64_t key, uint64_t chunk, uint32_t gen, uint8_t* dst, uint64_t len) {
  uint64_t st = amem_fp_splitmix64(key + chunk * 0x9E3779B97F4A7C15ull + gen);
  if (!st) st = 1;
  uint64_t i = 0;
  for (; i + 8 <= len; i += 8) {
    uint64_t v = amem_fp_next64(&st);
    memcpy(dst + i, &v, 8);
  }
  if (i < len) {
    uint64_t v = amem_fp_next64(&st);
    memcpy(dst + i, &v, len - i);
  }
}

struct fill_job {
  uint64_t key, c0, nchunks, bytes;
  const uint8_t* mask;
  const uint32_t* gen;
  uint8_t* buf;
  const uint8_t* cmp;
  int tid, nthreads;
  uint64_t mismatches;
};

static void* fill_worker(void* arg) {
  struct fill_job* j = (struct fill_job*)arg;
  uint8_t* tmp = j->cmp ? (uint8_t*)malloc(FP_CHUNK) : NULL;
  for (uint64_t k = j->tid; k < j->nchunks; k += j->nthreads) {
    uint64_t off = k * FP_CHUNK;
    uint64_t len = j->bytes - off < FP_CHUNK ? j->bytes - off : FP_CHUNK;
    uint64_t c = j->c0 + k;
    uint8_t* dst = j->cmp ? tmp : j->buf + off;
    if (j->mask && j->mask[c]) memset(dst, 0, len);
    else fill_chunk(j->key, c, j->gen ? j->gen[c] : 0, dst, len);
    if (j->cmp) {
      if (memcmp(tmp, j->cmp + off, len) != 0)
        for (uint64_t b = 0; b < len; ++b) j->mismatches += tmp[b] != j->cmp[off + b];
    }
  }
  free(tmp);
  return NULL;
}

static uint64_t run_jobs(uint64_t seed, uint64_t c0, uint64_t bytes, const uint8_t* mask, const uint32_t* gen,
                         uint8_t* buf, const uint8_t* cmp, int threads) {
  uint64_t nchunks = (bytes + FP_CHUNK - 1) / FP_CHUNK;
  if (threads < 1) threads = 1;
  if (threads > 64) threads = 64;
  if ((uint64_t)threads > nchunks) threads = nchunks ? (int)nchunks : 1;
  struct fill_job jobs[64];
  pthread_t th[64];
  uint64_t key = amem_fp_splitmix64(seed * 4 + 2);
  for (int t = 0; t < threads; ++t) {
    struct fill_job j = {key, c0, nchunks, bytes, mask, gen, buf, cmp, t, threads, 0};
    jobs[t] = j;
    if (t > 0) pthread_create(&th[t], NULL, fill_worker, &jobs[t]);
  }
  fill_worker(&jobs[0]);
  uint64_t bad = jobs[0].mismatches;
  for (int t = 1; t < threads; ++t) {
    pthread_join(th[t], NULL);
    bad += jobs[t].mismatches;
  }
  return bad;
}

/* Produce the bytes of a region whose first chunk has global chunk number `c0`.
 * mask/gen are indexed by global chunk number and may be NULL (no zero chunks / generation 0). */
FP_API void amem_fp_fill(uint64_t seed, uint64_t c0, uint64_t bytes, const uint8_t* mask, const uint32_t* gen,
                         uint8_t* buf, int threads) {
  run_jobs(seed, c0, bytes, mask, gen, buf, NULL, threads);
}

/* Compare `buf` with what amem_fp_fill would produce; returns the number of differing bytes. */
FP_API uint64_t amem_fp_check(uint64_t seed, uint64_t c0, uint64_t bytes, const uint8_t* mask, const uint32_t* gen,
                              const uint8_t* buf, int threads) {
  return run_jobs(seed, c0, bytes, mask, gen, NULL, buf, threads);
}

/* Writes between cycles (stream 3, advanced by `cycle`): `count` chunks are picked with
 * replacement; a zero chunk becomes non-zero, a non-zero chunk becomes zero on an even draw
 * and gets new contents on an odd one. Updates mask/gen in place and lists the touched
 * chunk numbers in out_chunks[0..count). */
FP_API void amem_fp_mutate(uint64_t seed, uint64_t cycle, uint64_t nchunks, uint64_t count, uint8_t* mask,
                           uint32_t* gen, uint64_t* out_chunks) {
  uint64_t st;
  amem_fp_rng_init(&st, seed, 3);
  st = amem_fp_splitmix64(st + cycle);
  if (!st) st = 1;
  for (uint64_t i = 0; i < count; ++i) {
    uint64_t c = amem_fp_next64(&st) % nchunks;
    uint32_t coin = amem_fp_next32(&st);
    if (mask[c]) { mask[c] = 0; gen[c]++; }
    else if ((coin & 1) == 0) mask[c] = 1;
    else gen[c]++;
    if (out_chunks) out_chunks[i] = c;
  }
}
