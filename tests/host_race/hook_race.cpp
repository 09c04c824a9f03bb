// TEST INFRASTRUCTURE. The allocator hook (csrc/rccl_hook.cpp) beside the engine, under ThreadSanitizer,
// on the host stand-in of the HIP calls: one thread plays RCCL's proxy thread and keeps exporting a
// buffer (the hook's hipMemExportToShareableHandle asks the registry which address the handle backs),
// while the main thread runs pause/resume cycles over a registry that grows between them, so that the
// engine frees and regrows its own tables inside a cycle (those hipFree calls land in the hook's hipFree
// while the engine holds the registry's locks). A hook that held its own lock while it called into the
// registry would close a lock cycle with that; the sanitizer's lock-order checker reports it even when the
// timing does not produce the deadlock. Built and run by tests/test_host_sanitizers.py.
#include <dlfcn.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include <atomic>
#include <thread>
#include <vector>

#include "../../include/amem.h"
#include "../../include/amem_testing.h"

static std::atomic<long> g_errors{0};
#define EXPECT(x) do { if (!(x)) { g_errors++; fprintf(stderr, "EXPECT failed line %d: %s\n", __LINE__, #x); } } while (0)

typedef int (*alloc_fn)(void**, size_t);
typedef int (*free_fn)(void*);
typedef int (*export_fn)(void*, int*);
typedef int (*plain_alloc_fn)(void**, size_t, unsigned int, int);
typedef int64_t (*count_fn)(void);

int main(int argc, char** argv) {
  if (argc < 2) { fprintf(stderr, "usage: hook_race <librccl_standin.so>\n"); return 2; }
  void* rccl = dlopen(argv[1], RTLD_NOW | RTLD_GLOBAL);
  if (!rccl) { fprintf(stderr, "dlopen: %s\n", dlerror()); return 2; }
  alloc_fn cumem_alloc = (alloc_fn)dlsym(rccl, "standin_cumem_alloc");
  free_fn cumem_free = (free_fn)dlsym(rccl, "standin_cumem_free");
  export_fn do_export = (export_fn)dlsym(rccl, "standin_export");
  plain_alloc_fn plain_alloc = (plain_alloc_fn)dlsym(rccl, "standin_plain_alloc");
  free_fn plain_free = (free_fn)dlsym(rccl, "standin_plain_free");
  count_fn registered = (count_fn)dlsym(RTLD_DEFAULT, "amem_rccl_hook_registered");
  if (!cumem_alloc || !cumem_free || !do_export || !plain_alloc || !plain_free || !registered) {
    fprintf(stderr, "missing symbol\n");
    return 2;
  }
  const uint64_t MiB = 1 << 20;
  EXPECT(amem_set_enabled(1) == 0);
  EXPECT(amem_set_option("verify", 1) == 0);
  std::vector<void*> bufs;
  auto add_buffers = [&](int n) {
    for (int i = 0; i < n; ++i) {
      void* p = nullptr;
      EXPECT(cumem_alloc(&p, (2 + 2 * (i % 2)) * MiB) == 0);
      std::vector<uint64_t> fill((2 + 2 * (i % 2)) * MiB / 8);
      for (size_t k = 0; k < fill.size(); ++k) fill[k] = (k >> 13) % 3 ? k * 0x9e3779b97f4a7c15ull + bufs.size() : 0;
      EXPECT(amem_copy_to_device((uint64_t)(uintptr_t)p, fill.data(), fill.size() * 8) == 0);
      bufs.push_back(p);
    }
  };
  add_buffers(4);
  void* served = nullptr;                                   // one plain allocation served through the VMM API:
  EXPECT(plain_alloc(&served, 2 * MiB, 0, 1) == 0);         // from here on hipFree consults the hook's tables
  EXPECT(registered() == 5);
  EXPECT(amem_get_slot() >= 0);                             // the hook notes exports only for a process that has a slot
  std::atomic<bool> stop{false};
  std::atomic<long> exports{0};
  void* const exported = bufs[0];
  std::thread proxy([&] {
    while (!stop.load()) {
      int fd = -1;
      const int rc = do_export(exported, &fd);             // fails while the buffer is released: that is fine
      if (rc == 0) { close(fd); exports++; }
      std::this_thread::yield();
    }
  });
  for (int cycle = 0; cycle < 6; ++cycle) {
    EXPECT(amem_mem_pause(0, 0) == 0);
    EXPECT(amem_check_paused(0) == 1);
    EXPECT(amem_mem_resume(0, 0) == 0);
    amem_cycle_stats st;
    amem_get_cycle_stats(&st);
    EXPECT(st.verify_mismatch == 0);
    add_buffers(4 << (cycle / 2));                          // more regions, more chunks: the engine's tables regrow
    usleep(2000);
  }
  stop.store(true);
  proxy.join();
  EXPECT(exports.load() > 0);
  EXPECT(registered() == (int64_t)bufs.size() + 1);
  for (void* p : bufs) EXPECT(cumem_free(p) == 0);
  EXPECT(plain_free(served) == 0);
  EXPECT(registered() == 0 && amem_region_count(0) == 0);
  printf("hook race done: %ld errors, %ld exports beside 6 cycles, %zu buffers\n", g_errors.load(), exports.load(), bufs.size());
  return g_errors.load() ? 1 : 0;
}
