// Race hammer for the host side of libamem_nccl: many threads drive the registry entry points
// at once while the socket service thread handles peer registrations. Built twice by
// tests/test_host_sanitizers.py, with -fsanitize=thread and with -fsanitize=address, from the
// library's own sources; it calls nothing that needs a GPU.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <thread>
#include <vector>

#include "../../include/amem.h"

static std::atomic<long> g_errors{0};
#define EXPECT(x) do { if (!(x)) { g_errors++; fprintf(stderr, "EXPECT failed line %d: %s\n", __LINE__, #x); } } while (0)

int main() {
  setenv("AMEM_ENABLE", "1", 1);
  EXPECT(amem_set_enabled(1) == 0);
  EXPECT(amem_set_option("peer_loopback", 1) == 0);
  EXPECT(amem_set_option("peer_timeout_ms", 5000) == 0);
  const int kThreads = 6, kPer = 400;
  const uint64_t MiB = 1 << 20;
  // a first region so that the context and the service exist before the threads start
  EXPECT(amem_add_alloc_info(0x7e0000000000ull, 2 * MiB, AMEM_TYPE_LOCAL, 0, 0x999, -1, 0, nullptr, 1) == 0);
  const int slot = amem_get_slot();
  EXPECT(slot >= 0);
  std::vector<std::thread> th;
  std::atomic<bool> stop{false};
  for (int t = 0; t < kThreads; ++t) {
    th.emplace_back([=] {
      const uint64_t base = 0x7f0000000000ull + ((uint64_t)t << 36);
      for (int i = 0; i < kPer; ++i) {
        const uint64_t va = base + (uint64_t)i * 4 * MiB, handle = 0x100000ull * (t + 1) + i;
        EXPECT(amem_add_alloc_info(va, 2 * MiB, AMEM_TYPE_LOCAL, 0, handle, -1, 0, nullptr, t % 8) == 0);
        EXPECT(amem_add_refcount((void*)va, 1) == 0);
        EXPECT(amem_add_peer_info(va, 0x5000 + i, (t + 1) % AMEM_MAX_DEVS) == 0);
        EXPECT(amem_handle_lookup(0, handle) == va);
        // an "import" of that region, registered with the owner through the socket service
        const uint64_t imp = base + (1ull << 34) + (uint64_t)i * 4 * MiB;
        EXPECT(amem_add_alloc_info(imp, 2 * MiB, AMEM_TYPE_PEER_POSIX, 0, handle + 0x80000, slot, handle, nullptr,
                                   AMEM_CALLER_P2P_PEER) == 0);
        amem_region_info info;
        EXPECT(amem_region_find(0, va, &info) == 0 && info.has_peer == 1 && info.peers[slot] == imp && info.refcount == 1);
        EXPECT(amem_check_paused(0) == 0);
        if (i % 3 == 0) {
          EXPECT(amem_del_alloc_info(imp, handle + 0x80000, 0) == 0);
          EXPECT(amem_del_alloc_info(va, handle, 0) == 0);
        }
      }
    });
  }
  std::thread reader([&] {
    amem_region_info info;
    amem_counters c;
    while (!stop.load()) {
      int64_t n = amem_region_count(0);
      for (int64_t k = 0; k < n; k += 17) (void)amem_region_at(0, k, &info);
      amem_get_counters(&c);
      amem_dump_alloc_stats(0);
    }
  });
  for (auto& x : th) x.join();
  stop.store(true);
  reader.join();
  amem_counters c;
  amem_get_counters(&c);
  const int64_t kept = (int64_t)kThreads * (kPer - (kPer + 2) / 3);
  EXPECT(amem_region_count(0) == 2 * kept + 1);
  EXPECT(amem_handle_count(0) == kept + 1);
  uint64_t bytes = 0;
  for (int i = 0; i < AMEM_MAX_CALLER; ++i) bytes += c.alloc_bytes[i];
  EXPECT(bytes == (uint64_t)(2 * kept + 1) * 2 * MiB);
  EXPECT(amem_shutdown() == 0);
  printf("hammer done: %ld errors\n", g_errors.load());
  return g_errors.load() ? 1 : 0;
}
