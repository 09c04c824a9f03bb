// TEST INFRASTRUCTURE. Drives the host stand-in build of the library (the library's own sources on a
// host-memory stand-in of the HIP calls) through whole pause/resume cycles with cross-rank imports while
// other threads keep calling the hook and inspection entry points: the engine's copy / unmap / release
// threads, the socket service threads and the callers' threads all run at once. Built and run under
// ThreadSanitizer and AddressSanitizer by tests/test_host_sanitizers.py.
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

static uint64_t mix(uint64_t x) { x ^= x >> 33; x *= 0xff51afd7ed558ccdull; x ^= x >> 33; return x; }

int main() {
  const uint64_t MiB = 1 << 20;
  EXPECT(amem_set_enabled(1) == 0);
  EXPECT(amem_set_option("peer_loopback", 1) == 0);
  EXPECT(amem_set_option("peer_timeout_ms", 20000) == 0);
  EXPECT(amem_set_option("verify", 1) == 0);
  EXPECT(amem_set_option("interleave_bytes", 1 << 20) == 0);   // many short launches: many hand-overs between the threads
  struct Reg { uint64_t va, handle, size; std::vector<uint8_t> data; };
  std::vector<Reg> regs;
  for (int i = 0; i < 24; ++i) {
    Reg r;
    EXPECT(amem_vmm_alloc((2 + 2 * (i % 3)) * MiB, 0, &r.va, &r.handle, &r.size) == 0);
    r.data.resize(r.size);
    for (uint64_t k = 0; k < r.size; k += 8) {
      const uint64_t chunk = k >> 16;
      const uint64_t v = (mix(chunk + 31 * i) % 3 == 0) ? 0 : mix(k + ((uint64_t)i << 40));   // a third of the chunks zero
      memcpy(&r.data[k], &v, 8);
    }
    EXPECT(amem_copy_to_device(r.va, r.data.data(), r.size) == 0);
    EXPECT(amem_add_alloc_info(r.va, r.size, AMEM_TYPE_LOCAL, 0, r.handle, -1, 0, nullptr, AMEM_CALLER_P2P) == 0);
    regs.push_back(std::move(r));
  }
  const int owner = amem_get_slot();
  EXPECT(owner >= 0);
  const int rank2 = amem_ipc_claim_slot(), rank3 = amem_ipc_claim_slot();
  EXPECT(rank2 >= 0 && rank3 >= 0 && rank2 != rank3);
  struct Imp { uint64_t va, size; size_t of; };
  std::vector<Imp> imports;
  for (int rank : {rank2, rank3}) {
    EXPECT(amem_ipc_act_as(rank) == 0);
    for (size_t i = 0; i < regs.size(); i += 2) {
      int fd = -1;
      uint64_t va = 0, h = 0;
      EXPECT(amem_vmm_export(regs[i].handle, &fd) == 0);
      EXPECT(amem_vmm_import(fd, regs[i].size, 0, &va, &h) == 0);
      close(fd);
      EXPECT(amem_add_alloc_info(va, regs[i].size, AMEM_TYPE_PEER_POSIX, 0, h, owner, regs[i].handle, nullptr,
                                 AMEM_CALLER_P2P_PEER) == 0);
      imports.push_back({va, regs[i].size, i});
    }
  }
  EXPECT(amem_ipc_act_as(-1) == 0);
  std::atomic<bool> stop{false};
  std::atomic<long> calls{0};
  std::vector<std::thread> others;
  for (int t = 0; t < 3; ++t) {
    others.emplace_back([&, t] {
      uint64_t n = 0;
      amem_region_info info;
      amem_counters c;
      amem_cycle_stats st;
      while (!stop.load()) {
        const uint64_t va = 0x7d0000000000ull + ((uint64_t)t << 36) + (n % 64) * 4 * MiB;
        // a hook call from a communication library's own thread: refused while paused, accepted otherwise
        const int rc = amem_add_alloc_info(va, 2 * MiB, AMEM_TYPE_LOCAL, 0, 0x900000 + n, -1, 0, nullptr, t);
        EXPECT(rc == 0 || rc == 1);
        if (rc == 0) EXPECT(amem_del_alloc_info(va, 0x900000 + n, 0) == 0);
        (void)amem_check_paused(0);
        (void)amem_region_count(0);
        (void)amem_region_at(0, (int64_t)(n % 40), &info);
        (void)amem_handle_lookup(0, regs[n % regs.size()].handle);
        amem_get_counters(&c);
        amem_get_cycle_stats(&st);
        ++n;
        calls++;
        if ((n & 15) == 0) std::this_thread::yield();
      }
    });
  }
  std::vector<uint8_t> back;
  for (int cycle = 0; cycle < 6; ++cycle) {
    EXPECT(amem_set_option("pause_path", cycle % 3 == 2 ? 1 : 2) == 0);   // the staged path now and then
    // (1 = invalid value: the pause caught one of the other threads' made-up regions between its add and
    // its delete, reported it as not being mapped memory, left it alone and paused everything else)
    const int rc = amem_mem_pause(0, 0);
    EXPECT(rc == 0 || rc == 1);
    EXPECT(amem_check_paused(0) == 1);
    EXPECT(amem_mem_resume(0, 0) == 0);
    amem_cycle_stats st;
    amem_get_cycle_stats(&st);
    EXPECT(st.verify_mismatch == 0);
    for (const Reg& r : regs) {
      back.assign(r.size, 0xEE);
      EXPECT(amem_copy_from_device(back.data(), r.va, r.size) == 0);
      EXPECT(memcmp(back.data(), r.data.data(), r.size) == 0);
    }
    for (const Imp& m : imports) {
      back.assign(m.size, 0xEE);
      EXPECT(amem_copy_from_device(back.data(), m.va, m.size) == 0);
      EXPECT(memcmp(back.data(), regs[m.of].data.data(), m.size) == 0);
    }
  }
  stop.store(true);
  for (auto& t : others) t.join();
  amem_counters c;
  amem_get_counters(&c);
  EXPECT(c.offload_cnt == 0 && c.release_local_cnt == 0 && c.release_shadow_cnt == 0 && c.paused == 0);
  EXPECT(c.pause_cnt == 6 && c.resume_cnt == 6);
  for (const Imp& m : imports) { amem_del_alloc_info(m.va, 0, 0); EXPECT(amem_vmm_free(m.va, m.size, 0) == 0); }
  for (const Reg& r : regs) { amem_del_alloc_info(r.va, 0, 0); EXPECT(amem_vmm_free(r.va, r.size, 0) == 0); }
  EXPECT(amem_shutdown() == 0);
  printf("cycle driver done: %ld errors, %ld calls from the other threads\n", g_errors.load(), calls.load());
  return g_errors.load() ? 1 : 0;
}
