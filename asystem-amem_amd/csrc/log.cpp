#include "log.h"

#include <execinfo.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <mutex>

namespace amem {

static std::atomic<int> g_level{INFO};
static std::mutex g_log_mtx;

int log_level() { return g_level.load(std::memory_order_relaxed); }

void set_log_level_from_env() {
  const char* e = getenv("GMM_LOG");
  int lv = e ? atoi(e) : (int)INFO;
  if (lv >= FATAL && lv <= VERBOSE) g_level.store(lv);
}

void log_line(int level, const char* file, const char* func, int line, const char* fmt, ...) {
  static const char* tag[] = {"[FATAL]", "[ERRO]", "[WARN]", "[INFO]", "[DEBG]", "[VERB]"};
  const char* base = strrchr(file, '/');
  base = base ? base + 1 : file;
  char msg[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(msg, sizeof(msg), fmt, ap);
  va_end(ap);
  std::lock_guard<std::mutex> lk(g_log_mtx);
  fprintf(stdout, "AMEM %s %s:%s:%d %s\n", tag[level], base, func, line, msg);
  if (level <= WARN) fflush(stdout);
}

// The call stack of the caller, in the layout of the reference's gtrace() (gmm_util.h:47-59).
void log_backtrace() {
  void* frames[96];
  const int n = backtrace(frames, 96);
  char** names = backtrace_symbols(frames, n);
  if (!names) return;
  std::lock_guard<std::mutex> lk(g_log_mtx);
  printf("------------------\n");
  for (int i = 0; i < n; ++i) printf("[%d] %s\n", i, names[i]);
  printf("------------------\n");
  fflush(stdout);
  free(names);
}

}  // namespace amem
