#include "log.h"

#include <stdarg.h>
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

}  // namespace amem
