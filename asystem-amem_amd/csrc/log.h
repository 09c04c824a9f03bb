// Logging in the reference's line format so existing log scrapers keep working:
//   "AMEM [INFO] file:function:line message"  (amem_nccl_plugin/gmm_util.h:157-195),
// level from GMM_LOG, 0 (fatal) .. 5 (verbose), default 3 (gmm_util.h:146-153).
#ifndef AMEM_LOG_H_
#define AMEM_LOG_H_

#include <stdio.h>

namespace amem {

enum LogLevel { FATAL = 0, ERROR = 1, WARN = 2, INFO = 3, DEBUG = 4, VERBOSE = 5 };

int log_level();
void set_log_level_from_env();
void log_line(int level, const char* file, const char* func, int line, const char* fmt, ...)
    __attribute__((format(printf, 5, 6)));
// Prints the caller's stack the way the reference's gtrace() does (gmm_util.h:47-59).
void log_backtrace();

}  // namespace amem

#define LOGGER(level, ...)                                                              \
  do {                                                                                  \
    if ((int)(amem::level) <= amem::log_level())                                        \
      amem::log_line((int)(amem::level), __FILE__, __FUNCTION__, __LINE__, __VA_ARGS__); \
  } while (0)

#endif
