// Library-level entry points of libpla_gfx950.so.
#include "common.h"

namespace pla {
char* error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}
}  // namespace pla

extern "C" const char* pla_version(void) { return "pla_gfx950 0.1 gfx950"; }
extern "C" const char* pla_last_error(void) { return pla::error_buffer(); }
