// Error text of the last failed call on this thread, for the Python side.
#include <cstdarg>

#include "common.h"

namespace lyp {
static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace lyp

extern "C" const char* lyp_last_error() { return lyp::g_error; }

// Which GPU architecture the code object was built for; lets the loader refuse
// a library that cannot run here before the first kernel is launched.
extern "C" const char* lyp_built_for() { return "gfx950"; }
