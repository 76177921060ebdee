// Error state and version of the C ABI.
#include <string>

#include "e3x_internal.h"

namespace e3x {

static thread_local std::string g_last_error;

int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}

}  // namespace e3x

extern "C" const char* e3x_last_error(void) { return e3x::g_last_error.c_str(); }
extern "C" int e3x_version(void) { return 100; }
