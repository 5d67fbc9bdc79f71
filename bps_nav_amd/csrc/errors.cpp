#include "errors.h"

#include "../../include/bpsx.h"

namespace bpsx {
namespace {
thread_local std::string g_last_error;
}
int fail(int code, const std::string& msg) {
  g_last_error = msg;
  return code;
}
const char* last_error_message() { return g_last_error.c_str(); }
}  // namespace bpsx

extern "C" const char* bpsx_last_error(void) { return bpsx::last_error_message(); }
