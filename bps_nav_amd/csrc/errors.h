// Error reporting shared by the host-side translation units of libbpsx: functions
// return negative BPSX_E_* codes and leave a message for bpsx_last_error().
#pragma once
#include <string>

namespace bpsx {
int fail(int code, const std::string& msg);  // records msg, returns code
const char* last_error_message();
}  // namespace bpsx
