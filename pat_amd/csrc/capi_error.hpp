// Thread-local error message shared by the C entry points.
#pragma once
#include <string>

namespace pat {
extern thread_local std::string g_last_error;
// Records msg as the calling thread's last error and returns code.
int fail(int code, const std::string& msg);
}  // namespace pat
