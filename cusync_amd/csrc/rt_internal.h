// Shared between the translation units of libcusync_amd.so; not installed.
#pragma once

#include <hip/hip_runtime.h>
#include <string>

namespace cusync {
namespace rt {
// Records `msg` as the text cusync_rt_last_error() returns (per host thread).
void setError(const std::string& msg);
// Returns 0 on hipSuccess; otherwise records a message and returns the code.
int check(hipError_t e, const char* what, const char* file, int line);
}  // namespace rt
}  // namespace cusync

#define CUSYNC_HIP(call) ::cusync::rt::check((call), #call, __FILE__, __LINE__)
