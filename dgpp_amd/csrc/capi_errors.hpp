// Error reporting shared by the translation units behind the C ABI: both record the message that
// dgpp_last_error() returns (thread-local) and give back the status code to return.
#pragma once
#include <hip/hip_runtime.h>

#include <string>

namespace dgpp_amd {
// DGPP_INVALID_ARGUMENT, the counterpart of the reference launchers' std::invalid_argument.
int report_invalid(const std::string& what);
// DGPP_OK for hipSuccess; else DGPP_RUNTIME_ERROR with the runtime's message, and the sticky error drained.
int report_hip(hipError_t err, const char* who);
}  // namespace dgpp_amd
