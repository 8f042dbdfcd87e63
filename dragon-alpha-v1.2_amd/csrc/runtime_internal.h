// Shared by the translation units of the runtime bridge.
#pragma once
#include <hip/hip_runtime.h>

namespace dragon_rt {
// remembers a failure for getLastExceptionType and returns the code as int
int note(hipError_t e);
}  // namespace dragon_rt
