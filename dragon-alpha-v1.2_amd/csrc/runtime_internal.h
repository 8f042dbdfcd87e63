// Shared by the translation units of the runtime bridge.
#pragma once
#include <hip/hip_runtime.h>

namespace dragon_rt {
// remembers a failure for getLastExceptionType and returns the code as int
int note(hipError_t e);
}  // namespace dragon_rt

namespace dragon {
// Device memory in [ptr, ptr + bytes) is about to be written (bytes == 0: from ptr to wherever its allocation
// ends, as when it is freed): a declined split-K call's partial buffer that overlaps it no longer counts as
// "known to hold zeros" (see the ledger in c_abi_gemm.hip).  Every entry point that writes device memory says
// so; costs one relaxed atomic load while no split has been declined.
void split_ledger_touch(const void* ptr, size_t bytes);
}  // namespace dragon
