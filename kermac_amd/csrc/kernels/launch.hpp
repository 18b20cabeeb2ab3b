// Kernel launch that reports its own status.  The <<<>>> form followed by
// hipGetLastError() returns, and clears, whatever error an earlier call on this
// thread left behind (another library's, for instance), which would then be blamed
// on this launch or lost to its owner; hipLaunchKernel returns the result of this
// launch alone and leaves the thread's error state as it found it.
#pragma once

#include <hip/hip_runtime.h>

namespace kmc_host {

template <typename Args>
inline hipError_t launch(void (*kernel)(const Args), dim3 grid, dim3 block, hipStream_t stream, const Args &args)
{
    void *kernel_args[] = {const_cast<Args *>(&args)};
    return hipLaunchKernel(reinterpret_cast<const void *>(kernel), grid, block, kernel_args, 0, stream);
}

}  // namespace kmc_host
