// Wait kernel: holds a stream back until a device-side semaphore reaches a value.
// Same entry point as src/include/cusync/wait-kernel.h:10 of the reference; the
// kernel itself lives in the library (cusync_wait_kernel in cusync_amd.h).
#pragma once

#include <stdint.h>
#include "../cusync_amd.h"

namespace cusync {
inline void invokeWaitKernel(uint32_t* semaphore, uint32_t givenValue, void* stream) {
  cusync_wait_kernel(semaphore, givenValue, stream);
}
}  // namespace cusync
