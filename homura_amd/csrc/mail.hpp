// The device side of a context's mailbox (see hmr_context in common.hpp): a kernel whose result the caller reads
// back at once - a check's verdict, a count - stores it in pinned host memory as well, and its launch's ticket
// after it.
#pragma once

#include <cstdint>

#include <hip/hip_runtime.h>

namespace hmr {

// Two words and then the ticket, release-ordered at system scope: a host thread that sees the ticket sees the words.
__device__ __forceinline__ void post(uint64_t *mailbox, uint64_t ticket, uint64_t first, uint64_t second) {
    __hip_atomic_store(&mailbox[0], first, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __hip_atomic_store(&mailbox[1], second, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    __hip_atomic_store(&mailbox[2], ticket, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

}  // namespace hmr
