// Process-wide access to the exhip contexts (one per HIP device ordinal) used by tensors and operators.
#pragma once
#include "../../../../include/exhip.h"
#include "logger.hpp"

namespace glasssix {
namespace memory {
// Context of `device` (created on first use); FATAL if the device cannot be opened.
exhip_ctx* device_context(int device);
// Size-bucketed cache of device allocations: operators allocate their outputs on every call, as in the
// reference (src/Excalibur/operation_convolution.cpp:277); blocks are recycled instead of hipMalloc'ed.
void* device_alloc(int device, size_t bytes);
void device_release(int device, void* ptr, size_t bytes);
}  // namespace memory
}  // namespace glasssix

#define EXHIP_FATAL(call)                                                             \
    do {                                                                              \
        int rc_ = (call);                                                             \
        if (rc_ != 0) LOG(FATAL) << #call << " failed (" << rc_ << "): " << exhip_last_error(); \
    } while (0)
