// Process-wide access to the exhip contexts (one per HIP device ordinal and stream slot) used by tensors and operators.
#pragma once
#include "../../../../include/exhip.h"
#include "logger.hpp"

namespace glasssix {
namespace memory {
// Stream slots. Every thread works in one slot at a time (0 unless it says otherwise); a slot has its own exhip context
// = HIP stream per device and its own cache of idle device blocks, so work issued in different slots may overlap on the
// GPU (two pipelines with a batch each in flight fill the launches' tails and the gaps between launches), while inside a
// slot everything stays ordered by the one stream, which is what lets a released block be reused without a wait.
// A pipeline belongs to the slot its constructing thread was in and does all its device work there, whichever thread
// calls it. Host <-> device copies of a tensor are synchronous, so a tensor filled in one slot may be read in another;
// what must not happen is freeing a tensor while another slot's queued kernels still use it: synchronise that slot first.
constexpr int kMaxStreamSlots = 8;
int stream_slot();
void set_stream_slot(int slot);
struct stream_scope {
    explicit stream_scope(int slot) : prev_(stream_slot()) { set_stream_slot(slot); }
    ~stream_scope() { set_stream_slot(prev_); }
    stream_scope(const stream_scope&) = delete;
    stream_scope& operator=(const stream_scope&) = delete;

private:
    int prev_;
};
// Context of `device` in the calling thread's slot (created on first use); FATAL if the device cannot be opened.
exhip_ctx* device_context(int device);
exhip_ctx* device_context(int device, int slot);
// Size-bucketed cache of device allocations: operators allocate their outputs on every call, as in the
// reference (src/Excalibur/operation_convolution.cpp:277); blocks are recycled instead of hipMalloc'ed. A block
// is taken from and returned to the cache of one slot: the calling thread's, or the one named.
void* device_alloc(int device, size_t bytes);
void device_release(int device, void* ptr, size_t bytes);
void* device_alloc(int device, int slot, size_t bytes);
void device_release(int device, int slot, void* ptr, size_t bytes);
}  // namespace memory
}  // namespace glasssix

#define EXHIP_FATAL(call)                                                             \
    do {                                                                              \
        int rc_ = (call);                                                             \
        if (rc_ != 0) LOG(FATAL) << #call << " failed (" << rc_ << "): " << exhip_last_error(); \
    } while (0)
