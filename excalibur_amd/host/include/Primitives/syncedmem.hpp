// Host/device mirror of one buffer with lazy synchronisation, the reference's syncedmem
// (include/Primitives/syncedmem.hpp, src/Primitives/syncedmem.cpp:100-276): UNINITIALIZED ->
// HEAD_AT_CPU / HEAD_AT_GPU -> SYNCED; first touch zero-fills; cpu_data()/gpu_data() copy across when the
// other side holds the newer bytes. The device side is HIP memory obtained through exhip.
#pragma once
#include <cstddef>

#include "device.hpp"

namespace glasssix {
namespace memory {

template <typename Dtype>
class pool_allocator;  // kept for signature compatibility with the reference's tensor constructors; unused

template <typename Dtype>
class syncedmem {
public:
    enum SyncedHead { UNINITIALIZED, HEAD_AT_CPU, HEAD_AT_GPU, SYNCED };

    explicit syncedmem(size_t size = 0, int device = -1);
    ~syncedmem();

    SyncedHead head() const { return head_; }
    size_t size() const { return size_; }
    // counts the mutable_*_data() calls: a holder that remembers the value can tell whether the bytes may have changed since
    unsigned long long writes() const { return writes_; }
    void set_allocator(pool_allocator<Dtype>*) {}
    const Dtype* cpu_data();
    const Dtype* gpu_data();
    Dtype* mutable_cpu_data();
    Dtype* mutable_gpu_data();

private:
    void to_cpu();
    void to_gpu(bool will_overwrite);
    Dtype* cpu_ptr_ = nullptr;
    Dtype* gpu_ptr_ = nullptr;
    size_t size_;
    SyncedHead head_ = UNINITIALIZED;
    unsigned long long writes_ = 0;
    int device_;
    int slot_;  // stream slot whose block cache gpu_ptr_ came from
    DISABLE_COPY_AND_ASSIGN(syncedmem);
};

}  // namespace memory
}  // namespace glasssix
