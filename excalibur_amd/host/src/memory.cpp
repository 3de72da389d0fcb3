// syncedmem / tensor / device contexts (the reference's src/Primitives/{syncedmem,tensor}.cpp roles).
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <tuple>

#include "../include/Primitives/tensor.hpp"

namespace glasssix {
namespace memory {

namespace {
std::mutex g_mu;
thread_local int t_slot = 0;
std::map<std::pair<int, int>, exhip_ctx*> g_ctx;                       // (device, slot)
std::map<std::tuple<int, int, size_t>, std::vector<void*>> g_free;     // (device, slot, rounded bytes) -> idle blocks
std::map<int, size_t> g_idle_bytes;                                    // device -> bytes held idle in g_free
// Idle blocks are kept for reuse up to this many bytes per device; beyond it a released block goes back to the driver, so
// a pipeline fed many different resolutions does not grow without bound.
constexpr size_t kIdleLimit = (size_t)8 << 30;

size_t round_block(size_t bytes) {
    size_t b = 256;
    while (b < bytes) b <<= 1;
    // above 1 MiB round to 1/8 of the power of two instead, to bound the slack
    if (b > (1u << 20)) {
        const size_t step = b >> 4;
        b = (bytes + step - 1) / step * step;
    }
    return b;
}
}  // namespace

int stream_slot() { return t_slot; }

void set_stream_slot(int slot) {
    if (slot < 0 || slot >= kMaxStreamSlots) LOG(FATAL) << "stream slot " << slot << " outside 0.." << kMaxStreamSlots - 1;
    t_slot = slot;
}

exhip_ctx* device_context(int device) { return device_context(device, t_slot); }

exhip_ctx* device_context(int device, int slot) {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_ctx.find({device, slot});
    if (it != g_ctx.end()) return it->second;
    exhip_ctx* ctx = nullptr;
    int rc = exhip_init(device, &ctx);
    if (rc != 0) LOG(FATAL) << "cannot open HIP device " << device << ": " << exhip_last_error();
    g_ctx[{device, slot}] = ctx;
    return ctx;
}

// Returns every idle block of a device to the driver, each through its own slot's context (exhip_free waits for that
// slot's stream first, behind which the block's last user is queued).
static void trim_idle(int device) {
    std::vector<std::pair<int, void*>> blocks;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        for (auto& kv : g_free)
            if (std::get<0>(kv.first) == device) {
                for (void* b : kv.second) blocks.push_back({std::get<1>(kv.first), b});
                kv.second.clear();
            }
        g_idle_bytes[device] = 0;
    }
    for (auto& b : blocks) exhip_free(device_context(device, b.first), b.second);
}

void* device_alloc(int device, size_t bytes) { return device_alloc(device, t_slot, bytes); }
void device_release(int device, void* ptr, size_t bytes) { device_release(device, t_slot, ptr, bytes); }

void* device_alloc(int device, int slot, size_t bytes) {
    exhip_ctx* ctx = device_context(device, slot);
    const size_t rb = round_block(bytes);
    {
        std::lock_guard<std::mutex> lock(g_mu);
        auto& pool = g_free[{device, slot, rb}];
        if (!pool.empty()) {
            void* p = pool.back();
            pool.pop_back();
            g_idle_bytes[device] -= rb;
            return p;
        }
    }
    void* p = nullptr;
    if (exhip_malloc(ctx, rb, &p) != 0) {  // out of device memory: give the idle blocks back and try once more
        trim_idle(device);
        EXHIP_FATAL(exhip_malloc(ctx, rb, &p));
    }
    return p;
}

void device_release(int device, int slot, void* ptr, size_t bytes) {
    if (!ptr) return;
    const size_t rb = round_block(bytes);
    {
        std::lock_guard<std::mutex> lock(g_mu);
        if (g_idle_bytes[device] + rb <= kIdleLimit) {
            g_free[{device, slot, rb}].push_back(ptr);
            g_idle_bytes[device] += rb;
            return;
        }
    }
    exhip_free(device_context(device, slot), ptr);  // over the limit: back to the driver (waits for the slot's stream)
}

template <typename Dtype>
syncedmem<Dtype>::syncedmem(size_t size, int device) : size_(size), device_(device), slot_(stream_slot()) {}

template <typename Dtype>
syncedmem<Dtype>::~syncedmem() {
    if (cpu_ptr_) std::free(cpu_ptr_);
    // Kernels using this buffer may still be queued, and that is fine: every device operation of a slot (kernels,
    // copies, fills) goes through that slot's one stream, and the block returns to the cache of the slot it was taken
    // from, so whatever touches the recycled block is queued behind them.
    if (gpu_ptr_) device_release(device_, slot_, gpu_ptr_, size_ * sizeof(Dtype));
}

template <typename Dtype>
void syncedmem<Dtype>::to_cpu() {
    const size_t bytes = size_ * sizeof(Dtype);
    switch (head_) {
    case UNINITIALIZED:
        cpu_ptr_ = static_cast<Dtype*>(std::aligned_alloc(64, (bytes + 63) / 64 * 64 + 64));
        std::memset(cpu_ptr_, 0, bytes);
        head_ = HEAD_AT_CPU;
        break;
    case HEAD_AT_GPU:
        if (!cpu_ptr_) cpu_ptr_ = static_cast<Dtype*>(std::aligned_alloc(64, (bytes + 63) / 64 * 64 + 64));
        // synchronises the stream of the slot the block was taken in (a pipeline's outputs: the pipeline's); a reader working
        // in another slot may have queued the writer there, so that stream is drained as well
        if (stream_slot() != slot_) EXHIP_FATAL(exhip_sync(device_context(device_)));
        EXHIP_FATAL(exhip_memcpy_d2h(device_context(device_, slot_), cpu_ptr_, gpu_ptr_, bytes));
        head_ = SYNCED;
        break;
    default: break;
    }
}

// will_overwrite: the caller asks for the buffer to write all of it (mutable_gpu_data of a fresh blob, which is how every
// layer makes its output): the zero fill the reference gives a fresh blob is then skipped. Reading a blob nobody wrote
// (gpu_data first) still yields zeros.
template <typename Dtype>
void syncedmem<Dtype>::to_gpu(bool will_overwrite) {
    if (device_ < 0) LOG(FATAL) << "gpu_data() on a tensor created without a device";
    const size_t bytes = size_ * sizeof(Dtype);
    exhip_ctx* ctx = device_context(device_);
    switch (head_) {
    case UNINITIALIZED:
        slot_ = stream_slot();  // the block comes from, is first used in, and returns to the slot of this call
        gpu_ptr_ = static_cast<Dtype*>(device_alloc(device_, bytes));
        if (!will_overwrite) EXHIP_FATAL(exhip_memset(ctx, gpu_ptr_, 0, bytes));
        head_ = HEAD_AT_GPU;
        break;
    case HEAD_AT_CPU:
        if (!gpu_ptr_) {
            slot_ = stream_slot();
            gpu_ptr_ = static_cast<Dtype*>(device_alloc(device_, bytes));
        }
        EXHIP_FATAL(exhip_memcpy_h2d(ctx, gpu_ptr_, cpu_ptr_, bytes));
        head_ = SYNCED;
        break;
    default: break;
    }
}

template <typename Dtype>
const Dtype* syncedmem<Dtype>::cpu_data() { to_cpu(); return cpu_ptr_; }
template <typename Dtype>
const Dtype* syncedmem<Dtype>::gpu_data() { to_gpu(false); return gpu_ptr_; }
template <typename Dtype>
Dtype* syncedmem<Dtype>::mutable_cpu_data() { to_cpu(); head_ = HEAD_AT_CPU; ++writes_; return cpu_ptr_; }
template <typename Dtype>
Dtype* syncedmem<Dtype>::mutable_gpu_data() { to_gpu(true); head_ = HEAD_AT_GPU; ++writes_; return gpu_ptr_; }

template <typename Dtype>
void tensor<Dtype>::init(const std::vector<int>& shape, int device) {
    shape_ = shape;
    device_ = device;
    data_ = std::make_shared<syncedmem<Dtype>>(static_cast<size_t>(count()), device);
}
template <typename Dtype>
tensor<Dtype>::tensor(orderType order, pool_allocator<Dtype>*) : order_(order) { init({0, 0, 0, 0}, -1); }
template <typename Dtype>
tensor<Dtype>::tensor(const int w, int device, orderType order, pool_allocator<Dtype>*) : order_(order) {
    init(order == NCHW ? std::vector<int>{1, 1, 1, w} : std::vector<int>{1, 1, w, 1}, device);
}
template <typename Dtype>
tensor<Dtype>::tensor(const int h, const int w, int device, orderType order, pool_allocator<Dtype>*) : order_(order) {
    init(order == NCHW ? std::vector<int>{1, 1, h, w} : std::vector<int>{1, h, w, 1}, device);
}
template <typename Dtype>
tensor<Dtype>::tensor(const int c, const int h, const int w, int device, orderType order, pool_allocator<Dtype>*) : order_(order) {
    init(order == NCHW ? std::vector<int>{1, c, h, w} : std::vector<int>{1, h, w, c}, device);
}
template <typename Dtype>
tensor<Dtype>::tensor(const std::vector<int>& shape, int device, orderType order, pool_allocator<Dtype>*) : order_(order) {
    std::vector<int> s = shape;
    while (s.size() < 4) s.insert(s.begin(), 1);
    init(s, device);
}
template <typename Dtype>
void tensor<Dtype>::copy_from(const void* data, size_t size) {
    CHECK_LE(size, static_cast<size_t>(count()) * sizeof(Dtype));
    std::memcpy(mutable_cpu_data(), data, size);
}

#define INSTANTIATE_MEMORY(T) \
    template class syncedmem<T>; \
    template class tensor<T>;
INSTANTIATE_MEMORY(float)
INSTANTIATE_MEMORY(double)
INSTANTIATE_MEMORY(int)
INSTANTIATE_MEMORY(signed char)
INSTANTIATE_MEMORY(unsigned char)
INSTANTIATE_MEMORY(unsigned short)

}  // namespace memory
}  // namespace glasssix
