// Four-dimensional blob in NCHW or NHWC order, dense, the reference's memory::tensor
// (include/Primitives/tensor.hpp:21-173): shape of four ints, shared syncedmem, device ordinal
// (-1 = host only). Same constructors and accessors, so operator code written against the reference
// compiles against this header.
#pragma once
#include <memory>
#include <vector>

#include "syncedmem.hpp"

namespace glasssix {
namespace memory {

enum orderType { NCHW, NHWC };

template <typename Dtype>
class tensor {
public:
    explicit tensor(orderType order = NCHW, pool_allocator<Dtype>* allocator = nullptr);
    explicit tensor(const int w, int device = -1, orderType order = NCHW, pool_allocator<Dtype>* allocator = nullptr);
    explicit tensor(const int h, const int w, int device = -1, orderType order = NCHW, pool_allocator<Dtype>* allocator = nullptr);
    explicit tensor(const int c, const int h, const int w, int device = -1, orderType order = NCHW,
                    pool_allocator<Dtype>* allocator = nullptr);
    explicit tensor(const std::vector<int>& shape, int device = -1, orderType order = NCHW,
                    pool_allocator<Dtype>* allocator = nullptr);

    bool empty() const { return data_ == nullptr || count() == 0; }
    const Dtype* cpu_data() const { return data_->cpu_data(); }
    const Dtype* gpu_data() const { return data_->gpu_data(); }
    Dtype* mutable_cpu_data() const { return data_->mutable_cpu_data(); }
    Dtype* mutable_gpu_data() const { return data_->mutable_gpu_data(); }
    unsigned long long writes() const { return data_->writes(); }  // mutable_*_data() calls so far
    void copy_from(const void* data, size_t size);

    int num() const { return shape_[0]; }
    int channels() const { return order_ == NCHW ? shape_[1] : shape_[3]; }
    int height() const { return order_ == NCHW ? shape_[2] : shape_[1]; }
    int width() const { return order_ == NCHW ? shape_[3] : shape_[2]; }
    int count(int start_axis, int end_axis) const {
        int c = 1;
        for (int i = start_axis; i < end_axis; ++i) c *= shape_[i];
        return c;
    }
    int count() const { return count(0, static_cast<int>(shape_.size())); }
    int device() const { return device_; }
    orderType order() const { return order_; }
    int offset(const int n, const int c = 0, const int h = 0, const int w = 0) const {
        return order_ == NCHW ? ((n * channels() + c) * height() + h) * width() + w
                              : ((n * height() + h) * width() + w) * channels() + c;
    }
    std::vector<int> data_shape() const { return shape_; }
    void reshape(std::vector<int> data_shape) { shape_ = data_shape; }
    pool_allocator<Dtype>* allocator() const { return nullptr; }

    // An int8 NHWC copy of this blob, q8(x * scale) with `stride` channels per pixel (pad channels zero), written by the
    // layer that produced the blob beside its float data, or instead of it (`only`: the float data was never written).
    // An int8 convolution that reads the blob with that scale and stride takes the copy in place of running its
    // quantizer. The pipeline sets this up and is the only one to hand out `only` blobs, to such readers alone.
    struct quantized_copy {
        std::shared_ptr<tensor<signed char>> data;
        float scale = 0.f;
        int stride = 0;
        bool only = false;
    };
    std::shared_ptr<quantized_copy> quantized;

private:
    void init(const std::vector<int>& shape, int device);
    std::shared_ptr<syncedmem<Dtype>> data_;
    std::vector<int> shape_;
    int device_ = -1;
    orderType order_;
};

}  // namespace memory
}  // namespace glasssix
