// Operator base class and parameter record with the reference's interface
// (include/Excalibur/operation.hpp:27-374): init_weights() / init_weights(FILE*), non-virtual
// forward_cpu / forward_gpu dispatching on the int8 flag to protected virtuals
// forward_{cpu,gpu}_{f32,f16,i8}. The GPU virtuals use the reference's non-CUDA signature (no library
// handle argument, :172-183,268-276,359-370): the stream lives in the device context.
// This backend has no CPU computation: forward_cpu is fatal.
#pragma once
#include <cstdio>
#include <memory>
#include <string>
#include <vector>

#include "../Primitives/tensor.hpp"

namespace glasssix {
namespace excalibur {

struct operation_param {
    std::string type_ = "N/A";      // layer type as written in the topology, e.g. Convolution
    std::string name_ = "N/A";      // unique layer name
    int input_count_ = 1;
    int output_count_ = 1;
    std::vector<std::string> input_featmaps_;
    std::vector<std::string> output_featmaps_;
    bool int8_quantization_ = false;
    bool brain_float16_ = false;
    bool float16_ = false;
    bool inplace_ = false;
    int device_ = -1;
    std::string specific_params_;   // "key=value key=value ..."

    void set_int8_quantization(bool v) { int8_quantization_ = v; }
    void set_brain_float16(bool v) { brain_float16_ = v; }
    void set_float16(bool v) { float16_ = v; }
};

// "a b  c" -> {"a","b","","c"} exactly like the reference helper (operation.hpp:91-107): empty fields between
// adjacent separators are kept, a trailing separator adds none.
std::vector<std::string> split_string(const std::string& s, const std::string& c);

// Test switch of this backend (process-wide): the fp16 pipeline keeps blobs NHWC between the layers whose kernels work on
// that layout; `true` keeps every blob NCHW as in the reference.
void set_f16_nchw_only(bool on);

// key=value attributes of a layer line, in order of appearance
struct layer_attr {
    std::string key;
    std::string value;
    int as_int() const { return std::atoi(value.c_str()); }
    float as_float() const { return static_cast<float>(std::atof(value.c_str())); }
};
std::vector<layer_attr> parse_attrs(const std::string& specific_params);

template <typename Dtype>
class operation {
public:
    template <typename T>
    using tensor_list = std::vector<std::shared_ptr<memory::tensor<T>>>;

    operation() {}
    explicit operation(const operation_param& param);
    virtual ~operation() {}

    virtual int init_weights() { return 0; }           // dummy weights
    virtual int init_weights(FILE*) { return 0; }      // returns bytes consumed from the model file

    void forward_cpu(const tensor_list<Dtype>& bottoms, tensor_list<Dtype>& tops);
    void forward_gpu(const tensor_list<Dtype>& bottoms, tensor_list<Dtype>& tops);

    tensor_list<double>& weights_d64() { return weights_d64_; }
    tensor_list<float>& weights_f32() { return weights_f32_; }
    tensor_list<unsigned short>& weights_f16() { return weights_f16_; }
    tensor_list<signed char>& weights_i8() { return weights_i8_; }
    const operation_param& param() const { return params_; }
    virtual const char* type() const { return "Unknown Type"; }

protected:
    tensor_list<double> weights_d64_;   // declared as in the reference (include/Excalibur/operation.hpp:158); no layer of the path fills it
    tensor_list<float> weights_f32_;
    tensor_list<unsigned short> weights_f16_;
    tensor_list<signed char> weights_i8_;
    operation_param params_;
    std::shared_ptr<memory::tensor<float>> weights_scaletable_i8_;
    std::shared_ptr<memory::tensor<float>> featmap_scaletable_i8_;

    virtual void forward_cpu_f32(const tensor_list<float>&, tensor_list<float>&) { NO_CPU; }
    virtual void forward_cpu_f16(const tensor_list<unsigned short>&, tensor_list<unsigned short>&) { NO_CPU; }
    virtual void forward_cpu_i8(const tensor_list<float>&, tensor_list<float>&) { NO_CPU; }
    virtual void forward_gpu_f32(const tensor_list<float>&, tensor_list<float>&) { NOT_IMPLEMENTED; }
    // the reference's double-precision hooks (include/Excalibur/operation.hpp:185-201): NOT_IMPLEMENTED there and here
    virtual void forward_cpu_d64(const tensor_list<double>&, tensor_list<double>&) { NOT_IMPLEMENTED; }
    virtual void forward_gpu_d64(const tensor_list<double>&, tensor_list<double>&) { NOT_IMPLEMENTED; }
    // Default fp16 layer: the float32 operator on converted data, as the reference's CPU wrapper does
    // (include/Excalibur/operation.hpp:204-266): half -> float, forward_gpu_f32, float -> half.
    virtual void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops);
    virtual void forward_gpu_i8(const tensor_list<float>&, tensor_list<float>&) {
        NOT_IMPLEMENTED << " This function should be overrided in derived class";
    }

    exhip_ctx* ctx() const { return memory::device_context(params_.device_); }

private:
    DISABLE_COPY_AND_ASSIGN(operation);
};

}  // namespace excalibur
}  // namespace glasssix
