// The operators of the CNN forward hot path, under the reference's class names so that an unmodified
// topology resolves to them through the registry: operation_convolution (on operation_general_conv),
// operation_convolutiondepthwise, operation_pooling, operation_eltwise, operation_binaryop, operation_relu,
// operation_innerproduct, operation_split. Each overrides the forward_gpu_* virtuals and calls the exhip C ABI.
#pragma once
#include <map>

#include "operation.hpp"

namespace glasssix {
namespace excalibur {

// Convolution hyper-parameters as parsed by the reference (src/Excalibur/operation_general_conv.cpp:9-124),
// member names kept.
template <typename Dtype>
class operation_general_conv : public operation<Dtype> {
public:
    explicit operation_general_conv(const operation_param& param);
    const char* type() const override { return this->params_.type_.c_str(); }

    int output_channel_ = 0;
    int kernel_size_w_ = 0, kernel_size_h_ = 0;
    int dilation_w_ = 1, dilation_h_ = 1;
    int stride_w_ = 1, stride_h_ = 1;
    int group_ = 1;
    int pad_left_ = 0, pad_right_ = 0, pad_top_ = 0, pad_bottom_ = 0;
    bool int8_scale_term_ = false;
    bool bias_term_ = false;
    int weight_data_size_ = 0;
    int activation_type_ = 0;
    int impl_type_ = 0;
    int output_pad_right_ = 0, output_pad_bottom_ = 0, output_dim_h_ = 0, output_dim_w_ = 0;
    int input_channels() const { return weight_data_size_ * group_ / output_channel_ / kernel_size_h_ / kernel_size_w_; }
};

template <typename Dtype>
class operation_convolution : public operation_general_conv<Dtype> {
public:
    template <typename T>
    using tensor_list = typename operation<Dtype>::template tensor_list<T>;
    explicit operation_convolution(const operation_param& param);
    ~operation_convolution() override;
    int init_weights() override;
    int init_weights(FILE* fp) override;

    // Dequantization scale per output channel, fabs(ws) <= 1e-6 ? 0 : 1.0f / (ws * fs), computed on the
    // host in float exactly as src/Excalibur/operation_convolution.cpp:400-403.
    std::vector<float> dequantize_scales() const;
    float featmap_scale() const;
    // device copies (created on first use)
    const float* bias_gpu();
    const float* scale_gpu();
    // weights packed for the MFMA kernel for one input geometry; cached per (dtype, n, h, w, c_stride)
    const void* packed_weights(int dtype, const exhip_conv_desc& d);
    exhip_conv_desc describe(int n, int h, int w, int c_stride, int k_stride) const;

protected:
    void forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_i8(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) override;
    bool mfma_path_ok() const;

private:
    struct packed_entry { void* ptr; size_t bytes; };
    std::map<std::vector<int>, packed_entry> packed_;
    std::shared_ptr<memory::tensor<float>> scale_dev_;
};

template <typename Dtype>
class operation_convolutiondepthwise : public operation_convolution<Dtype> {
public:
    template <typename T>
    using tensor_list = typename operation<Dtype>::template tensor_list<T>;
    explicit operation_convolutiondepthwise(const operation_param& param) : operation_convolution<Dtype>(param) {}

protected:
    void forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_i8(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) override;
    bool fast3x3() const;
};

template <typename Dtype>
class operation_pooling : public operation<Dtype> {
public:
    template <typename T>
    using tensor_list = typename operation<Dtype>::template tensor_list<T>;
    explicit operation_pooling(const operation_param& param);
    const char* type() const override { return this->params_.type_.c_str(); }

    int kernel_size_w_ = 0, kernel_size_h_ = 0, stride_w_ = 1, stride_h_ = 1;
    int pad_left_ = 0, pad_right_ = 0, pad_top_ = 0, pad_bottom_ = 0;
    int type_ = 0;  // 0 MAX, 1 AVE
    bool global_pooling_ = false;
    int pad_mode_ = 1;  // 0 ceil, 1 floor
    int avgpool_count_include_pad_ = 0;
    // effective window for an input of h x w (global pooling overrides kernel, stride and padding)
    void geometry(int h, int w, int* kh, int* kw, int* sh, int* sw, int* pt, int* pb, int* pl, int* pr, int* oh, int* ow) const;

protected:
    void forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) override;
};

template <typename Dtype>
class operation_eltwise : public operation<Dtype> {
public:
    template <typename T>
    using tensor_list = typename operation<Dtype>::template tensor_list<T>;
    explicit operation_eltwise(const operation_param& param);
    const char* type() const override { return this->params_.type_.c_str(); }
    enum eltwise_type { PROD = 0, SUM = 1, MAX = 2 };
    int type_ = SUM;
    std::vector<float> coeffs_;

protected:
    void forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) override;
};

template <typename Dtype>
class operation_binaryop : public operation<Dtype> {
public:
    template <typename T>
    using tensor_list = typename operation<Dtype>::template tensor_list<T>;
    explicit operation_binaryop(const operation_param& param);
    const char* type() const override { return this->params_.type_.c_str(); }
    int op_type_ = 0;  // 0 ADD (the only one on the hot path)
    int with_scalar_ = 0;
    float coef_ = 0.f;

protected:
    void forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) override;
};

template <typename Dtype>
class operation_relu : public operation<Dtype> {
public:
    template <typename T>
    using tensor_list = typename operation<Dtype>::template tensor_list<T>;
    explicit operation_relu(const operation_param& param);
    const char* type() const override { return this->params_.type_.c_str(); }
    float slope_ = 0.f;  // parsed and ignored, as in the reference (src/Excalibur/operation_relu.cpp:14-17)

protected:
    void forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) override;
};

template <typename Dtype>
class operation_split : public operation<Dtype> {
public:
    template <typename T>
    using tensor_list = typename operation<Dtype>::template tensor_list<T>;
    explicit operation_split(const operation_param& param) : operation<Dtype>(param) {}
    const char* type() const override { return this->params_.type_.c_str(); }

protected:
    void forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) override;
};

template <typename Dtype>
class operation_innerproduct : public operation<Dtype> {
public:
    template <typename T>
    using tensor_list = typename operation<Dtype>::template tensor_list<T>;
    explicit operation_innerproduct(const operation_param& param);
    const char* type() const override { return this->params_.type_.c_str(); }
    int init_weights() override;
    int init_weights(FILE* fp) override;
    int num_output_ = 0;
    bool bias_term_ = false;
    int weight_data_size_ = 0;
    bool int8_scale_term_ = false;
    int activation_type_ = 0;  // parsed, never applied (as in the reference)

protected:
    void forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) override;
    void forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) override;
};

}  // namespace excalibur
}  // namespace glasssix
