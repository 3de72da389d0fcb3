// Operator implementations: parameter parsing and weight loading as the reference does them, computation
// through the exhip C ABI on the operator's device. Tensors at this interface are the reference's dense NCHW
// blobs; the kernels' NHWC / int8 forms are produced and consumed inside each forward call.
#include "../include/Excalibur/operators.hpp"

#include <cstdlib>
#include <cmath>
#include <cstring>
#include <random>

#include "../include/Excalibur/operation_reflector.hpp"

namespace glasssix {
namespace excalibur {

using memory::tensor;

std::vector<std::string> split_string(const std::string& s, const std::string& c) {
    std::vector<std::string> out;
    size_t from = 0, at;
    while ((at = s.find(c, from)) != std::string::npos) {
        out.push_back(s.substr(from, at - from));
        from = at + c.size();
    }
    if (from != s.length()) out.push_back(s.substr(from));
    return out;
}

std::vector<layer_attr> parse_attrs(const std::string& specific_params) {
    std::vector<layer_attr> attrs;
    for (const std::string& tok : split_string(specific_params, " ")) {
        if (tok.empty()) continue;
        const size_t eq = tok.find('=');
        attrs.push_back({tok.substr(0, eq), eq == std::string::npos ? std::string() : tok.substr(eq + 1)});
    }
    return attrs;
}

template <typename Dtype>
operation<Dtype>::operation(const operation_param& param) : params_(param) {
    if (sizeof(Dtype) == 2) params_.set_float16(true);  // pipeline<unsigned short> is the fp16 pipeline (operation.cpp:13-16)
}

template <>
void operation<float>::forward_cpu(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    if (params_.int8_quantization_) forward_cpu_i8(bottoms, tops);
    else forward_cpu_f32(bottoms, tops);
}
template <>
void operation<float>::forward_gpu(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    if (params_.int8_quantization_) forward_gpu_i8(bottoms, tops);
    else forward_gpu_f32(bottoms, tops);
}
template <>
void operation<unsigned short>::forward_cpu(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    forward_cpu_f16(bottoms, tops);
}
template <>
void operation<unsigned short>::forward_gpu(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    forward_gpu_f16(bottoms, tops);
}
// pipeline<double>: the reference dispatches to forward_*_d64, which no operator of this path overrides
// (include/Excalibur/operation.hpp:185-201): NOT_IMPLEMENTED.
template <>
void operation<double>::forward_cpu(const tensor_list<double>&, tensor_list<double>&) { NO_CPU; }
template <>
void operation<double>::forward_gpu(const tensor_list<double>&, tensor_list<double>&) {
    NOT_IMPLEMENTED << " double-precision layers have no forward";
}
template class operation<float>;
template class operation<double>;
template class operation<unsigned short>;

namespace {

inline int pad_to(int v, int m) { return (v + m - 1) / m * m; }

template <typename T>
std::shared_ptr<tensor<T>> new_tensor(std::vector<int> shape, int device, memory::orderType order = memory::NCHW) {
    return std::make_shared<tensor<T>>(shape, device, order, nullptr);
}

// 1 x 1 x 1 x n vector blob (the reference's tensor(w, device, order, allocator) constructor)
template <typename T>
std::shared_ptr<tensor<T>> vec_tensor(int n, int device) {
    return std::make_shared<tensor<T>>(n, device, memory::NCHW, nullptr);
}

// float -> IEEE half bits, round to nearest even
unsigned short half_bits_rne(float f) {
    unsigned int u;
    std::memcpy(&u, &f, 4);
    const unsigned int sign = (u >> 16) & 0x8000u;
    unsigned int a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return static_cast<unsigned short>(sign | 0x7E00u);
    if (a >= 0x47800000u) return static_cast<unsigned short>(sign | 0x7C00u);
    if (a < 0x38800000u) {
        if (a < 0x33000000u) return static_cast<unsigned short>(sign);
        const int e = static_cast<int>(a >> 23);
        const unsigned int m = (a & 0x7FFFFFu) | 0x800000u;
        const int shift = 126 - e;
        unsigned int r = m >> shift;
        const unsigned int rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (r & 1))) ++r;
        return static_cast<unsigned short>(sign | r);
    }
    unsigned int r = (a - 0x38000000u) >> 13;
    const unsigned int rem = a & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) ++r;
    return static_cast<unsigned short>(sign | r);
}

// input channel stride (elements) the MFMA convolution wants for a dtype / kernel width
int conv_in_stride(int c, int dtype, int kw) {
    const int es = dtype == EXHIP_I8 ? 1 : dtype == EXHIP_F16 ? 2 : 4;
    if (c <= 4 && ((dtype == EXHIP_I8 && kw <= 8) || (dtype == EXHIP_F16 && kw <= 4))) return 4;
    return pad_to(c * es, 32) / es;
}

void require_nchw(memory::orderType o) {
    if (o != memory::NCHW) LOG(FATAL) << "this backend takes NCHW blobs at the operator interface";
}

// The fp16 pipeline keeps blobs NHWC between the layers whose kernels work on that layout (convolution, depthwise,
// pooling, the elementwise and per-channel layers): a blob of order NHWC has shape {n, h, w, c} (the reference's
// convention for that order, include/Primitives/tensor.hpp:124-134), channel stride == c, c a multiple of 8. Every other
// layer, and whoever reads a blob from outside, gets the NCHW form through as_nchw.
using half_ptr = std::shared_ptr<tensor<unsigned short>>;
// set_f16_nchw_only(true) keeps every blob NCHW, the form the NHWC-resident one is checked against.
bool g_f16_nchw_only = false;
bool nhwc_allowed() { return !g_f16_nchw_only; }
bool nhwc_channels_ok(int c) { return c % 8 == 0 && nhwc_allowed(); }

half_ptr as_nchw(exhip_ctx* ctx, const half_ptr& t, int device) {
    if (t->order() == memory::NCHW) return t;
    auto out = new_tensor<unsigned short>({t->num(), t->channels(), t->height(), t->width()}, device);
    EXHIP_FATAL(exhip_nhwc_f16_to_nchw_f16(ctx, t->gpu_data(), t->num(), t->channels(), t->height(), t->width(), t->channels(),
                                           out->mutable_gpu_data()));
    return out;
}

half_ptr as_order(exhip_ctx* ctx, const half_ptr& t, memory::orderType order, int device);

half_ptr as_nhwc(exhip_ctx* ctx, const half_ptr& t, int device) {
    if (t->order() == memory::NHWC) return t;
    auto out = new_tensor<unsigned short>({t->num(), t->height(), t->width(), t->channels()}, device, memory::NHWC);
    EXHIP_FATAL(exhip_nchw_f16_to_nhwc_f16(ctx, t->gpu_data(), t->num(), t->channels(), t->height(), t->width(), t->channels(),
                                           out->mutable_gpu_data()));
    return out;
}

half_ptr as_order(exhip_ctx* ctx, const half_ptr& t, memory::orderType order, int device) {
    return order == memory::NHWC ? as_nhwc(ctx, t, device) : as_nchw(ctx, t, device);
}

}  // namespace

void set_f16_nchw_only(bool on) { g_f16_nchw_only = on; }

// ------------------------------------------------------------------ convolution parameters
template <typename Dtype>
operation_general_conv<Dtype>::operation_general_conv(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        const int v = a.as_int();
        switch (key) {
        case 0: output_channel_ = v; break;
        case 1: kernel_size_w_ = kernel_size_h_ = v; break;
        case 2: dilation_w_ = dilation_h_ = v; break;
        case 3: stride_w_ = stride_h_ = v; break;
        case 4: pad_left_ = pad_right_ = pad_top_ = pad_bottom_ = v; break;
        case 5: bias_term_ = v != 0; break;
        case 6: weight_data_size_ = v; break;
        case 7: group_ = v; break;
        case 8:
            int8_scale_term_ = v != 0;
            this->params_.set_int8_quantization(int8_scale_term_);
            break;
        case 9: activation_type_ = v; break;
        case 10: NOT_IMPLEMENTED; break;
        case 11: kernel_size_h_ = v; break;
        case 12: dilation_h_ = v; break;
        case 13: stride_h_ = v; break;
        case 14: pad_top_ = v; break;
        case 15: pad_right_ = v; break;
        case 16: pad_bottom_ = v; break;
        case 17: impl_type_ = v; break;
        case 18: output_pad_right_ = output_pad_bottom_ = v; break;
        case 19: output_pad_bottom_ = v; break;
        case 20: output_dim_h_ = output_dim_w_ = v; break;
        case 21: output_dim_w_ = v; break;
        case -23330: break;
        default: LOG(FATAL) << "Un-supported Convolution Attribution " << a.key;
        }
    }
    CHECK_GT(group_, 0);
    CHECK_EQ(output_channel_ % group_, 0);
}

// ------------------------------------------------------------------ convolution
template <typename Dtype>
operation_convolution<Dtype>::operation_convolution(const operation_param& param) : operation_general_conv<Dtype>(param) {}

template <typename Dtype>
operation_convolution<Dtype>::~operation_convolution() {
    for (auto& kv : packed_) memory::device_release(this->params_.device_, kv.second.ptr, kv.second.bytes);
}

// Weight blob, src/Excalibur/operation_convolution.cpp:71-152: int32 tag; tag 0: float W (OIHW) then float bias[K];
// tag 871224: int8 W padded to a multiple of 4 bytes, float bias[K], float ws[K], float fs[1]. In the int8 case the
// bias sits in weights_f32_[1] behind a one-element placeholder (:121-126).
template <typename Dtype>
int operation_convolution<Dtype>::init_weights(FILE* fp) {
    const int dev = this->params_.device_;
    int tag = 0;
    if (fread(&tag, 1, sizeof(int), fp) != sizeof(int)) LOG(FATAL) << "model file ended inside layer " << this->params_.name_;
    int mem = 0;
    const int k = this->output_channel_;
    auto read_into = [&](void* dst, size_t bytes) {
        if (fread(dst, 1, bytes, fp) != bytes) LOG(FATAL) << "model file ended inside layer " << this->params_.name_;
        mem += static_cast<int>(bytes);
    };
    if (tag == 0) {
        this->weights_f32_.push_back(vec_tensor<float>(this->weight_data_size_, dev));
        read_into(this->weights_f32_[0]->mutable_cpu_data(), sizeof(float) * this->weight_data_size_);
        if (this->bias_term_) {
            this->weights_f32_.push_back(vec_tensor<float>(k, dev));
            read_into(this->weights_f32_[1]->mutable_cpu_data(), sizeof(float) * k);
        }
    } else if (tag == 871224) {
        const int aligned = (this->weight_data_size_ + 3) & ~3;
        this->weights_i8_.push_back(vec_tensor<signed char>(aligned, dev));
        read_into(this->weights_i8_[0]->mutable_cpu_data(), aligned);
        if (this->bias_term_) {
            this->weights_f32_.push_back(vec_tensor<float>(1, dev));
            this->weights_f32_.push_back(vec_tensor<float>(k, dev));
            read_into(this->weights_f32_[1]->mutable_cpu_data(), sizeof(float) * k);
        }
        this->weights_scaletable_i8_ = vec_tensor<float>(k, dev);
        read_into(this->weights_scaletable_i8_->mutable_cpu_data(), sizeof(float) * k);
        this->featmap_scaletable_i8_ = vec_tensor<float>(1, dev);
        read_into(this->featmap_scaletable_i8_->mutable_cpu_data(), sizeof(float));
    } else {
        NOT_IMPLEMENTED;
    }
    return mem;
}

// Dummy weights, src/Excalibur/operation_convolution.cpp:155-248: a default-seeded std::default_random_engine
// drawn in this order: weights, bias, (int8: weight scales, feature-map scale).
template <typename Dtype>
int operation_convolution<Dtype>::init_weights() {
    const int dev = this->params_.device_;
    std::default_random_engine e;
    std::normal_distribution<float> n(0, 0.3);
    std::uniform_int_distribution<int> u(-128, 127);
    const int k = this->output_channel_;
    int mem = 0;
    if (!this->params_.int8_quantization_) {
        this->weights_f32_.push_back(vec_tensor<float>(this->weight_data_size_, dev));
        float* w = this->weights_f32_[0]->mutable_cpu_data();
        for (int i = 0; i < this->weight_data_size_; ++i) w[i] = n(e);
        mem += this->weight_data_size_ * sizeof(float);
        if (this->bias_term_) {
            this->weights_f32_.push_back(vec_tensor<float>(k, dev));
            float* b = this->weights_f32_[1]->mutable_cpu_data();
            for (int i = 0; i < k; ++i) b[i] = n(e);
            mem += k * sizeof(float);
        }
    } else {
        const int aligned = (this->weight_data_size_ + 3) & ~3;
        this->weights_i8_.push_back(vec_tensor<signed char>(aligned, dev));
        signed char* w = this->weights_i8_[0]->mutable_cpu_data();
        for (int i = 0; i < aligned; ++i) w[i] = static_cast<signed char>(u(e));
        mem += aligned;
        if (this->bias_term_) {
            this->weights_f32_.push_back(vec_tensor<float>(1, dev));
            this->weights_f32_.push_back(vec_tensor<float>(k, dev));
            float* b = this->weights_f32_[1]->mutable_cpu_data();
            for (int i = 0; i < k; ++i) b[i] = n(e);
            mem += k * sizeof(float);
        }
        this->weights_scaletable_i8_ = vec_tensor<float>(k, dev);
        float* ws = this->weights_scaletable_i8_->mutable_cpu_data();
        for (int i = 0; i < k; ++i) ws[i] = n(e);
        this->featmap_scaletable_i8_ = vec_tensor<float>(1, dev);
        this->featmap_scaletable_i8_->mutable_cpu_data()[0] = n(e);
        mem += (k + 1) * sizeof(float);
    }
    return mem;
}

template <typename Dtype>
float operation_convolution<Dtype>::featmap_scale() const {
    CHECK(this->featmap_scaletable_i8_ != nullptr) << "layer " << this->params_.name_ << " has no int8 scales";
    return this->featmap_scaletable_i8_->cpu_data()[0];
}

template <typename Dtype>
std::vector<float> operation_convolution<Dtype>::dequantize_scales() const {
    const int k = this->output_channel_;
    const float fs = featmap_scale();
    const float* ws = this->weights_scaletable_i8_->cpu_data();
    const int n_ws = this->weights_scaletable_i8_->count();
    std::vector<float> s(k);
    for (int q = 0; q < k; ++q) {
        const float w = n_ws == 1 ? ws[0] : ws[q];
        volatile float prod = w * fs;  // float product, then float division
        s[q] = (std::fabs(w) <= 1e-6) ? 0.f : (1.0f / prod);
    }
    return s;
}

template <typename Dtype>
const float* operation_convolution<Dtype>::bias_gpu() {
    if (!this->bias_term_) return nullptr;
    return this->weights_f32_[1]->gpu_data();
}

template <typename Dtype>
const float* operation_convolution<Dtype>::scale_gpu() {
    if (!scale_dev_) {
        const std::vector<float> s = dequantize_scales();
        scale_dev_ = vec_tensor<float>(static_cast<int>(s.size()), this->params_.device_);
        std::memcpy(scale_dev_->mutable_cpu_data(), s.data(), s.size() * sizeof(float));
    }
    return scale_dev_->gpu_data();
}

template <typename Dtype>
exhip_conv_desc operation_convolution<Dtype>::describe(int n, int h, int w, int c_stride, int k_stride) const {
    exhip_conv_desc d;
    std::memset(&d, 0, sizeof(d));
    d.n = n; d.c = this->input_channels(); d.h = h; d.w = w; d.k = this->output_channel_;
    d.kh = this->kernel_size_h_; d.kw = this->kernel_size_w_; d.sh = this->stride_h_; d.sw = this->stride_w_;
    d.pt = this->pad_top_; d.pb = this->pad_bottom_; d.pl = this->pad_left_; d.pr = this->pad_right_;
    d.act = this->activation_type_; d.c_stride = c_stride; d.k_stride = k_stride;
    d.post_relu = post_relu_ ? 1 : 0; d.post_op = post_op_; d.post_alpha = post_alpha_; d.post_beta = post_beta_;
    d.post_slope = post_slope_; d.post_slope_shared = post_slope_shared_ ? 1 : 0;
    return d;
}

template <typename Dtype>
bool operation_convolution<Dtype>::set_post_prelu(const float* slopes, bool shared) {
    if (!slopes || this->group_ != 1 || this->stride_h_ != this->stride_w_) return false;
    post_op_ = EXHIP_POST_PRELU; post_alpha_ = post_beta_ = 0.f; post_relu_ = false;
    post_slope_ = slopes; post_slope_shared_ = shared;
    return true;
}

template <typename Dtype>
bool operation_convolution<Dtype>::set_post_activation(int post_op, float alpha, float beta, bool relu) {
    if ((post_op || relu) && (this->group_ != 1 || this->stride_h_ != this->stride_w_ || post_op == 1 + EXHIP_UNARY_SIGMOID))
        return false;
    post_op_ = post_op; post_alpha_ = alpha; post_beta_ = beta; post_relu_ = relu;
    post_slope_ = nullptr; post_slope_shared_ = false;
    return true;
}

template <typename Dtype>
bool operation_convolution<Dtype>::set_quantized_output(float fs, int stride, bool only) {
    if (fs != 0.f && (!this->params_.int8_quantization_ || this->group_ != 1 || this->stride_h_ != this->stride_w_ ||
                      stride < this->output_channel_ || stride % 32 != 0))
        return false;
    q_out_fs_ = fs; q_out_stride_ = fs != 0.f ? stride : 0; q_out_only_ = fs != 0.f && only;
    return true;
}

template <typename Dtype>
void operation_convolution<Dtype>::quantized_input(float* fs, int* stride) const {
    *fs = 0.f; *stride = 0;
    if (!this->params_.int8_quantization_ || this->group_ != 1 || this->stride_h_ != this->stride_w_) return;
    if (!this->featmap_scaletable_i8_ || this->featmap_scaletable_i8_->count() != 1) return;
    *fs = featmap_scale();
    *stride = conv_in_stride(this->input_channels(), EXHIP_I8, this->kernel_size_w_);
}

template <typename Dtype>
const void* operation_convolution<Dtype>::packed_weights(int dtype, const exhip_conv_desc& d) {
    const std::vector<int> key{dtype, d.n, d.h, d.w, d.c_stride};
    auto it = packed_.find(key);
    if (it != packed_.end()) {
        it->second.last_use = ++packed_clock_;
        return it->second.ptr;
    }
    // One packed copy per input geometry, the few most recently used: a detector fed many resolutions would otherwise
    // keep a copy of its weights for each. Copies a fused plan holds are pinned and stay.
    for (;;) {
        size_t loose = 0;
        auto oldest = packed_.end();
        for (auto jt = packed_.begin(); jt != packed_.end(); ++jt) {
            if (jt->second.pins > 0) continue;
            ++loose;
            if (oldest == packed_.end() || jt->second.last_use < oldest->second.last_use) oldest = jt;
        }
        if (loose < 4) break;
        memory::device_release(this->params_.device_, oldest->second.ptr, oldest->second.bytes);
        packed_.erase(oldest);
    }
    const size_t bytes = exhip_conv_packed_bytes(&d, dtype);
    if (bytes == 0) LOG(FATAL) << "layer " << this->params_.name_ << ": " << exhip_last_error();
    std::vector<char> host(bytes);
    std::vector<unsigned short> half_w;
    const void* src = nullptr;
    if (dtype == EXHIP_I8) {
        src = this->weights_i8_[0]->cpu_data();
    } else if (dtype == EXHIP_F32) {
        src = this->weights_f32_[0]->cpu_data();
    } else {
        // fp16 MFMA operands: float weights rounded to nearest-even half once, here
        const float* w = this->weights_f32_[0]->cpu_data();
        half_w.resize(this->weight_data_size_);
        for (int i = 0; i < this->weight_data_size_; ++i) half_w[i] = half_bits_rne(w[i]);
        src = half_w.data();
    }
    EXHIP_FATAL(exhip_conv_pack_weights(&d, dtype, src, host.data()));
    void* dev = memory::device_alloc(this->params_.device_, bytes);
    EXHIP_FATAL(exhip_memcpy_h2d(this->ctx(), dev, host.data(), bytes));
    packed_[key] = {dev, bytes, ++packed_clock_, 0};
    return dev;
}

template <typename Dtype>
const void* operation_convolution<Dtype>::pin_packed_weights(int dtype, const exhip_conv_desc& d) {
    const void* ptr = packed_weights(dtype, d);
    for (auto& kv : packed_)
        if (kv.second.ptr == ptr) ++kv.second.pins;
    return ptr;
}

template <typename Dtype>
void operation_convolution<Dtype>::unpin_packed_weights(const void* ptr) {
    for (auto& kv : packed_)
        if (kv.second.ptr == ptr && kv.second.pins > 0) --kv.second.pins;
}

template <typename Dtype>
bool operation_convolution<Dtype>::mfma_path_ok() const {
    if (this->dilation_h_ != 1 || this->dilation_w_ != 1)
        LOG(FATAL) << "layer " << this->params_.name_ << ": dilation is ignored by the reference's x86 path and not supported here";
    return this->group_ == 1 && this->stride_h_ == this->stride_w_;
}

template <typename Dtype>
void operation_convolution<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    require_nchw(bottoms[0]->order());
    const int dev = this->params_.device_;
    const int n = bottoms[0]->num(), c = bottoms[0]->channels(), h = bottoms[0]->height(), w = bottoms[0]->width();
    CHECK_EQ(c, this->input_channels());
    exhip_conv_desc d = describe(n, h, w, c, this->output_channel_);
    int oh, ow;
    EXHIP_FATAL(exhip_conv_out_hw(&d, &oh, &ow));
    tops[0] = new_tensor<float>({n, this->output_channel_, oh, ow}, dev);
    if (!mfma_path_ok()) {
        EXHIP_FATAL(exhip_conv2d_direct_nchw(this->ctx(), &d, this->group_, bottoms[0]->gpu_data(), this->weights_f32_[0]->gpu_data(),
                                             nullptr, 1.f, nullptr, bias_gpu(), tops[0]->mutable_gpu_data()));
        return;
    }
    d.c_stride = conv_in_stride(c, EXHIP_F32, d.kw);
    auto x = new_tensor<float>({n, h, w, d.c_stride}, dev);
    EXHIP_FATAL(exhip_nchw_f32_to_nhwc_f32(this->ctx(), bottoms[0]->gpu_data(), n, c, h, w, d.c_stride, x->mutable_gpu_data()));
    EXHIP_FATAL(exhip_conv2d_f32(this->ctx(), &d, x->gpu_data(), packed_weights(EXHIP_F32, d), bias_gpu(), nullptr, nullptr,
                                 tops[0]->mutable_gpu_data()));
}

template <typename Dtype>
void operation_convolution<Dtype>::forward_gpu_i8(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    require_nchw(bottoms[0]->order());
    const int dev = this->params_.device_;
    const int n = bottoms[0]->num(), c = bottoms[0]->channels(), h = bottoms[0]->height(), w = bottoms[0]->width();
    CHECK_EQ(c, this->input_channels());
    // Both loaders of the reference give a convolution exactly one feature-map scale (model file: operation_convolution.cpp:130-131,
    // dummy weights: :230-231), so the per-input-channel branch of its quantizer (operation_general_conv.cpp:596) cannot be
    // reached through this operator; the quantizer entry point of the C ABI covers that branch on its own.
    CHECK_EQ(this->featmap_scaletable_i8_->count(), 1) << "a convolution carries one feature-map scale";
    exhip_conv_desc d = describe(n, h, w, c, this->output_channel_);
    int oh, ow;
    EXHIP_FATAL(exhip_conv_out_hw(&d, &oh, &ow));
    tops[0] = new_tensor<float>({n, this->output_channel_, oh, ow}, dev);
    if (!mfma_path_ok()) {
        EXHIP_FATAL(exhip_conv2d_direct_nchw(this->ctx(), &d, this->group_, bottoms[0]->gpu_data(), nullptr,
                                             this->weights_i8_[0]->gpu_data(), featmap_scale(), scale_gpu(), bias_gpu(),
                                             tops[0]->mutable_gpu_data()));
        return;
    }
    d.c_stride = conv_in_stride(c, EXHIP_I8, d.kw);
    // the producer's int8 copy of the input if it was made with this layer's scale and stride, else the quantizer
    std::shared_ptr<tensor<signed char>> q;
    const auto& copy = bottoms[0]->quantized;
    if (copy && copy->scale == featmap_scale() && copy->stride == d.c_stride &&
        copy->data->data_shape() == std::vector<int>{n, h, w, d.c_stride}) {
        q = copy->data;
    } else {
        if (copy && copy->only) LOG(FATAL) << "layer " << this->params_.name_ << ": the input blob holds int8 data for another reader";
        q = new_tensor<signed char>({n, h, w, d.c_stride}, dev);
        EXHIP_FATAL(exhip_quantize_nchw_f32_to_nhwc_i8(this->ctx(), bottoms[0]->gpu_data(), n, c, h, w, featmap_scale(), nullptr,
                                                       d.c_stride, reinterpret_cast<int8_t*>(q->mutable_gpu_data())));
    }
    int8_t* y_q = nullptr;
    if (q_out_fs_ != 0.f) {
        auto out = std::make_shared<typename tensor<float>::quantized_copy>();
        out->data = new_tensor<signed char>({n, oh, ow, q_out_stride_}, dev);
        out->scale = q_out_fs_; out->stride = q_out_stride_; out->only = q_out_only_;
        tops[0]->quantized = out;
        y_q = reinterpret_cast<int8_t*>(out->data->mutable_gpu_data());
        d.fs_out = q_out_fs_;
        d.k_stride = q_out_stride_;
    }
    EXHIP_FATAL(exhip_conv2d_i8(this->ctx(), &d, reinterpret_cast<const int8_t*>(q->gpu_data()), packed_weights(EXHIP_I8, d),
                                scale_gpu(), bias_gpu(), nullptr, y_q, nullptr, q_out_only_ ? nullptr : tops[0]->mutable_gpu_data(),
                                nullptr));
}

template <typename Dtype>
void operation_convolution<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const int dev = this->params_.device_;
    const int n = bottoms[0]->num(), c = bottoms[0]->channels(), h = bottoms[0]->height(), w = bottoms[0]->width();
    CHECK_EQ(c, this->input_channels());
    exhip_conv_desc d = describe(n, h, w, c, this->output_channel_);
    int oh, ow;
    EXHIP_FATAL(exhip_conv_out_hw(&d, &oh, &ow));
    if (!mfma_path_ok()) {
        // definition-order kernel in float on converted tensors, result rounded to half
        const half_ptr in = as_nchw(this->ctx(), bottoms[0], dev);
        tops[0] = new_tensor<unsigned short>({n, this->output_channel_, oh, ow}, dev);
        auto xf = new_tensor<float>({n, c, h, w}, dev);
        auto yf = new_tensor<float>({n, this->output_channel_, oh, ow}, dev);
        EXHIP_FATAL(exhip_f16_to_f32(this->ctx(), in->gpu_data(), xf->mutable_gpu_data(), xf->count()));
        EXHIP_FATAL(exhip_conv2d_direct_nchw(this->ctx(), &d, this->group_, xf->gpu_data(), this->weights_f32_[0]->gpu_data(), nullptr,
                                             1.f, nullptr, bias_gpu(), yf->mutable_gpu_data()));
        EXHIP_FATAL(exhip_f32_to_f16(this->ctx(), yf->gpu_data(), tops[0]->mutable_gpu_data(), yf->count()));
        return;
    }
    // The kernel reads NHWC with the channel stride it wants (16 halves per 32-byte step) and writes NHWC, NCHW or both:
    // an NHWC blob with such a stride goes in as it is, and the result stays NHWC where its channel count allows.
    d.c_stride = conv_in_stride(c, EXHIP_F16, d.kw);
    half_ptr x;
    if (bottoms[0]->order() == memory::NHWC && d.c_stride == c) {
        x = bottoms[0];
    } else {
        const half_ptr in = as_nchw(this->ctx(), bottoms[0], dev);
        x = new_tensor<unsigned short>({n, h, w, d.c_stride}, dev);
        EXHIP_FATAL(exhip_nchw_f16_to_nhwc_f16(this->ctx(), in->gpu_data(), n, c, h, w, d.c_stride, x->mutable_gpu_data()));
    }
    const bool out_nhwc = this->output_channel_ % 16 == 0 && nhwc_allowed();
    tops[0] = out_nhwc ? new_tensor<unsigned short>({n, oh, ow, this->output_channel_}, dev, memory::NHWC)
                       : new_tensor<unsigned short>({n, this->output_channel_, oh, ow}, dev);
    unsigned short* y = tops[0]->mutable_gpu_data();
    const unsigned short* residual = nullptr;
    if (post_sum_ && out_nhwc && post_sum_->order() == memory::NHWC && post_sum_->data_shape() == tops[0]->data_shape() &&
        (post_sum_last_ || (!post_op_ && !post_relu_))) {
        residual = post_sum_->gpu_data();
        d.residual_last = post_sum_last_ ? 1 : 0;
        post_sum_used_ = true;
    }
    EXHIP_FATAL(exhip_conv2d_f16(this->ctx(), &d, x->gpu_data(), packed_weights(EXHIP_F16, d), bias_gpu(), residual,
                                 out_nhwc ? y : nullptr, out_nhwc ? nullptr : y, nullptr));
}

// ------------------------------------------------------------------ depthwise convolution
template <typename Dtype>
bool operation_convolutiondepthwise<Dtype>::fast3x3() const {
    return this->kernel_size_h_ == 3 && this->kernel_size_w_ == 3 && this->stride_h_ == this->stride_w_ &&
           (this->stride_h_ == 1 || this->stride_h_ == 2);
}

template <typename Dtype>
void operation_convolutiondepthwise<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    CHECK_EQ(this->output_channel_, this->group_);
    CHECK_EQ(bottoms[0]->channels(), this->output_channel_);
    if (!fast3x3()) {  // the reference falls back to the grouped dense convolution (operation_convolutiondepthwise.cpp:118)
        operation_convolution<Dtype>::forward_gpu_f32(bottoms, tops);
        return;
    }
    require_nchw(bottoms[0]->order());
    const int n = bottoms[0]->num(), c = bottoms[0]->channels(), h = bottoms[0]->height(), w = bottoms[0]->width();
    const int oh = (h + this->pad_top_ + this->pad_bottom_ - 3) / this->stride_h_ + 1;
    const int ow = (w + this->pad_left_ + this->pad_right_ - 3) / this->stride_w_ + 1;
    tops[0] = new_tensor<float>({n, c, oh, ow}, this->params_.device_);
    if (this->post_slope_) {  // the PReLU layer behind this one in the same kernel, or as a second launch where the shape needs it
        const int rc = exhip_dwconv3x3_nchw_f32_prelu(this->ctx(), bottoms[0]->gpu_data(), this->weights_f32_[0]->gpu_data(), this->bias_gpu(),
                                                      this->post_slope_, this->post_slope_shared_, tops[0]->mutable_gpu_data(), n, c, h, w,
                                                      this->stride_h_, this->pad_top_, this->pad_bottom_, this->pad_left_, this->pad_right_);
        if (rc != EXHIP_ERR_UNSUPPORTED) {
            EXHIP_FATAL(rc);
            return;
        }
        auto mid = new_tensor<float>({n, c, oh, ow}, this->params_.device_);
        EXHIP_FATAL(exhip_dwconv3x3_nchw_f32(this->ctx(), bottoms[0]->gpu_data(), this->weights_f32_[0]->gpu_data(), this->bias_gpu(),
                                             mid->mutable_gpu_data(), n, c, h, w, this->stride_h_, this->pad_top_, this->pad_bottom_,
                                             this->pad_left_, this->pad_right_, 0));
        EXHIP_FATAL(exhip_channelwise_f32(this->ctx(), EXHIP_CHANNEL_PRELU, mid->gpu_data(), tops[0]->mutable_gpu_data(), n, c, oh * ow,
                                          this->post_slope_, nullptr, this->post_slope_shared_ ? 1 : 0));
        return;
    }
    EXHIP_FATAL(exhip_dwconv3x3_nchw_f32(this->ctx(), bottoms[0]->gpu_data(), this->weights_f32_[0]->gpu_data(), this->bias_gpu(),
                                         tops[0]->mutable_gpu_data(), n, c, h, w, this->stride_h_, this->pad_top_, this->pad_bottom_,
                                         this->pad_left_, this->pad_right_, this->activation_type_));
}

template <typename Dtype>
bool operation_convolutiondepthwise<Dtype>::set_post_prelu(const float* slopes, bool shared) {
    if (!slopes || !fast3x3() || this->activation_type_ != 0 || this->output_channel_ != this->group_) return false;
    this->post_op_ = EXHIP_POST_PRELU; this->post_slope_ = slopes; this->post_slope_shared_ = shared;
    return true;
}

// Weight-only quantization: the int8 weights are dequantized once and the float path runs
// (src/Excalibur/operation_convolutiondepthwise.cpp:184-222).
template <typename Dtype>
void operation_convolutiondepthwise<Dtype>::forward_gpu_i8(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    if (this->int8_scale_term_) {
        const int aligned = (this->weight_data_size_ + 3) & ~3;
        auto wf = vec_tensor<float>(aligned, this->params_.device_);
        EXHIP_FATAL(exhip_dw_dequant_weights(this->ctx(), reinterpret_cast<const int8_t*>(this->weights_i8_[0]->gpu_data()),
                                             this->weights_scaletable_i8_->gpu_data(), wf->mutable_gpu_data(), this->output_channel_,
                                             aligned / this->group_));
        if (this->weights_f32_.empty()) this->weights_f32_.push_back(wf);
        else this->weights_f32_[0] = wf;
        this->int8_scale_term_ = false;
    }
    forward_gpu_f32(bottoms, tops);
}

template <typename Dtype>
void operation_convolutiondepthwise<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms,
                                                            tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    CHECK_EQ(this->output_channel_, this->group_);
    if (!fast3x3()) {
        operation_convolution<Dtype>::forward_gpu_f16(bottoms, tops);
        return;
    }
    const int dev = this->params_.device_;
    const int n = bottoms[0]->num(), c = bottoms[0]->channels(), h = bottoms[0]->height(), w = bottoms[0]->width();
    const int oh = (h + this->pad_top_ + this->pad_bottom_ - 3) / this->stride_h_ + 1;
    const int ow = (w + this->pad_left_ + this->pad_right_ - 3) / this->stride_w_ + 1;
    if (nhwc_channels_ok(c)) {  // NHWC in, NHWC out
        const half_ptr x = as_nhwc(this->ctx(), bottoms[0], dev);
        tops[0] = new_tensor<unsigned short>({n, oh, ow, c}, dev, memory::NHWC);
        if (this->post_slope_) {
            const int rc = exhip_dwconv3x3_nhwc_f16_prelu(this->ctx(), x->gpu_data(), this->weights_f32_[0]->gpu_data(), this->bias_gpu(),
                                                          this->post_slope_, this->post_slope_shared_, tops[0]->mutable_gpu_data(), n, c, h,
                                                          w, c, this->stride_h_, this->pad_top_, this->pad_bottom_, this->pad_left_,
                                                          this->pad_right_);
            if (rc != EXHIP_ERR_UNSUPPORTED) {
                EXHIP_FATAL(rc);
                return;
            }
            auto mid = new_tensor<unsigned short>({n, oh, ow, c}, dev, memory::NHWC);
            EXHIP_FATAL(exhip_dwconv3x3_nhwc_f16(this->ctx(), x->gpu_data(), this->weights_f32_[0]->gpu_data(), this->bias_gpu(),
                                                 mid->mutable_gpu_data(), n, c, h, w, c, this->stride_h_, this->pad_top_,
                                                 this->pad_bottom_, this->pad_left_, this->pad_right_, 0));
            EXHIP_FATAL(exhip_channelwise_nhwc_f16(this->ctx(), EXHIP_CHANNEL_PRELU, mid->gpu_data(), tops[0]->mutable_gpu_data(),
                                                   static_cast<size_t>(n) * oh * ow, c, this->post_slope_, nullptr,
                                                   this->post_slope_shared_ ? 1 : 0));
            return;
        }
        EXHIP_FATAL(exhip_dwconv3x3_nhwc_f16(this->ctx(), x->gpu_data(), this->weights_f32_[0]->gpu_data(), this->bias_gpu(),
                                             tops[0]->mutable_gpu_data(), n, c, h, w, c, this->stride_h_, this->pad_top_,
                                             this->pad_bottom_, this->pad_left_, this->pad_right_, this->activation_type_));
        return;
    }
    const half_ptr in = as_nchw(this->ctx(), bottoms[0], dev);
    const int cs = pad_to(c, 8);
    auto x = new_tensor<unsigned short>({n, h, w, cs}, dev);
    auto y = new_tensor<unsigned short>({n, oh, ow, cs}, dev);
    tops[0] = new_tensor<unsigned short>({n, c, oh, ow}, dev);
    EXHIP_FATAL(exhip_nchw_f16_to_nhwc_f16(this->ctx(), in->gpu_data(), n, c, h, w, cs, x->mutable_gpu_data()));
    EXHIP_FATAL(exhip_dwconv3x3_nhwc_f16(this->ctx(), x->gpu_data(), this->weights_f32_[0]->gpu_data(), this->bias_gpu(),
                                         y->mutable_gpu_data(), n, c, h, w, cs, this->stride_h_, this->pad_top_, this->pad_bottom_,
                                         this->pad_left_, this->pad_right_, this->activation_type_));
    if (this->post_slope_) {  // channel counts off the NHWC layout: the PReLU layer as a launch of its own on the NCHW result
        auto mid = new_tensor<unsigned short>({n, c, oh, ow}, dev);
        EXHIP_FATAL(exhip_nhwc_f16_to_nchw_f16(this->ctx(), y->gpu_data(), n, c, oh, ow, cs, mid->mutable_gpu_data()));
        EXHIP_FATAL(exhip_channelwise_f16(this->ctx(), EXHIP_CHANNEL_PRELU, mid->gpu_data(), tops[0]->mutable_gpu_data(), n, c, oh * ow,
                                          this->post_slope_, nullptr, this->post_slope_shared_ ? 1 : 0));
        return;
    }
    EXHIP_FATAL(exhip_nhwc_f16_to_nchw_f16(this->ctx(), y->gpu_data(), n, c, oh, ow, cs, tops[0]->mutable_gpu_data()));
}

// ------------------------------------------------------------------ pooling
template <typename Dtype>
operation_pooling<Dtype>::operation_pooling(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int v = a.as_int();
        switch (std::atoi(a.key.c_str())) {
        case 0: type_ = v; break;
        case 1: kernel_size_w_ = kernel_size_h_ = v; break;
        case 2: stride_w_ = stride_h_ = v; break;
        case 3: pad_left_ = pad_right_ = pad_top_ = pad_bottom_ = v; break;
        case 4: global_pooling_ = v != 0; break;
        case 5: pad_mode_ = v; break;
        case 6: avgpool_count_include_pad_ = v; break;
        case 11: kernel_size_h_ = v; break;
        case 12: stride_h_ = v; break;
        case 13: pad_top_ = v; break;
        case 14: pad_right_ = v; break;
        case 15: pad_bottom_ = v; break;
        case -23330: break;
        default: LOG(FATAL) << "Un-supported Pooling Attribution " << a.key;
        }
    }
}

template <typename Dtype>
void operation_pooling<Dtype>::geometry(int h, int w, int* kh, int* kw, int* sh, int* sw, int* pt, int* pb, int* pl, int* pr,
                                        int* oh, int* ow) const {
    *kh = kernel_size_h_; *kw = kernel_size_w_; *sh = stride_h_; *sw = stride_w_;
    *pt = pad_top_; *pb = pad_bottom_; *pl = pad_left_; *pr = pad_right_;
    if (global_pooling_) {  // src/Excalibur/operation_pooling.cpp:90-100
        *kh = h; *kw = w; *sh = *sw = 1; *pt = *pb = *pl = *pr = 0;
    }
    if (type_ != 0 && type_ != 1) LOG(FATAL) << "Unknown pooling method.";
    if (pad_mode_ != 0 && pad_mode_ != 1) NOT_IMPLEMENTED;
    EXHIP_FATAL(exhip_pool_out_hw(h, w, *kh, *kw, *sh, *sw, *pt, *pb, *pl, *pr, pad_mode_, oh, ow));
}

template <typename Dtype>
void operation_pooling<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        require_nchw(bottoms[i]->order());
        const int n = bottoms[i]->num(), c = bottoms[i]->channels(), h = bottoms[i]->height(), w = bottoms[i]->width();
        int kh, kw, sh, sw, pt, pb, pl, pr, oh, ow;
        geometry(h, w, &kh, &kw, &sh, &sw, &pt, &pb, &pl, &pr, &oh, &ow);
        tops[i] = new_tensor<float>({n, c, oh, ow}, this->params_.device_);
        EXHIP_FATAL(exhip_pool2d_nchw_f32(this->ctx(), bottoms[i]->gpu_data(), tops[i]->mutable_gpu_data(), n, c, h, w, oh, ow, type_,
                                          kh, kw, sh, sw, pt, pb, pl, pr, avgpool_count_include_pad_));
    }
}

template <typename Dtype>
void operation_pooling<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    const int dev = this->params_.device_;
    for (size_t i = 0; i < bottoms.size(); ++i) {
        const int n = bottoms[i]->num(), c = bottoms[i]->channels(), h = bottoms[i]->height(), w = bottoms[i]->width();
        int kh, kw, sh, sw, pt, pb, pl, pr, oh, ow;
        geometry(h, w, &kh, &kw, &sh, &sw, &pt, &pb, &pl, &pr, &oh, &ow);
        if (nhwc_channels_ok(c)) {  // NHWC in, NHWC out
            const half_ptr x = as_nhwc(this->ctx(), bottoms[i], dev);
            tops[i] = new_tensor<unsigned short>({n, oh, ow, c}, dev, memory::NHWC);
            if (type_ == 0 && kh == kw && (kh == 5 || kh == 9 || kh == 13) && sh == 1 && sw == 1 && pt == kh / 2 && pb == kh / 2 &&
                pl == kh / 2 && pr == kh / 2 && oh == h && ow == w) {  // the detection topologies' 5 / 9 / 13 pyramid: rows, then columns
                auto tmp = new_tensor<unsigned short>({n, h, w, c}, dev, memory::NHWC);
                EXHIP_FATAL(exhip_maxpool_same_nhwc_f16(this->ctx(), x->gpu_data(), tmp->mutable_gpu_data(), tops[i]->mutable_gpu_data(), n,
                                                        c, h, w, kh));
                continue;
            }
            EXHIP_FATAL(exhip_pool2d_nhwc_f16(this->ctx(), x->gpu_data(), tops[i]->mutable_gpu_data(), n, c, h, w, c, oh, ow, type_, kh,
                                              kw, sh, sw, pt, pb, pl, pr, avgpool_count_include_pad_));
            continue;
        }
        const half_ptr in = as_nchw(this->ctx(), bottoms[i], dev);
        const int cs = pad_to(c, 8);
        auto x = new_tensor<unsigned short>({n, h, w, cs}, dev);
        auto y = new_tensor<unsigned short>({n, oh, ow, cs}, dev);
        tops[i] = new_tensor<unsigned short>({n, c, oh, ow}, dev);
        EXHIP_FATAL(exhip_nchw_f16_to_nhwc_f16(this->ctx(), in->gpu_data(), n, c, h, w, cs, x->mutable_gpu_data()));
        EXHIP_FATAL(exhip_pool2d_nhwc_f16(this->ctx(), x->gpu_data(), y->mutable_gpu_data(), n, c, h, w, cs, oh, ow, type_, kh, kw, sh,
                                          sw, pt, pb, pl, pr, avgpool_count_include_pad_));
        EXHIP_FATAL(exhip_nhwc_f16_to_nchw_f16(this->ctx(), y->gpu_data(), n, c, oh, ow, cs, tops[i]->mutable_gpu_data()));
    }
}

// ------------------------------------------------------------------ eltwise / binaryop / relu / split
template <typename Dtype>
operation_eltwise<Dtype>::operation_eltwise(const operation_param& param) : operation<Dtype>(param) {
    coeffs_.assign(param.input_count_, 1.0f);
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) {
            type_ = a.as_int();
        } else if (key == -23301) {
            // "n,c0,c1,...": the reference reads entries 1 .. n-1 into coeffs_[0 .. n-2] (operation_eltwise.cpp:26-33)
            const std::vector<std::string> parts = split_string(a.value, ",");
            CHECK_EQ(type_, static_cast<int>(SUM));
            const int cnt = parts.empty() ? 0 : std::atoi(parts[0].c_str());
            for (int j = 1; j < cnt && j < static_cast<int>(parts.size()) && j - 1 < static_cast<int>(coeffs_.size()); ++j)
                coeffs_[j - 1] = static_cast<float>(std::atof(parts[j].c_str()));
        } else if (key != -23330) {
            LOG(FATAL) << "Un-supported Eltwise Attribution " << a.key;
        }
    }
}

template <typename Dtype>
void operation_eltwise<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_GE(bottoms.size(), 2);
    CHECK_EQ(tops.size(), 1);
    for (size_t i = 1; i < bottoms.size(); ++i) CHECK(bottoms[i]->data_shape() == bottoms[0]->data_shape());
    if (type_ < 0 || type_ > 2) LOG(FATAL) << "Unknown elementwise operation.";
    tops[0] = std::make_shared<tensor<float>>(bottoms[0]->data_shape(), this->params_.device_, bottoms[0]->order());
    std::vector<const float*> in;
    for (auto& b : bottoms) in.push_back(b->gpu_data());
    EXHIP_FATAL(exhip_eltwise_f32(this->ctx(), in.data(), static_cast<int>(in.size()), coeffs_.data(), type_,
                                  tops[0]->mutable_gpu_data(), tops[0]->count()));
}

template <typename Dtype>
void operation_eltwise<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    // fp16 layer = float operator on half-rounded inputs, result rounded to half
    CHECK_GE(bottoms.size(), 2);
    CHECK_EQ(tops.size(), 1);
    const int dev = this->params_.device_;
    if (type_ == 1 && bottoms.size() == 2 && coeffs_[0] == 1.f && coeffs_[1] == 1.f) {  // the residual add, in one pass
        const half_ptr b1 = as_order(this->ctx(), bottoms[1], bottoms[0]->order(), dev);  // element by element: any common layout
        CHECK(b1->data_shape() == bottoms[0]->data_shape());
        tops[0] = std::make_shared<tensor<unsigned short>>(bottoms[0]->data_shape(), dev, bottoms[0]->order());
        EXHIP_FATAL(exhip_add_f16(this->ctx(), bottoms[0]->gpu_data(), b1->gpu_data(), tops[0]->mutable_gpu_data(), tops[0]->count(), 0));
        return;
    }
    // the general form in NCHW: the SUM kernel reproduces a rounding that depends on an element's position in the blob
    tensor_list<unsigned short> nchw;
    for (const auto& b : bottoms) nchw.push_back(as_nchw(this->ctx(), b, dev));
    eltwise_general_f16(nchw, tops);
}

template <typename Dtype>
void operation_eltwise<Dtype>::eltwise_general_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    const int dev = this->params_.device_;
    tensor_list<float> f(bottoms.size());
    std::vector<const float*> in;
    for (size_t i = 0; i < bottoms.size(); ++i) {
        CHECK(bottoms[i]->data_shape() == bottoms[0]->data_shape());
        f[i] = std::make_shared<tensor<float>>(bottoms[i]->data_shape(), dev, bottoms[i]->order());
        EXHIP_FATAL(exhip_f16_to_f32(this->ctx(), bottoms[i]->gpu_data(), f[i]->mutable_gpu_data(), f[i]->count()));
        in.push_back(f[i]->gpu_data());
    }
    auto y = std::make_shared<tensor<float>>(bottoms[0]->data_shape(), dev, bottoms[0]->order());
    EXHIP_FATAL(exhip_eltwise_f32(this->ctx(), in.data(), static_cast<int>(in.size()), coeffs_.data(), type_, y->mutable_gpu_data(),
                                  y->count()));
    tops[0] = std::make_shared<tensor<unsigned short>>(bottoms[0]->data_shape(), dev, bottoms[0]->order());
    EXHIP_FATAL(exhip_f32_to_f16(this->ctx(), y->gpu_data(), tops[0]->mutable_gpu_data(), y->count()));
}

template <typename Dtype>
operation_binaryop<Dtype>::operation_binaryop(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        switch (std::atoi(a.key.c_str())) {
        case 0: op_type_ = a.as_int(); break;
        case 1: with_scalar_ = a.as_int(); break;
        case 2: coef_ = a.as_float(); break;
        default: LOG(FATAL) << "Un-supported BinaryOp Attribution " << a.key;
        }
    }
}

template <typename Dtype>
void operation_binaryop<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_GE(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    if (with_scalar_ || bottoms.size() != 2 || op_type_ < 0 || op_type_ > 3) NOT_IMPLEMENTED << " BinaryOp with a scalar, one operand or op " << op_type_;
    require_nchw(bottoms[0]->order());
    if (op_type_ == 0 && bottoms[0]->data_shape() == bottoms[1]->data_shape()) {  // the residual add
        tops[0] = std::make_shared<tensor<float>>(bottoms[0]->data_shape(), this->params_.device_, bottoms[0]->order());
        EXHIP_FATAL(exhip_add_f32(this->ctx(), bottoms[0]->gpu_data(), bottoms[1]->gpu_data(), tops[0]->mutable_gpu_data(), tops[0]->count(), 0));
        return;
    }
    // which operand gives the output its shape: src/Excalibur/operation_binaryop.cpp:9-42
    auto dims_of = [](const tensor<float>& t) { return (t.width() != 1) + (t.height() != 1) + (t.channels() != 1); };
    const std::vector<int> s1 = bottoms[0]->data_shape(), s2 = bottoms[1]->data_shape();
    bool second_larger = false;
    if (s1 != s2) {
        const int d1 = dims_of(*bottoms[0]), d2 = dims_of(*bottoms[1]);
        if (d2 > d1) second_larger = true;
        else if (d2 == d1)
            for (int i = 1; i < 4; ++i)
                if (s2[i] > s1[i]) { second_larger = true; break; }
    }
    const auto& large = second_larger ? bottoms[1] : bottoms[0];
    const auto& small = second_larger ? bottoms[0] : bottoms[1];
    const int hw = large->height() * large->width();
    const int small_chw = small->channels() * small->height() * small->width();
    const int large_dims = std::max(1, dims_of(*large)), small_dims = std::max(1, dims_of(*small));
    int mode = -1;
    if (s1 == s2) mode = EXHIP_BINARY_EQUAL;
    else if (small_chw == 1) mode = EXHIP_BINARY_PER_IMAGE;
    else if (large_dims == 3 && small_dims == 2 && small->channels() == 1 && small->height() * small->width() == hw) mode = EXHIP_BINARY_PER_PIXEL;
    else if (large_dims == 3 && small_dims == 1 && small->channels() > 1 && small->channels() == large->channels()) mode = EXHIP_BINARY_PER_CHANNEL;
    if (mode < 0) NOT_IMPLEMENTED << " BinaryOp on these two shapes";
    tops[0] = std::make_shared<tensor<float>>(large->data_shape(), this->params_.device_, large->order());
    EXHIP_FATAL(exhip_binaryop_f32(this->ctx(), op_type_, mode, large->gpu_data(), small->gpu_data(), tops[0]->mutable_gpu_data(),
                                   large->num(), large->channels(), hw, small->num()));
}

template <typename Dtype>
void operation_binaryop<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(tops.size(), 1);
    const int dev = this->params_.device_;
    const bool same_blob_shape = bottoms.size() == 2 && bottoms[0]->num() == bottoms[1]->num() &&
                                 bottoms[0]->channels() == bottoms[1]->channels() && bottoms[0]->height() == bottoms[1]->height() &&
                                 bottoms[0]->width() == bottoms[1]->width();
    if (op_type_ != 0 || with_scalar_ || !same_blob_shape) {
        operation<Dtype>::forward_gpu_f16(bottoms, tops);  // everything but the residual add: convert, float kernel, convert back
        return;
    }
    const half_ptr b1 = as_order(this->ctx(), bottoms[1], bottoms[0]->order(), dev);  // element by element: any common layout
    tops[0] = std::make_shared<tensor<unsigned short>>(bottoms[0]->data_shape(), dev, bottoms[0]->order());
    EXHIP_FATAL(exhip_add_f16(this->ctx(), bottoms[0]->gpu_data(), b1->gpu_data(), tops[0]->mutable_gpu_data(), tops[0]->count(), 0));
}

template <typename Dtype>
operation_relu<Dtype>::operation_relu(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) slope_ = a.as_float();
        else if (key != -23330) LOG(FATAL) << "Un-supported ReLU Attribution " << a.key;
    }
    this->params_.inplace_ = true;
}

template <typename Dtype>
void operation_relu<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        tops[i] = std::make_shared<tensor<float>>(bottoms[i]->data_shape(), this->params_.device_, bottoms[i]->order());
        EXHIP_FATAL(exhip_relu_f32(this->ctx(), bottoms[i]->gpu_data(), tops[i]->mutable_gpu_data(), tops[i]->count()));
    }
}

template <typename Dtype>
void operation_relu<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        tops[i] = std::make_shared<tensor<unsigned short>>(bottoms[i]->data_shape(), this->params_.device_, bottoms[i]->order());
        EXHIP_FATAL(exhip_relu_f16(this->ctx(), bottoms[i]->gpu_data(), tops[i]->mutable_gpu_data(), tops[i]->count()));
    }
}

// Split hands the same blob to every consumer (src/Excalibur/operation_split.cpp:14-23).
template <typename Dtype>
void operation_split<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    for (auto& t : tops) t = bottoms[0];
}
template <typename Dtype>
void operation_split<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    for (auto& t : tops) t = bottoms[0];
}

// ------------------------------------------------------------------ inner product
template <typename Dtype>
operation_innerproduct<Dtype>::operation_innerproduct(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int v = a.as_int();
        switch (std::atoi(a.key.c_str())) {
        case 0: num_output_ = v; break;
        case 1: bias_term_ = v != 0; break;
        case 2: weight_data_size_ = v; break;
        case 8:
            int8_scale_term_ = v != 0;
            this->params_.set_int8_quantization(int8_scale_term_);
            break;
        case 9: activation_type_ = v; break;
        case 10: NOT_IMPLEMENTED; break;
        case -23330: break;
        default: LOG(FATAL) << "Un-supported InnerProduct Attribution " << a.key;
        }
    }
}

// src/Excalibur/operation_innerproduct.cpp:77-120: like the convolution blob, with a single weight scale.
template <typename Dtype>
int operation_innerproduct<Dtype>::init_weights(FILE* fp) {
    const int dev = this->params_.device_;
    int tag = 0, mem = 0;
    if (fread(&tag, 1, sizeof(int), fp) != sizeof(int)) LOG(FATAL) << "model file ended inside layer " << this->params_.name_;
    auto read_into = [&](void* dst, size_t bytes) {
        if (fread(dst, 1, bytes, fp) != bytes) LOG(FATAL) << "model file ended inside layer " << this->params_.name_;
        mem += static_cast<int>(bytes);
    };
    if (tag == 0) {
        this->weights_f32_.push_back(vec_tensor<float>(weight_data_size_, dev));
        read_into(this->weights_f32_[0]->mutable_cpu_data(), sizeof(float) * weight_data_size_);
        if (bias_term_) {
            this->weights_f32_.push_back(vec_tensor<float>(num_output_, dev));
            read_into(this->weights_f32_[1]->mutable_cpu_data(), sizeof(float) * num_output_);
        }
    } else if (tag == 871224) {
        const int aligned = (weight_data_size_ + 3) & ~3;
        this->weights_i8_.push_back(vec_tensor<signed char>(aligned, dev));
        read_into(this->weights_i8_[0]->mutable_cpu_data(), aligned);
        if (bias_term_) {
            this->weights_f32_.push_back(vec_tensor<float>(1, dev));
            this->weights_f32_.push_back(vec_tensor<float>(num_output_, dev));
            read_into(this->weights_f32_[1]->mutable_cpu_data(), sizeof(float) * num_output_);
        }
        this->weights_scaletable_i8_ = vec_tensor<float>(1, dev);
        read_into(this->weights_scaletable_i8_->mutable_cpu_data(), sizeof(float));
        this->featmap_scaletable_i8_ = vec_tensor<float>(1, dev);
        read_into(this->featmap_scaletable_i8_->mutable_cpu_data(), sizeof(float));
    } else {
        NOT_IMPLEMENTED;
    }
    return mem;
}

template <typename Dtype>
int operation_innerproduct<Dtype>::init_weights() {
    std::default_random_engine e;
    std::normal_distribution<float> n(0, 0.3);
    const int dev = this->params_.device_;
    this->weights_f32_.push_back(vec_tensor<float>(weight_data_size_, dev));
    float* w = this->weights_f32_[0]->mutable_cpu_data();
    for (int i = 0; i < weight_data_size_; ++i) w[i] = n(e);
    int mem = weight_data_size_ * sizeof(float);
    if (bias_term_) {
        this->weights_f32_.push_back(vec_tensor<float>(num_output_, dev));
        float* b = this->weights_f32_[1]->mutable_cpu_data();
        for (int i = 0; i < num_output_; ++i) b[i] = n(e);
        mem += num_output_ * sizeof(float);
    }
    return mem;
}

// Y[m,n] = sum_k X[m,k] W[n,k] (+ b[n]); when exactly two of (C,H,W) differ from 1 the reference treats the H rows
// of each image as a batch of W-long vectors and adds no bias (src/Excalibur/operation_innerproduct.cpp:197-212).
template <typename Dtype>
void operation_innerproduct<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    require_nchw(bottoms[0]->order());
    if (this->weights_f32_.empty()) NOT_IMPLEMENTED << " (int8 InnerProduct has no CPU counterpart in the reference)";
    const int dev = this->params_.device_;
    const int m = bottoms[0]->num(), n = num_output_, c = bottoms[0]->channels(), h = bottoms[0]->height(), w = bottoms[0]->width();
    const float* bias = bias_term_ ? this->weights_f32_[1]->gpu_data() : nullptr;
    const int dims = (w == 1 ? 0 : 1) + (h == 1 ? 0 : 1) + (c == 1 ? 0 : 1);
    if (dims == 2) {
        tops[0] = new_tensor<float>({m, 1, h, n}, dev);
        for (int i = 0; i < m; ++i)
            EXHIP_FATAL(exhip_innerproduct_f32(this->ctx(), bottoms[0]->gpu_data() + bottoms[0]->offset(i), this->weights_f32_[0]->gpu_data(),
                                               nullptr, tops[0]->mutable_gpu_data() + tops[0]->offset(i), h, n, w));
        return;
    }
    const int k = bottoms[0]->count(1, 4);
    CHECK_EQ(k * n, weight_data_size_);
    tops[0] = new_tensor<float>({m, n, 1, 1}, dev);
    EXHIP_FATAL(exhip_innerproduct_f32(this->ctx(), bottoms[0]->gpu_data(), this->weights_f32_[0]->gpu_data(), bias,
                                       tops[0]->mutable_gpu_data(), m, n, k));
}

template <typename Dtype>
void operation_innerproduct<Dtype>::forward_gpu_i8(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    require_nchw(bottoms[0]->order());
    if (this->weights_i8_.empty()) {  // a float blob in a layer flagged int8: the float path
        forward_gpu_f32(bottoms, tops);
        return;
    }
    const int dev = this->params_.device_;
    const int m = bottoms[0]->num(), n = num_output_, k = bottoms[0]->count(1, 4);
    CHECK_EQ(k * n, weight_data_size_);
    const float fs = this->featmap_scaletable_i8_->cpu_data()[0];
    if (!scale_dev_) {
        const float ws = this->weights_scaletable_i8_->cpu_data()[0];
        volatile float prod = ws * fs;  // float product, then float division, as for the convolution
        const float s = std::fabs(ws) <= 1e-6 ? 0.f : 1.0f / prod;
        scale_dev_ = vec_tensor<float>(n, dev);
        for (int i = 0; i < n; ++i) scale_dev_->mutable_cpu_data()[i] = s;
    }
    exhip_conv_desc d;
    std::memset(&d, 0, sizeof(d));
    d.n = m; d.c = k; d.h = 1; d.w = 1; d.k = n; d.kh = d.kw = 1; d.sh = d.sw = 1;
    d.c_stride = k; d.k_stride = n;
    tops[0] = new_tensor<float>({m, n, 1, 1}, dev);
    EXHIP_FATAL(exhip_conv2d_direct_nchw(this->ctx(), &d, 1, bottoms[0]->gpu_data(), nullptr,
                                         reinterpret_cast<const int8_t*>(this->weights_i8_[0]->gpu_data()), fs, scale_dev_->gpu_data(),
                                         bias_term_ ? this->weights_f32_[1]->gpu_data() : nullptr, tops[0]->mutable_gpu_data()));
}

template <typename Dtype>
void operation_innerproduct<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const int dev = this->params_.device_;
    tensor_list<float> fb(1), ft(1);
    const half_ptr in = as_nchw(this->ctx(), bottoms[0], dev);  // the flattening order is NCHW's
    fb[0] = std::make_shared<tensor<float>>(in->data_shape(), dev, in->order());
    EXHIP_FATAL(exhip_f16_to_f32(this->ctx(), in->gpu_data(), fb[0]->mutable_gpu_data(), fb[0]->count()));
    forward_gpu_f32(fb, ft);
    tops[0] = std::make_shared<tensor<unsigned short>>(ft[0]->data_shape(), dev, ft[0]->order());
    EXHIP_FATAL(exhip_f32_to_f16(this->ctx(), ft[0]->gpu_data(), tops[0]->mutable_gpu_data(), ft[0]->count()));
}

// ------------------------------------------------------------------ default fp16 layer
template <typename Dtype>
void operation<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    tensor_list<float> in32, out32(tops.size());
    for (const auto& blob : bottoms) {
        const half_ptr b = as_nchw(ctx(), blob, params_.device_);  // the float layers take NCHW
        auto f = std::make_shared<tensor<float>>(b->data_shape(), params_.device_, b->order());
        EXHIP_FATAL(exhip_f16_to_f32(ctx(), b->gpu_data(), f->mutable_gpu_data(), f->count()));
        in32.push_back(f);
    }
    forward_gpu_f32(in32, out32);
    for (size_t i = 0; i < tops.size(); ++i) {
        tops[i] = std::make_shared<tensor<unsigned short>>(out32[i]->data_shape(), params_.device_, out32[i]->order());
        EXHIP_FATAL(exhip_f32_to_f16(ctx(), out32[i]->gpu_data(), tops[i]->mutable_gpu_data(), tops[i]->count()));
    }
}
template void operation<float>::forward_gpu_f16(const tensor_list<unsigned short>&, tensor_list<unsigned short>&);
template void operation<unsigned short>::forward_gpu_f16(const tensor_list<unsigned short>&, tensor_list<unsigned short>&);

// ------------------------------------------------------------------ activation / glue layers
template <typename Dtype>
operation_unary<Dtype>::operation_unary(const operation_param& param, int op, float alpha, float beta, int n_keys)
    : operation<Dtype>(param), op_(op), alpha_(alpha), beta_(beta) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0 && n_keys >= 1) alpha_ = a.as_float();
        else if (key == 1 && n_keys >= 2) beta_ = a.as_float();
        else if (key != -23330) LOG(FATAL) << "Un-supported " << param.type_ << " Attribution " << a.key;
    }
}

template <typename Dtype>
void operation_unary<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        tops[i] = std::make_shared<tensor<float>>(bottoms[i]->data_shape(), this->params_.device_, bottoms[i]->order());
        EXHIP_FATAL(exhip_unary_f32(this->ctx(), op_, bottoms[i]->gpu_data(), tops[i]->mutable_gpu_data(), tops[i]->count(), alpha_, beta_));
    }
}

template <typename Dtype>
void operation_unary<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        tops[i] = std::make_shared<tensor<unsigned short>>(bottoms[i]->data_shape(), this->params_.device_, bottoms[i]->order());
        EXHIP_FATAL(exhip_unary_f16(this->ctx(), op_, bottoms[i]->gpu_data(), tops[i]->mutable_gpu_data(), tops[i]->count(), alpha_, beta_));
    }
}

template <typename Dtype>
operation_prelu<Dtype>::operation_prelu(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) {
            num_slope_ = a.as_int();
            CHECK_GE(num_slope_, 1);
            share_channel_ = num_slope_ == 1;
        } else if (key != -23330) {
            LOG(FATAL) << "Un-supported PReLU Attribution " << a.key;
        }
    }
    this->params_.inplace_ = true;
}

template <typename Dtype>
int operation_prelu<Dtype>::init_weights(FILE* fp) {
    this->weights_f32_.push_back(vec_tensor<float>(num_slope_, this->params_.device_));
    if (std::fread(this->weights_f32_[0]->mutable_cpu_data(), sizeof(float), num_slope_, fp) != static_cast<size_t>(num_slope_))
        LOG(FATAL) << "PReLU: model file too short";
    return num_slope_ * static_cast<int>(sizeof(float));
}

template <typename Dtype>
int operation_prelu<Dtype>::init_weights() {
    this->weights_f32_.push_back(vec_tensor<float>(num_slope_, this->params_.device_));
    // dummy weights as the reference draws them (src/Excalibur/operation_prelu.cpp:45-55): |N(0, 0.3)| from a
    // default-seeded engine
    std::default_random_engine e;
    std::normal_distribution<float> n(0, 0.3);
    float* s = this->weights_f32_[0]->mutable_cpu_data();
    for (int i = 0; i < num_slope_; ++i) s[i] = std::fabs(n(e));
    return num_slope_ * static_cast<int>(sizeof(float));
}

template <typename Dtype>
void operation_prelu<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        const auto& b = bottoms[i];
        if (b->order() != memory::NCHW) NOT_IMPLEMENTED;
        if (!share_channel_) CHECK_EQ(b->channels(), num_slope_);
        tops[i] = std::make_shared<tensor<float>>(b->data_shape(), this->params_.device_, b->order());
        EXHIP_FATAL(exhip_channelwise_f32(this->ctx(), EXHIP_CHANNEL_PRELU, b->gpu_data(), tops[i]->mutable_gpu_data(), b->num(), b->channels(),
                                          b->height() * b->width(), this->weights_f32_[0]->gpu_data(), nullptr, share_channel_ ? 1 : 0));
    }
}

template <typename Dtype>
void operation_prelu<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        const auto& b = bottoms[i];
        if (!share_channel_) CHECK_EQ(b->channels(), num_slope_);
        tops[i] = std::make_shared<tensor<unsigned short>>(b->data_shape(), this->params_.device_, b->order());
        if (b->order() == memory::NHWC) {
            EXHIP_FATAL(exhip_channelwise_nhwc_f16(this->ctx(), EXHIP_CHANNEL_PRELU, b->gpu_data(), tops[i]->mutable_gpu_data(),
                                                   static_cast<size_t>(b->num()) * b->height() * b->width(), b->channels(),
                                                   this->weights_f32_[0]->gpu_data(), nullptr, share_channel_ ? 1 : 0));
            continue;
        }
        EXHIP_FATAL(exhip_channelwise_f16(this->ctx(), EXHIP_CHANNEL_PRELU, b->gpu_data(), tops[i]->mutable_gpu_data(), b->num(), b->channels(),
                                          b->height() * b->width(), this->weights_f32_[0]->gpu_data(), nullptr, share_channel_ ? 1 : 0));
    }
}

template <typename Dtype>
operation_batchnorm<Dtype>::operation_batchnorm(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) channels_ = a.as_int();
        else if (key == 1) eps_ = static_cast<float>(std::atof(a.value.c_str()));
        else LOG(FATAL) << "Un-supported Batchnorm Attribution " << a.key;
    }
    this->params_.inplace_ = true;
}

// a = bias - slope*mean/sqrt(var + eps), b = slope/sqrt(var + eps) in float, the root taken in double
// (src/Excalibur/operation_batchnorm.cpp:52-64)
template <typename Dtype>
void operation_batchnorm<Dtype>::fold() {
    const float *slope = this->weights_f32_[0]->cpu_data(), *mean = this->weights_f32_[1]->cpu_data(),
                *var = this->weights_f32_[2]->cpu_data(), *bias = this->weights_f32_[3]->cpu_data();
    a_ = vec_tensor<float>(channels_, this->params_.device_);
    b_ = vec_tensor<float>(channels_, this->params_.device_);
    float *a = a_->mutable_cpu_data(), *b = b_->mutable_cpu_data();
    for (int i = 0; i < channels_; ++i) {
        volatile float sum = var[i] + eps_;
        const float sqrt_var = static_cast<float>(std::sqrt(static_cast<double>(sum)));
        volatile float prod = slope[i] * mean[i];
        volatile float quot = prod / sqrt_var;
        a[i] = bias[i] - quot;
        b[i] = slope[i] / sqrt_var;
    }
}

template <typename Dtype>
int operation_batchnorm<Dtype>::init_weights(FILE* fp) {
    for (int k = 0; k < 4; ++k) {
        this->weights_f32_.push_back(vec_tensor<float>(channels_, this->params_.device_));
        if (std::fread(this->weights_f32_[k]->mutable_cpu_data(), sizeof(float), channels_, fp) != static_cast<size_t>(channels_))
            LOG(FATAL) << "BatchNorm: model file too short";
    }
    fold();
    return channels_ * static_cast<int>(sizeof(float)) * 4;
}

template <typename Dtype>
int operation_batchnorm<Dtype>::init_weights() {
    // dummy weights as the reference draws them (src/Excalibur/operation_batchnorm.cpp:69-121): slope, mean, var and
    // bias are N(0, 0.3) from one default-seeded engine; a negative var gives NaN there and here
    std::default_random_engine e;
    std::normal_distribution<float> n(0, 0.3);
    for (int k = 0; k < 4; ++k) {
        this->weights_f32_.push_back(vec_tensor<float>(channels_, this->params_.device_));
        float* p = this->weights_f32_[k]->mutable_cpu_data();
        for (int i = 0; i < channels_; ++i) p[i] = n(e);
    }
    fold();
    return channels_ * static_cast<int>(sizeof(float)) * 4;
}

template <typename Dtype>
void operation_batchnorm<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        const auto& b = bottoms[i];
        if (b->order() != memory::NCHW) NOT_IMPLEMENTED;
        CHECK_EQ(b->channels(), channels_);
        tops[i] = std::make_shared<tensor<float>>(b->data_shape(), this->params_.device_, b->order());
        EXHIP_FATAL(exhip_channelwise_f32(this->ctx(), EXHIP_CHANNEL_BATCHNORM, b->gpu_data(), tops[i]->mutable_gpu_data(), b->num(),
                                          b->channels(), b->height() * b->width(), a_->gpu_data(), b_->gpu_data(), 0));
    }
}

template <typename Dtype>
void operation_batchnorm<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        const auto& b = bottoms[i];
        CHECK_EQ(b->channels(), channels_);
        tops[i] = std::make_shared<tensor<unsigned short>>(b->data_shape(), this->params_.device_, b->order());
        if (b->order() == memory::NHWC) {
            const size_t pixels = static_cast<size_t>(b->num()) * b->height() * b->width();
            if (post_unary_ >= 0 && bottoms.size() == 1 && b->channels() % 8 == 0) {
                const unsigned short* src = b->gpu_data();
                const int ch = b->channels();
                EXHIP_FATAL(exhip_concat_batchnorm_unary_nhwc_f16(this->ctx(), &src, &ch, 1, pixels, a_->gpu_data(), b_->gpu_data(), post_unary_,
                                                                  post_alpha_, post_beta_, tops[i]->mutable_gpu_data()));
                post_used_ = true;
                continue;
            }
            EXHIP_FATAL(exhip_channelwise_nhwc_f16(this->ctx(), EXHIP_CHANNEL_BATCHNORM, b->gpu_data(), tops[i]->mutable_gpu_data(), pixels,
                                                   b->channels(), a_->gpu_data(), b_->gpu_data(), 0));
            continue;
        }
        EXHIP_FATAL(exhip_channelwise_f16(this->ctx(), EXHIP_CHANNEL_BATCHNORM, b->gpu_data(), tops[i]->mutable_gpu_data(), b->num(),
                                          b->channels(), b->height() * b->width(), a_->gpu_data(), b_->gpu_data(), 0));
    }
}

template <typename Dtype>
operation_input<Dtype>::operation_input(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) w_ = a.as_int();
        else if (key == 1) h_ = a.as_int();
        else if (key == 2) c_ = a.as_int();
        else if (key == 3) {
            for (const std::string& v : split_string(a.value, ",")) means_.push_back(static_cast<float>(std::atof(v.c_str())));
        } else if (key == 4) {
            for (const std::string& v : split_string(a.value, ",")) vars_.push_back(static_cast<float>(std::atof(v.c_str())));
            if (c_ != 1 && c_ != static_cast<int>(vars_.size())) {  // one scale given for several channels (:42-48)
                if (!vars_.empty()) vars_.resize(1);
                for (int i = 1; i < c_; ++i) vars_.push_back(vars_[0]);
            }
        } else if (key != -23330) {
            LOG(FATAL) << "Un-supported Input Attribution " << a.key;
        }
    }
}

template <typename Dtype>
void operation_input<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        const auto& b = bottoms[i];
        const int ch = b->channels();
        if (ch != 1 && ch != 3) LOG(FATAL) << "Un-supprted channel num: " << ch;
        if (b->order() != memory::NCHW) NOT_IMPLEMENTED;
        CHECK_EQ(static_cast<size_t>(ch), means_.size());
        CHECK_GE(vars_.size(), static_cast<size_t>(ch));
        if (!means_dev_) {
            means_dev_ = vec_tensor<float>(ch, this->params_.device_);
            vars_dev_ = vec_tensor<float>(ch, this->params_.device_);
            for (int c = 0; c < ch; ++c) {
                means_dev_->mutable_cpu_data()[c] = means_[c];
                vars_dev_->mutable_cpu_data()[c] = vars_[c];
            }
        }
        tops[i] = std::make_shared<tensor<float>>(b->data_shape(), this->params_.device_, b->order());
        EXHIP_FATAL(exhip_channelwise_f32(this->ctx(), EXHIP_CHANNEL_INPUT, b->gpu_data(), tops[i]->mutable_gpu_data(), b->num(), ch,
                                          b->height() * b->width(), means_dev_->gpu_data(), vars_dev_->gpu_data(), 0));
    }
}

template <typename Dtype>
void operation_input<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        const half_ptr b = as_nchw(this->ctx(), bottoms[i], this->params_.device_);
        const int ch = b->channels();
        if (ch != 1 && ch != 3) LOG(FATAL) << "Un-supprted channel num: " << ch;
        CHECK_EQ(static_cast<size_t>(ch), means_.size());
        CHECK_GE(vars_.size(), static_cast<size_t>(ch));
        if (!means_dev_) {
            means_dev_ = vec_tensor<float>(ch, this->params_.device_);
            vars_dev_ = vec_tensor<float>(ch, this->params_.device_);
            for (int c = 0; c < ch; ++c) {
                means_dev_->mutable_cpu_data()[c] = means_[c];
                vars_dev_->mutable_cpu_data()[c] = vars_[c];
            }
        }
        tops[i] = std::make_shared<tensor<unsigned short>>(b->data_shape(), this->params_.device_, b->order());
        EXHIP_FATAL(exhip_channelwise_f16(this->ctx(), EXHIP_CHANNEL_INPUT, b->gpu_data(), tops[i]->mutable_gpu_data(), b->num(), ch,
                                          b->height() * b->width(), means_dev_->gpu_data(), vars_dev_->gpu_data(), 0));
    }
}

template <typename Dtype>
operation_concat<Dtype>::operation_concat(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) axis_ = static_cast<int>(std::atof(a.value.c_str()));
        else if (key != -23330) LOG(FATAL) << "Un-supported Concat Attribution " << a.key;
    }
}

template <typename Dtype>
void operation_concat<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_GE(bottoms.size(), 2);
    CHECK_EQ(tops.size(), 1);
    const int concat_axis = axis_ + 2;  // the files store the axis shifted (src/Excalibur/operation_concat.cpp:36-40)
    if (concat_axis != 1 || bottoms[0]->order() != memory::NCHW) NOT_IMPLEMENTED << " Concat along axis " << concat_axis;
    std::vector<const float*> ptrs;
    std::vector<int> channels;
    int total = 0;
    for (const auto& b : bottoms) {
        CHECK_EQ(b->num(), bottoms[0]->num());
        CHECK_EQ(b->height(), bottoms[0]->height());
        CHECK_EQ(b->width(), bottoms[0]->width());
        ptrs.push_back(b->gpu_data());
        channels.push_back(b->channels());
        total += b->channels();
    }
    const auto& b0 = bottoms[0];
    tops[0] = new_tensor<float>({b0->num(), total, b0->height(), b0->width()}, this->params_.device_);
    EXHIP_FATAL(exhip_concat_channels_f32(this->ctx(), ptrs.data(), channels.data(), static_cast<int>(ptrs.size()), b0->num(),
                                          b0->height() * b0->width(), tops[0]->mutable_gpu_data()));
}

template <typename Dtype>
void operation_concat<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_GE(bottoms.size(), 2);
    CHECK_EQ(tops.size(), 1);
    bool nhwc = axis_ + 2 == 1 && bottoms.size() <= 8;
    for (const auto& b : bottoms) nhwc = nhwc && nhwc_channels_ok(b->channels());
    if (!nhwc) {
        operation<Dtype>::forward_gpu_f16(bottoms, tops);  // convert, float kernel, convert back
        return;
    }
    const int dev = this->params_.device_;
    tensor_list<unsigned short> in;
    std::vector<const unsigned short*> ptrs;
    std::vector<int> channels;
    int total = 0;
    for (const auto& blob : bottoms) {
        const half_ptr b = as_nhwc(this->ctx(), blob, dev);
        CHECK_EQ(b->num(), bottoms[0]->num());
        CHECK_EQ(b->height(), bottoms[0]->height());
        CHECK_EQ(b->width(), bottoms[0]->width());
        in.push_back(b);
        ptrs.push_back(b->gpu_data());
        channels.push_back(b->channels());
        total += b->channels();
    }
    const auto& b0 = in[0];
    tops[0] = new_tensor<unsigned short>({b0->num(), b0->height(), b0->width(), total}, dev, memory::NHWC);
    const size_t pixels = static_cast<size_t>(b0->num()) * b0->height() * b0->width();
    if (post_set_) {
        EXHIP_FATAL(exhip_concat_batchnorm_unary_nhwc_f16(this->ctx(), ptrs.data(), channels.data(), static_cast<int>(ptrs.size()), pixels,
                                                          post_bn_a_, post_bn_b_, post_unary_, post_alpha_, post_beta_,
                                                          tops[0]->mutable_gpu_data()));
        post_used_ = true;
        return;
    }
    EXHIP_FATAL(exhip_concat_channels_nhwc_f16(this->ctx(), ptrs.data(), channels.data(), static_cast<int>(ptrs.size()), pixels,
                                               tops[0]->mutable_gpu_data()));
}

template <typename Dtype>
operation_interp<Dtype>::operation_interp(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        switch (std::atoi(a.key.c_str())) {
        case 0: resize_type_ = a.as_int(); break;
        case 1: width_scale_ = a.as_float(); break;   // sic: key 1 feeds the width scale (operation_interp.cpp:196-201)
        case 2: height_scale_ = a.as_float(); break;
        case 3: output_width_ = a.as_int(); break;
        case 4: output_height_ = a.as_int(); break;
        case 6: align_corner_ = a.as_int(); break;
        default: LOG(FATAL) << "Un-supported Interp Attribution " << a.key;
        }
    }
}

template <typename Dtype>
void operation_interp<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const auto& b = bottoms[0];
    if (resize_type_ != 1 || align_corner_ != 0 || b->order() != memory::NCHW) NOT_IMPLEMENTED << " Interp type " << resize_type_;
    int oh = output_height_, ow = output_width_;
    if (oh == 0 || ow == 0) {
        oh = static_cast<int>(b->height() * height_scale_);
        ow = static_cast<int>(b->width() * width_scale_);
    }
    tops[0] = new_tensor<float>({b->num(), b->channels(), oh, ow}, this->params_.device_);
    EXHIP_FATAL(exhip_interp_nearest_f32(this->ctx(), b->gpu_data(), tops[0]->mutable_gpu_data(), b->num(), b->channels(), b->height(),
                                         b->width(), oh, ow));
}

template <typename Dtype>
void operation_interp<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const auto& blob = bottoms[0];
    if (resize_type_ != 1 || align_corner_ != 0 || !nhwc_channels_ok(blob->channels())) {
        operation<Dtype>::forward_gpu_f16(bottoms, tops);  // convert, float kernel, convert back
        return;
    }
    const int dev = this->params_.device_;
    const half_ptr b = as_nhwc(this->ctx(), blob, dev);
    int oh = output_height_, ow = output_width_;
    if (oh == 0 || ow == 0) {
        oh = static_cast<int>(b->height() * height_scale_);
        ow = static_cast<int>(b->width() * width_scale_);
    }
    tops[0] = new_tensor<unsigned short>({b->num(), oh, ow, b->channels()}, dev, memory::NHWC);
    EXHIP_FATAL(exhip_interp_nearest_nhwc_f16(this->ctx(), b->gpu_data(), tops[0]->mutable_gpu_data(), b->num(), b->channels(),
                                              b->height(), b->width(), oh, ow));
}

template <typename Dtype>
void operation_yolov5focus<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const auto& b = bottoms[0];
    if (b->order() != memory::NCHW) NOT_IMPLEMENTED;
    tops[0] = new_tensor<float>({b->num(), b->channels() * 4, b->height() / 2, b->width() / 2}, this->params_.device_);
    EXHIP_FATAL(exhip_focus_f32(this->ctx(), b->gpu_data(), tops[0]->mutable_gpu_data(), b->num(), b->channels(), b->height(), b->width()));
}

// The fp16 pipeline's form: the layer only moves values, so it moves the halves (NCHW, as the float layer).
template <typename Dtype>
void operation_yolov5focus<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const half_ptr b = as_nchw(this->ctx(), bottoms[0], this->params_.device_);
    tops[0] = new_tensor<unsigned short>({b->num(), b->channels() * 4, b->height() / 2, b->width() / 2}, this->params_.device_);
    EXHIP_FATAL(exhip_focus_f16(this->ctx(), b->gpu_data(), tops[0]->mutable_gpu_data(), b->num(), b->channels(), b->height(), b->width()));
}

template <typename Dtype>
operation_reshape<Dtype>::operation_reshape(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) w_ = a.as_int();
        else if (key == 1) h_ = a.as_int();
        else if (key == 2) c_ = a.as_int();
        else if (key == 3) permute_ = a.as_int();
        else if (key != -23330) LOG(FATAL) << "Un-supported Reshape Attribution " << a.key;
    }
    this->params_.inplace_ = true;
}

template <typename Dtype>
std::vector<int> operation_reshape<Dtype>::new_shape(const std::vector<int>& old_shape, int count) const {
    std::vector<int> shape = old_shape;
    if (n_ > 0) shape[0] = n_;
    if (c_ > 0) shape[1] = c_;
    if (h_ > 0) shape[2] = h_;
    if (w_ > 0) shape[3] = w_;
    // absent or negative dimensions follow from the element count, each from the values the earlier steps left
    auto derive = [&](int axis) {
        int others = 1;
        for (int i = 0; i < 4; ++i)
            if (i != axis) others *= shape[i];
        CHECK_EQ(count % others, 0);
        shape[axis] = count / others;
    };
    if (n_ < 0) derive(0);
    if (c_ < 0) derive(1);
    if (h_ < 0) derive(2);
    if (w_ < 0) derive(3);
    CHECK_EQ(shape[0] * shape[1] * shape[2] * shape[3], count);
    return shape;
}

template <typename Dtype>
void operation_reshape<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    if (bottoms[0]->order() != memory::NCHW) NOT_IMPLEMENTED;
    bottoms[0]->reshape(new_shape(bottoms[0]->data_shape(), static_cast<int>(bottoms[0]->count())));
    tops[0] = bottoms[0];
}

// The fp16 pipeline's form: the NCHW blob itself takes the new shape, as in the float layer; an NHWC blob is brought
// into NCHW order first (a new tensor, which then takes the shape).
template <typename Dtype>
void operation_reshape<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const half_ptr b = as_nchw(this->ctx(), bottoms[0], this->params_.device_);
    b->reshape(new_shape(b->data_shape(), static_cast<int>(b->count())));
    tops[0] = b;
}

template <typename Dtype>
operation_flatten<Dtype>::operation_flatten(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) axis_ = a.as_int();
        else if (key != -23330) LOG(FATAL) << "Un-supported flatten Attribution " << a.key;
    }
}

template <typename Dtype>
void operation_flatten<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const auto& b = bottoms[0];
    const int bw = b->width(), bh = b->height(), bc = b->channels();
    int w = 0, h = 0;
    if (axis_ == 0) { w = 1; h = bw * bh * bc; }
    else if (axis_ == 1) { w = bw; h = bh * bc; }
    else if (axis_ == 2) { w = bw * bh; h = bc; }
    else { w = bw * bh * bc; h = 1; }  // the reference's last test is an assignment: every other axis lands here
    tops[0] = new_tensor<float>({b->num(), 1, h, w}, this->params_.device_);
    EXHIP_FATAL(exhip_memcpy_d2d(this->ctx(), tops[0]->mutable_gpu_data(), b->gpu_data(), b->count() * sizeof(float)));
}

template <typename Dtype>
operation_softmax<Dtype>::operation_softmax(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) axis_ = a.as_int();
        else if (key != 1 && key != -23330) LOG(FATAL) << "Un-supported Softmax Attribution " << a.key;
    }
}

template <typename Dtype>
void operation_softmax<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), tops.size());
    for (size_t i = 0; i < bottoms.size(); ++i) {
        const auto& b = bottoms[i];
        if (b->order() != memory::NCHW) NOT_IMPLEMENTED;
        tops[i] = std::make_shared<tensor<float>>(b->data_shape(), this->params_.device_, b->order());
        EXHIP_FATAL(exhip_softmax_channels_f32(this->ctx(), b->gpu_data(), tops[i]->mutable_gpu_data(), b->num(), b->channels(),
                                               b->height() * b->width()));
    }
}

template <typename Dtype>
operation_transpose<Dtype>::operation_transpose(const operation_param& param) : operation<Dtype>(param) {
    for (const layer_attr& a : parse_attrs(param.specific_params_)) {
        const int key = std::atoi(a.key.c_str());
        if (key == 0) {
            perms_.clear();
            size_t pos = 0;
            while (pos <= a.value.size()) {
                const size_t comma = a.value.find(',', pos);
                const std::string item = a.value.substr(pos, comma == std::string::npos ? std::string::npos : comma - pos);
                if (!item.empty()) perms_.push_back(std::atoi(item.c_str()));
                if (comma == std::string::npos) break;
                pos = comma + 1;
            }
            CHECK_EQ(perms_.size(), 3);
        } else if (key != -23330) {
            LOG(FATAL) << "Un-supported Transpose Attribution " << a.key;
        }
    }
}

template <typename Dtype>
void operation_transpose<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const auto& b = bottoms[0];
    if (b->order() != memory::NCHW) NOT_IMPLEMENTED;
    if (perms_[0] == 0 && perms_[1] == 1 && perms_[2] == 2) {
        tops[0] = bottoms[0];
    } else if (perms_[0] == 1 && perms_[1] == 0 && perms_[2] == 2) {
        tops[0] = new_tensor<float>({b->num(), b->channels(), b->width(), b->height()}, this->params_.device_);
        EXHIP_FATAL(exhip_transpose_hw_f32(this->ctx(), b->gpu_data(), tops[0]->mutable_gpu_data(), b->num() * b->channels(),
                                           b->height(), b->width()));
    } else {
        NOT_IMPLEMENTED << " Transpose order " << perms_[0] << "," << perms_[1] << "," << perms_[2];
    }
}

template <typename Dtype>
void operation_transpose<Dtype>::forward_gpu_f16(const tensor_list<unsigned short>& bottoms, tensor_list<unsigned short>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const half_ptr b = as_nchw(this->ctx(), bottoms[0], this->params_.device_);
    if (perms_[0] == 0 && perms_[1] == 1 && perms_[2] == 2) {
        tops[0] = b;
    } else if (perms_[0] == 1 && perms_[1] == 0 && perms_[2] == 2) {
        tops[0] = new_tensor<unsigned short>({b->num(), b->channels(), b->width(), b->height()}, this->params_.device_);
        EXHIP_FATAL(exhip_transpose_hw_f16(this->ctx(), b->gpu_data(), tops[0]->mutable_gpu_data(), b->num() * b->channels(),
                                           b->height(), b->width()));
    } else {
        NOT_IMPLEMENTED << " Transpose order " << perms_[0] << "," << perms_[1] << "," << perms_[2];
    }
}

template <typename Dtype>
int operation_deconvolution<Dtype>::init_weights(FILE* fp) {
    int tag = 0;
    if (std::fread(&tag, sizeof(int), 1, fp) != 1) LOG(FATAL) << "Deconvolution: model file too short";
    if (tag != 0) NOT_IMPLEMENTED << " quantized Deconvolution";
    int mem = 0;
    this->weights_f32_.push_back(vec_tensor<float>(this->weight_data_size_, this->params_.device_));
    if (std::fread(this->weights_f32_[0]->mutable_cpu_data(), sizeof(float), this->weight_data_size_, fp) !=
        static_cast<size_t>(this->weight_data_size_))
        LOG(FATAL) << "Deconvolution: model file too short";
    mem += this->weight_data_size_ * static_cast<int>(sizeof(float));
    if (this->bias_term_) {
        this->weights_f32_.push_back(vec_tensor<float>(this->output_channel_, this->params_.device_));
        if (std::fread(this->weights_f32_[1]->mutable_cpu_data(), sizeof(float), this->output_channel_, fp) !=
            static_cast<size_t>(this->output_channel_))
            LOG(FATAL) << "Deconvolution: model file too short";
        mem += this->output_channel_ * static_cast<int>(sizeof(float));
    }
    return mem;
}

template <typename Dtype>
int operation_deconvolution<Dtype>::init_weights() {
    if (this->params_.int8_quantization_) NOT_IMPLEMENTED;
    this->weights_f32_.push_back(vec_tensor<float>(this->weight_data_size_, this->params_.device_));
    // dummy weights as the reference draws them (src/Excalibur/operation_deconvolution.cpp:44-76)
    std::default_random_engine e;
    std::normal_distribution<float> n(0, 0.3);
    float* w = this->weights_f32_[0]->mutable_cpu_data();
    for (int i = 0; i < this->weight_data_size_; ++i) w[i] = n(e);
    int mem = this->weight_data_size_ * static_cast<int>(sizeof(float));
    if (this->bias_term_) {
        this->weights_f32_.push_back(vec_tensor<float>(this->output_channel_, this->params_.device_));
        float* b = this->weights_f32_[1]->mutable_cpu_data();
        for (int i = 0; i < this->output_channel_; ++i) b[i] = n(e);
        mem += this->output_channel_ * static_cast<int>(sizeof(float));
    }
    return mem;
}

template <typename Dtype>
void operation_deconvolution<Dtype>::forward_gpu_f32(const tensor_list<float>& bottoms, tensor_list<float>& tops) {
    CHECK_EQ(bottoms.size(), 1);
    CHECK_EQ(tops.size(), 1);
    const auto& b = bottoms[0];
    if (b->order() != memory::NCHW || this->group_ != 1 || this->dilation_h_ != 1 || this->dilation_w_ != 1)
        NOT_IMPLEMENTED << " Deconvolution with groups, dilation or NHWC input";
    const int c = b->channels();
    CHECK_EQ(c * this->output_channel_ * this->kernel_size_h_ * this->kernel_size_w_, this->weight_data_size_);
    const int oh = (b->height() - 1) * this->stride_h_ + this->kernel_size_h_ - (this->pad_top_ + this->pad_bottom_);
    const int ow = (b->width() - 1) * this->stride_w_ + this->kernel_size_w_ - (this->pad_left_ + this->pad_right_);
    tops[0] = new_tensor<float>({b->num(), this->output_channel_, oh, ow}, this->params_.device_);
    EXHIP_FATAL(exhip_deconv2d_f32(this->ctx(), b->gpu_data(), this->weights_f32_[0]->gpu_data(),
                                   this->bias_term_ ? this->weights_f32_[1]->gpu_data() : nullptr, tops[0]->mutable_gpu_data(), b->num(), c,
                                   b->height(), b->width(), this->output_channel_, this->kernel_size_h_, this->kernel_size_w_, this->stride_h_,
                                   this->stride_w_, this->pad_top_, this->pad_bottom_, this->pad_left_, this->pad_right_));
}

INSTANCE_CLASS(operation_general_conv);
INSTANCE_CLASS(operation_convolution);
INSTANCE_CLASS(operation_convolutiondepthwise);
INSTANCE_CLASS(operation_pooling);
INSTANCE_CLASS(operation_eltwise);
INSTANCE_CLASS(operation_binaryop);
INSTANCE_CLASS(operation_relu);
INSTANCE_CLASS(operation_split);
INSTANCE_CLASS(operation_innerproduct);
INSTANCE_CLASS(operation_unary);
INSTANCE_CLASS(operation_hardswish);
INSTANCE_CLASS(operation_leakyrelu);
INSTANCE_CLASS(operation_sigmoid);
INSTANCE_CLASS(operation_hardsigmoid);
INSTANCE_CLASS(operation_prelu);
INSTANCE_CLASS(operation_batchnorm);
INSTANCE_CLASS(operation_input);
INSTANCE_CLASS(operation_concat);
INSTANCE_CLASS(operation_interp);
INSTANCE_CLASS(operation_yolov5focus);
INSTANCE_CLASS(operation_deconvolution);
INSTANCE_CLASS(operation_clip);
INSTANCE_CLASS(operation_reshape);
INSTANCE_CLASS(operation_flatten);
INSTANCE_CLASS(operation_softmax);
INSTANCE_CLASS(operation_transpose);

REGISTE(operation_convolution);
REGISTE(operation_convolutiondepthwise);
REGISTE(operation_pooling);
REGISTE(operation_eltwise);
REGISTE(operation_binaryop);
REGISTE(operation_relu);
REGISTE(operation_split);
REGISTE(operation_innerproduct);
REGISTE(operation_hardswish);
REGISTE(operation_leakyrelu);
REGISTE(operation_sigmoid);
REGISTE(operation_hardsigmoid);
REGISTE(operation_prelu);
REGISTE(operation_batchnorm);
REGISTE(operation_input);
REGISTE(operation_concat);
REGISTE(operation_interp);
REGISTE(operation_yolov5focus);
REGISTE(operation_deconvolution);
REGISTE(operation_clip);
REGISTE(operation_reshape);
REGISTE(operation_flatten);
REGISTE(operation_softmax);
REGISTE(operation_transpose);

}  // namespace excalibur
}  // namespace glasssix
