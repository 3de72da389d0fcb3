/* CPU restatement of the arithmetic of Excalibur's CNN forward hot path.
 *
 * TEST INFRASTRUCTURE ONLY. This is the checker the HIP kernels are compared
 * against. Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py may load it; the product library never links, loads or calls it.
 *
 * Every function states the reference file:line it follows (paths relative to
 * the Excalibur source tree). All tensors are dense NCHW unless noted, weights
 * are OIHW, exactly as the reference holds them at its API boundary
 * (include/Primitives/tensor.hpp:124-134, src/Excalibur/operation_convolution.cpp:78-79).
 *
 * Pinning status (what fixes each function besides this text):
 *   exo_float32_to_int8, exo_quantize      closed form + exhaustive tie cases + reference fixtures
 *   exo_conv2d_i8_acc                      brute-force definition, linearity, 1x1==GEMM, reference fixtures
 *   exo_conv2d_i8 (dequant+bias+act)       reference fixtures (bit-exact) + live reference build
 *   exo_conv2d_f32, exo_innerproduct_f32   float64 direct evaluation, reference fixtures at 1e-4
 *   exo_dwconv_f32                         reference fixtures (bit-exact order) + float64 direct evaluation
 *   exo_pool2d_f32, exo_eltwise_f32,
 *   exo_binaryop_add_f32, exo_relu_f32     reference fixtures (bit-exact)
 *   exo_float2half / exo_half2float        exhaustive round trip over all 65536 halfs + reference fixtures
 *   exo_hardswish / leakyrelu / sigmoid /
 *   hardsigmoid / prelu / batchnorm / input /
 *   concat_channels / interp_nearest       reference fixtures (bit-exact), element counts with and without a vector tail
 *   exo_deconv2d_f32                       float64 evaluation of the definition, reference fixtures at 1e-4
 *   exo_focus_f32                          reference fixture (bit-exact) for one image; further images by the same formula
 *   exo_clip_f32, exo_transpose_hw_f32     reference fixtures (bit-exact)
 *   exo_binaryop_f32                       reference fixtures (bit-exact) for every op and every restated shape pair
 *   exo_softmax_channels_f32               reference fixtures at 1e-4; rows sum to 1, invariance under a shift of the input
 * No function here is "parity unpinned".
 */
#ifndef EXCALIBUR_ORACLE_H_
#define EXCALIBUR_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Geometry of one convolution / pooling window op. */
typedef struct exo_geom {
    int n, c, h, w;          /* input NCHW */
    int k;                   /* output channels */
    int kh, kw, sh, sw;      /* kernel, stride */
    int pt, pb, pl, pr;      /* zero padding: top, bottom, left, right */
    int groups;
} exo_geom;

enum { EXO_ACT_NONE = 0, EXO_ACT_RELU = 1, EXO_ACT_RELU6_ZEROING = 3, EXO_ACT_SIGMOID = 4, EXO_ACT_MISH = 5 };

int exo_out_dim(int in, int pad_a, int pad_b, int kernel, int stride);

int8_t exo_float32_to_int8(float v);
void exo_quantize_f32_i8(const float* x, int8_t* q, int n, int c, int hw, const float* fs, int fs_count);

void exo_conv2d_i8_acc(const int8_t* q, const int8_t* w, int32_t* acc, const exo_geom* g);
float exo_dequant_scale(float ws, float fs);
void exo_dequant_i32_f32(const int32_t* acc, float* y, int n, int k, int hw, const float* ws, int ws_count,
                         const float* fs, int fs_count, const float* bias);
void exo_activation_f32(float* y, long count, int act);
void exo_conv2d_i8(const float* x, const int8_t* w, const float* bias, const float* ws, int ws_count, const float* fs,
                   int fs_count, int act, float* y, int32_t* acc_or_null, const exo_geom* g);

void exo_conv2d_f32(const float* x, const float* w, const float* bias, int act, float* y, const exo_geom* g);

void exo_dw_dequant_weights(const int8_t* w, float* wf, int k, int per_group, const float* ws);
void exo_dwconv_f32(const float* x, const float* w, const float* bias, int act, float* y, const exo_geom* g);

enum { EXO_POOL_MAX = 0, EXO_POOL_AVE = 1 };
int exo_pool_out_dim(int in, int pad_a, int pad_b, int kernel, int stride, int pad_mode);
void exo_pool2d_f32(const float* x, float* y, int n, int c, int h, int w, int type, int kh, int kw, int sh, int sw,
                    int pt, int pb, int pl, int pr, int global, int pad_mode, int count_include_pad);

enum { EXO_ELT_PROD = 0, EXO_ELT_SUM = 1, EXO_ELT_MAX = 2 };
void exo_eltwise_f32(const float* const* inputs, int n_inputs, const float* coeffs, int type, float* y, long count);
void exo_binaryop_add_f32(const float* a, const float* b, float* y, long count);
void exo_relu_f32(const float* x, float* y, long count);

void exo_innerproduct_f32(const float* x, const float* w, const float* bias, float* y, int m, int n_out, int k_in);

uint16_t exo_float32_to_float16(float v);
float exo_float16_to_float32(uint16_t v);
void exo_float2half(const float* x, uint16_t* y, int length);
void exo_half2float(const uint16_t* x, float* y, int length);

void exo_hardswish_f32(const float* x, float* y, long count, float alpha, float beta);
void exo_leakyrelu_f32(const float* x, float* y, long count, float alpha);
void exo_sigmoid_f32(const float* x, float* y, long count);
void exo_hardsigmoid_f32(const float* x, float* y, long count, float alpha, float beta);
void exo_clip_f32(const float* x, float* y, long count, float lo, float hi);
int exo_binaryop_f32(int op, const float* a, const int* a_shape, const float* b, const int* b_shape, float* y, int* y_shape);
void exo_softmax_channels_f32(const float* x, float* y, int n, int c, int hw);
void exo_transpose_hw_f32(const float* x, float* y, long planes, int h, int w);
void exo_prelu_f32(const float* x, float* y, int n, int c, int hw, const float* slope, int shared);
void exo_batchnorm_f32(const float* x, float* y, int n, int c, int hw, const float* slope, const float* mean,
                       const float* var, const float* bias, float eps, float* ab);
void exo_input_f32(const float* x, float* y, int n, int c, int hw, const float* mean, const float* scale);
void exo_concat_channels_f32(const float* const* xs, const int* channels, int n_inputs, int n, int hw, float* y);
void exo_interp_nearest_f32(const float* x, float* y, int n, int c, int h, int w, int oh, int ow);
void exo_focus_f32(const float* x, float* y, int n, int c, int h, int w);

void exo_deconv2d_f32(const float* x, const float* w, const float* bias, float* y, int n, int c, int h, int wd, int k, int kh,
                      int kw, int sh, int sw, int pt, int pb, int pl, int pr);

#ifdef __cplusplus
}
#endif
#endif
