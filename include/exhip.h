/* exhip: C ABI of the MI355X (gfx950) backend for Excalibur's CNN forward hot path.
 *
 * Plain pointers and sizes only. Every function returns 0 on success and a non-zero code on
 * failure (a hipError_t, or EXHIP_ERR_* for argument errors); nothing throws. exhip_last_error()
 * returns a text for the last failure on the calling thread. Device pointers are raw HIP device
 * addresses; the library never owns or frees caller memory.
 *
 * The reference (zhousheng-zser/Excalibur) has no C interface for its operators: each entry below
 * states the C++ member function whose device-side work it replaces (paths relative to the reference
 * tree). The C++ operator classes of this repository (excalibur_amd/host) override the reference's
 * forward_gpu_{f32,f16,i8} virtuals (include/Excalibur/operation.hpp:172-183,268-276,359-370) and call
 * only these functions.
 *
 * Tensor layouts
 *   NCHW f32 / f16 : the reference's boundary layout (include/Primitives/tensor.hpp:124-134), dense.
 *   NHWC i8/f16/f32: internal, channel-fastest with a channel stride `c_stride` >= C elements (pad
 *                    channels hold zeros). Convolution inputs need c_stride * sizeof(elem) to be a
 *                    multiple of 32 bytes, or exactly 4 bytes (i8, C <= 4) / 8 bytes (f16, C <= 4)
 *                    for the packed first-layer form.
 */
#ifndef EXHIP_H_
#define EXHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EXHIP_ERR_ARG 10001        /* invalid argument / unsupported geometry */
#define EXHIP_ERR_UNSUPPORTED 10002

typedef struct exhip_ctx exhip_ctx; /* one device + one stream; not thread-safe, like a reference pipeline */

/* ---- runtime: replaces syncedmem's cudaMalloc/cudaMemcpy use, src/Primitives/syncedmem.cpp:176-276 ---- */
int exhip_init(int device, exhip_ctx** ctx);
int exhip_destroy(exhip_ctx* ctx);
int exhip_malloc(exhip_ctx* ctx, size_t bytes, void** dptr);
int exhip_free(exhip_ctx* ctx, void* dptr);
int exhip_memset(exhip_ctx* ctx, void* dptr, int value, size_t bytes);
int exhip_memcpy_h2d(exhip_ctx* ctx, void* dst, const void* src, size_t bytes);
int exhip_memcpy_d2h(exhip_ctx* ctx, void* dst, const void* src, size_t bytes);
int exhip_memcpy_d2d(exhip_ctx* ctx, void* dst, const void* src, size_t bytes);
int exhip_sync(exhip_ctx* ctx);
const char* exhip_last_error(void);
/* Switches for tests and development (no counterpart in the reference; the library reads nothing from the environment):
 * "force_variant" / "force_chunk" / "force_rs" / "force_abufs" pin the convolution planner's tile variant, channel chunk
 * bytes, filter rows per stage and activation tile buffers, "debug_plan" prints one line per planned layer,
 * "dw_band_rows" pins the depthwise strip kernels' band height, "force_splits" the groups per tile of the convolution's
 * split reduction (1 = never split). 0 (-1 for force_variant) restores the planner's choice. "share_gpu" = 1 tells the
 * planner that launches of several streams overlap on the GPU (it then prefers one more group per CU over fewer rounds
 * of a launch: measured 3 % faster with two forwards in flight, 2 % slower alone; off unless set).
 * "lean" / "lean_cfg" / "lean_wres" / "lean_groups" / "lean_f16" choose the form of the lean 3x3 kernel for int8 / fp16
 * layers (0 = the general kernel), "pw" the fp16 / int8 kernel without staging for pointwise layers and "direct" its
 * form for layers with a filter (1 where it measured faster, 2 wherever it can run, 0 never), "pw_tile" that kernel's wave
 * tile (0 = 32 pixels x 64 channels, 2 = 64 x 64 for large launches), "stem" the one-kernel stem: every form computes
 * the same values.
 * Process-wide; packed weights depend on the first three, so set them before packing. */
int exhip_set_option(const char* name, int value);
int exhip_device_name(exhip_ctx* ctx, char* buf, size_t len);

/* HIP events on the context's stream, for timing kernels where they are launched
 * (the reference times with a host clock, include/Primitives/profiler.hpp:186-226). */
int exhip_event_create(void** ev);
int exhip_event_destroy(void* ev);
int exhip_event_record(exhip_ctx* ctx, void* ev);
int exhip_event_elapsed_ms(void* ev_start, void* ev_stop, float* ms); /* synchronises on ev_stop */

/* A fixed sequence of launches recorded once and replayed as one HIP graph (no counterpart in the reference, whose
 * executor issues one call per layer, src/Excalibur/pipeline.cpp:326-392): between exhip_graph_begin and exhip_graph_end
 * every kernel an entry point of this library launches on the context's stream is recorded instead of run (entry points
 * that copy, fill or synchronise must not be called there); exhip_graph_launch replays the recording with the pointers
 * and sizes it was made with. */
int exhip_graph_begin(exhip_ctx* ctx);
int exhip_graph_end(exhip_ctx* ctx, void** graph_exec);
int exhip_graph_launch(exhip_ctx* ctx, void* graph_exec);
int exhip_graph_destroy(void* graph_exec);

/* ---- layout / precision conversion at the boundary ---- */
/* quantize_float32_to_int8 (src/Excalibur/operation_general_conv.cpp:584-720) fused with NCHW->NHWC:
 * y[n,h,w,c] = sat8(trunc(x[n,c,h,w]*fs +- 0.5)); fs per tensor (fs_per_channel == NULL) or a device
 * array of C per-input-channel scales. Pad channels c in [C, c_stride) are written as 0. */
int exhip_quantize_nchw_f32_to_nhwc_i8(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, float fs,
                                       const float* fs_per_channel, int c_stride, int8_t* y);
/* NCHW f32 -> NHWC f32 / f16 (round to nearest even) with zero pad channels; NCHW f16 -> NHWC f16. */
int exhip_nchw_f32_to_nhwc_f32(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, int c_stride, float* y);
int exhip_nchw_f32_to_nhwc_f16(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, int c_stride, uint16_t* y);
int exhip_nchw_f16_to_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, int n, int c, int h, int w, int c_stride, uint16_t* y);
/* NHWC -> NCHW f32 (drops pad channels). */
int exhip_nhwc_f32_to_nchw_f32(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, int c_stride, float* y);
int exhip_nhwc_f16_to_nchw_f32(exhip_ctx* ctx, const uint16_t* x, int n, int c, int h, int w, int c_stride, float* y);
int exhip_nhwc_f16_to_nchw_f16(exhip_ctx* ctx, const uint16_t* x, int n, int c, int h, int w, int c_stride, uint16_t* y);
/* float2half / half2float on flat arrays (src/Primitives/simd_types.cpp:198-252); round to nearest even. */
int exhip_f32_to_f16(exhip_ctx* ctx, const float* x, uint16_t* y, size_t count);
int exhip_f16_to_f32(exhip_ctx* ctx, const uint16_t* x, float* y, size_t count);

/* ---- dense convolution as an implicit GEMM on MFMA ---- */
enum { EXHIP_I8 = 0, EXHIP_F16 = 1, EXHIP_F32 = 2 };
/* activation codes of the reference's key 9 (src/Excalibur/operation_general_conv.cpp:127-272):
 * 0 none, 1 ReLU, 3 "ReLU6" that zeroes values above 6, 4 sigmoid, 5 mish. */

typedef struct exhip_conv_desc {
    int n, c, h, w;             /* logical input shape */
    int k;                      /* output channels */
    int kh, kw, sh, sw;         /* kernel and stride (dilation 1 only, as the reference's AVX paths) */
    int pt, pb, pl, pr;         /* zero padding top/bottom/left/right */
    int act;                    /* fused activation applied to conv + bias */
    int c_stride;               /* channel stride of the NHWC input, in elements */
    int k_stride;               /* channel stride of the NHWC outputs, in elements (>= k) */
    int post_relu;              /* ReLU applied after the residual add (0/1) */
    float fs_out;               /* scale of the optional int8 output: q = sat8(trunc(v*fs_out +- 0.5)) */
    int post_op;                /* 0, or 1 + EXHIP_UNARY_*: the activation layer behind the convolution, applied to the
                                 * value the convolution layer would have stored (rounded to half first in the fp16
                                 * kernel); with exhip_conv2d_i8_projection and exhip_conv2d_i8_maxpool3x3s2 it must be 0 */
    float post_alpha, post_beta; /* that layer's parameters (operation_hardswish.cpp:32-63, operation_leakyrelu.cpp:31-58) */
    const float* post_slope;    /* post_op == EXHIP_POST_PRELU: the PReLU layer behind the convolution
                                 * (operation_prelu.cpp:57-124), v >= 0 ? v : slope * v with these device-resident
                                 * slopes, one per output channel, or one for all if post_slope_shared */
    int post_slope_shared;
    int residual_last;          /* 1: the shortcut is added behind post_relu / post_op instead of in front of them (a sum
                                 * layer behind the activation layer that follows the convolution) */
    /* exhip_conv2d_i8, 1x1 stride-1 layers with NHWC results only: the BatchNorm layer (operation_batchnorm.cpp:122-156)
     * that follows the layer through a Concat, applied in front of post_op: v = fmaf(post_bn_b[k], v, post_bn_a[k]) with
     * device arrays of k floats (the layer's a / b for this convolution's channels); both NULL = none */
    const float* post_bn_a;
    const float* post_bn_b;
    int exact_k;                /* the same layers: 1 = write channels [0, k) only (k a multiple of 32), no zeros into the
                                 * pad channels up to k_stride: the outputs point into a wider tensor that other layers
                                 * fill beside this one (a Concat's buffer). EXHIP_ERR_UNSUPPORTED where the kernel that
                                 * has these two features cannot take the layer */
} exhip_conv_desc;
#define EXHIP_POST_PRELU 16

/* Output spatial size, (H + pt + pb - kh)/sh + 1 (src/Excalibur/operation_convolution.cpp:270-271). */
int exhip_conv_out_hw(const exhip_conv_desc* d, int* oh, int* ow);

/* Weight pre-packing, the counterpart of the reference's load-time weight transforms
 * (conv3x3s1_winograd23_tr_kernel*, forward_im2col*_tr_kernel, src/Excalibur/operation_convolution.cpp:90-97,136-143).
 * Runs on the host: w is OIHW (int8 / IEEE half bits / float per dtype), `packed` a host buffer of
 * exhip_conv_packed_bytes() bytes that the caller then uploads. */
size_t exhip_conv_packed_bytes(const exhip_conv_desc* d, int dtype);
int exhip_conv_pack_weights(const exhip_conv_desc* d, int dtype, const void* w_oihw, void* packed);

/* operation_convolution::forward_cpu_i8 after quantization (src/Excalibur/operation_convolution.cpp:373-408):
 * acc = int8 x int8 -> int32 convolution; v = fmaf((float)acc, scale[k], bias[k]) (bias NULL = 0);
 * v = act(v); if residual: v += residual[n,oh,ow,k] (NHWC f32, stride k_stride); if post_relu: v = max(0, v).
 * Any non-NULL output is written: y_i8 NHWC (requantized with fs_out, pad channels zeroed),
 * y_f32_nhwc, y_f32_nchw (the reference's boundary layout), acc_nchw (raw int32 accumulators).
 * `scale` is the per-output-channel dequantization scale the host computes exactly as the reference,
 * fabs(ws) <= 1e-6 ? 0 : 1.0f/(ws*fs) (:400-403). */
int exhip_conv2d_i8(exhip_ctx* ctx, const exhip_conv_desc* d, const int8_t* x_nhwc, const void* w_packed,
                    const float* scale, const float* bias, const float* residual_nhwc, int8_t* y_i8_nhwc,
                    float* y_f32_nhwc, float* y_f32_nchw, int32_t* acc_nchw);

/* exhip_conv2d_i8 followed by operation_pooling::forward_cpu_f32's MAX pooling
 * (src/Excalibur/operation_pooling.cpp:80-190) with a 3x3 window and stride 2, in one kernel: the
 * convolution's own output never reaches memory. pool_pt / pool_pl (0 or 1) are the pool's top / left
 * padding, pool_oh x pool_ow its output size (exhip_pool_out_hw); windows are clipped to the convolution's
 * output exactly as the reference clips them. Outputs (either may be NULL): pooled NHWC int8 requantized
 * with d->fs_out, pooled NHWC float32. Needs d->k % 64 == 0, k_stride == k, act 0 or 1; returns
 * EXHIP_ERR_UNSUPPORTED when the layer's packed weights use a tiling the pooled kernel cannot share (the
 * caller then runs exhip_conv2d_i8 and exhip_maxpool2d_nhwc_f32). w_packed is exhip_conv_pack_weights' output. */
int exhip_conv2d_i8_maxpool3x3s2(exhip_ctx* ctx, const exhip_conv_desc* d, int pool_pt, int pool_pl, int pool_oh,
                                 int pool_ow, const int8_t* x_nhwc, const void* w_packed, const float* scale,
                                 const float* bias, int8_t* y_i8_nhwc, float* y_f32_nhwc);

/* A residual block's closing layers in one kernel: the 1x1 projection of the block's input (d_proj: kernel 1, stride 1 or
 * 2, no padding, no activation; operation_convolution::forward_cpu_i8, src/Excalibur/operation_convolution.cpp:373-408),
 * the 3x3 stride-1 convolution d of the block's inner tensor, their sum (BinaryOp ADD, src/Excalibur/operation_binaryop.cpp)
 * and the ReLU behind it (d->post_relu), which the reference runs as four layers (src/Excalibur/pipeline.cpp:326-392).
 * Values are those of exhip_conv2d_i8 for the projection (float32 result) followed by exhip_conv2d_i8 for d with that
 * result as residual_nhwc; the projection's float32 tensor is never stored. Both outputs are required: y_i8_nhwc
 * (requantized with d->fs_out > 0) and y_f32_nhwc. w_packed / w_packed_proj are exhip_conv_pack_weights' outputs for d /
 * d_proj. EXHIP_ERR_UNSUPPORTED, with nothing launched, for shapes outside the kernel's (channel strides not multiples
 * of 64, other activations, launches too small to fill the chip): the caller then issues the two calls. */
int exhip_conv2d_i8_projection(exhip_ctx* ctx, const exhip_conv_desc* d, const int8_t* x_nhwc, const void* w_packed,
                               const float* scale, const float* bias, const exhip_conv_desc* d_proj, const int8_t* x_proj_nhwc,
                               const void* w_packed_proj, const float* scale_proj, const float* bias_proj, int8_t* y_i8_nhwc,
                               float* y_f32_nhwc);

/* The stem of an int8 network in one kernel: quantize_float32_to_int8 of the float32 NCHW input with the per-tensor scale
 * fs_in (src/Excalibur/operation_general_conv.cpp:584-720), the first convolution (operation_convolution::forward_cpu_i8,
 * src/Excalibur/operation_convolution.cpp:373-408) and MAX pooling 3x3 stride 2 (src/Excalibur/operation_pooling.cpp:145-159)
 * as in exhip_conv2d_i8_maxpool3x3s2; neither the quantized input nor the convolution's output reaches memory. d describes
 * the convolution on 4-byte pixels (c <= 4, c_stride 4, kw <= 8, kh 3 / 5 / 7, stride 2, k % 64 == 0, act 0 or 1), w_packed
 * is exhip_conv_pack_weights' output for it. The maximum is taken on the int32 accumulators, which is the reference's
 * result when no dequantization scale is negative: the caller states that with scales_nonnegative != 0.
 * EXHIP_ERR_UNSUPPORTED for anything else (the caller then runs the quantizer and exhip_conv2d_i8_maxpool3x3s2). */
int exhip_stem_f32_conv_i8_maxpool3x3s2(exhip_ctx* ctx, const exhip_conv_desc* d, int pool_pt, int pool_pl, int pool_oh,
                                        int pool_ow, const float* x_f32_nchw, float fs_in, const void* w_packed,
                                        const float* scale, int scales_nonnegative, const float* bias, int8_t* y_i8_nhwc,
                                        float* y_f32_nhwc);

/* operation_convolution::forward_cpu_f32 (src/Excalibur/operation_convolution.cpp:251-329) with fp16
 * storage and f32 accumulation (include/Excalibur/operation.hpp:234-260 describes the fp16 layer):
 * x NHWC f16; outputs NHWC f16 and/or NCHW f16 and/or NCHW f32. residual_nhwc (NHWC f16, the output's shape and
 * stride) is the other operand of the two-input sum layer behind the convolution (operation_eltwise.cpp:43-94 SUM,
 * operation_binaryop.cpp:75-84): added to the layer's result rounded to half, as that layer would read it. */
int exhip_conv2d_f16(exhip_ctx* ctx, const exhip_conv_desc* d, const uint16_t* x_nhwc, const void* w_packed,
                     const float* bias, const uint16_t* residual_nhwc, uint16_t* y_f16_nhwc, uint16_t* y_f16_nchw,
                     float* y_f32_nchw);

/* operation_convolution::forward_cpu_f32 in fp32 (f32 MFMA): x NHWC f32; outputs NHWC and/or NCHW f32. */
int exhip_conv2d_f32(exhip_ctx* ctx, const exhip_conv_desc* d, const float* x_nhwc, const void* w_packed,
                     const float* bias, const float* residual_nhwc, float* y_f32_nhwc, float* y_f32_nchw);

/* Any geometry incl. groups, straight from the definition on NCHW f32 (slow; used for shapes the
 * MFMA path does not take). int8 mode when w_i8 != NULL: quantizes x with fs on the fly and applies
 * fmaf(acc, scale[k], bias[k]); otherwise f32 weights. */
int exhip_conv2d_direct_nchw(exhip_ctx* ctx, const exhip_conv_desc* d, int groups, const float* x, const float* w_f32,
                             const int8_t* w_i8, float fs, const float* scale, const float* bias, float* y);

/* ---- bandwidth-bound operators ---- */
/* operation_convolutiondepthwise::forward_cpu_f32, 3x3 stride 1/2 (src/Excalibur/operation_convolutiondepthwise.cpp:321-626):
 * per pixel three vertical fused multiply-adds per kernel column, then bias + col0 + col1 + col2; act fused.
 * NCHW f32 (boundary layout) and NHWC f16 (between fp16 layers; f32 math, result rounded to half). */
int exhip_dwconv3x3_nchw_f32(exhip_ctx* ctx, const float* x, const float* w9, const float* bias, float* y, int n,
                             int c, int h, int w, int stride, int pt, int pb, int pl, int pr, int act);
int exhip_dwconv3x3_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, const float* w9, const float* bias, uint16_t* y,
                             int n, int c, int h, int w, int c_stride, int stride, int pt, int pb, int pl, int pr,
                             int act);
/* operation_convolutiondepthwise::dequantize_int8 (:195-222): wf = w_i8 * (ws <= 1e-6 ? 0 : 1/ws). */
/* The same followed by the PReLU layer behind it (operation_prelu.cpp:57-124), v >= 0 ? v : slope * v on the value the
 * depthwise layer stores (the rounded half in the f16 form), slopes per channel or one for all; the layer's own activation
 * is none. EXHIP_ERR_UNSUPPORTED for shapes only the general kernel takes: run the two layers one after the other then. */
int exhip_dwconv3x3_nchw_f32_prelu(exhip_ctx* ctx, const float* x, const float* w9, const float* bias, const float* slope,
                                   int slope_shared, float* y, int n, int c, int h, int w, int stride, int pt, int pb, int pl,
                                   int pr);
int exhip_dwconv3x3_nhwc_f16_prelu(exhip_ctx* ctx, const uint16_t* x, const float* w9, const float* bias, const float* slope,
                                   int slope_shared, uint16_t* y, int n, int c, int h, int w, int cs, int stride, int pt, int pb,
                                   int pl, int pr);
int exhip_dw_dequant_weights(exhip_ctx* ctx, const int8_t* w, const float* ws, float* wf, int k, int per_group);

/* operation_pooling::forward_cpu_f32 (src/Excalibur/operation_pooling.cpp:80-208). type 0 max, 1 average.
 * Output size is computed by the caller with exhip_pool_out_hw (pad_mode 0 ceil, 1 floor). */
int exhip_pool_out_hw(int h, int w, int kh, int kw, int sh, int sw, int pt, int pb, int pl, int pr, int pad_mode,
                      int* oh, int* ow);
int exhip_pool2d_nchw_f32(exhip_ctx* ctx, const float* x, float* y, int n, int c, int h, int w, int oh, int ow,
                          int type, int kh, int kw, int sh, int sw, int pt, int pb, int pl, int pr,
                          int count_include_pad);
/* NHWC variants used between fused layers. The int8 one exists because max commutes with the
 * (monotone) quantizer; the f32 one can also emit the requantized int8 copy (y_i8 may be NULL). */
int exhip_maxpool2d_nhwc_f32(exhip_ctx* ctx, const float* x, float* y, int8_t* y_i8, float fs_out, int n, int c,
                             int h, int w, int c_stride, int oh, int ow, int kh, int kw, int sh, int sw, int pt,
                             int pl);
/* The same MAX pooling (operation_pooling.cpp:145-159) on an int8 NHWC tensor, c_stride a multiple of 16: what the layer's
 * float result would quantize to, since max commutes with the monotone quantizer (taps outside the image do not count). */
int exhip_maxpool2d_nhwc_i8(exhip_ctx* ctx, const int8_t* x, int8_t* y, int n, int c, int h, int w, int c_stride, int oh, int ow,
                            int kh, int kw, int sh, int sw, int pt, int pl);
/* The pooling pyramid of a detection network's SPP block (models/yolov5s_simp.phai: three Pooling layers, windows 5 / 9 / 13,
 * stride 1, "same" padding, over one tensor) on the int8 tensor in one launch: y1 = pool_k(x), y2 = pool_k(y1),
 * y3 = pool_k(y2), which are the maxima over windows k, 2k - 1 and 3k - 2 of x (operation_pooling.cpp:145-159: taps outside
 * the image count in no maximum). y3, or y2 and y3, may be NULL. k odd; tensors [n][h][w][cs], cs a multiple of 16. */
int exhip_maxpool_same_pyramid_nhwc_i8(exhip_ctx* ctx, const int8_t* x, int8_t* y1, int8_t* y2, int8_t* y3, int n, int c, int h, int w,
                                       int cs, int k);
int exhip_pool2d_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int h, int w, int c_stride,
                          int oh, int ow, int type, int kh, int kw, int sh, int sw, int pt, int pb, int pl, int pr,
                          int count_include_pad);

/* operation_eltwise::forward_cpu_f32 (src/Excalibur/operation_eltwise.cpp:43-94): type 0 PROD, 1 SUM
 * (coeffs host array or NULL = ones), 2 MAX over n_inputs same-shape device arrays (inputs: host array
 * of device pointers). SUM follows the reference's saxpby rounding (body unfused, last count%8 fused). */
int exhip_eltwise_f32(exhip_ctx* ctx, const float* const* inputs, int n_inputs, const float* coeffs, int type,
                      float* y, size_t count);
/* operation_binaryop equal-shape ADD (src/Excalibur/operation_binaryop.cpp:75-84) with optional fused ReLU
 * (operation_relu, src/Excalibur/operation_relu.cpp:31-81) and optional requantized NHWC/flat int8 copy. */
int exhip_add_f32(exhip_ctx* ctx, const float* a, const float* b, float* y, size_t count, int relu);
int exhip_relu_f32(exhip_ctx* ctx, const float* x, float* y, size_t count);
int exhip_add_f16(exhip_ctx* ctx, const uint16_t* a, const uint16_t* b, uint16_t* y, size_t count, int relu);
int exhip_relu_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, size_t count);

/* operation_binaryop::forward_cpu_f32 beyond the equal-shape add (src/Excalibur/operation_binaryop.cpp:44-199,395-448):
 * op 0 ADD, 1 SUB, 2 MUL, 3 DIV; `large` [n][c][hw] gives the output its shape, `small` is, by mode, the same shape
 * (op(large, small)), one value per image (op(large, value)), [small_n][c] (op(value, large): the reference puts the
 * smaller operand first here) or [small_n][hw] (op(value, large)); its images repeat modulo small_n. */
#define EXHIP_BINARY_EQUAL 0
#define EXHIP_BINARY_PER_IMAGE 1
#define EXHIP_BINARY_PER_CHANNEL 2
#define EXHIP_BINARY_PER_PIXEL 3
int exhip_binaryop_f32(exhip_ctx* ctx, int op, int mode, const float* large, const float* small, float* y, int n, int c, int hw,
                       int small_n);

/* Elementwise activations of the shipped topologies. HardSwish x * clamp(alpha*x + beta, 0, 1)
 * (src/Excalibur/operation_hardswish.cpp:32-63), LeakyReLU (operation_leakyrelu.cpp:31-58), sigmoid evaluated in double
 * (operation_sigmoid.cpp:17-33), HardSigmoid clamp(alpha*x + beta, 0, 1) (operation_hardsigmoid.cpp:33-46). */
#define EXHIP_UNARY_HARDSWISH 0
#define EXHIP_UNARY_LEAKYRELU 1
#define EXHIP_UNARY_SIGMOID 2
#define EXHIP_UNARY_HARDSIGMOID 3
#define EXHIP_UNARY_CLIP 4 /* max(alpha, min(beta, x)), src/Excalibur/operation_clip.cpp:32-58 */
int exhip_unary_f32(exhip_ctx* ctx, int op, const float* x, float* y, size_t count, float alpha, float beta);
/* The same on half storage: the reference's fp16 layer is float2half(op(half2float(x))) (include/Excalibur/operation.hpp:204-266);
 * here in one pass, rounding to nearest even. */
int exhip_unary_f16(exhip_ctx* ctx, int op, const uint16_t* x, uint16_t* y, size_t count, float alpha, float beta);
/* Per-channel layers on NCHW float tensors: PReLU, p0 = slope[c] or one shared slope (operation_prelu.cpp:57-124);
 * BatchNorm as fma(p1[c], x, p0[c]) with a = p0, b = p1 computed at load time (operation_batchnorm.cpp:52-64,122-156);
 * Input (x - p0[c]) * p1[c] (operation_input.cpp:61-151). p0 / p1: device arrays of c floats. */
#define EXHIP_CHANNEL_PRELU 0
#define EXHIP_CHANNEL_BATCHNORM 1
#define EXHIP_CHANNEL_INPUT 2
int exhip_channelwise_f32(exhip_ctx* ctx, int op, const float* x, float* y, int n, int c, int hw, const float* p0,
                          const float* p1, int shared);
/* The same on half storage (float parameters and arithmetic, one rounding to half). */
int exhip_channelwise_f16(exhip_ctx* ctx, int op, const uint16_t* x, uint16_t* y, int n, int c, int hw, const float* p0,
                          const float* p1, int shared);
/* ... and on NHWC half storage with channel stride == c (a multiple of 8): the layout the fp16 pipeline keeps between
 * its convolution, depthwise and pooling layers. */
int exhip_channelwise_nhwc_f16(exhip_ctx* ctx, int op, const uint16_t* x, uint16_t* y, size_t pixels, int c,
                               const float* p0, const float* p1, int shared);
/* Layers that only move or compare values, on those NHWC half blobs (channel counts multiples of 8): Concat along the
 * channels (src/Excalibur/operation_concat.cpp:31-103; inputs: host array of up to 8 device pointers), nearest Interp
 * (operation_interp.cpp:247-268) and the stride-1 max pooling with window k = 5 / 9 / 13 and padding k / 2 of the
 * detection topologies (operation_pooling.cpp:145-159), as a row pass into tmp (same size as x) and a column pass. */
int exhip_concat_channels_nhwc_f16(exhip_ctx* ctx, const uint16_t* const* inputs, const int* channels, int n_inputs,
                                   size_t pixels, uint16_t* y);
/* exhip_concat_channels_nhwc_f16 with the layers a detection topology puts behind its Concat applied on the way:
 * BatchNorm (operation_batchnorm.cpp:122-156; bn_a / bn_b as exhip_channelwise_*'s p0 / p1 for the concatenated
 * channels, both NULL = none) and then an activation layer (unary_op = EXHIP_UNARY_HARDSWISH / LEAKYRELU / HARDSIGMOID /
 * CLIP, -1 = none). The results are those of the separate layers, each of which stores halves: the value is rounded
 * to half after the BatchNorm step when an activation follows. n_inputs = 1: the two layers on one blob. */
int exhip_concat_batchnorm_unary_nhwc_f16(exhip_ctx* ctx, const uint16_t* const* inputs, const int* channels, int n_inputs,
                                          size_t pixels, const float* bn_a, const float* bn_b, int unary_op, float alpha,
                                          float beta, uint16_t* y);
/* The same layers on float32 NHWC blobs (operation_concat.cpp:31-103, operation_batchnorm.cpp:122-156 and the activation
 * layers' forward_cpu_f32), for an int8 network's executor: input i has channels[i] channels (multiples of 4) at a
 * channel stride of strides[i] elements; the result has out_stride elements per pixel (pad channels zero) and is
 * written as float32 (y_f32) and / or as the int8 tensor an int8 convolution's quantizer
 * (operation_general_conv.cpp:584-720) would make of it, q8(v * fs_out) (y_i8); either may be NULL. Without BatchNorm
 * and activation and with one input it is that quantizer on an NHWC blob. */
int exhip_concat_batchnorm_unary_nhwc_f32(exhip_ctx* ctx, const float* const* inputs, const int* channels, const int* strides,
                                          int n_inputs, size_t pixels, const float* bn_a, const float* bn_b, int unary_op,
                                          float alpha, float beta, int out_stride, float* y_f32, int8_t* y_i8, float fs_out);
int exhip_interp_nearest_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int h, int w, int oh, int ow);
int exhip_maxpool_same_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* tmp, uint16_t* y, int n, int c, int h, int w, int k);
/* exhip_maxpool_same_nhwc_f16 for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. The row pass's intermediate tensor
 * lives in a static device array of exhip_static_scratch_bytes() bytes (8 MiB) per GPU instead of a caller workspace;
 * a tensor of more than that many bytes (n*h*w*c*2) is refused with EXHIP_ERR_ARG. The call allocates and frees
 * nothing. All calls on one GPU share that array: calls that overlap on one GPU (two contexts, two threads) race. */
size_t exhip_static_scratch_bytes(void);
int exhip_maxpool_same_nhwc_f16_static(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int h, int w, int k);
/* operation_concat::forward_cpu_f32 along the channel axis (operation_concat.cpp:31-103): inputs is a host array of
 * device pointers to NCHW tensors [n][channels[i]][hw]. */
int exhip_concat_channels_f32(exhip_ctx* ctx, const float* const* inputs, const int* channels, int n_inputs, int n, int hw,
                              float* y);
/* operation_interp::forward_cpu_f32, nearest branch (operation_interp.cpp:247-268). */
int exhip_interp_nearest_f32(exhip_ctx* ctx, const float* x, float* y, int n, int c, int h, int w, int oh, int ow);
/* operation_yolov5focus::forward_cpu_f32 (operation_yolov5focus.cpp:17-50), for every image of the batch
 * (the reference fills image 0 only). y: [n][4c][h/2][w/2]. */
int exhip_focus_f32(exhip_ctx* ctx, const float* x, float* y, int n, int c, int h, int w);
/* The front of an int8 detection network in one pass: the Input layer (src/Excalibur/operation_input.cpp:10-151, host
 * arrays means[c] / scales[c]: (x - mean) * scale), YoloV5Focus (operation_yolov5focus.cpp:12-50) and the first
 * convolution's quantizer (operation_general_conv.cpp:584-720, q8(v * fs)), float32 NCHW -> int8 NHWC. Takes c == 3,
 * c_stride == 32 and even h, w; EXHIP_ERR_UNSUPPORTED otherwise (the caller then runs the three layers). */
int exhip_input_focus_quantize_nchw_f32_to_nhwc_i8(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, const float* means,
                                                   const float* scales, float fs, int c_stride, int8_t* y);
/* A detection head's Reshape (operation_reshape.cpp:8-131) to groups x per_group x pixels followed by the Transpose of the
 * last two axes (operation_transpose.cpp), on the convolution's float32 NHWC result:
 * y[n][g][pixel][j] = x[n][pixel][g * per_group + j]. */
int exhip_nhwc_f32_to_grouped_f32(exhip_ctx* ctx, const float* x, int n, int hw, int groups, int per_group, int c_stride, float* y);
/* The same on half storage: the reference's fp16 layer converts, runs the float layer and converts back
 * (include/Excalibur/operation.hpp:204-266), which for a layer that only moves values is the move itself. */
int exhip_focus_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int h, int w);

/* operation_softmax::forward_cpu_f32, NCHW branch (src/Excalibur/operation_softmax.cpp:36-96): softmax over the channels of
 * every (image, position); x, y [n][c][hw]. */
int exhip_softmax_channels_f32(exhip_ctx* ctx, const float* x, float* y, int n, int c, int hw);
/* operation_transpose::forward_cpu_f32, order (1, 0, 2) (src/Excalibur/operation_transpose.cpp:51-70): rows and columns of
 * each of `planes` planes change places, y[p][i][j] = x[p][j][i]; x [planes][h][w], y [planes][w][h]. */
int exhip_transpose_hw_f32(exhip_ctx* ctx, const float* x, float* y, int planes, int h, int w);
int exhip_transpose_hw_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int planes, int h, int w);  /* on half storage */

/* operation_deconvolution::forward_cpu_f32 (src/Excalibur/operation_deconvolution.cpp:80-171), group 1, dilation 1:
 * x NCHW, w [c][k][kh][kw], y [n][k][(h-1)*sh + kh - pt - pb][(w-1)*sw + kw - pl - pr] = scatter of W^T x (+ bias). */
int exhip_deconv2d_f32(exhip_ctx* ctx, const float* x, const float* w, const float* bias, float* y, int n, int c, int h, int wd,
                       int k, int kh, int kw, int sh, int sw, int pt, int pb, int pl, int pr);

/* operation_innerproduct::forward_cpu_f32 (src/Excalibur/operation_innerproduct.cpp:176-224):
 * y[m,n] = sum_k x[m,k]*w[n,k] + bias[n]; x [m][k_in], w [n_out][k_in] row-major f32. */
int exhip_innerproduct_f32(exhip_ctx* ctx, const float* x, const float* w, const float* bias, float* y, int m,
                           int n_out, int k_in);

#ifdef __cplusplus
}
#endif
#endif /* EXHIP_H_ */
