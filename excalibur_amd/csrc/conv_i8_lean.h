// The 3x3 stride-1 int8 convolution with the fused epilogue as a lean, optionally persistent kernel
// (conv_i8_lean.hip). conv_igemm.hip plans the layer and hands the launch over when the geometry fits.
#pragma once
#include "common.h"

struct exhip_lean_geom {
    int n, h, w, c_bytes, k, oh, ow;     // input / output shape; c_bytes: bytes per input pixel (a multiple of 64)
    int pt, pl;                          // top / left zero padding
    int ph, pw, ih, iw;                  // output patch of a group and its staged input tile, in pixels
    int tiles_x, tiles_y, ktiles;        // patches per image and 64-channel slabs
    int act, post_relu;                  // ReLU before / after the shortcut sum
    float fs_out;                        // scale of the int8 output
};

// A 1x1 convolution of another int8 tensor (stride 1 or 2, no padding, no activation) whose float32 result is the
// shortcut the 3x3 layer adds: a residual block's projection. The kernel accumulates it beside the 3x3 products, from
// the pixels under the patch, and adds it in the epilogue in place of a shortcut tensor read from memory.
struct exhip_lean_proj {
    const int8_t* x;       // NHWC int8, h x w pixels of c_bytes bytes (a multiple of 64); output pixel (y, x) reads (y * stride, x * stride)
    const void* wp;        // the 1x1 layer's packed weights: 64-channel slabs, 64-byte chunks (4 KiB per slab and chunk)
    const float* scale;
    const float* bias;     // may be NULL
    int h, w, c_bytes, stride;
};

// The layers behind the convolution that the epilogue applies (both data types): an activation layer, and a sum layer
// behind it instead of in front of it.
struct exhip_lean_f16_epilogue {
    int post_op;              // 0, or 1 + EXHIP_UNARY_*: the activation layer behind the convolution
    float post_alpha, post_beta;
    int residual_last;        // the shortcut is added behind post_relu / post_op
};

// Returns 0 when launched, EXHIP_ERR_UNSUPPORTED when the geometry is outside what the kernel takes (the caller then
// runs the general kernel), another code on failure. Weights are the general kernel's packing for 64-channel slabs and
// 64-byte channel chunks. `post` (may be NULL): not together with a projection.
int exhip_conv3x3_i8_lean(exhip_ctx* ctx, const exhip_lean_geom& g, const int8_t* x, const void* wp, const float* scale,
                          const float* bias, const float* residual, int8_t* y_q, float* y_f, float* y_nchw,
                          const exhip_lean_proj* proj = nullptr, const exhip_lean_f16_epilogue* post = nullptr);

// The fp16 3x3 stride-1 layer on the same kernel: half operands and result, the general kernel's fp16 epilogue.
int exhip_conv3x3_f16_lean(exhip_ctx* ctx, const exhip_lean_geom& g, const exhip_lean_f16_epilogue& e, const uint16_t* x, const void* wp,
                           const float* bias, const uint16_t* residual, uint16_t* y);
