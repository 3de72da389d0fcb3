// The 1x1 stride-1 fp16 / int8 convolution (a pointwise layer: a matrix product over the flattened pixels) as a kernel
// without LDS staging and without barriers (conv_pw.hip). conv_igemm.hip plans the layer and hands the launch over when the
// geometry fits; the weights are the general kernel's packing.
#pragma once
#include "common.h"

struct exhip_pw_geom {
    long long pixels;           // N * H * W: rows of the NHWC input and output
    int c_bytes;                // bytes per input pixel (channel stride * element size), a multiple of 32
    int k, k_stride;            // output channels and the output's channel stride, in elements
    int slab_blocks, slabs;     // the packing: 32-channel blocks per slab (2 or 4) and slabs
    int act, post_relu, post_op, post_slope_shared;
    int residual_last;          // the shortcut is added behind post_relu / post_op
    float post_alpha, post_beta;
    const float* post_slope;
    float fs_out;               // int8 layers: the scale of the requantized int8 result
    // int8 layers: a BatchNorm layer in front of post_op (device arrays of k floats, both or neither), and whether only
    // channels [0, k) are written (the results point into a wider tensor; k a multiple of 32). Either makes the kernel
    // take the layer whatever its size.
    const float* post_bn_a;
    const float* post_bn_b;
    int exact_k;
};

// A layer with a filter, a stride or padding on the same kernel (`taps` below; NULL: the pointwise layer). The wave's
// pixel fragments then come from the filter's taps around each output pixel -- still straight from the NHWC rows into
// registers, a tap outside the image reading zeros -- in the order of the packing's k-steps. g.pixels counts output pixels.
struct exhip_pw_taps {
    int n, in_h, in_w, out_h, out_w;   // images, input and output maps
    int kh, kw, stride, pad_t, pad_l;  // at most 32 taps
    int n_chunks, chunk_b;             // the packing: channel chunks of chunk_b bytes (a multiple of 32), n_chunks * chunk_b bytes per pixel
};

// Returns 0 when launched, EXHIP_ERR_UNSUPPORTED when the geometry is outside what the kernel takes (the caller then
// runs the general kernel), another code on failure. Semantics as exhip_conv2d_f16 with only the NHWC half output.
int exhip_conv1x1_f16_pw(exhip_ctx* ctx, const exhip_pw_geom& g, const uint16_t* x, const void* wp, const float* bias,
                         const uint16_t* residual, uint16_t* y, const exhip_pw_taps* taps = nullptr);
// The int8 layer: semantics as exhip_conv2d_i8 with the NHWC results only (y_i8 and / or y_f32; k_stride a multiple of 16).
int exhip_conv1x1_i8_pw(exhip_ctx* ctx, const exhip_pw_geom& g, const int8_t* x, const void* wp, const float* scale, const float* bias,
                        const float* residual, int8_t* y_i8, float* y_f32, const exhip_pw_taps* taps = nullptr);
