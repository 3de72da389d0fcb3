// conv1x1_f16_pw_kernel: the pointwise (1x1, stride 1, no padding) fp16 convolution, y[pixel][k] = sum_c x[pixel][c] * w[k][c].
//
// A pointwise layer of a detection or mobile network moves a few tens of MB for a few GFLOP: what it costs is the
// length of one group's chain from launch to last store, and the memory system's rate. So nothing is staged: a wave
// owns 32 * NT pixels x 32 * MT output channels and fetches its MFMA operands straight into registers, 16 bytes per
// lane and k-step -- the weight fragments in the general kernel's packing (one contiguous KiB per 32-channel block and
// k-step), the pixel fragments from the NHWC rows themselves (lane = pixel, the two half-waves the two 16-byte halves
// of a 32-byte k-step). No LDS, no barrier, no tile geometry: the pixels of all images form one list. The four waves of
// a group are neighbours in (pixel tile, channel group) order with the channel group running fastest, so the waves that
// read the same pixels sit on one CU; the pixel rows come from HBM once and from the caches after that.
//
// Arithmetic and roundings are the general kernel's (conv_igemm.hip, general epilogue): float32 accumulation in
// v_mfma_f32_32x32x16_f16, bias, activation, the optional shortcut added to the value rounded to half, ReLU / the
// activation layer behind the convolution applied to the rounded half, one final rounding.
//
// The int8 layer (DT == EXHIP_I8) is the same kernel on the same byte geometry -- a 32-byte k-step is 32 int8 channels,
// v_mfma_i32_32x32x32_i8 on the same 16-byte fragments -- with the int8 epilogue of the general kernel: dequantization
// fmaf((float)acc, scale, bias), activation, float32 shortcut, ReLU / activation layer, float32 NHWC and / or
// requantized int8 NHWC results.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <type_traits>

#include "conv_pw.h"

namespace {

typedef exhip_v4i v4i;
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr unsigned kRsrcWord3 = 0x00020000u;  // raw buffer: out-of-range loads return 0
constexpr int kOutOfRange = 0x7ffff000;       // a lane offset beyond every view
constexpr int kMaxDirectSteps = 40;           // k-steps of a layer with a filter (taps x 32-byte steps per pixel)
constexpr int kTapShift = 27;                 // a step's table entry: byte offset below, tap number above

struct PwParams {
    const char* x;
    const char* wp;
    const float* bias;
    const uint16_t* residual;
    uint16_t* y;
    const float* post_slope;
    // int8 layers: dequantization scales, float32 shortcut, float32 and int8 results
    const float* scale;
    const float* residual_f;
    float* y_f;
    int8_t* y_q;
    float fs_out;
    const float* post_bn_a;   // BatchNorm in front of post_op: fmaf(post_bn_b[ch], v, post_bn_a[ch])
    const float* post_bn_b;
    int exact;                // channels [0, K) only: blocks past K are not written (the results lie inside a wider tensor)
    unsigned pixels, x_bytes, w_bytes;
    unsigned items, ch_groups;   // waves with work; 32 * MT channel groups per pixel tile
    int xs_b;                    // bytes per input pixel
    int n_ksteps;                // 32-byte k-steps per pixel
    int mts;                     // 32-channel blocks per packed slab
    int K, kstride;
    int act, post_relu, post_op, post_slope_shared, residual_last;
    float post_alpha, post_beta;
    // the form with a filter (TAPS): output pixel (img, oy, ox) reads input pixel (oy * stride - pt + r, ox * stride - pl + q)
    // for k-step s of tap r * kw + q, that many bytes behind its top-left input pixel
    int in_h, in_w, out_h, out_w, stride, pad_t, pad_l, kh, kw;
    int step[kMaxDirectSteps];   // offset | tap << kTapShift
};

__device__ __forceinline__ float fast_activation(float v, int act) {
    if (act == 1) return (0.f > v) ? 0.f : v;
    if (act == 3) { const float d = (0.f > v) ? 0.f : v; return d <= 6.f ? d : 0.f; }
    return v;
}
__device__ __noinline__ float slow_activation(float v, int act) { return exhip_act(v, act); }

template <int OP>
__device__ __forceinline__ void post_activation_op(float (&v)[16], float alpha, float beta) {
#pragma unroll
    for (int e = 0; e < 16; ++e) v[e] = unary_value<OP>(exhip_h2f(exhip_f2h(v[e])), alpha, beta);
}

// The bias values of a lane's 16 channels per 32-channel block (zeros beyond K).
template <int MT>
__device__ __forceinline__ void load_bias(const PwParams& p, int kb0, int lane, float (&bi)[MT][16]) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int ch0 = (kb0 + m) * 32 + (lane >> 5) * 16;
#pragma unroll
        for (int e = 0; e < 16; ++e) bi[m][e] = (p.bias && ch0 + e < p.K) ? p.bias[ch0 + e] : 0.f;
    }
}

// Epilogue of one wave tile: a lane holds 16 consecutive channels of its pixel per 32-channel block.
template <int MT, int NT>
__device__ __forceinline__ void pw_epilogue(const PwParams& p, const v16f (&acc)[MT][NT], const unsigned (&pix)[NT], int kb0, int lane,
                                            const float (&bi)[MT][16]) {
    const bool odd = lane & 1;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int ch0 = (kb0 + m) * 32 + (lane >> 5) * 16;
        if (ch0 >= p.kstride && ch0 >= p.K) continue;
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            const bool valid = pix[n] < p.pixels;
            float v[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) v[e] = acc[m][n][e] + bi[m][e];
            if (p.act >= 4) {
#pragma unroll 1
                for (int e = 0; e < 16; ++e) v[e] = slow_activation(v[e], p.act);
            } else if (p.act) {
#pragma unroll
                for (int e = 0; e < 16; ++e) v[e] = fast_activation(v[e], p.act);
            }
            auto add_shortcut = [&]() {
                // the add layer behind this one reads the stored (rounded) half
                const uint16_t* r = p.residual + (size_t)pix[n] * p.kstride + ch0;
                if (ch0 + 16 <= p.K) {
                    const v4i r0 = reinterpret_cast<const v4i*>(r)[0], r1 = reinterpret_cast<const v4i*>(r)[1];
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int word = e < 8 ? r0[e >> 1] : r1[(e - 8) >> 1];
                        v[e] = exhip_h2f(exhip_f2h(v[e])) + exhip_h2f((uint16_t)(((uint32_t)word >> ((e & 1) * 16)) & 0xffff));
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        if (ch0 + e < p.K) v[e] = exhip_h2f(exhip_f2h(v[e])) + exhip_h2f(r[e]);
                }
            };
            if (p.residual && valid && !p.residual_last) add_shortcut();
            if (p.post_relu) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    v[e] = exhip_h2f(exhip_f2h(v[e]));
                    v[e] = (0.f > v[e]) ? 0.f : v[e];
                }
            }
            if (p.post_op == EXHIP_POST_PRELU) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float t = exhip_h2f(exhip_f2h(v[e]));
                    const float slope = p.post_slope[p.post_slope_shared || ch0 + e >= p.K ? 0 : ch0 + e];
                    v[e] = t >= 0.f ? t : slope * t;
                }
            } else if (p.post_op) {
                switch (p.post_op - 1) {
                case EXHIP_UNARY_HARDSWISH: post_activation_op<0>(v, p.post_alpha, p.post_beta); break;
                case EXHIP_UNARY_LEAKYRELU: post_activation_op<1>(v, p.post_alpha, p.post_beta); break;
                case EXHIP_UNARY_HARDSIGMOID: post_activation_op<3>(v, p.post_alpha, p.post_beta); break;
                default: post_activation_op<4>(v, p.post_alpha, p.post_beta); break;
                }
            }
            if (p.residual && valid && p.residual_last) add_shortcut();
#pragma unroll
            for (int e = 0; e < 16; ++e)
                if (ch0 + e >= p.K) v[e] = 0.f;  // pad channels hold zeros
            v4i o[2];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t lo = exhip_f2h(v[2 * e]), hi = exhip_f2h(v[2 * e + 1]);
                o[e >> 2][e & 3] = (int)(lo | (hi << 16));
            }
            char* const yb = reinterpret_cast<char*>(p.y) + ch0 * 2;
            if (ch0 + 16 <= p.kstride) {
                if (__builtin_amdgcn_ballot_w64(valid) == ~0ull) {
                    // the whole wave stores: a lane's 32 bytes and its neighbour's trade halves, so that four lanes (p,
                    // p + 1 and the same two of the other half-wave) write 64 contiguous bytes of one pixel per instruction
                    pair_exchange4(o[0], o[1], odd);
                    const unsigned mine = pix[n], other = (unsigned)lane_neighbour((int)mine);
                    const size_t even_pix = odd ? other : mine, odd_pix = odd ? mine : other;
                    const int sub = odd ? 16 : 0;
                    *reinterpret_cast<v4i*>(yb + even_pix * p.kstride * 2 + sub) = o[0];
                    *reinterpret_cast<v4i*>(yb + odd_pix * p.kstride * 2 + sub) = o[1];
                } else if (valid) {
                    v4i* y = reinterpret_cast<v4i*>(yb + (size_t)pix[n] * p.kstride * 2);
                    y[0] = o[0];
                    y[1] = o[1];
                }
            } else if (valid) {
                uint16_t* y = reinterpret_cast<uint16_t*>(yb + (size_t)pix[n] * p.kstride * 2);
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if (ch0 + e < p.kstride) y[e] = (uint16_t)(((uint32_t)o[e >> 3][(e >> 1) & 3] >> ((e & 1) * 16)) & 0xffff);
            }
            // one 32 x 32 block at a time: interleaving the blocks buys nothing (they do not depend on each other's loads)
            // and costs the registers of their temporaries
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// The int8 layer's epilogue: the general kernel's, value by value.
template <int MT, int NT>
__device__ __forceinline__ void pw_epilogue_i8(const PwParams& p, const v16i (&acc)[MT][NT], const unsigned (&pix)[NT], int kb0, int lane) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int ch0 = (kb0 + m) * 32 + (lane >> 5) * 16;
        if (ch0 >= p.K && (p.exact || ch0 >= p.kstride)) continue;
        // FULL: every channel of the block exists (wave-uniform), and the per-value tests against K fall away
        auto block = [&](auto full_c) {
        constexpr bool FULL = decltype(full_c)::value;
        float sc[16], bi[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            sc[e] = (FULL || ch0 + e < p.K) ? p.scale[ch0 + e] : 0.f;
            bi[e] = (p.bias && (FULL || ch0 + e < p.K)) ? p.bias[ch0 + e] : 0.f;
        }
        const bool vec_ok = ch0 + 16 <= p.kstride;
        float bna[16], bnb[16];  // the BatchNorm's parameters of these channels (identity beyond K)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            bna[e] = (p.post_bn_a && (FULL || ch0 + e < p.K)) ? p.post_bn_a[ch0 + e] : 0.f;
            bnb[e] = (p.post_bn_a && (FULL || ch0 + e < p.K)) ? p.post_bn_b[ch0 + e] : 1.f;
        }
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            const bool valid = pix[n] < p.pixels;
            const size_t at = (size_t)pix[n] * p.kstride + ch0;
            float v[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) v[e] = __builtin_fmaf((float)acc[m][n][e], sc[e], bi[e]);
            if (p.act >= 4) {
#pragma unroll 1
                for (int e = 0; e < 16; ++e) v[e] = slow_activation(v[e], p.act);
            } else if (p.act) {
#pragma unroll
                for (int e = 0; e < 16; ++e) v[e] = fast_activation(v[e], p.act);
            }
            float r[16];
            if (p.residual_f) {
#pragma unroll
                for (int e = 0; e < 16; ++e) r[e] = 0.f;
                if (valid && (FULL || ch0 + 16 <= p.K)) {
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4) {
                        const v4f t = *reinterpret_cast<const v4f*>(p.residual_f + at + e4 * 4);
#pragma unroll
                        for (int e = 0; e < 4; ++e) r[e4 * 4 + e] = t[e];
                    }
                } else if (valid) {
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        if (ch0 + e < p.K) r[e] = p.residual_f[at + e];
                }
            }
            if (p.residual_f && !p.residual_last) {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if (FULL || ch0 + e < p.K) v[e] += r[e];
            }
            if (p.post_relu) {
#pragma unroll
                for (int e = 0; e < 16; ++e) v[e] = (0.f > v[e]) ? 0.f : v[e];
            }
            if (p.post_bn_a) {  // the BatchNorm layer between this layer (through a Concat) and its activation layer
#pragma unroll
                for (int e = 0; e < 16; ++e) v[e] = __builtin_fmaf(bnb[e], v[e], bna[e]);
            }
            if (p.post_op == EXHIP_POST_PRELU) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float slope = p.post_slope[p.post_slope_shared || (!FULL && ch0 + e >= p.K) ? 0 : ch0 + e];
                    v[e] = v[e] >= 0.f ? v[e] : slope * v[e];
                }
            } else if (p.post_op) {
                auto apply = [&](auto op) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) v[e] = unary_value<decltype(op)::value>(v[e], p.post_alpha, p.post_beta);
                };
                switch (p.post_op - 1) {
                case EXHIP_UNARY_HARDSWISH: apply(std::integral_constant<int, 0>{}); break;
                case EXHIP_UNARY_LEAKYRELU: apply(std::integral_constant<int, 1>{}); break;
                case EXHIP_UNARY_HARDSIGMOID: apply(std::integral_constant<int, 3>{}); break;
                default: apply(std::integral_constant<int, 4>{}); break;
                }
            }
            if (p.residual_f && p.residual_last) {
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if (FULL || ch0 + e < p.K) v[e] += r[e];
            }
#pragma unroll
            for (int e = 0; e < 16; ++e)
                if (!FULL && ch0 + e >= p.K) v[e] = 0.f;  // pad channels hold zeros
            if (p.y_f && (kb0 + m) * 32 + 32 <= p.kstride && __builtin_amdgcn_ballot_w64(valid) == ~0ull) {
                // the whole wave stores a whole 32-channel block: the two half-waves trade 16-byte pieces and neighbouring
                // lanes trade pixels, so that four lanes (p, p + 1 and the same two of the other half-wave) write 64
                // contiguous bytes of one pixel per instruction instead of 16-byte pieces of 64 pixels
                v4i o4[4];
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    const v4f o = {v[e4 * 4], v[e4 * 4 + 1], v[e4 * 4 + 2], v[e4 * 4 + 3]};
                    o4[e4] = __builtin_bit_cast(v4i, o);
                }
                const bool odd = lane & 1;
                half_swap4(o4[0], o4[1]);   // o4[0], o4[2]: channels 0-7 and 8-15 of the block; o4[1], o4[3]: 16-23 and 24-31
                half_swap4(o4[2], o4[3]);
                pair_exchange4(o4[0], o4[2], odd);
                pair_exchange4(o4[1], o4[3], odd);
                const unsigned mine = pix[n], other = (unsigned)lane_neighbour((int)mine);
                const size_t even_pix = odd ? other : mine, odd_pix = odd ? mine : other;
                char* const yb = reinterpret_cast<char*>(p.y_f) + (size_t)(kb0 + m) * 128 + (odd ? 32 : 0) + (lane >> 5) * 16;
                *reinterpret_cast<v4i*>(yb + even_pix * p.kstride * 4) = o4[0];
                *reinterpret_cast<v4i*>(yb + even_pix * p.kstride * 4 + 64) = o4[1];
                *reinterpret_cast<v4i*>(yb + odd_pix * p.kstride * 4) = o4[2];
                *reinterpret_cast<v4i*>(yb + odd_pix * p.kstride * 4 + 64) = o4[3];
            } else if (p.y_f && valid) {
                float* y = p.y_f + at;
                if (vec_ok) {
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4) {
                        const v4f o = {v[e4 * 4], v[e4 * 4 + 1], v[e4 * 4 + 2], v[e4 * 4 + 3]};
                        *reinterpret_cast<v4f*>(y + e4 * 4) = o;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        if (ch0 + e < p.kstride) y[e] = v[e];
                }
            }
            if (p.y_q && valid && vec_ok) {
                v4i o;
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    uint32_t w = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) w |= (uint32_t)(exhip_q8(v[e4 * 4 + e] * p.fs_out) & 0xff) << (8 * e);
                    o[e4] = (int)w;
                }
                *reinterpret_cast<v4i*>(p.y_q + at) = o;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        };
        // (the 64 x 64 tile keeps the one general form: with both its epilogue no longer fits the register file)
        if constexpr (MT + NT < 4 || MT == 1) {
            if ((kb0 + m) * 32 + 32 <= p.K) block(std::true_type{});
            else block(std::false_type{});
        } else {
            block(std::false_type{});
        }
    }
}

template <int DT, int MT, int NT, bool TAPS>
__global__ __launch_bounds__(256, 2) void conv1x1_pw_kernel(const PwParams p) {
    constexpr int U = MT + NT > 4 ? 2 : 4;  // k-steps fetched per request round; two rounds are in flight
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // workgroup ids are dealt round-robin to the 8 XCDs: give each XCD one contiguous run of items, so that the channel
    // groups of a pixel tile (and the weights' re-reads) share that XCD's L2
    unsigned bid = blockIdx.x;
    {
        const unsigned per = gridDim.x >> 3;
        if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
    }
    const unsigned item = __builtin_amdgcn_readfirstlane(bid * 4 + wave);
    if (item >= p.items) return;  // wave-uniform; the kernel has no barrier
    const unsigned tile = __builtin_amdgcn_readfirstlane(item / p.ch_groups);
    const int kb0 = __builtin_amdgcn_readfirstlane((int)(item - tile * p.ch_groups) * MT);  // first 32-channel block

    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(p.x), 0, (int)p.x_bytes, kRsrcWord3);
    const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(p.wp), 0, (int)p.w_bytes, kRsrcWord3);

    // pixel fragments: lane = pixel (lane & 31), 16-byte half (lane >> 5) of each 32-byte k-step
    unsigned pix[NT];
    int xoff[NT];
    unsigned taps_in[NT];  // TAPS: bit r * kw + q set where that tap of the pixel lies inside the image
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        pix[nt] = (tile * NT + nt) * 32 + (lane & 31);
        if constexpr (TAPS) {
            // the filter's top-left input pixel; its offset may lie in front of the tensor (padding), the taps inside the
            // image never do, and 32-bit wrap-around of the sum gives their offsets
            const unsigned per_image = (unsigned)(p.out_h * p.out_w);
            const unsigned img = pix[nt] / per_image, rem = pix[nt] - img * per_image;
            const int oy = (int)(rem / (unsigned)p.out_w), ox = (int)(rem - (unsigned)oy * (unsigned)p.out_w);
            const int iy = oy * p.stride - p.pad_t, ix = ox * p.stride - p.pad_l;
            xoff[nt] = (((int)img * p.in_h + iy) * p.in_w + ix) * p.xs_b + (lane >> 5) * 16;
            unsigned m = 0;
            if (pix[nt] < p.pixels) {
                for (int r = 0; r < p.kh; ++r)
                    for (int q = 0; q < p.kw; ++q)
                        if ((unsigned)(iy + r) < (unsigned)p.in_h && (unsigned)(ix + q) < (unsigned)p.in_w) m |= 1u << (r * p.kw + q);
            }
            taps_in[nt] = m;
        } else {
            xoff[nt] = pix[nt] < p.pixels ? (int)(pix[nt] * (unsigned)p.xs_b) + (lane >> 5) * 16 : kOutOfRange;
        }
    }
    // weight fragments: block kb of slab kb / mts lies at ((slab * n_ksteps + ks) * mts + kb % mts) KiB; the MT blocks
    // of a wave are neighbours in one slab (mts is a multiple of MT)
    const int w_step = p.mts * 1024;
    const int w_base = __builtin_amdgcn_readfirstlane(((kb0 / p.mts) * p.n_ksteps * p.mts + kb0 % p.mts) * 1024);
    const int woff = lane * 16;

    typedef typename std::conditional<DT == EXHIP_I8, v16i, v16f>::type acc_t;
    acc_t acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < NT; ++n)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[m][n][e] = 0;

    v4i a[2][U][MT], b[2][U][NT];
    const int nks = p.n_ksteps;
    auto request = [&](auto buf_c, int ks0) {
        constexpr int buf = decltype(buf_c)::value;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (ks0 + u < nks) {
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    a[buf][u][m] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wr, woff + m * 1024, w_base + (ks0 + u) * w_step, 0));
                if constexpr (TAPS) {
                    const int entry = p.step[ks0 + u];
                    const int off = entry & ((1 << kTapShift) - 1);
                    const unsigned bit = 1u << ((unsigned)entry >> kTapShift);
#pragma unroll
                    for (int n = 0; n < NT; ++n)
                        b[buf][u][n] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(xr, (taps_in[n] & bit) ? xoff[n] + off : kOutOfRange, 0, 0));
                } else {
#pragma unroll
                    for (int n = 0; n < NT; ++n)
                        b[buf][u][n] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(xr, xoff[n], (ks0 + u) * 32, 0));
                }
            }
        }
    };
    auto compute = [&](auto buf_c, int ks0) {
        constexpr int buf = decltype(buf_c)::value;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (ks0 + u < nks) {
#pragma unroll
                for (int m = 0; m < MT; ++m)
#pragma unroll
                    for (int n = 0; n < NT; ++n) {
                        if constexpr (DT == EXHIP_I8)
                            acc[m][n] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[buf][u][m], b[buf][u][n], acc[m][n], 0, 0, 0);
                        else
                            acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a[buf][u][m]), __builtin_bit_cast(v8h, b[buf][u][n]),
                                                                               acc[m][n], 0, 0, 0);
                    }
            }
        }
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    request(B0{}, 0);
    for (int ks0 = 0; ks0 < nks; ks0 += 2 * U) {
        request(B1{}, ks0 + U);
        compute(B0{}, ks0);
        request(B0{}, ks0 + 2 * U);
        compute(B1{}, ks0 + U);
    }

    if constexpr (DT == EXHIP_I8) {
        pw_epilogue_i8<MT, NT>(p, acc, pix, kb0, lane);
    } else {
        float bi[MT][16];
        load_bias<MT>(p, kb0, lane, bi);
        pw_epilogue<MT, NT>(p, acc, pix, kb0, lane, bi);
    }
}

template <int DT, int MT, int NT, bool TAPS = false>
int launch(exhip_ctx* ctx, PwParams& p, int kblocks) {
    const long long tiles = ((long long)p.pixels + 32 * NT - 1) / (32 * NT);
    p.ch_groups = (unsigned)((kblocks + MT - 1) / MT);
    const long long items = tiles * p.ch_groups;
    if (items >= (1ll << 31)) return EXHIP_ERR_UNSUPPORTED;
    p.items = (unsigned)items;
    const unsigned grid = (unsigned)((items + 3) / 4);
    hipLaunchKernelGGL((conv1x1_pw_kernel<DT, MT, NT, TAPS>), dim3(grid), dim3(256), 0, ctx->stream, p);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

}  // namespace

namespace {

// Layers of more than 32 output channels take the 32-pixel x 64-channel wave tile whatever their size: half the registers of
// the 64 x 64 tile, so more waves hide each other's loads and epilogues. Measured on whole forwards against "64 x 64 from
// 2048 waves on" (option pw_tile = 2): int8 64 -> 64 at 16 x 160 x 160 41 -> 30 us, a detection network's int8 forward
// 1.44 -> 1.35 ms, its fp16 forward 1.81 -> 1.79 ms, two mobile networks' fp16 forwards 0.435 -> 0.42 and 0.82 -> 0.805 ms.
template <int DT>
bool small_tile() { return g_exhip_options.pw_tile != 2; }

// A layer with a filter, a stride or padding on the same kernel: g.pixels counts output pixels, the k-steps walk the
// packing's order (channel chunk, filter row, tap, 32-byte step).
template <int DT>
int run_taps(exhip_ctx* ctx, const exhip_pw_geom& g, const exhip_pw_taps& t, PwParams& p, bool has_residual) {
    if (g_exhip_options.direct == 0) return EXHIP_ERR_UNSUPPORTED;
    if (g.post_bn_a || g.post_bn_b || g.exact_k) return EXHIP_ERR_UNSUPPORTED;
    const long long n_ksteps = (long long)t.n_chunks * t.kh * t.kw * (t.chunk_b / 32);
    if (g.pixels <= 0 || g.c_bytes <= 0 || g.c_bytes % 32 != 0 || t.chunk_b % 32 != 0 || t.n_chunks * t.chunk_b != g.c_bytes ||
        (g.slab_blocks != 2 && g.slab_blocks != 4) || g.k_stride % 8 != 0 || n_ksteps > kMaxDirectSteps || t.kh * t.kw > (1 << (32 - kTapShift)) || t.stride < 1 || t.pad_t < 0 || t.pad_l < 0)
        return EXHIP_ERR_UNSUPPORTED;
    const long long x_bytes = (long long)t.n * t.in_h * t.in_w * g.c_bytes;
    const long long w_bytes = (long long)g.slabs * n_ksteps * g.slab_blocks * 1024;
    const long long reach = ((long long)(t.kh - 1) * t.in_w + t.kw) * g.c_bytes;   // the furthest step behind a pixel's top-left tap
    if (x_bytes >= kOutOfRange || w_bytes >= kOutOfRange || reach >= (1ll << kTapShift) || g.pixels != (long long)t.n * t.out_h * t.out_w ||
        g.pixels * 4 * g.k_stride >= (1ll << 40) || g.pixels >= (1ll << 31))
        return EXHIP_ERR_UNSUPPORTED;
    if (g.post_op && g.post_op != EXHIP_POST_PRELU && (g.post_op < 1 || g.post_op > 1 + EXHIP_UNARY_CLIP || g.post_op == 1 + EXHIP_UNARY_SIGMOID))
        return EXHIP_ERR_UNSUPPORTED;
    const int kblocks = std::min(g.slabs * g.slab_blocks, (std::max(g.k, g.k_stride) + 31) / 32);
    // Measured inside two detection networks at 16 x 3 x 640 x 640 and two mobile networks: the fp16 layers the lean
    // kernel leaves (stride 2, 12 or 32 input channels, ragged output channels) are faster here as a whole (0.88 -> 0.85 ms
    // and 1.83 -> 1.81 ms per forward of the detection networks); of the int8 layers only a few deep ones are (3x3
    // stride 2 from 40 x 40: 29 -> 23 us) while the wide first layers lose (12 -> 32 channels at 320 x 320: 81 -> 94 us),
    // so int8 layers stay with the staged kernels unless the option asks.
    // A lone 32-channel block (its 128-pixel tile with the tap bookkeeping fills the register file) never wins: 12 -> 32
    // at 16 x 320 x 320 78 against 80 us, 16 -> 32 stride 2 at 224 x 224 11.5 against 9 us in either data type.
    const bool take = kblocks > 1 && (DT == EXHIP_F16 || g.c_bytes == 32 || (g.pixels <= 32768 && kblocks <= 4) || g.pixels <= 6400);
    if (g_exhip_options.direct != 2 && !take) return EXHIP_ERR_UNSUPPORTED;
    p.post_slope = g.post_slope;
    p.pixels = (unsigned)g.pixels; p.x_bytes = (unsigned)x_bytes; p.w_bytes = (unsigned)w_bytes;
    p.xs_b = g.c_bytes; p.n_ksteps = (int)n_ksteps; p.mts = g.slab_blocks;
    p.K = g.k; p.kstride = g.k_stride;
    p.act = g.act; p.post_relu = g.post_relu; p.post_op = g.post_op; p.post_slope_shared = g.post_slope_shared;
    p.residual_last = g.residual_last && has_residual;
    p.post_alpha = g.post_alpha; p.post_beta = g.post_beta;
    p.in_h = t.in_h; p.in_w = t.in_w; p.out_h = t.out_h; p.out_w = t.out_w; p.stride = t.stride; p.pad_t = t.pad_t; p.pad_l = t.pad_l;
    p.kh = t.kh; p.kw = t.kw;
    int s = 0;
    for (int cc = 0; cc < t.n_chunks; ++cc)
        for (int r = 0; r < t.kh; ++r)
            for (int q = 0; q < t.kw; ++q)
                for (int j = 0; j < t.chunk_b / 32; ++j)
                    p.step[s++] = ((r * t.in_w + q) * g.c_bytes + cc * t.chunk_b + j * 32) | (int)((unsigned)(r * t.kw + q) << kTapShift);
    if (kblocks == 1) return launch<DT, 1, 4, true>(ctx, p, kblocks);
    const long long waves64 = ((g.pixels + 63) / 64) * ((kblocks + 1) / 2);
    if (waves64 < 2048 || small_tile<DT>()) return launch<DT, 2, 1, true>(ctx, p, kblocks);
    return launch<DT, 2, 2, true>(ctx, p, kblocks);
}

// Geometry checks and the wave tile, shared by the two data types. `es`: bytes per input element.
template <int DT>
int run_pw(exhip_ctx* ctx, const exhip_pw_geom& g, PwParams& p, int es, bool has_residual, const exhip_pw_taps* t = nullptr) {
    if (g_exhip_options.pw == 0) return EXHIP_ERR_UNSUPPORTED;
    if (t) return run_taps<DT>(ctx, g, *t, p, has_residual);
    // Measured per layer against the general kernel inside a detection and two mobile networks (16 and 64 images, kernel
    // traces): this form wins where a launch is short -- every layer of at most 32 768 pixels up to about 7 GFLOP (twice
    // as fast on 20 x 20 maps) --, for a lone 32-channel block (which the general kernel pads to a 64-channel slab), and on
    // larger maps while the input is narrow: fp16 up to 64 input channels (64 -> 64 at 16 x 160 x 160: 42 against 49 us)
    // and 128 -> 64 at 80 x 80; int8 up to 64 channels at 131 072 pixels, and layers with only a float32 result (its
    // 64-byte store runs against the general epilogue's 16-byte pieces: 41 against 60 us on a 128 -> 255 head at
    // 16 x 80 x 80). Beyond that the general kernel's staged tiles re-read less and win (128 -> 128 at 80 x 80).
    // Option pw = 2 takes every layer the kernel can (tests), 0 none.
    const bool joined = g.post_bn_a || g.exact_k;  // only this kernel has those: it takes the layer whatever its size
    if (joined && (DT != EXHIP_I8 || (g.post_bn_a == nullptr) != (g.post_bn_b == nullptr) || (g.exact_k && g.k % 32 != 0))) return EXHIP_ERR_UNSUPPORTED;
    const int out_channels = g.exact_k ? g.k : std::max(g.k, g.k_stride);  // channels this launch writes
    const int blocks_needed = (out_channels + 31) / 32;
    const double flop = 2.0 * (double)g.pixels * (g.c_bytes / es) * g.k;
    bool take = joined || blocks_needed == 1 || (flop <= 8.0e9 && g.pixels <= 32768);
    if (DT == EXHIP_I8 && g.pixels <= 131072 && (g.c_bytes <= 64 || (p.y_f && !p.y_q))) take = true;
    if (DT == EXHIP_I8 && g_exhip_options.pw_tile != 2 && g.c_bytes <= 512) take = true;  // with the small tile: every layer measured
    // With the small tile: every fp16 layer. Launched thirty times alone, long reductions on large maps lose a little
    // (256 -> 256 at 64 x 28 x 28: 33 against 32 us, 512 -> 512 at 16 x 40 x 40: 49 against 46 us); inside the networks,
    // between other layers, taking them too is what measured faster (same box, two runs each: a detection network 1.752
    // -> 1.738 ms, another 0.820 -> 0.805 ms, a depthwise / pointwise network 0.772 -> 0.761 ms), and the networks decide.
    if (DT == EXHIP_F16 && g_exhip_options.pw_tile != 2) take = true;
    if (DT == EXHIP_F16 && ((g.c_bytes <= 128 && g.pixels <= 524288) || (g.c_bytes <= 256 && g.k <= 64 && g.pixels <= 131072))) take = true;
    if (g_exhip_options.pw != 2 && !take) return EXHIP_ERR_UNSUPPORTED;
    if (g.pixels <= 0 || g.c_bytes <= 0 || g.c_bytes % 32 != 0 || (g.slab_blocks != 2 && g.slab_blocks != 4) || g.k_stride % 8 != 0)
        return EXHIP_ERR_UNSUPPORTED;
    // lane offsets are 32-bit: the input tensor and the packed weights must stay below the out-of-range sentinel
    const long long x_bytes = g.pixels * g.c_bytes;
    const long long n_ksteps = g.c_bytes / 32;
    const long long w_bytes = (long long)g.slabs * n_ksteps * g.slab_blocks * 1024;
    if (x_bytes >= kOutOfRange || w_bytes >= kOutOfRange || g.pixels * 4 * g.k_stride >= (1ll << 40)) return EXHIP_ERR_UNSUPPORTED;
    if (g.post_op && g.post_op != EXHIP_POST_PRELU && (g.post_op < 1 || g.post_op > 1 + EXHIP_UNARY_CLIP || g.post_op == 1 + EXHIP_UNARY_SIGMOID))
        return EXHIP_ERR_UNSUPPORTED;
    p.post_slope = g.post_slope;
    p.pixels = (unsigned)g.pixels; p.x_bytes = (unsigned)x_bytes; p.w_bytes = (unsigned)w_bytes;
    p.xs_b = g.c_bytes; p.n_ksteps = (int)n_ksteps; p.mts = g.slab_blocks;
    p.K = g.k; p.kstride = g.k_stride;
    p.act = g.act; p.post_relu = g.post_relu; p.post_op = g.post_op; p.post_slope_shared = g.post_slope_shared;
    p.residual_last = g.residual_last && has_residual;
    p.post_alpha = g.post_alpha; p.post_beta = g.post_beta;
    // every packed block that holds a channel below max(k, k_stride): pad channels of the output are written as zeros
    // (exact_k: only the blocks of the k channels themselves)
    const int kblocks = std::min(g.slabs * g.slab_blocks, (out_channels + 31) / 32);
    // 64 x 64 per wave unless that leaves SIMDs without a wave: then 64 channels x 32 pixels; a lone 32-channel block
    // takes 128 pixels per wave
    if (kblocks == 1) return launch<DT, 1, 4>(ctx, p, kblocks);
    const long long waves64 = ((g.pixels + 63) / 64) * ((kblocks + 1) / 2);
    if (waves64 < 2048 || small_tile<DT>()) return launch<DT, 2, 1>(ctx, p, kblocks);
    return launch<DT, 2, 2>(ctx, p, kblocks);
}

}  // namespace

int exhip_conv1x1_f16_pw(exhip_ctx* ctx, const exhip_pw_geom& g, const uint16_t* x, const void* wp, const float* bias,
                         const uint16_t* residual, uint16_t* y, const exhip_pw_taps* taps) {
    PwParams p = {};
    p.x = reinterpret_cast<const char*>(x); p.wp = reinterpret_cast<const char*>(wp); p.bias = bias; p.residual = residual; p.y = y;
    return run_pw<EXHIP_F16>(ctx, g, p, 2, residual != nullptr, taps);
}

int exhip_conv1x1_i8_pw(exhip_ctx* ctx, const exhip_pw_geom& g, const int8_t* x, const void* wp, const float* scale, const float* bias,
                        const float* residual, int8_t* y_i8, float* y_f32, const exhip_pw_taps* taps) {
    if (!scale || (!y_i8 && !y_f32) || g.k_stride % 16 != 0) return EXHIP_ERR_UNSUPPORTED;
    PwParams p = {};
    p.x = reinterpret_cast<const char*>(x); p.wp = reinterpret_cast<const char*>(wp); p.bias = bias; p.scale = scale;
    p.residual_f = residual; p.y_f = y_f32; p.y_q = y_i8; p.fs_out = g.fs_out;
    p.post_bn_a = g.post_bn_a; p.post_bn_b = g.post_bn_b; p.exact = g.exact_k;
    return run_pw<EXHIP_I8>(ctx, g, p, 1, residual != nullptr, taps);
}
