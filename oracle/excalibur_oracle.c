/* CPU restatement of the arithmetic of Excalibur's CNN forward hot path.
 * TEST INFRASTRUCTURE ONLY: see excalibur_oracle.h. Built with -ffp-contract=off so
 * that every fused multiply-add below is one written on purpose with fmaf().
 */
#include "excalibur_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* conv output size: src/Excalibur/operation_convolution.cpp:270-271 (integer division). */
int exo_out_dim(int in, int pad_a, int pad_b, int kernel, int stride) { return (in + pad_a + pad_b - kernel) / stride + 1; }

/* src/Primitives/simd_types.cpp:140-152 — round half away from zero by adding +-0.5 and
 * truncating, saturating to [-128, 127]. */
int8_t exo_float32_to_int8(float v) {
    float t = v >= 0.f ? v + 0.5f : v - 0.5f;
    if (t > 127) return 127;
    if (t < -128) return -128;
    return (int8_t)t;
}

/* src/Excalibur/operation_general_conv.cpp:584-720 (x86 path): q = float32_to_int8(x * fs),
 * fs per tensor (fs_count == 1) or per input channel (:596). The product is rounded to
 * float before the +-0.5 (the conversion is a call into another library). */
void exo_quantize_f32_i8(const float* x, int8_t* q, int n, int c, int hw, const float* fs, int fs_count) {
    for (int in = 0; in < n; ++in)
        for (int ic = 0; ic < c; ++ic) {
            const float scale = fs_count == 1 ? fs[0] : fs[ic];
            const float* src = x + ((size_t)in * c + ic) * hw;
            int8_t* dst = q + ((size_t)in * c + ic) * hw;
            for (int i = 0; i < hw; ++i) {
                volatile float prod = src[i] * scale;
                dst[i] = exo_float32_to_int8(prod);
            }
        }
}

/* The integer convolution both int8 CPU paths evaluate exactly:
 * Winograd F(2,3) with int16 transforms and >>2 (src/Excalibur/operation_convolution.cpp:1783-2161)
 * and im2col + 8x8 int32 tiles (:2269-2978). acc[n,k,oh,ow] = sum q[n,c,oh*s-pt+i,ow*s-pl+j] * w[k,c,i,j],
 * zero outside the image (make_border with pad_value_ 0, :373-380). Groups as in :2292. */
void exo_conv2d_i8_acc(const int8_t* q, const int8_t* w, int32_t* acc, const exo_geom* g) {
    const int oh = exo_out_dim(g->h, g->pt, g->pb, g->kh, g->sh);
    const int ow = exo_out_dim(g->w, g->pl, g->pr, g->kw, g->sw);
    const int cg = g->c / g->groups, kg = g->k / g->groups;
    memset(acc, 0, sizeof(int32_t) * (size_t)g->n * g->k * oh * ow);
    for (int n = 0; n < g->n; ++n)
        for (int k = 0; k < g->k; ++k) {
            const int grp = k / kg;
            int32_t* out = acc + ((size_t)n * g->k + k) * oh * ow;
            for (int c = 0; c < cg; ++c) {
                const int8_t* in = q + ((size_t)n * g->c + grp * cg + c) * g->h * g->w;
                const int8_t* wk = w + (((size_t)k * cg + c) * g->kh) * g->kw;
                for (int i = 0; i < g->kh; ++i)
                    for (int j = 0; j < g->kw; ++j) {
                        const int wv = wk[i * g->kw + j];
                        if (wv == 0) continue;
                        for (int y = 0; y < oh; ++y) {
                            const int iy = y * g->sh - g->pt + i;
                            if (iy < 0 || iy >= g->h) continue;
                            /* valid ox range: 0 <= ox*sw - pl + j < w */
                            int x0 = 0, x1 = ow;
                            while (x0 < ow && x0 * g->sw - g->pl + j < 0) ++x0;
                            while (x1 > x0 && (x1 - 1) * g->sw - g->pl + j >= g->w) --x1;
                            const int8_t* row = in + (size_t)iy * g->w - g->pl + j;
                            int32_t* orow = out + (size_t)y * ow;
                            if (g->sw == 1) {
                                for (int x = x0; x < x1; ++x) orow[x] += wv * row[x];
                            } else {
                                for (int x = x0; x < x1; ++x) orow[x] += wv * row[x * g->sw];
                            }
                        }
                    }
            }
        }
}

/* src/Excalibur/operation_convolution.cpp:400-403 and operation_general_conv.cpp:756:
 * scale = fabs(ws) <= 1e-6 ? 0 : 1.0f / (ws * fs), float multiply then float divide. */
float exo_dequant_scale(float ws, float fs) {
    if (fabs((double)ws) <= 1e-6) return 0.f;
    volatile float prod = ws * fs;
    return 1.0f / prod;
}

/* src/Excalibur/operation_general_conv.cpp:724-941 (scalar `*intptr * scale + bias`, :842) and the
 * vector epilogue src/Excalibur/operation_convolution.cpp:2497-2513 (cvtepi32_ps then fmadd):
 * under the reference's flags both are one fused multiply-add on the RNE-converted accumulator. */
void exo_dequant_i32_f32(const int32_t* acc, float* y, int n, int k, int hw, const float* ws, int ws_count,
                         const float* fs, int fs_count, const float* bias) {
    for (int in = 0; in < n; ++in)
        for (int ik = 0; ik < k; ++ik) {
            const float s = exo_dequant_scale(ws_count == 1 ? ws[0] : ws[ik], fs_count == 1 ? fs[0] : fs[ik]);
            const float b = bias ? bias[ik] : 0.f;
            const int32_t* a = acc + ((size_t)in * k + ik) * hw;
            float* o = y + ((size_t)in * k + ik) * hw;
            for (int i = 0; i < hw; ++i) o[i] = fmaf((float)a[i], s, b);
        }
}

/* src/Excalibur/operation_general_conv.cpp:127-272. 1: max(0,x) keeping -0.0 and mapping NaN to NaN
 * as _mm256_max_ps(zero, x) does (:157); 3: the reference's "ReLU6" zeroes values above 6
 * (:206-229); 4: sigmoid evaluated in double (:251); 5: mish in double (:264: the unqualified exp / log / tanh
 * on a float resolve to the C library's double functions; pinned by the fixtures conv_f32_mish / conv_i8_mish of
 * the compiled reference, which the float functions expf / logf / tanhf miss in half of the elements). */
void exo_activation_f32(float* y, long count, int act) {
    switch (act) {
    case EXO_ACT_NONE: return;
    case EXO_ACT_RELU:
        for (long i = 0; i < count; ++i) y[i] = (0.f > y[i]) ? 0.f : y[i];
        return;
    case EXO_ACT_RELU6_ZEROING:
        for (long i = 0; i < count; ++i) {
            float d = (0.f > y[i]) ? 0.f : y[i];
            y[i] = (d <= 6.0f) ? d : 0.f;
        }
        return;
    case EXO_ACT_SIGMOID:
        for (long i = 0; i < count; ++i) y[i] = (float)(1. / (1. + exp(-(double)y[i])));
        return;
    case EXO_ACT_MISH:
        for (long i = 0; i < count; ++i) y[i] = (float)((double)y[i] * tanh(log(1 + exp((double)y[i]))));
        return;
    default: abort();
    }
}

/* operation_convolution::forward_cpu_i8, src/Excalibur/operation_convolution.cpp:332-409:
 * float in -> quantize -> integer conv -> dequant(+bias) -> activation -> float out.
 * Unlike the reference's im2col path (:2284-2300) every image of the batch is computed. */
void exo_conv2d_i8(const float* x, const int8_t* w, const float* bias, const float* ws, int ws_count, const float* fs,
                   int fs_count, int act, float* y, int32_t* acc_or_null, const exo_geom* g) {
    const int oh = exo_out_dim(g->h, g->pt, g->pb, g->kh, g->sh);
    const int ow = exo_out_dim(g->w, g->pl, g->pr, g->kw, g->sw);
    const size_t in_count = (size_t)g->n * g->c * g->h * g->w, out_count = (size_t)g->n * g->k * oh * ow;
    int8_t* q = (int8_t*)malloc(in_count);
    int32_t* acc = acc_or_null ? acc_or_null : (int32_t*)malloc(out_count * sizeof(int32_t));
    exo_quantize_f32_i8(x, q, g->n, g->c, g->h * g->w, fs, fs_count);
    exo_conv2d_i8_acc(q, w, acc, g);
    exo_dequant_i32_f32(acc, y, g->n, g->k, oh * ow, ws, ws_count, fs, fs_count, bias);
    exo_activation_f32(y, (long)out_count, act);
    free(q);
    if (!acc_or_null) free(acc);
}

/* operation_convolution::forward_cpu_f32, src/Excalibur/operation_convolution.cpp:251-329. The reference
 * evaluates y = act(conv(x, W) + b) in float through Winograd F(2,3) (:470-870) or an im2col GEMM
 * (:974-1725); both agree with the exact sum to ~1e-6 relative. This restatement accumulates the
 * definition in double and rounds once, which is the value both are compared to at 1e-4. */
void exo_conv2d_f32(const float* x, const float* w, const float* bias, int act, float* y, const exo_geom* g) {
    const int oh = exo_out_dim(g->h, g->pt, g->pb, g->kh, g->sh);
    const int ow = exo_out_dim(g->w, g->pl, g->pr, g->kw, g->sw);
    const int cg = g->c / g->groups, kg = g->k / g->groups;
    double* accd = (double*)malloc(sizeof(double) * (size_t)oh * ow);
    for (int n = 0; n < g->n; ++n)
        for (int k = 0; k < g->k; ++k) {
            const int grp = k / kg;
            for (int i = 0; i < oh * ow; ++i) accd[i] = 0.0;
            for (int c = 0; c < cg; ++c) {
                const float* in = x + ((size_t)n * g->c + grp * cg + c) * g->h * g->w;
                const float* wk = w + (((size_t)k * cg + c) * g->kh) * g->kw;
                for (int i = 0; i < g->kh; ++i)
                    for (int j = 0; j < g->kw; ++j) {
                        const double wv = wk[i * g->kw + j];
                        for (int yy = 0; yy < oh; ++yy) {
                            const int iy = yy * g->sh - g->pt + i;
                            if (iy < 0 || iy >= g->h) continue;
                            for (int xx = 0; xx < ow; ++xx) {
                                const int ix = xx * g->sw - g->pl + j;
                                if (ix < 0 || ix >= g->w) continue;
                                accd[yy * ow + xx] += wv * (double)in[(size_t)iy * g->w + ix];
                            }
                        }
                    }
            }
            float* out = y + ((size_t)n * g->k + k) * oh * ow;
            const double b = bias ? (double)bias[k] : 0.0;
            for (int i = 0; i < oh * ow; ++i) out[i] = (float)(accd[i] + b);
        }
    free(accd);
    exo_activation_f32(y, (long)g->n * g->k * oh * ow, act);
}

/* operation_convolutiondepthwise::dequantize_int8, src/Excalibur/operation_convolutiondepthwise.cpp:195-222:
 * weight-only quantization, w_f = w_i8 * (ws <= 1e-6 ? 0 : 1.f / ws) (no fabs: a negative scale gives 0). */
void exo_dw_dequant_weights(const int8_t* w, float* wf, int k, int per_group, const float* ws) {
    for (int q = 0; q < k; ++q) {
        const float s = ws[q] <= 1e-6 ? 0.f : 1.f / ws[q];
        for (int i = 0; i < per_group; ++i) wf[(size_t)q * per_group + i] = (float)w[(size_t)q * per_group + i] * s;
    }
}

/* operation_convolutiondepthwise::forward_cpu_f32, src/Excalibur/operation_convolutiondepthwise.cpp:18-181.
 * 3x3 stride 1 (:321-503) and 3x3 stride 2 (:506-626) use this exact order per output pixel:
 * three vertical fused multiply-adds per kernel column starting from 0, then bias + col0 + col1 + col2.
 * Every other kernel shape goes through the dense grouped convolution (:118). */
void exo_dwconv_f32(const float* x, const float* w, const float* bias, int act, float* y, const exo_geom* g) {
    const int oh = exo_out_dim(g->h, g->pt, g->pb, g->kh, g->sh);
    const int ow = exo_out_dim(g->w, g->pl, g->pr, g->kw, g->sw);
    const int fast = g->kh == 3 && g->kw == 3 && g->sh == g->sw && (g->sh == 1 || g->sh == 2);
    if (!fast) {
        exo_conv2d_f32(x, w, bias, act, y, g);
        return;
    }
    for (int n = 0; n < g->n; ++n)
        for (int c = 0; c < g->c; ++c) {
            const float* in = x + ((size_t)n * g->c + c) * g->h * g->w;
            const float* k = w + (size_t)c * 9;
            const float b = bias ? bias[c] : 0.f;
            float* out = y + ((size_t)n * g->c + c) * oh * ow;
            for (int yy = 0; yy < oh; ++yy)
                for (int xx = 0; xx < ow; ++xx) {
                    float col[3];
                    for (int j = 0; j < 3; ++j) {
                        float s = 0.f;
                        for (int i = 0; i < 3; ++i) {
                            const int iy = yy * g->sh - g->pt + i, ix = xx * g->sw - g->pl + j;
                            const float v = (iy >= 0 && iy < g->h && ix >= 0 && ix < g->w) ? in[(size_t)iy * g->w + ix] : 0.f;
                            s = fmaf(v, k[i * 3 + j], s);
                        }
                        col[j] = s;
                    }
                    float sum = b;
                    sum += col[0];
                    sum += col[1];
                    sum += col[2];
                    out[yy * ow + xx] = 0.f + sum; /* the reference adds into a zero-filled output (:434) */
                }
        }
    exo_activation_f32(y, (long)g->n * g->c * oh * ow, act);
}

/* src/Excalibur/operation_pooling.cpp:103-121: pad_mode 0 = ceil, 1 = floor, on a float quotient. */
int exo_pool_out_dim(int in, int pad_a, int pad_b, int kernel, int stride, int pad_mode) {
    const float q = (float)(in + pad_a + pad_b - kernel) / stride;
    return (int)(pad_mode == 0 ? ceilf(q) : floorf(q)) + 1;
}

/* operation_pooling::forward_cpu_f32, NCHW branch, src/Excalibur/operation_pooling.cpp:80-208.
 * MAX: window clipped to the image, start value -FLT_MAX (:145-159). AVE: running float sum over
 * the valid cells in row-major order, divided by the valid count, or by the padded window size when
 * count_include_pad is set (:181-201). global: kernel = HxW, stride 1, no padding (:90-100). */
void exo_pool2d_f32(const float* x, float* y, int n, int c, int h, int w, int type, int kh, int kw, int sh, int sw,
                    int pt, int pb, int pl, int pr, int global, int pad_mode, int count_include_pad) {
    if (global) { kh = h; kw = w; pt = pb = pl = pr = 0; sh = sw = 1; }
    const int oh = exo_pool_out_dim(h, pt, pb, kh, sh, pad_mode), ow = exo_pool_out_dim(w, pl, pr, kw, sw, pad_mode);
    for (int nc = 0; nc < n * c; ++nc) {
        const float* in = x + (size_t)nc * h * w;
        float* out = y + (size_t)nc * oh * ow;
        for (int ph = 0; ph < oh; ++ph)
            for (int pw = 0; pw < ow; ++pw) {
                int hs = ph * sh - pt, wsx = pw * sw - pl;
                if (type == EXO_POOL_MAX) {
                    int he = hs + kh < h ? hs + kh : h, we = wsx + kw < w ? wsx + kw : w;
                    if (hs < 0) hs = 0;
                    if (wsx < 0) wsx = 0;
                    float v = -FLT_MAX;
                    for (int a = hs; a < he; ++a)
                        for (int b = wsx; b < we; ++b) v = v < in[a * w + b] ? in[a * w + b] : v;
                    out[ph * ow + pw] = v;
                } else {
                    int he = hs + kh < h + pb ? hs + kh : h + pb, we = wsx + kw < w + pr ? wsx + kw : w + pr;
                    int pool_size = (he - hs) * (we - wsx);
                    if (hs < 0) hs = 0;
                    if (wsx < 0) wsx = 0;
                    if (he > h) he = h;
                    if (we > w) we = w;
                    float s = 0.f;
                    int area = 0;
                    for (int a = hs; a < he; ++a)
                        for (int b = wsx; b < we; ++b) { s += in[a * w + b]; ++area; }
                    if (count_include_pad == 0) pool_size = area;
                    out[ph * ow + pw] = s / pool_size;
                }
            }
    }
}

/* operation_eltwise::forward_cpu_f32, src/Excalibur/operation_eltwise.cpp:43-94.
 * SUM: top = 0, then top = coeff_i * x_i + 1.0f * top per input through cblas_saxpby
 * (src/Julius/julius_axpby.cpp:12-40). Its 8-wide body, over the first count - count % 8 elements, is
 * add(mul(x, alpha), mul(y, beta)) with both products rounded; its scalar tail
 * `alpha * x + beta * y` (:36-39) is compiled to one fused multiply-add under the reference's flags
 * (observed on the compiled reference). Both are the exact x0 + x1 for unit coefficients.
 * MAX / PROD: pairwise left to right. */
void exo_eltwise_f32(const float* const* inputs, int n_inputs, const float* coeffs, int type, float* y, long count) {
    if (type == EXO_ELT_SUM) {
        for (long i = 0; i < count; ++i) y[i] = 0.f;
        for (int k = 0; k < n_inputs; ++k) {
            const float a = coeffs ? coeffs[k] : 1.f;
            const long body = count - count % 8;
            for (long i = 0; i < body; ++i) y[i] = inputs[k][i] * a + y[i] * 1.0f;
            for (long i = body; i < count; ++i) y[i] = fmaf(a, inputs[k][i], y[i] * 1.0f);
        }
    } else if (type == EXO_ELT_MAX) {
        for (long i = 0; i < count; ++i) y[i] = inputs[0][i] < inputs[1][i] ? inputs[1][i] : inputs[0][i];
        for (int k = 2; k < n_inputs; ++k)
            for (long i = 0; i < count; ++i) y[i] = y[i] < inputs[k][i] ? inputs[k][i] : y[i];
    } else if (type == EXO_ELT_PROD) {
        for (long i = 0; i < count; ++i) y[i] = inputs[0][i] * inputs[1][i];
        for (int k = 2; k < n_inputs; ++k)
            for (long i = 0; i < count; ++i) y[i] = y[i] * inputs[k][i];
    } else {
        abort();
    }
}

/* operation_binaryop, equal-shape ADD branch, src/Excalibur/operation_binaryop.cpp:75-84,297-303. */
void exo_binaryop_add_f32(const float* a, const float* b, float* y, long count) {
    for (long i = 0; i < count; ++i) y[i] = a[i] + b[i];
}

/* operation_relu::forward_cpu_f32, src/Excalibur/operation_relu.cpp:31-81: max(0, x) into a new tensor. */
void exo_relu_f32(const float* x, float* y, long count) {
    for (long i = 0; i < count; ++i) y[i] = (0.f > x[i]) ? 0.f : x[i];
}

/* operation_innerproduct::forward_cpu_f32, src/Excalibur/operation_innerproduct.cpp:176-224 (the
 * m x n x 1 x 1 branch): Y[m,n] = sum_k X[m,k] * W[n,k] (+ b[n]). Julius sgemm sums in float in its own
 * blocked order; this restatement sums in double and rounds once (compared at 1e-4). */
void exo_innerproduct_f32(const float* x, const float* w, const float* bias, float* y, int m, int n_out, int k_in) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n_out; ++j) {
            double s = 0.0;
            for (int k = 0; k < k_in; ++k) s += (double)x[(size_t)i * k_in + k] * (double)w[(size_t)j * k_in + k];
            if (bias) s += (double)bias[j];
            y[(size_t)i * n_out + j] = (float)s;
        }
}

/* src/Primitives/simd_types.cpp:8-69: float -> half by truncating the mantissa (no rounding),
 * float denormals flush to zero, half denormals by shifting, NaN -> quiet NaN. */
uint16_t exo_float32_to_float16(float value) {
    union { uint32_t u; float f; } t;
    t.f = value;
    const uint16_t sign = (uint16_t)((t.u & 0x80000000u) >> 31);
    const int exponent = (int)((t.u & 0x7F800000u) >> 23);
    const uint32_t sig = t.u & 0x7FFFFFu;
    if (exponent == 0) return (uint16_t)(sign << 15);
    if (exponent == 0xFF) return (uint16_t)((sign << 15) | (0x1F << 10) | (sig ? 0x200 : 0));
    const int newexp = exponent - 127 + 15;
    if (newexp >= 31) return (uint16_t)((sign << 15) | (0x1F << 10));
    if (newexp <= 0) {
        if (newexp >= -10) return (uint16_t)((sign << 15) | ((sig | 0x800000u) >> (14 - newexp)));
        return (uint16_t)(sign << 15);
    }
    return (uint16_t)((sign << 15) | (newexp << 10) | (sig >> 13));
}

/* src/Primitives/simd_types.cpp:71-122: exact half -> float. */
float exo_float16_to_float32(uint16_t v) {
    const uint32_t sign = (v & 0x8000u) >> 15;
    uint32_t exponent = (v & 0x7c00u) >> 10, sig = v & 0x3FFu;
    union { uint32_t u; float f; } t;
    if (exponent == 0) {
        if (sig == 0) {
            t.u = sign << 31;
        } else {
            exponent = 0;
            while ((sig & 0x200u) == 0) { sig <<= 1; ++exponent; }
            sig = (sig << 1) & 0x3FFu;
            t.u = (sign << 31) | ((uint32_t)(112 - (int)exponent) << 23) | (sig << 13);
        }
    } else if (exponent == 0x1F) {
        t.u = (sign << 31) | (0xFFu << 23) | (sig << 13);
    } else {
        t.u = (sign << 31) | ((exponent + 112) << 23) | (sig << 13);
    }
    return t.f;
}

static uint16_t rne_half(float f) {
    /* round-to-nearest-even conversion, what _mm256_cvtps_ph(v, 0) computes */
    union { uint32_t u; float f; } t;
    t.f = f;
    const uint32_t sign = (t.u >> 16) & 0x8000u;
    uint32_t a = t.u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu));
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7C00u); /* >= 65536 -> inf (65520 rounds up below) */
    if (a < 0x38800000u) { /* half subnormal or zero */
        if (a < 0x33000000u) return (uint16_t)sign; /* < 2^-25 */
        const int e = (int)(a >> 23);
        uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
        const int shift = 126 - e; /* 14..24 */
        const uint32_t half_m = m >> shift, rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
        uint32_t r = half_m;
        if (rem > halfway || (rem == halfway && (half_m & 1))) ++r;
        return (uint16_t)(sign | r);
    }
    uint32_t r = ((a - 0x38000000u) >> 13);
    const uint32_t rem = a & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) ++r;
    return (uint16_t)(sign | r);
}

/* float2half, src/Primitives/simd_types.cpp:198-224, on a CPU with F16C: the first length % 8
 * elements are converted with round-to-nearest-even (one 8-wide F16C conversion whose upper lanes
 * are then overwritten), all remaining elements by the truncating scalar routine above.
 * Arrays shorter than 8 are converted entirely with round-to-nearest-even. */
void exo_float2half(const float* x, uint16_t* y, int length) {
    const int partl = length % 8;
    for (int i = 0; i < length; ++i) y[i] = (i < partl) ? rne_half(x[i]) : exo_float32_to_float16(x[i]);
}

/* half2float, src/Primitives/simd_types.cpp:226-252: exact in both of its branches. */
void exo_half2float(const uint16_t* x, float* y, int length) {
    for (int i = 0; i < length; ++i) y[i] = exo_float16_to_float32(x[i]);
}

/* ---- activation / glue layers of the shipped topologies ---- */

/* operation_hardswish::forward_cpu_f32, src/Excalibur/operation_hardswish.cpp:32-63: y = x * clamp(alpha*x + beta, 0, 1).
 * The vector body fuses alpha*x + beta (_mm256_fmadd_ps, :45); the scalar tail's alpha*x + beta (:59) is contracted to an
 * FMA by the reference's compiler flags as well. */
void exo_hardswish_f32(const float* x, float* y, long count, float alpha, float beta) {
    for (long i = 0; i < count; ++i) {
        float t = fmaf(x[i], alpha, beta);
        t = t > 0.f ? t : 0.f;
        t = t < 1.f ? t : 1.f;
        y[i] = t * x[i];
    }
}

/* operation_leakyrelu::forward_cpu_f32, src/Excalibur/operation_leakyrelu.cpp:31-58: body max(0,x) + min(0,x)*alpha,
 * tail x < 0 ? alpha*x : x: the same values (the sign of a zero result aside). */
void exo_leakyrelu_f32(const float* x, float* y, long count, float alpha) {
    for (long i = 0; i < count; ++i) y[i] = x[i] < 0.f ? alpha * x[i] : x[i];
}

/* operation_sigmoid::forward_cpu_f32, src/Excalibur/operation_sigmoid.cpp:17-33: 1. / (1. + exp(-x)) in double. */
void exo_sigmoid_f32(const float* x, float* y, long count) {
    for (long i = 0; i < count; ++i) y[i] = (float)(1. / (1. + exp(-(double)x[i])));
}

/* operation_hardsigmoid::forward_cpu_f32, src/Excalibur/operation_hardsigmoid.cpp:33-46:
 * max(0, min(1, alpha*x + beta)), the sum contracted to an FMA by the reference's compiler flags. */
void exo_hardsigmoid_f32(const float* x, float* y, long count, float alpha, float beta) {
    for (long i = 0; i < count; ++i) {
        float t = fmaf(alpha, x[i], beta);
        t = 1.f < t ? 1.f : t;
        y[i] = 0.f < t ? t : 0.f;
    }
}

/* operation_prelu::forward_cpu_f32, src/Excalibur/operation_prelu.cpp:57-124 (NCHW): slope per channel, or one shared
 * slope when 0=1 (:19-22); body max(0,x) + slope*min(0,x), tail x >= 0 ? x : slope*x. */
void exo_prelu_f32(const float* x, float* y, int n, int c, int hw, const float* slope, int shared) {
    for (int i = 0; i < n * c; ++i) {
        const float s = slope[shared ? 0 : i % c];
        for (int j = 0; j < hw; ++j) {
            const float v = x[(size_t)i * hw + j];
            y[(size_t)i * hw + j] = v >= 0.f ? v : s * v;
        }
    }
}

/* operation_batchnorm, src/Excalibur/operation_batchnorm.cpp:33-66 (load time) and :122-156 (forward):
 * sqrt_var = (float)sqrt(var + eps); a = bias - slope*mean/sqrt_var; b = slope/sqrt_var; y = b*x + a, which the
 * reference's flags contract to an FMA. a and b are returned for the caller that wants them (ab may be NULL). */
void exo_batchnorm_f32(const float* x, float* y, int n, int c, int hw, const float* slope, const float* mean,
                       const float* var, const float* bias, float eps, float* ab) {
    for (int ch = 0; ch < c; ++ch) {
        const float sqrt_var = (float)sqrt((double)(var[ch] + eps));
        const float a = bias[ch] - slope[ch] * mean[ch] / sqrt_var;
        const float b = slope[ch] / sqrt_var;
        if (ab) { ab[ch] = a; ab[c + ch] = b; }
        for (int i = 0; i < n; ++i)
            for (int j = 0; j < hw; ++j) {
                const size_t o = ((size_t)i * c + ch) * hw + j;
                y[o] = fmaf(b, x[o], a);
            }
    }
}

/* operation_input::forward_cpu_f32, src/Excalibur/operation_input.cpp:61-151 (NCHW): (x - mean[c]) * var[c];
 * only 1- and 3-channel tensors are accepted (:78,126,143-146). */
void exo_input_f32(const float* x, float* y, int n, int c, int hw, const float* mean, const float* scale) {
    if (c != 1 && c != 3) abort();
    for (int i = 0; i < n * c; ++i)
        for (int j = 0; j < hw; ++j) y[(size_t)i * hw + j] = (x[(size_t)i * hw + j] - mean[i % c]) * scale[i % c];
}

/* operation_concat::forward_cpu_f32, channel axis (file key 0=-1 -> axis 1), NCHW,
 * src/Excalibur/operation_concat.cpp:31-103: per image, the inputs' channel blocks one after the other. */
void exo_concat_channels_f32(const float* const* xs, const int* channels, int n_inputs, int n, int hw, float* y) {
    int total = 0;
    for (int i = 0; i < n_inputs; ++i) total += channels[i];
    for (int img = 0; img < n; ++img) {
        size_t off = 0;
        for (int i = 0; i < n_inputs; ++i) {
            const size_t cnt = (size_t)channels[i] * hw;
            memcpy(y + (size_t)img * total * hw + off, xs[i] + (size_t)img * cnt, cnt * sizeof(float));
            off += cnt;
        }
    }
}

/* operation_interp::forward_cpu_f32, nearest branch (0=1, align_corner 0), src/Excalibur/operation_interp.cpp:247-268:
 * in_y = min((int)(y * hs), h - 1) with hs = h / (float)oh, likewise for x; oh = (int)(h * height_scale) (:232-233). */
void exo_interp_nearest_f32(const float* x, float* y, int n, int c, int h, int w, int oh, int ow) {
    const float hs = h / (float)oh, ws = w / (float)ow;
    for (int i = 0; i < n * c; ++i)
        for (int oy = 0; oy < oh; ++oy) {
            int iy = (int)(oy * hs);
            if (iy > h - 1) iy = h - 1;
            for (int ox = 0; ox < ow; ++ox) {
                int ix = (int)(ox * ws);
                if (ix > w - 1) ix = w - 1;
                y[((size_t)i * oh + oy) * ow + ox] = x[((size_t)i * h + iy) * w + ix];
            }
        }
}

/* operation_yolov5focus::forward_cpu_f32, src/Excalibur/operation_yolov5focus.cpp:17-50: space to depth,
 * out[p][i][j] = in[p % C][2i + (p / C) % 2][2j + (p / C) / 2], p < 4C. The reference fills image 0 only
 * (offset(0, ...), :36-37); this restatement does every image the same way. */
void exo_focus_f32(const float* x, float* y, int n, int c, int h, int w) {
    const int oh = h / 2, ow = w / 2;
    for (int img = 0; img < n; ++img)
        for (int p = 0; p < 4 * c; ++p) {
            const int g = p / c, ch = p % c, dy = g % 2, dx = g / 2;
            for (int i = 0; i < oh; ++i)
                for (int j = 0; j < ow; ++j)
                    y[(((size_t)img * 4 * c + p) * oh + i) * ow + j] = x[(((size_t)img * c + ch) * h + 2 * i + dy) * w + 2 * j + dx];
        }
}

/* operation_deconvolution::forward_cpu_f32, src/Excalibur/operation_deconvolution.cpp:80-171 (group 1, dilation 1):
 * col = W^T x per image (W stored [C][K][kh][kw]), col2im scatters col[k][r][s][i][j] to
 * y[k][i*sh - pt + r][j*sw - pl + s], then the bias is added; OH = (H-1)*sh + kh - (pt+pb). The reference sums
 * in float in its GEMM's order; this restatement sums each output in double and rounds once (compared at 1e-4). */
void exo_deconv2d_f32(const float* x, const float* w, const float* bias, float* y, int n, int c, int h, int wd, int k, int kh,
                      int kw, int sh, int sw, int pt, int pb, int pl, int pr) {
    const int oh = (h - 1) * sh + kh - (pt + pb), ow = (wd - 1) * sw + kw - (pl + pr);
    for (int img = 0; img < n; ++img)
        for (int ko = 0; ko < k; ++ko)
            for (int oy = 0; oy < oh; ++oy)
                for (int ox = 0; ox < ow; ++ox) {
                    double s = 0.0;
                    for (int r = 0; r < kh; ++r) {
                        const int ty = oy + pt - r;
                        if (ty < 0 || ty % sh) continue;
                        const int iy = ty / sh;
                        if (iy >= h) continue;
                        for (int q = 0; q < kw; ++q) {
                            const int tx = ox + pl - q;
                            if (tx < 0 || tx % sw) continue;
                            const int ix = tx / sw;
                            if (ix >= wd) continue;
                            for (int ci = 0; ci < c; ++ci)
                                s += (double)x[(((size_t)img * c + ci) * h + iy) * wd + ix] *
                                     (double)w[(((size_t)ci * k + ko) * kh + r) * kw + q];
                        }
                    }
                    if (bias) s += (double)bias[ko];
                    y[(((size_t)img * k + ko) * oh + oy) * ow + ox] = (float)s;
                }
}

/* operation_clip::forward_cpu_f32, src/Excalibur/operation_clip.cpp:32-58: max(lo, min(hi, x)) (vector body and scalar
 * tail agree for lo <= hi). */
void exo_clip_f32(const float* x, float* y, long count, float lo, float hi) {
    for (long i = 0; i < count; ++i) {
        const float t = hi < x[i] ? hi : x[i];
        y[i] = lo < t ? t : lo;
    }
}

/* operation_softmax::forward_cpu_f32, NCHW branch, src/Excalibur/operation_softmax.cpp:36-96: over the channels of each
 * (image, position): subtract the maximum (exactly x - m, the GEMM update has a single product per element), exponentiate,
 * divide by the sum over channels. The reference sums in its GEMV's order; here channels are added in ascending order
 * (compared at 1e-4). */
void exo_softmax_channels_f32(const float* x, float* y, int n, int c, int hw) {
    for (int img = 0; img < n; ++img)
        for (int k = 0; k < hw; ++k) {
            const float* in = x + (size_t)img * c * hw + k;
            float* out = y + (size_t)img * c * hw + k;
            float m = in[0];
            for (int j = 0; j < c; ++j) m = m < in[(size_t)j * hw] ? in[(size_t)j * hw] : m;
            float sum = 0.f;
            for (int j = 0; j < c; ++j) {
                out[(size_t)j * hw] = expf(in[(size_t)j * hw] - m);
                sum += out[(size_t)j * hw];
            }
            for (int j = 0; j < c; ++j) out[(size_t)j * hw] = out[(size_t)j * hw] / sum;
        }
}

/* operation_transpose::forward_cpu_f32, order (1, 0, 2), src/Excalibur/operation_transpose.cpp:51-70: rows and columns
 * of every channel plane change places, y[n][c][i][j] = x[n][c][j][i], output shape [n][c][w][h]. */
void exo_transpose_hw_f32(const float* x, float* y, long planes, int h, int w) {
    for (long p = 0; p < planes; ++p)
        for (int i = 0; i < w; ++i)
            for (int j = 0; j < h; ++j) y[((size_t)p * w + i) * h + j] = x[((size_t)p * h + j) * w + i];
}

/* operation_binaryop::forward_cpu_f32 without the scalar form, src/Excalibur/operation_binaryop.cpp:9-96,152-199,395-448:
 * op 0 ADD, 1 SUB, 2 MUL, 3 DIV on two NCHW tensors. The operand with more non-unit dimensions among (C, H, W) (on a
 * tie: the second if one of its dimensions is larger) is the "larger" one and gives the output its shape. Cases
 * restated: equal shapes, op(a, b); a smaller operand of one value per image, op(large, value); [N][C][H][W] with
 * [N][C][1][1], op(small[c], large) -- the small operand comes first; [N][C][H][W] with [N][1][H][W],
 * op(small[pixel], large). The smaller operand's images repeat modulo its batch size. Returns 0, or -1 for a shape
 * pair the reference does not implement or that is not restated here. */
static float exo_binop(int op, float x, float y) {
    switch (op) {
    case 0: return x + y;
    case 1: return x - y;
    case 2: return x * y;
    default: return x / y;
    }
}
int exo_binaryop_f32(int op, const float* a, const int* a_shape, const float* b, const int* b_shape, float* y, int* y_shape) {
    int second_larger = 0, same = 1;
    for (int i = 0; i < 4; ++i) same = same && a_shape[i] == b_shape[i];
    if (!same) {
        const int d1 = (a_shape[3] != 1) + (a_shape[2] != 1) + (a_shape[1] != 1);
        const int d2 = (b_shape[3] != 1) + (b_shape[2] != 1) + (b_shape[1] != 1);
        if (d2 > d1) second_larger = 1;
        else if (d2 == d1)
            for (int i = 1; i < 4; ++i)
                if (b_shape[i] > a_shape[i]) { second_larger = 1; break; }
    }
    const float* big = second_larger ? b : a;
    const float* small = second_larger ? a : b;
    const int* bs = second_larger ? b_shape : a_shape;
    const int* ss = second_larger ? a_shape : b_shape;
    for (int i = 0; i < 4; ++i) y_shape[i] = bs[i];
    const long chw = (long)bs[1] * bs[2] * bs[3], hw = (long)bs[2] * bs[3], small_chw = (long)ss[1] * ss[2] * ss[3];
    int big_dims = (bs[3] != 1) + (bs[2] != 1) + (bs[1] != 1), small_dims = (ss[3] != 1) + (ss[2] != 1) + (ss[1] != 1);
    big_dims = big_dims ? big_dims : 1;
    small_dims = small_dims ? small_dims : 1;
    if (same) {
        for (long i = 0; i < bs[0] * chw; ++i) y[i] = exo_binop(op, big[i], small[i]);
        return 0;
    }
    if (small_chw == 1) {
        for (int n = 0; n < bs[0]; ++n)
            for (long i = 0; i < chw; ++i) y[n * chw + i] = exo_binop(op, big[n * chw + i], small[n % ss[0]]);
        return 0;
    }
    if (big_dims == 3 && small_dims == 2 && ss[1] == 1 && (long)ss[2] * ss[3] == hw) {
        for (int n = 0; n < bs[0]; ++n)
            for (int c = 0; c < bs[1]; ++c)
                for (long i = 0; i < hw; ++i)
                    y[n * chw + c * hw + i] = exo_binop(op, small[(n % ss[0]) * small_chw + i], big[n * chw + c * hw + i]);
        return 0;
    }
    if (big_dims == 3 && small_dims == 1 && ss[1] > 1 && ss[1] == bs[1]) {
        for (int n = 0; n < bs[0]; ++n)
            for (int c = 0; c < bs[1]; ++c)
                for (long i = 0; i < hw; ++i)
                    y[n * chw + c * hw + i] = exo_binop(op, small[(n % ss[0]) * small_chw + c], big[n * chw + c * hw + i]);
        return 0;
    }
    return -1;
}
