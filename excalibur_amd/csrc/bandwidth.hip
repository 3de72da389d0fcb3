// Bandwidth-bound operators of the CNN forward path: layout / precision conversion, depthwise 3x3,
// pooling, elementwise, inner product, and a definition-order convolution for shapes the MFMA path
// does not take. All are one pass over their operands; arithmetic follows the reference's CPU order
// where that order is observable in the result (depthwise columns, average-pool row-major sums,
// saxpby rounding), so these kernels are bit-exact against it in fp32.
#include <float.h>

#include <mutex>
#include <type_traits>

#include "common.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v8f __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

namespace {

constexpr int kBlock = 256;
inline unsigned blocks_for(size_t n, int per_block = kBlock) { return (unsigned)((n + per_block - 1) / per_block); }

// ---------------------------------------------------------------------------------------------
// NCHW -> NHWC with optional quantization. One workgroup moves 64 pixels x 64 channels through LDS:
// reads are coalesced along pixels of a channel plane, writes are 16-byte runs of channels.
// MODE 0: f32 -> i8 (quantize), 1: f32 -> f32, 2: f32 -> f16, 3: f16 -> f16
// ---------------------------------------------------------------------------------------------
template <int MODE> struct Conv;
template <> struct Conv<0> { typedef float in_t; typedef int8_t out_t; };
template <> struct Conv<1> { typedef float in_t; typedef float out_t; };
template <> struct Conv<2> { typedef float in_t; typedef uint16_t out_t; };
template <> struct Conv<3> { typedef uint16_t in_t; typedef uint16_t out_t; };

template <int MODE>
__global__ __launch_bounds__(kBlock) void nchw_to_nhwc_kernel(const typename Conv<MODE>::in_t* __restrict__ x,
                                                              typename Conv<MODE>::out_t* __restrict__ y, int C, int HW,
                                                              int c_stride, float fs, const float* __restrict__ fs_pc,
                                                              int quads) {
    typedef typename Conv<MODE>::out_t out_t;
    constexpr int ES = sizeof(out_t);
    constexpr int ROW = 64 * ES + 4;  // bytes per pixel row in LDS; ROW/4 is odd: conflict-free column writes
    __shared__ __attribute__((aligned(16))) char tile[64 * ROW];
    const int n = blockIdx.y, p0 = blockIdx.x * 64, tid = threadIdx.x;
    const int px = tid & 63, csub = tid >> 6;
    for (int c0 = 0; c0 < c_stride; c0 += 64) {
        if (quads) {
            // four pixels of one channel per load: 16 pixel quads x 16 channels per pass
            const int quad = tid & 15, crow = tid >> 4;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int cl = i * 16 + crow, c = c0 + cl, p = p0 + 4 * quad;
                typename Conv<MODE>::in_t in[4] = {0, 0, 0, 0};
                const bool live = c < C && p < HW;
                if (live) {
                    const auto* src = x + ((size_t)n * C + c) * HW + p;
                    if constexpr (sizeof(in[0]) == 4) {
                        const v4f v = *reinterpret_cast<const v4f*>(src);
#pragma unroll
                        for (int e = 0; e < 4; ++e) in[e] = v[e];
                    } else {
                        const v2i v = *reinterpret_cast<const v2i*>(src);
#pragma unroll
                        for (int e = 0; e < 4; ++e) in[e] = (uint16_t)(((uint32_t)v[e >> 1] >> ((e & 1) * 16)) & 0xffff);
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    out_t v = 0;
                    if (live) {
                        if constexpr (MODE == 0) v = (out_t)exhip_q8(in[e] * (fs_pc ? fs_pc[c] : fs));
                        else if constexpr (MODE == 2) v = exhip_f2h(in[e]);
                        else v = in[e];
                    }
                    *reinterpret_cast<out_t*>(tile + (4 * quad + e) * ROW + cl * ES) = v;
                }
            }
        } else
#pragma unroll 4
        for (int i = 0; i < 16; ++i) {
            const int cl = i * 4 + csub, c = c0 + cl, p = p0 + px;
            out_t v = 0;
            if (c < C && p < HW) {
                const auto in = x[((size_t)n * C + c) * HW + p];
                if constexpr (MODE == 0) v = (out_t)exhip_q8(in * (fs_pc ? fs_pc[c] : fs));
                else if constexpr (MODE == 2) v = exhip_f2h(in);
                else v = in;
            }
            *reinterpret_cast<out_t*>(tile + px * ROW + cl * ES) = v;
        }
        __syncthreads();
        // 64 pixels x (64*ES/16) vectors of 16 bytes
        constexpr int VPP = 64 * ES / 16;
        for (int v = tid; v < 64 * VPP; v += kBlock) {
            const int pp = v / VPP, part = v % VPP;
            const int cbase = c0 + part * (16 / ES);
            if (p0 + pp < HW && cbase < c_stride) {
                const int* src = reinterpret_cast<const int*>(tile + pp * ROW + part * 16);
                out_t* dst = y + ((size_t)n * HW + p0 + pp) * c_stride + cbase;
                if (cbase + 16 / ES <= c_stride && (c_stride * ES) % 16 == 0) {
                    v4i o = {src[0], src[1], src[2], src[3]};
                    *reinterpret_cast<v4i*>(dst) = o;
                } else {
                    const out_t* s = reinterpret_cast<const out_t*>(src);
                    for (int e = 0; e < 16 / ES && cbase + e < c_stride; ++e) dst[e] = s[e];
                }
            }
        }
        __syncthreads();
    }
}

// First-layer form: C <= 4 channels packed into one 4-byte int8 pixel (one thread per pixel).
__global__ __launch_bounds__(kBlock) void quantize_nchw_to_nhwc4_kernel(const float* __restrict__ x, int* __restrict__ y,
                                                                        int C, int HW, float fs,
                                                                        const float* __restrict__ fs_pc) {
    const int n = blockIdx.y;
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= HW) return;
    uint32_t w = 0;
    for (int c = 0; c < C; ++c) {
        const float v = x[((size_t)n * C + c) * HW + p] * (fs_pc ? fs_pc[c] : fs);
        w |= (uint32_t)(exhip_q8(v) & 0xff) << (8 * c);
    }
    y[(size_t)n * HW + p] = (int)w;
}

// The same with four pixels per thread: 16-byte loads from each channel plane and one 16-byte store
// (HW a multiple of 4, 16-byte aligned tensors).
__global__ __launch_bounds__(kBlock) void quantize_nchw_to_nhwc4_x4_kernel(const float* __restrict__ x, int4* __restrict__ y,
                                                                           int C, int HW4, float fs,
                                                                           const float* __restrict__ fs_pc) {
    const int n = blockIdx.y;
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= HW4) return;
    uint32_t w[4] = {0, 0, 0, 0};
    for (int c = 0; c < C; ++c) {
        const float s = fs_pc ? fs_pc[c] : fs;
        const float4 v = reinterpret_cast<const float4*>(x + ((size_t)n * C + c) * HW4 * 4)[p];
        w[0] |= (uint32_t)(exhip_q8(v.x * s) & 0xff) << (8 * c);
        w[1] |= (uint32_t)(exhip_q8(v.y * s) & 0xff) << (8 * c);
        w[2] |= (uint32_t)(exhip_q8(v.z * s) & 0xff) << (8 * c);
        w[3] |= (uint32_t)(exhip_q8(v.w * s) & 0xff) << (8 * c);
    }
    y[(size_t)n * HW4 + p] = make_int4((int)w[0], (int)w[1], (int)w[2], (int)w[3]);
}

// Half NCHW planes of an image with at most four channels -> NHWC pixels of four halves (the packed first-layer form of
// the fp16 convolution; absent channels are zero). Eight pixels per thread: one 16-byte load per plane, four 16-byte
// stores (HW a multiple of 8, 16-byte aligned tensors).
__global__ __launch_bounds__(kBlock) void nchw_f16_to_nhwc4_x8_kernel(const uint16_t* __restrict__ x, v4i* __restrict__ y, int C, int HW8) {
    const int n = blockIdx.y;
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= HW8) return;
    v4i plane[4] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
    for (int c = 0; c < 4; ++c)
        if (c < C) plane[c] = reinterpret_cast<const v4i*>(x + ((size_t)n * C + c) * HW8 * 8)[p];
    auto half_of = [](const v4i& v, int i) { return ((unsigned)v[i >> 1] >> ((i & 1) * 16)) & 0xffffu; };
    v4i* dst = y + ((size_t)n * HW8 + p) * 4;   // eight pixels x 8 bytes = four 16-byte vectors
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        v4i o;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int px = 2 * q + e;
            o[2 * e] = (int)(half_of(plane[0], px) | (half_of(plane[1], px) << 16));
            o[2 * e + 1] = (int)(half_of(plane[2], px) | (half_of(plane[3], px) << 16));
        }
        dst[q] = o;
    }
}

// NHWC -> NCHW (graph outputs; small). MODE 0: f32->f32, 1: f16->f32, 2: f16->f16
template <int MODE, typename Tin, typename Tout>
__global__ __launch_bounds__(kBlock) void nhwc_to_nchw_kernel(const Tin* __restrict__ x, Tout* __restrict__ y, int C, int HW,
                                                              int c_stride, size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int p = (int)(i % HW);
    const size_t nc = i / HW;
    const int c = (int)(nc % C);
    const size_t n = nc / C;
    const Tin v = x[(n * HW + p) * c_stride + c];
    if constexpr (MODE == 1) y[i] = exhip_h2f(v);
    else y[i] = v;
}

// Precision conversion, eight values per thread over the 16-byte aligned body and one per thread over the rest.
// The same through LDS for tensors of some size: a workgroup moves 64 pixels x 64 channels; 16-byte reads along the
// channels of a pixel, stores of 64 consecutive pixels of a channel plane.
template <int MODE, typename Tin, typename Tout>
__global__ __launch_bounds__(kBlock) void nhwc_to_nchw_tiled_kernel(const Tin* __restrict__ x, Tout* __restrict__ y, int C, int HW,
                                                                    int c_stride) {
    constexpr int VE = 16 / sizeof(Tin);  // elements per 16-byte read
    constexpr int VPP = 64 / VE;          // reads per pixel of the tile
    constexpr int PITCH = 65;             // words per channel row in LDS: odd, so pixel columns spread over the banks
    __shared__ Tout tile[64 * PITCH];
    const int n = blockIdx.y, p0 = blockIdx.x * 64, tid = threadIdx.x;
    for (int c0 = 0; c0 < C; c0 += 64) {
        for (int v = tid; v < 64 * VPP; v += kBlock) {
            const int pp = v / VPP, part = v % VPP;
            const int cb = c0 + part * VE;
            if (p0 + pp < HW && cb < c_stride) {
                const v4i raw = *reinterpret_cast<const v4i*>(x + ((size_t)n * HW + p0 + pp) * c_stride + cb);
                if constexpr (sizeof(Tin) == 4) {
                    const v4f f = __builtin_bit_cast(v4f, raw);
#pragma unroll
                    for (int e = 0; e < 4; ++e) tile[(part * VE + e) * PITCH + pp] = (Tout)f[e];
                } else {
                    const v8h hv = __builtin_bit_cast(v8h, raw);
                    const v4i words = raw;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if constexpr (MODE == 1) tile[(part * VE + e) * PITCH + pp] = (float)hv[e];
                        else tile[(part * VE + e) * PITCH + pp] = (Tout)(((uint32_t)words[e >> 1] >> ((e & 1) * 16)) & 0xffff);
                    }
                }
            }
        }
        __syncthreads();
        const int px = tid & 63, csub = tid >> 6;
#pragma unroll 4
        for (int i = 0; i < 16; ++i) {
            const int cl = i * 4 + csub, c = c0 + cl;
            if (c < C && p0 + px < HW) y[((size_t)n * C + c) * HW + p0 + px] = tile[cl * PITCH + px];
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(kBlock) void f32_to_f16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y, size_t n8,
                                                            size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n8) {
        const v4f a = reinterpret_cast<const v4f*>(x)[2 * i], b = reinterpret_cast<const v4f*>(x)[2 * i + 1];
        const v2i lo = __builtin_bit_cast(v2i, __builtin_convertvector(a, v4h)), hi = __builtin_bit_cast(v2i, __builtin_convertvector(b, v4h));
        const v4i o = {lo[0], lo[1], hi[0], hi[1]};
        reinterpret_cast<v4i*>(y)[i] = o;
    } else {
        const size_t j = n8 * 8 + (i - n8);
        if (j < n) y[j] = exhip_f2h(x[j]);
    }
}
__global__ __launch_bounds__(kBlock) void f16_to_f32_kernel(const uint16_t* __restrict__ x, float* __restrict__ y, size_t n8,
                                                            size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n8) {
        const v8h v = __builtin_bit_cast(v8h, reinterpret_cast<const v4i*>(x)[i]);
        const v8f f = __builtin_convertvector(v, v8f);
        const v4f a = {f[0], f[1], f[2], f[3]}, b = {f[4], f[5], f[6], f[7]};
        reinterpret_cast<v4f*>(y)[2 * i] = a;
        reinterpret_cast<v4f*>(y)[2 * i + 1] = b;
    } else {
        const size_t j = n8 * 8 + (i - n8);
        if (j < n) y[j] = exhip_h2f(x[j]);
    }
}

// ---------------------------------------------------------------------------------------------
// Depthwise 3x3. Column order of the reference: col_j = fma(r2j,k2j, fma(r1j,k1j, fma(r0j,k0j,0)));
// out = ((bias + col0) + col1) + col2; then the fused activation.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float dw_pixel(const float r[3][3], const float* k, float bias) {
    float col[3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 3; ++i) s = __builtin_fmaf(r[i][j], k[i * 3 + j], s);
        col[j] = s;
    }
    float sum = bias;
    sum += col[0];
    sum += col[1];
    sum += col[2];
    return sum;
}

// Workgroup ids are dealt round-robin to the chip's 8 XCDs, each with an L2 of its own. Remapped like this every XCD
// works on one contiguous run of a kernel's blocks, so that neighbouring blocks (row bands of one image, which read each
// other's border rows) meet in one L2.
__device__ __forceinline__ unsigned xcd_contiguous_block() {
    const unsigned per = gridDim.x >> 3, b = blockIdx.x;
    return b < (per << 3) ? (b & 7) * per + (b >> 3) : b;
}

__global__ __launch_bounds__(kBlock) void dwconv3x3_nchw_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                    const float* __restrict__ bias, float* __restrict__ y,
                                                                    int C, int H, int W, int OH, int OW, int stride, int pt,
                                                                    int pl, int act, size_t total) {
    const size_t gi = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (gi >= total) return;
    const size_t nc = gi / ((size_t)OH * OW);
    const int c = (int)(nc % C);
    const int o = (int)(gi - nc * ((size_t)OH * OW));
    const int oy = o / OW, ox = o - oy * OW;
    const float* in = x + (size_t)nc * H * W;
    float k[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) k[i] = w[c * 9 + i];
    float r[3][3];
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const int iy = oy * stride - pt + i, ix = ox * stride - pl + j;
            r[i][j] = (iy >= 0 && iy < H && ix >= 0 && ix < W) ? in[(size_t)iy * W + ix] : 0.f;
        }
    y[(size_t)nc * OH * OW + o] = exhip_act(dw_pixel(r, k, bias ? bias[c] : 0.f), act);
}

// Strip form of the NCHW float kernel for stride 1 and 2, rows a multiple of four floats long, left padding 0 or 1
// and the activations that need no transcendental: a thread makes four neighbouring outputs of a row and walks a
// band of output rows with the three input rows it needs in registers. A row arrives as one (stride 1) or two
// (stride 2) aligned 16-byte loads plus the halo floats the padding asks for, through a buffer descriptor whose
// range check turns taps outside the image into zeros. slot i of a row holds column c0 - 1 + i.
constexpr int kDwPrelu = 100;  // ACT of the strip kernels: no activation of the layer's own, then the PReLU layer behind it
template <int STRIDE, int ACT, int PL>
__global__ __launch_bounds__(kBlock) void dwconv3x3_nchw_f32_strip_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                          const float* __restrict__ bias, float* __restrict__ y,
                                                                          int C, int H, int W, int OH, int OW, int pt,
                                                                          int band_rows, int bands, int strips, unsigned x_bytes,
                                                                          unsigned y_bytes, size_t total,
                                                                          const float* __restrict__ slope, int slope_shared) {
    constexpr int pl = PL;  // left padding (0 or 1) as a constant: which register a tap reads is then fixed, and the halo
                            // floats that this padding does not use are not loaded
    constexpr int CH = STRIDE == 1 ? 1 : 2;  // aligned 16-byte chunks per row
    constexpr int NI = 4 * CH + 3, KEEP = 3 - STRIDE;
    constexpr unsigned kRowOutside = 0x80000000u, kColOutside = 0x40000000u;  // tensors are at most 2^30 bytes
    const size_t gi = (size_t)xcd_contiguous_block() * kBlock + threadIdx.x;
    if (gi >= total) return;
    const int t = (int)(gi % strips);
    size_t rest = gi / strips;
    const int band = (int)(rest % bands);
    const int nc = (int)(rest / bands);
    const int c = nc % C;
    float k[9];
#pragma unroll
    for (int q = 0; q < 9; ++q) k[q] = w[c * 9 + q];
    const float b = bias ? bias[c] : 0.f;
    const float sl = ACT == kDwPrelu ? slope[slope_shared ? 0 : c] : 0.f;  // the PReLU layer behind this one
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x), 0, (int)x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(y, 0, (int)y_bytes, 0x00020000);
    const int c0 = 4 * CH * t;
    unsigned chunk_off[CH], halo_off[3];  // halo slots: 0, NI - 2, NI - 1
#pragma unroll
    for (int q = 0; q < CH; ++q) chunk_off[q] = c0 + 4 * q < W ? (unsigned)((c0 + 4 * q) * 4) : kColOutside;
    {
        const int cols[3] = {c0 - 1, c0 + 4 * CH, c0 + 4 * CH + 1};
        const bool used[3] = {pl == 1, STRIDE == 1 || pl == 0, STRIDE == 1 && pl == 0};
#pragma unroll
        for (int q = 0; q < 3; ++q) halo_off[q] = used[q] && cols[q] >= 0 && cols[q] < W ? (unsigned)(cols[q] * 4) : kColOutside;
    }
    const int plane_off = nc * H * W * 4;
    float r[3][NI], nxt[STRIDE][NI];
    auto fetch = [&](int iy, float (&dst)[NI]) {
        const unsigned row_off = iy >= 0 && iy < H ? (unsigned)(plane_off + iy * W * 4) : kRowOutside;
#pragma unroll
        for (int q = 0; q < CH; ++q) {
            const v4f v = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(xr, (int)(row_off + chunk_off[q]), 0, 0));
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[1 + 4 * q + e] = v[e];
        }
        dst[0] = dst[NI - 2] = dst[NI - 1] = 0.f;
        if constexpr (pl == 1) dst[0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, (int)(row_off + halo_off[0]), 0, 0));
        if constexpr (STRIDE == 1 || pl == 0)
            dst[NI - 2] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, (int)(row_off + halo_off[1]), 0, 0));
        if constexpr (STRIDE == 1 && pl == 0)
            dst[NI - 1] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xr, (int)(row_off + halo_off[2]), 0, 0));
    };
    const int oy0 = band * band_rows, oy1 = min(OH, oy0 + band_rows);
#pragma unroll
    for (int a = 0; a < KEEP; ++a) fetch(oy0 * STRIDE - pt + a, r[STRIDE + a]);
#pragma unroll
    for (int a = 0; a < STRIDE; ++a) fetch(oy0 * STRIDE - pt + KEEP + a, nxt[a]);
    unsigned out_off = (unsigned)(((nc * OH + oy0) * OW + 4 * t) * 4);
    const bool whole = (OW & 3) == 0;
    for (int oy = oy0; oy < oy1; ++oy, out_off += OW * 4) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
#pragma unroll
            for (int a = 0; a < KEEP; ++a) r[a][i] = r[a + STRIDE][i];
#pragma unroll
            for (int a = 0; a < STRIDE; ++a) r[KEEP + a][i] = nxt[a][i];
        }
        if (oy + 1 < oy1) {
#pragma unroll
            for (int a = 0; a < STRIDE; ++a) fetch((oy + 1) * STRIDE - pt + KEEP + a, nxt[a]);
        }
        v4f out;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float sum = b;
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                float col = 0.f;
#pragma unroll
                for (int a = 0; a < 3; ++a) col = __builtin_fmaf(pl == 1 ? r[a][j * STRIDE + q] : r[a][j * STRIDE + q + 1], k[a * 3 + q], col);
                sum += col;
            }
            if (ACT == kDwPrelu) sum = sum >= 0.f ? sum : sl * sum;
            else if (ACT != 0) sum = (0.f > sum) ? 0.f : sum;
            if (ACT == 3) sum = sum <= 6.f ? sum : 0.f;
            out[j] = sum;
        }
        const v4i bits = __builtin_bit_cast(v4i, out);  // cast the whole vector: a cast of one element picks element 0
        if (whole) {
            __builtin_amdgcn_raw_buffer_store_b128(bits, yr, (int)out_off, 0, 0);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                __builtin_amdgcn_raw_buffer_store_b32(bits[j], yr,
                                                      (int)(4 * t + j < OW ? out_off + 4 * j : kRowOutside), 0, 0);
        }
    }
}

// NHWC half storage, 8 channels (16 bytes) per thread, f32 math in the same order.
__global__ __launch_bounds__(kBlock) void dwconv3x3_nhwc_f16_kernel(const uint16_t* __restrict__ x, const float* __restrict__ w,
                                                                    const float* __restrict__ bias, uint16_t* __restrict__ y,
                                                                    int C, int H, int W, int cs, int OH, int OW, int stride,
                                                                    int pt, int pl, int act, size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int groups = cs / 8;
    const int g = (int)(i % groups);
    size_t pix = i / groups;
    const int ox = (int)(pix % OW);
    pix /= OW;
    const int oy = (int)(pix % OH);
    const size_t n = pix / OH;
    float r[8][3][3];
#pragma unroll
    for (int a = 0; a < 3; ++a)
#pragma unroll
        for (int b = 0; b < 3; ++b) {
            const int iy = oy * stride - pt + a, ix = ox * stride - pl + b;
            v4i v = {0, 0, 0, 0};
            if (iy >= 0 && iy < H && ix >= 0 && ix < W)
                v = *reinterpret_cast<const v4i*>(x + ((n * H + iy) * W + ix) * cs + g * 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                r[2 * e][a][b] = exhip_h2f((uint16_t)(v[e] & 0xffff));
                r[2 * e + 1][a][b] = exhip_h2f((uint16_t)((uint32_t)v[e] >> 16));
            }
        }
    v4i o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int c = g * 8 + e;
        float res = 0.f;
        if (c < C) {
            float k[9];
#pragma unroll
            for (int q = 0; q < 9; ++q) k[q] = w[c * 9 + q];
            res = exhip_act(dw_pixel(r[e], k, bias ? bias[c] : 0.f), act);
        }
        const uint32_t h = exhip_f2h(res);
        if (e & 1) o[e >> 1] |= (int)(h << 16);
        else o[e >> 1] = (int)h;
    }
    *reinterpret_cast<v4i*>(y + ((n * OH + oy) * OW + ox) * cs + g * 8) = o;
}

// Strip form of the same layer for stride 1 and 2 and the activations that need no transcendental: a thread owns
// 4 channels (8 bytes) of a strip of PX output pixels and walks a band of output rows, keeping the three input
// rows it needs as stored (two halves to a register), so every input value is fetched once per band and the 36
// weights once per thread. The next step's rows are requested before the current outputs are computed. Loads and
// stores go through buffer descriptors over the whole tensors: a tap outside the image, or an output pixel beyond
// the row's end, gets an offset beyond the descriptor's range and reads as zero / is dropped. The kernel is bound
// by vector ALU issue as much as by memory, hence the template on the activation and the masked, packed stores.
// Arithmetic order per output is that of dw_pixel.
template <int STRIDE, int PX, int ACT>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(3, 4))) void dwconv3x3_nhwc_f16_strip_kernel(const uint16_t* __restrict__ x,
                                                                          const float* __restrict__ w,
                                                                          const float* __restrict__ bias,
                                                                          uint16_t* __restrict__ y, int C, int H, int W,
                                                                          int cs, int OH, int OW, int pt, int pl,
                                                                          int band_rows, int bands, int strips,
                                                                          unsigned x_bytes, unsigned y_bytes, size_t total,
                                                                          const float* __restrict__ slope, int slope_shared) {
    constexpr int NC = (PX - 1) * STRIDE + 3, KEEP = 3 - STRIDE;
    // out-of-range markers: a tensor is at most 2^30 bytes, so a valid row offset plus the column marker, the row
    // marker plus anything, and both markers together all land beyond the descriptor's range without wrapping
    constexpr unsigned kRowOutside = 0x80000000u, kColOutside = 0x40000000u;
    const size_t i = (size_t)xcd_contiguous_block() * kBlock + threadIdx.x;
    if (i >= total) return;
    const int groups = cs / 4;
    const int g = (int)(i % groups);
    size_t t = i / groups;
    const int xs = (int)(t % strips);
    t /= strips;
    const int band = (int)(t % bands);
    const int n = (int)(t / bands);
    const int c0 = g * 4;
    float k[4][9], b[4];
    if (c0 + 4 <= C) {  // 36 consecutive floats, 16-byte aligned
        v4f kv[9];
#pragma unroll
        for (int q = 0; q < 9; ++q) kv[q] = reinterpret_cast<const v4f*>(w + c0 * 9)[q];
#pragma unroll
        for (int q = 0; q < 36; ++q) k[q / 9][q % 9] = kv[q / 4][q % 4];
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int c = min(c0 + e, C - 1);
#pragma unroll
            for (int q = 0; q < 9; ++q) k[e][q] = w[c * 9 + q];
        }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) b[e] = bias ? bias[min(c0 + e, C - 1)] : 0.f;
    float sl[4] = {0.f, 0.f, 0.f, 0.f};  // the PReLU layer behind this one
    if (ACT == kDwPrelu) {
#pragma unroll
        for (int e = 0; e < 4; ++e) sl[e] = slope[slope_shared ? 0 : min(c0 + e, C - 1)];
    }
    // channels of the padding are stored as zero halves
    const int keep_lo = (c0 < C ? 0xffff : 0) | (c0 + 1 < C ? 0xffff0000 : 0);
    const int keep_hi = (c0 + 2 < C ? 0xffff : 0) | (c0 + 3 < C ? 0xffff0000 : 0);
    const bool ragged_c = (C & 3) != 0 || cs != C;  // uniform over the launch: whole groups of four channels need no masks
    const int oy0 = band * band_rows, oy1 = min(OH, oy0 + band_rows);
    const int ox0 = xs * PX, ix0 = ox0 * STRIDE - pl;
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(x), 0, (int)x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(y, 0, (int)y_bytes, 0x00020000);
    const int row_b = W * cs * 2, orow_b = OW * cs * 2;
    const int img_off = n * H * row_b + c0 * 2;
    unsigned col_off[NC], ocol_off[PX];  // byte offsets within a row, or the marker
#pragma unroll
    for (int cidx = 0; cidx < NC; ++cidx) {
        const int ix = ix0 + cidx;
        col_off[cidx] = ix >= 0 && ix < W ? (unsigned)(ix * cs * 2) : kColOutside;
    }
#pragma unroll
    for (int px = 0; px < PX; ++px) ocol_off[px] = ox0 + px < OW ? (unsigned)((ox0 + px) * cs * 2) : kColOutside;
    // The input rows live in a ring of 3 + D * STRIDE register rows: output row t reads ring slots (t * STRIDE + a) % R,
    // a = 0 .. 2, while the rows the next D output rows add are already on their way into the slots behind them. The
    // row loop is unrolled over one turn of the ring, so every slot index is a constant and no row is ever copied.
    // D: how many output rows ahead the input rows are requested (two at stride 1, where a row's arithmetic is too short to
    // cover the memory latency with three waves per SIMD).
    constexpr int D = STRIDE == 1 ? 2 : 1;
    constexpr int R = 3 + D * STRIDE, TURN = R;  // R and STRIDE are coprime (4 or 5 and 1, 5 and 2): a turn is R output rows
    v4h r[R][NC];
    auto fetch = [&](int iy, v4h (&dst)[NC]) {
        const unsigned row_off = iy >= 0 && iy < H ? (unsigned)(img_off + iy * row_b) : kRowOutside;
#pragma unroll
        for (int cidx = 0; cidx < NC; ++cidx)
            dst[cidx] = __builtin_bit_cast(v4h, __builtin_amdgcn_raw_buffer_load_b64(xr, (int)(row_off + col_off[cidx]), 0, 0));
    };
#pragma unroll
    for (int a = 0; a < (D - 1) * STRIDE + 3; ++a) fetch(oy0 * STRIDE - pt + a, r[a]);
    unsigned orow_off = (unsigned)((n * OH + oy0) * orow_b + c0 * 2);
    // one output row, PH = its position in the turn
    auto row = [&](auto ph, int oy) {
        constexpr int PH = decltype(ph)::value;
        if (oy + D < oy1) {
#pragma unroll
            for (int a = 0; a < STRIDE; ++a)
                fetch((oy + D) * STRIDE - pt + 3 - STRIDE + a, r[((PH + D) * STRIDE + 3 - STRIDE + a) % R]);
        }
#pragma unroll
        for (int px = 0; px < PX; ++px) {
            v4f res;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float sum = b[e];
#pragma unroll
                for (int j = 0; j < 3; ++j) {
                    float s = 0.f;
#pragma unroll
                    for (int a = 0; a < 3; ++a) s = __builtin_fmaf((float)r[(PH * STRIDE + a) % R][px * STRIDE + j][e], k[e][a * 3 + j], s);
                    sum += s;
                }
                // activations 0 (none), 1 (ReLU), 3 (ReLU6 as the reference writes it)
                if (ACT == kDwPrelu) {
                    sum = exhip_h2f(exhip_f2h(sum));  // the PReLU layer reads the stored half
                    sum = sum >= 0.f ? sum : sl[e] * sum;
                } else if (ACT != 0) {
                    sum = (0.f > sum) ? 0.f : sum;
                }
                if (ACT == 3) sum = sum <= 6.f ? sum : 0.f;
                res[e] = sum;
            }
            v2i o = __builtin_bit_cast(v2i, __builtin_convertvector(res, v4h));
            if (ragged_c) {
                o[0] &= keep_lo;
                o[1] &= keep_hi;
            }
            __builtin_amdgcn_raw_buffer_store_b64(o, yr, (int)(orow_off + ocol_off[px]), 0, 0);
        }
        orow_off += orow_b;
    };
    auto turn = [&](auto self, auto ph, int oy) -> void {
        constexpr int PH = decltype(ph)::value;
        if constexpr (PH < TURN) {
            if (oy < oy1) {
                row(ph, oy);
                self(self, std::integral_constant<int, PH + 1>{}, oy + 1);
            }
        }
    };
    for (int oy = oy0; oy < oy1; oy += TURN) turn(turn, std::integral_constant<int, 0>{}, oy);
}

__global__ __launch_bounds__(kBlock) void dw_dequant_kernel(const int8_t* __restrict__ w, const float* __restrict__ ws,
                                                            float* __restrict__ wf, int k, int per_group) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= k * per_group) return;
    const float s = ws[i / per_group] <= 1e-6f ? 0.f : 1.f / ws[i / per_group];
    wf[i] = (float)w[i] * s;
}

// ---------------------------------------------------------------------------------------------
// Pooling
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void pool2d_nchw_f32_kernel(const float* __restrict__ x, float* __restrict__ y, int H, int W,
                                                                 int OH, int OW, int type, int kh, int kw, int sh, int sw,
                                                                 int pt, int pb, int pl, int pr, int include_pad,
                                                                 size_t total) {
    // flat index over (plane, output pixel): global pooling then runs one plane per thread
    const size_t gi = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (gi >= total) return;
    const size_t nc = gi / ((size_t)OH * OW);
    const int o = (int)(gi - nc * ((size_t)OH * OW));
    const int ph = o / OW, pw = o - ph * OW;
    const float* in = x + (size_t)nc * H * W;
    int hs = ph * sh - pt, wsx = pw * sw - pl;
    float out;
    if (type == 0) {
        const int he = min(hs + kh, H), we = min(wsx + kw, W);
        hs = max(hs, 0);
        wsx = max(wsx, 0);
        float v = -FLT_MAX;
        for (int a = hs; a < he; ++a)
            for (int b = wsx; b < we; ++b) {
                const float t = in[(size_t)a * W + b];
                v = v < t ? t : v;
            }
        out = v;
    } else {
        int he = min(hs + kh, H + pb), we = min(wsx + kw, W + pr);
        int pool = (he - hs) * (we - wsx);
        hs = max(hs, 0);
        wsx = max(wsx, 0);
        he = min(he, H);
        we = min(we, W);
        float s = 0.f;
        for (int a = hs; a < he; ++a)
            for (int b = wsx; b < we; ++b) s += in[(size_t)a * W + b];
        if (!include_pad) pool = (he - hs) * (we - wsx);
        out = s / (float)pool;
    }
    y[(size_t)nc * OH * OW + o] = out;
}

// Stride-2 pooling with a 2x2 or 3x3 window over planes whose rows are a multiple of four floats long: a thread
// makes four neighbouring outputs of one row from two aligned 16-byte loads per input row (plus one halo float to
// the left for left padding 1, or to the right for a 3-wide window without left padding), so a wave reads whole
// rows contiguously. Window clipping, the divisor and the row-major summation order are those of the general kernel.
template <int K, int TYPE, int ROWS, int PL>
__global__ __launch_bounds__(kBlock) void pool_s2_nchw_f32_strip_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                        int H, int W, int OH, int OW, int pt, int pb,
                                                                        int pr, int include_pad, int strips, int row_blocks,
                                                                        size_t total) {
    constexpr int pl = PL;  // left padding, 0 or 1: a constant so that every index into v[] is one (registers, not scratch)
    const size_t gi = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (gi >= total) return;
    const int t = (int)(gi % strips);
    const size_t rest = gi / strips;
    const int ph0 = (int)(rest % row_blocks) * ROWS;  // this thread's first output row; it makes ROWS of them
    const size_t nc = rest / row_blocks;
    const float* in = x + nc * H * W;
    const int c0 = 8 * t;  // first column of the aligned chunk; v[i] below holds column c0 - 1 + i
    const float fill = TYPE == 0 ? -FLT_MAX : 0.f;
    constexpr int NR = 2 * (ROWS - 1) + K;  // input rows under ROWS consecutive windows: neighbouring windows share K - 2 of them
    float v[NR][10];
    const int hs00 = ph0 * 2 - pt;
#pragma unroll
    for (int a = 0; a < NR; ++a) {
        const int iy = hs00 + a;
        const bool row_ok = iy >= 0 && iy < H;
        const float* row = in + (size_t)iy * W;
        v4f lo = {fill, fill, fill, fill}, hi = lo;
        if (row_ok && c0 < W) lo = *reinterpret_cast<const v4f*>(row + c0);
        if (row_ok && c0 + 4 < W) hi = *reinterpret_cast<const v4f*>(row + c0 + 4);
        v[a][0] = pl == 1 && row_ok && c0 >= 1 && c0 - 1 < W ? row[c0 - 1] : fill;
        v[a][9] = K == 3 && pl == 0 && row_ok && c0 + 8 < W ? row[c0 + 8] : fill;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[a][1 + e] = lo[e];
            v[a][5 + e] = hi[e];
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int ph = ph0 + r, hs0 = hs00 + 2 * r;
        const bool row_out = ph < OH;  // no early exit: the loop must unroll for v[] to stay in registers
        v4f out;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int first = 2 * j - pl + 1;  // index into v[] of the window's first column
            float res;
            if (TYPE == 0) {
                res = -FLT_MAX;
#pragma unroll
                for (int a = 0; a < K; ++a)
#pragma unroll
                    for (int b = 0; b < K; ++b) {
                        const float tap = v[2 * r + a][first + b];
                        res = res < tap ? tap : res;
                    }
            } else {
                const int pw = 4 * t + j;
                int hs = hs0, wsx = pw * 2 - pl;
                int he = min(hs + K, H + pb), we = min(wsx + K, W + pr);
                int pool = (he - hs) * (we - wsx);
                hs = max(hs, 0);
                wsx = max(wsx, 0);
                he = min(he, H);
                we = min(we, W);
                if (!include_pad) pool = (he - hs) * (we - wsx);
                res = 0.f;
#pragma unroll
                for (int a = 0; a < K; ++a)
#pragma unroll
                    for (int b = 0; b < K; ++b) {
                        const int iy = hs0 + a, ix = pw * 2 - pl + b;
                        if (iy >= hs && iy < he && ix >= wsx && ix < we) res += v[2 * r + a][first + b];
                    }
                res = res / (float)pool;
            }
            out[j] = res;
        }
        float* dst = y + (nc * OH + ph) * OW + 4 * t;
        if ((OW & 3) == 0) {
            if (row_out) *reinterpret_cast<v4f*>(dst) = out;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (row_out && 4 * t + j < OW) dst[j] = out[j];
        }
    }
}

// Stride-1 max pooling with an odd window and "same" padding (the 5 / 9 / 13 pyramid of the detection topologies):
// the maximum is separable, so a workgroup stages a 32 x 32 output tile's halo in LDS, takes row maxima into a second
// LDS array and column maxima of those into the output: 2K compares per output instead of K * K. Cells outside the
// image hold -FLT_MAX, the clipped window's identity.
template <int K>
__global__ __launch_bounds__(kBlock) void maxpool_same_nchw_f32_kernel(const float* __restrict__ x, float* __restrict__ y, int H,
                                                                       int W) {
    constexpr int P = K / 2, T = 32, S = T + 2 * P;
    __shared__ float in[S][S + 1];
    __shared__ float rowmax[S][T + 1];
    const size_t plane = blockIdx.z;
    const int x0 = blockIdx.x * T, y0 = blockIdx.y * T;
    const float* src = x + plane * H * W;
    for (int i = threadIdx.x; i < S * S; i += kBlock) {
        const int r = i / S, c = i - r * S;
        const int gy = y0 - P + r, gx = x0 - P + c;
        in[r][c] = (gy >= 0 && gy < H && gx >= 0 && gx < W) ? src[(size_t)gy * W + gx] : -FLT_MAX;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < S * T; i += kBlock) {
        const int r = i / T, c = i - r * T;
        float m = in[r][c];
#pragma unroll
        for (int k = 1; k < K; ++k) m = m < in[r][c + k] ? in[r][c + k] : m;
        rowmax[r][c] = m;
    }
    __syncthreads();
    float* dst = y + plane * H * W;
    for (int i = threadIdx.x; i < T * T; i += kBlock) {
        const int r = i / T, c = i - r * T;
        if (y0 + r >= H || x0 + c >= W) continue;
        float m = rowmax[r][c];
#pragma unroll
        for (int k = 1; k < K; ++k) m = m < rowmax[r + k][c] ? rowmax[r + k][c] : m;
        dst[(size_t)(y0 + r) * W + x0 + c] = m;
    }
}

__global__ __launch_bounds__(kBlock) void maxpool_nhwc_f32_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                  int8_t* __restrict__ yq, float fs_out, int H, int W, int cs,
                                                                  int OH, int OW, int kh, int kw, int sh, int sw, int pt,
                                                                  int pl, size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int groups = cs / 4;
    const int g = (int)(i % groups);
    size_t pix = i / groups;
    const int ox = (int)(pix % OW);
    pix /= OW;
    const int oy = (int)(pix % OH);
    const size_t n = pix / OH;
    const int hs = max(oy * sh - pt, 0), wsx = max(ox * sw - pl, 0);
    const int he = min(oy * sh - pt + kh, H), we = min(ox * sw - pl + kw, W);
    v4f m = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
    for (int a = hs; a < he; ++a)
        for (int b = wsx; b < we; ++b) {
            const v4f t = *reinterpret_cast<const v4f*>(x + ((n * H + a) * W + b) * cs + g * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) m[e] = m[e] < t[e] ? t[e] : m[e];
        }
    const size_t o = ((n * OH + oy) * OW + ox) * cs + g * 4;
    if (y) *reinterpret_cast<v4f*>(y + o) = m;
    if (yq) {
        uint32_t w = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) w |= (uint32_t)(exhip_q8(m[e] * fs_out) & 0xff) << (8 * e);
        *reinterpret_cast<int*>(yq + o) = (int)w;
    }
}

// The same pooling on an int8 NHWC tensor (the int8 executor: the quantizer is monotone, so the maximum of the quantized
// values is the quantized maximum). 16 channels per thread; the running maxima stay unpacked over the window.
__global__ __launch_bounds__(kBlock) void maxpool_nhwc_i8_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y, int H, int W, int cs,
                                                                 int OH, int OW, int kh, int kw, int sh, int sw, int pt, int pl,
                                                                 size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int groups = cs / 16;
    const int g = (int)(i % groups);
    size_t pix = i / groups;
    const int ox = (int)(pix % OW);
    pix /= OW;
    const int oy = (int)(pix % OH);
    const size_t n = pix / OH;
    const int hs = max(oy * sh - pt, 0), wsx = max(ox * sw - pl, 0);
    const int he = min(oy * sh - pt + kh, H), we = min(ox * sw - pl + kw, W);
    int m[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) m[e] = -128;
    for (int a = hs; a < he; ++a)
        for (int b = wsx; b < we; ++b) {
            const v4i t = *reinterpret_cast<const v4i*>(x + ((n * H + a) * W + b) * cs + g * 16);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int v = (t[e >> 2] << (24 - 8 * (e & 3))) >> 24;  // byte e, sign-extended
                m[e] = m[e] < v ? v : m[e];
            }
        }
    v4i o;
#pragma unroll
    for (int q = 0; q < 4; ++q)
        o[q] = (m[4 * q] & 0xff) | ((m[4 * q + 1] & 0xff) << 8) | ((m[4 * q + 2] & 0xff) << 16) | (m[4 * q + 3] << 24);
    *reinterpret_cast<v4i*>(y + ((n * OH + oy) * OW + ox) * cs + g * 16) = o;
}

// A pyramid of stride-1 "same" max pools on an int8 NHWC tensor in one launch: y1 = pool_k(x), y2 = pool_k(y1), y3 = pool_k(y2)
// (windows k, 2k - 1, 3k - 2 over x: 5 / 9 / 13). One group per image and 16-channel slab keeps the slab's map in LDS as
// int16 pairs (v_pk_max_i16 takes two channels per instruction) and pools it separably, rows then columns, level after
// level; taps outside the image count in no maximum. kPyrPixels bounds the map (two buffers of 32 bytes per pixel).
constexpr int kPyrPixels = 960;
typedef short v2s __attribute__((ext_vector_type(2)));
struct PyrPixel { v2s c[8]; };  // 16 channels
__global__ __launch_bounds__(kBlock) void maxpool_pyramid_nhwc_i8_kernel(const int8_t* __restrict__ x, int8_t* __restrict__ y1, int8_t* __restrict__ y2,
                                                                        int8_t* __restrict__ y3, int H, int W, int cs, int k) {
    __shared__ PyrPixel buf[2][kPyrPixels];
    const int slab = blockIdx.x, n = blockIdx.y, px = H * W, r = k / 2;
    const size_t base = (size_t)n * px * cs + (size_t)slab * 16;
    for (int i = threadIdx.x; i < px; i += kBlock) {
        const v4i t = *reinterpret_cast<const v4i*>(x + base + (size_t)i * cs);
        PyrPixel o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int w = t[e >> 1] >> ((e & 1) * 16);                       // bytes 2e, 2e + 1 in the low half
            o.c[e] = v2s{(short)((w << 24) >> 24), (short)((w << 16) >> 24)};  // sign-extended
        }
        buf[0][i] = o;
    }
    __syncthreads();
    int8_t* const outs[3] = {y1, y2, y3};
#pragma unroll 1
    for (int level = 0; level < 3; ++level) {
        int8_t* const y = outs[level];
        if (!y) break;  // uniform
        // rows: buf[0] -> buf[1]
        for (int i = threadIdx.x; i < px; i += kBlock) {
            const int yy = i / W, xx = i - yy * W;
            const int lo = xx - r < 0 ? 0 : xx - r, hi = xx + r >= W ? W - 1 : xx + r;
            PyrPixel m = buf[0][yy * W + lo];
            for (int b = lo + 1; b <= hi; ++b) {
                const PyrPixel t = buf[0][yy * W + b];
#pragma unroll
                for (int e = 0; e < 8; ++e) m.c[e] = __builtin_elementwise_max(m.c[e], t.c[e]);
            }
            buf[1][i] = m;
        }
        __syncthreads();
        // columns: buf[1] -> buf[0] (the level's result, the next level's input) and out
        for (int i = threadIdx.x; i < px; i += kBlock) {
            const int yy = i / W, xx = i - yy * W;
            const int lo = yy - r < 0 ? 0 : yy - r, hi = yy + r >= H ? H - 1 : yy + r;
            PyrPixel m = buf[1][lo * W + xx];
            for (int a = lo + 1; a <= hi; ++a) {
                const PyrPixel t = buf[1][a * W + xx];
#pragma unroll
                for (int e = 0; e < 8; ++e) m.c[e] = __builtin_elementwise_max(m.c[e], t.c[e]);
            }
            buf[0][i] = m;
            v4i o;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                o[q] = (m.c[2 * q][0] & 0xff) | ((m.c[2 * q][1] & 0xff) << 8) | ((m.c[2 * q + 1][0] & 0xff) << 16) | ((int)m.c[2 * q + 1][1] << 24);
            *reinterpret_cast<v4i*>(y + base + (size_t)i * cs) = o;
        }
        __syncthreads();
    }
}

// 3x3 stride-2 max pooling on NHWC float32, a 2 x 2 block of output pixels per thread (four channels each): the four
// windows share a row and a column, so 25 loads instead of 36, all in flight at once. Taps outside the image count as
// -FLT_MAX, the clipped window of the general kernel. Optional requantized int8 copy as there.
__global__ __launch_bounds__(kBlock) void maxpool3x3s2_nhwc_f32_block_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                                             int8_t* __restrict__ yq, float fs_out, int H, int W,
                                                                             int cs, int OH, int OW, int pt, int pl, size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int groups = cs / 4, pairs = (OW + 1) / 2, row_pairs = (OH + 1) / 2;
    const int g = (int)(i % groups);
    size_t pix = i / groups;
    const int ox = (int)(pix % pairs) * 2;
    pix /= pairs;
    const int oy = (int)(pix % row_pairs) * 2;
    const size_t n = pix / row_pairs;
    const int iy0 = oy * 2 - pt, ix0 = ox * 2 - pl;
    const v4f lowest = {-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
    v4f t[5][5];
#pragma unroll
    for (int a = 0; a < 5; ++a)
#pragma unroll
        for (int b = 0; b < 5; ++b) {
            const int iy = iy0 + a, ix = ix0 + b;
            const bool ok = (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
            t[a][b] = ok ? *reinterpret_cast<const v4f*>(x + ((n * H + iy) * W + ix) * cs + g * 4) : lowest;
        }
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            v4f m = lowest;
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int b = 0; b < 3; ++b)
#pragma unroll
                    for (int e = 0; e < 4; ++e) m[e] = m[e] < t[2 * r + a][2 * j + b][e] ? t[2 * r + a][2 * j + b][e] : m[e];
            if (oy + r < OH && ox + j < OW) {
                const size_t o = ((n * OH + oy + r) * OW + ox + j) * cs + g * 4;
                if (y) *reinterpret_cast<v4f*>(y + o) = m;
                if (yq) {
                    uint32_t w = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e) w |= (uint32_t)(exhip_q8(m[e] * fs_out) & 0xff) << (8 * e);
                    *reinterpret_cast<int*>(yq + o) = (int)w;
                }
            }
        }
}

// Max pooling with a small fixed window on half storage: the maximum of halves is exact, so the taps are compared
// as packed halves, all window loads in flight at once. Taps outside the image count as -inf (the clipped window of
// the general kernel); an all-padding window cannot occur for the output sizes the layer computes.
template <int K, int S>
__global__ __launch_bounds__(kBlock) void maxpool_nhwc_f16_window_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                                         int H, int W, int cs, int OH, int OW, int pt, int pl,
                                                                         size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int groups = cs / 8;
    const int g = (int)(i % groups);
    size_t pix = i / groups;
    const int ox = (int)(pix % OW);
    pix /= OW;
    const int oy = (int)(pix % OH);
    const size_t n = pix / OH;
    const _Float16 ninf = -__builtin_inff16();
    const v8h lowest = {ninf, ninf, ninf, ninf, ninf, ninf, ninf, ninf};
    v8h tap[K][K];
#pragma unroll
    for (int a = 0; a < K; ++a)
#pragma unroll
        for (int b = 0; b < K; ++b) {
            const int iy = oy * S - pt + a, ix = ox * S - pl + b;
            tap[a][b] = lowest;
            if (iy >= 0 && iy < H && ix >= 0 && ix < W)
                tap[a][b] = __builtin_bit_cast(v8h, *reinterpret_cast<const v4i*>(x + ((n * H + iy) * W + ix) * cs + g * 8));
        }
    v8h best = lowest;
#pragma unroll
    for (int a = 0; a < K; ++a)
#pragma unroll
        for (int b = 0; b < K; ++b) best = __builtin_elementwise_max(best, tap[a][b]);
    *reinterpret_cast<v4i*>(y + ((n * OH + oy) * OW + ox) * cs + g * 8) = __builtin_bit_cast(v4i, best);
}

// The 3x3 stride-2 window on half storage, a 2 x 2 block of output pixels per thread (eight channels each): 25 loads
// instead of 36, since neighbouring windows share a row and a column.
__global__ __launch_bounds__(kBlock) void maxpool3x3s2_nhwc_f16_block_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                                             int H, int W, int cs, int OH, int OW, int pt, int pl,
                                                                             size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int groups = cs / 8, pairs = (OW + 1) / 2, row_pairs = (OH + 1) / 2;
    const int g = (int)(i % groups);
    size_t pix = i / groups;
    const int ox = (int)(pix % pairs) * 2;
    pix /= pairs;
    const int oy = (int)(pix % row_pairs) * 2;
    const size_t n = pix / row_pairs;
    const int iy0 = oy * 2 - pt, ix0 = ox * 2 - pl;
    const _Float16 ninf = -__builtin_inff16();
    const v8h lowest = {ninf, ninf, ninf, ninf, ninf, ninf, ninf, ninf};
    v8h tap[5][5];
#pragma unroll
    for (int a = 0; a < 5; ++a)
#pragma unroll
        for (int b = 0; b < 5; ++b) {
            const int iy = iy0 + a, ix = ix0 + b;
            tap[a][b] = lowest;
            if ((unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W)
                tap[a][b] = __builtin_bit_cast(v8h, *reinterpret_cast<const v4i*>(x + ((n * H + iy) * W + ix) * cs + g * 8));
        }
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            v8h best = lowest;
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int b = 0; b < 3; ++b) best = __builtin_elementwise_max(best, tap[2 * r + a][2 * j + b]);
            if (oy + r < OH && ox + j < OW)
                *reinterpret_cast<v4i*>(y + ((n * OH + oy + r) * OW + ox + j) * cs + g * 8) = __builtin_bit_cast(v4i, best);
        }
}

__global__ __launch_bounds__(kBlock) void pool2d_nhwc_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y, int H,
                                                                 int W, int cs, int OH, int OW, int type, int kh, int kw,
                                                                 int sh, int sw, int pt, int pb, int pl, int pr,
                                                                 int include_pad, size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int groups = cs / 8;
    const int g = (int)(i % groups);
    size_t pix = i / groups;
    const int ox = (int)(pix % OW);
    pix /= OW;
    const int oy = (int)(pix % OH);
    const size_t n = pix / OH;
    int hs = oy * sh - pt, wsx = ox * sw - pl;
    int he = min(hs + kh, type == 0 ? H : H + pb), we = min(wsx + kw, type == 0 ? W : W + pr);
    int pool = (he - hs) * (we - wsx);
    hs = max(hs, 0);
    wsx = max(wsx, 0);
    he = min(he, H);
    we = min(we, W);
    if (!include_pad) pool = (he - hs) * (we - wsx);
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = type == 0 ? -FLT_MAX : 0.f;
    // eight taps of a row are loaded before the first is used (a global pool is one thread walking the whole plane);
    // the taps are taken in window order, as in the definition
    for (int a = hs; a < he; ++a)
        for (int b0 = wsx; b0 < we; b0 += 8) {
            v4i v[8];
#pragma unroll
            for (int t = 0; t < 8; ++t)
                v[t] = *reinterpret_cast<const v4i*>(x + ((n * H + a) * W + min(b0 + t, we - 1)) * cs + g * 8);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const bool in_window = b0 + t < we;  // a select, not a branch: the loads above stay ahead of all of this
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float f = exhip_h2f((uint16_t)(((uint32_t)v[t][e >> 1] >> ((e & 1) * 16)) & 0xffff));
                    const float next = type == 0 ? (acc[e] < f ? f : acc[e]) : acc[e] + f;
                    acc[e] = in_window ? next : acc[e];
                }
            }
        }
    v4i o = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float r = type == 0 ? acc[e] : acc[e] / (float)pool;
        o[e >> 1] |= (int)((uint32_t)exhip_f2h(r) << ((e & 1) * 16));
    }
    *reinterpret_cast<v4i*>(y + ((n * OH + oy) * OW + ox) * cs + g * 8) = o;
}

// Global average pooling, src/Excalibur/operation_pooling.cpp:90-100,181-201 with the window = the whole plane. The
// reference adds a plane's values one after the other; here a plane is cut into interleaved runs that are summed side by
// side and combined in a fixed order (a launch gives the same bits every time; against the reference the float sum differs
// in its last bits, inside the 1e-4 the path allows for this layer).
// NHWC half: a block takes G groups of 8 channels of one image; thread (phase, group) adds pixels phase, phase + P, ...
// of its group, the P partial sums of a group meet in LDS and are added in phase order.
__global__ __launch_bounds__(kBlock) void global_avgpool_nhwc_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                                         int HW, int cs, int G, int slabs) {
    __shared__ float part[kBlock][9];  // 8 sums per thread, rows padded against bank conflicts
    const int n = blockIdx.x / slabs, slab = blockIdx.x % slabs;
    const int P = kBlock / G;
    const int g = threadIdx.x % G, phase = threadIdx.x / G;
    const int group = slab * G + g;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (group * 8 < cs && phase < P) {
        const uint16_t* src = x + (size_t)n * HW * cs + group * 8;
        for (int p = phase; p < HW; p += P) {
            const v8h v = __builtin_bit_cast(v8h, *reinterpret_cast<const v4i*>(src + (size_t)p * cs));
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += (float)v[e];
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part[threadIdx.x][e] = acc[e];
    __syncthreads();
    if (phase == 0 && group * 8 < cs) {
        float s[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) s[e] = part[g][e];
        for (int q = 1; q < P; ++q)
#pragma unroll
            for (int e = 0; e < 8; ++e) s[e] += part[q * G + g][e];
        v8h o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (_Float16)(s[e] / (float)HW);
        *reinterpret_cast<v4i*>(y + (size_t)n * cs + group * 8) = __builtin_bit_cast(v4i, o);
    }
}

// NCHW float: one wave per plane; lane l adds elements l, l + 64, ..., then the 64 partial sums are folded
// 32 + 32, 16 + 16, ... in a fixed tree.
__global__ __launch_bounds__(kBlock) void global_avgpool_nchw_f32_kernel(const float* __restrict__ x, float* __restrict__ y, int HW,
                                                                         size_t planes) {
    const size_t plane = (size_t)blockIdx.x * (kBlock / 64) + threadIdx.x / 64;
    if (plane >= planes) return;
    const int lane = threadIdx.x & 63;
    const float* src = x + plane * HW;
    float s = 0.f;
    for (int i = lane; i < HW; i += 64) s += src[i];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) s += __shfl_down(s, d, 64);
    if (lane == 0) y[plane] = s / (float)HW;
}

// ---------------------------------------------------------------------------------------------
// Elementwise
// ---------------------------------------------------------------------------------------------
struct EltArgs {
    const float* in[8];
    float coeff[8];
    int n;
};

__global__ __launch_bounds__(kBlock) void eltwise_f32_kernel(EltArgs a, int type, float* __restrict__ y, size_t count, size_t body) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= count) return;
    float r;
    if (type == 1) {  // SUM through saxpby: body unfused, tail fused
        r = 0.f;
        for (int k = 0; k < a.n; ++k) {
            const float xv = a.in[k][i];
            if (i < body) r = xv * a.coeff[k] + r * 1.0f;
            else r = __builtin_fmaf(a.coeff[k], xv, r * 1.0f);
        }
    } else if (type == 2) {
        r = a.in[0][i] < a.in[1][i] ? a.in[1][i] : a.in[0][i];
        for (int k = 2; k < a.n; ++k) r = r < a.in[k][i] ? a.in[k][i] : r;
    } else {
        r = a.in[0][i] * a.in[1][i];
        for (int k = 2; k < a.n; ++k) r = r * a.in[k][i];
    }
    y[i] = r;
}

// Four floats per thread over the unfused body (a multiple of eight floats), the fused tail one per thread
template <int TYPE>
__global__ __launch_bounds__(kBlock) void eltwise_f32_v4_kernel(EltArgs a, float* __restrict__ y, size_t count, size_t body) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t n4 = body / 4;
    if (i < n4) {
        v4f r;
        if (TYPE == 1) {
            r = (v4f){0.f, 0.f, 0.f, 0.f};
            for (int k = 0; k < a.n; ++k) {
                const v4f xv = reinterpret_cast<const v4f*>(a.in[k])[i];
#pragma unroll
                for (int e = 0; e < 4; ++e) r[e] = xv[e] * a.coeff[k] + r[e] * 1.0f;
            }
        } else {
            r = reinterpret_cast<const v4f*>(a.in[0])[i];
            for (int k = 1; k < a.n; ++k) {
                const v4f xv = reinterpret_cast<const v4f*>(a.in[k])[i];
#pragma unroll
                for (int e = 0; e < 4; ++e) r[e] = TYPE == 2 ? (r[e] < xv[e] ? xv[e] : r[e]) : r[e] * xv[e];
            }
        }
        reinterpret_cast<v4f*>(y)[i] = r;
        return;
    }
    const size_t j = body + (i - n4);
    if (j >= count) return;
    float r;
    if (TYPE == 1) {
        r = 0.f;
        for (int k = 0; k < a.n; ++k) r = __builtin_fmaf(a.coeff[k], a.in[k][j], r * 1.0f);
    } else {
        r = a.in[0][j];
        for (int k = 1; k < a.n; ++k) r = TYPE == 2 ? (r < a.in[k][j] ? a.in[k][j] : r) : r * a.in[k][j];
    }
    y[j] = r;
}

// BinaryOp ADD / SUB / MUL / DIV (OP 0..3) with a smaller second operand. MODE 0: equal shapes, op(large, small);
// 1: one value per image, op(large, value); 2: one value per (image, channel), op(value, large) -- the reference puts
// the smaller operand first there; 3: one value per (image, pixel), op(value, large). The smaller operand's images
// repeat modulo its batch size. Four floats per thread along a plane.
template <int OP>
__device__ __forceinline__ float binop_value(float x, float y) {
    if constexpr (OP == 0) return x + y;
    else if constexpr (OP == 1) return x - y;
    else if constexpr (OP == 2) return x * y;
    else return x / y;
}
template <int OP, int MODE, int VEC>
__global__ __launch_bounds__(kBlock) void binaryop_f32_kernel(const float* __restrict__ big, const float* __restrict__ small,
                                                              float* __restrict__ y, int C, int HW, int small_n, size_t total) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;  // one thread per VEC consecutive values of a plane
    if (t >= total) return;
    const int per_plane = HW / VEC;
    const size_t plane = t / per_plane;
    const int p = (int)(t - plane * per_plane) * VEC;
    const int c = (int)(plane % C);
    const size_t img = plane / C;
    const size_t at = plane * HW + p;
    const size_t simg = img % small_n;
    float b[VEC], s[VEC], r[VEC];
    if constexpr (VEC == 4) {
        const v4f v = *reinterpret_cast<const v4f*>(big + at);
#pragma unroll
        for (int e = 0; e < 4; ++e) b[e] = v[e];
    } else {
        b[0] = big[at];
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        if constexpr (MODE == 0) s[e] = small[at + e];
        else if constexpr (MODE == 1) s[e] = small[simg];
        else if constexpr (MODE == 2) s[e] = small[simg * C + c];
        else s[e] = small[simg * HW + p + e];
        r[e] = MODE <= 1 ? binop_value<OP>(b[e], s[e]) : binop_value<OP>(s[e], b[e]);
    }
    if constexpr (VEC == 4) {
        const v4f o = {r[0], r[1], r[2], r[3]};
        *reinterpret_cast<v4f*>(y + at) = o;
    } else {
        y[at] = r[0];
    }
}

// ---- activation / glue layers ----

template <int OP>
__global__ __launch_bounds__(kBlock) void unary_f32_kernel(const float* __restrict__ x, float* __restrict__ y, size_t n4,
                                                           size_t count, float alpha, float beta) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n4) {
        const v4f v = reinterpret_cast<const v4f*>(x)[i];
        v4f r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = unary_value<OP>(v[e], alpha, beta);
        reinterpret_cast<v4f*>(y)[i] = r;
    } else {
        const size_t j = n4 * 4 + (i - n4);
        if (j < count) y[j] = unary_value<OP>(x[j], alpha, beta);
    }
}

// The same on half storage: widened to float, the float formula, rounded to half once (what the reference's fp16 layers
// do through their convert-and-call wrapper). Eight values per thread over the aligned body.
template <int OP>
__global__ __launch_bounds__(kBlock) void unary_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y, size_t n8,
                                                           size_t count, float alpha, float beta) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n8) {
        v8f v = __builtin_convertvector(__builtin_bit_cast(v8h, reinterpret_cast<const v4i*>(x)[i]), v8f);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = unary_value<OP>(v[e], alpha, beta);
        reinterpret_cast<v4i*>(y)[i] = __builtin_bit_cast(v4i, __builtin_convertvector(v, v8h));
    } else {
        const size_t j = n8 * 8 + (i - n8);
        if (j < count) y[j] = exhip_f2h(unary_value<OP>(exhip_h2f(x[j]), alpha, beta));
    }
}

template <int OP>
__device__ __forceinline__ float channel_value(float v, float a, float b) {
    if constexpr (OP == 0) return v >= 0.f ? v : a * v;
    else if constexpr (OP == 1) return __builtin_fmaf(b, v, a);
    else return (v - a) * b;
}

// Per-channel layers on NCHW half storage, one block row per (image, channel) plane, eight values per thread where the
// plane is a multiple of eight halves long.
template <int OP, int VEC>
__global__ __launch_bounds__(kBlock) void channelwise_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y, int C,
                                                                 int HW, const float* __restrict__ p0,
                                                                 const float* __restrict__ p1, int shared) {
    const int plane = blockIdx.y;
    const int c = plane % C;
    const float a = p0[shared ? 0 : c];
    const float b = p1 ? p1[c] : 0.f;
    const size_t base = (size_t)plane * HW;
    for (int j = (blockIdx.x * kBlock + threadIdx.x) * VEC; j < HW; j += gridDim.x * kBlock * VEC) {
        if constexpr (VEC == 8) {
            v8f v = __builtin_convertvector(__builtin_bit_cast(v8h, *reinterpret_cast<const v4i*>(x + base + j)), v8f);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = channel_value<OP>(v[e], a, b);
            *reinterpret_cast<v4i*>(y + base + j) = __builtin_bit_cast(v4i, __builtin_convertvector(v, v8h));
        } else {
            y[base + j] = exhip_f2h(channel_value<OP>(exhip_h2f(x[base + j]), a, b));
        }
    }
}

// The per-channel layers on NHWC half storage (channel = element index modulo C, C a multiple of eight): eight
// consecutive channels of one pixel per 16-byte vector. The launch has a multiple of C / 8 threads, so a thread's
// vectors (one every `gridDim.x * kBlock`) all belong to the same eight channels and their parameters are read once.
template <int OP, bool VEC_PARAMS>
__global__ __launch_bounds__(kBlock) void channelwise_nhwc_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                                      size_t n8, unsigned groups, const float* __restrict__ p0,
                                                                      const float* __restrict__ p1, int shared) {
    const unsigned first = blockIdx.x * kBlock + threadIdx.x;
    const size_t step = (size_t)gridDim.x * kBlock;
    const unsigned c0 = (first % groups) * 8;
    float a[8], b[8];
    if constexpr (VEC_PARAMS) {
        const v4f a0 = shared ? v4f{p0[0], p0[0], p0[0], p0[0]} : *reinterpret_cast<const v4f*>(p0 + c0);
        const v4f a1 = shared ? a0 : *reinterpret_cast<const v4f*>(p0 + c0 + 4);
        const v4f b0 = p1 ? *reinterpret_cast<const v4f*>(p1 + c0) : v4f{0.f, 0.f, 0.f, 0.f};
        const v4f b1 = p1 ? *reinterpret_cast<const v4f*>(p1 + c0 + 4) : b0;
#pragma unroll
        for (int e = 0; e < 4; ++e) { a[e] = a0[e]; a[e + 4] = a1[e]; b[e] = b0[e]; b[e + 4] = b1[e]; }
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) { a[e] = p0[shared ? 0 : c0 + e]; b[e] = p1 ? p1[c0 + e] : 0.f; }
    }
    for (size_t i = first; i < n8; i += step) {
        v8f v = __builtin_convertvector(__builtin_bit_cast(v8h, reinterpret_cast<const v4i*>(x)[i]), v8f);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = channel_value<OP>(v[e], a[e], b[e]);
        reinterpret_cast<v4i*>(y)[i] = __builtin_bit_cast(v4i, __builtin_convertvector(v, v8h));
    }
}

// Per-channel layers on NCHW. OP 0 PReLU (p0 = slope, one per channel or one shared), 1 BatchNorm as
// fma(p1[c], x, p0[c]) with the load-time a / b, 2 Input (x - p0[c]) * p1[c]. One block row per (image, channel) plane.
template <int OP>
__global__ __launch_bounds__(kBlock) void channelwise_f32_kernel(const float* __restrict__ x, float* __restrict__ y, int C,
                                                                 int HW, const float* __restrict__ p0,
                                                                 const float* __restrict__ p1, int shared) {
    const int plane = blockIdx.y;
    const int c = plane % C;
    const float a = p0[shared ? 0 : c];
    const float b = p1 ? p1[c] : 0.f;
    const size_t base = (size_t)plane * HW;
    for (int j = blockIdx.x * kBlock + threadIdx.x; j < HW; j += gridDim.x * kBlock) {
        const float v = x[base + j];
        float r;
        if constexpr (OP == 0) r = v >= 0.f ? v : a * v;
        else if constexpr (OP == 1) r = __builtin_fmaf(b, v, a);
        else r = (v - a) * b;
        y[base + j] = r;
    }
}

// The same, four floats per thread, for planes a multiple of four floats long
template <int OP>
__global__ __launch_bounds__(kBlock) void channelwise_f32_v4_kernel(const float* __restrict__ x, float* __restrict__ y, int C,
                                                                    int HW4, const float* __restrict__ p0,
                                                                    const float* __restrict__ p1, int shared) {
    const int plane = blockIdx.y;
    const int c = plane % C;
    const float a = p0[shared ? 0 : c];
    const float b = p1 ? p1[c] : 0.f;
    const v4f* src = reinterpret_cast<const v4f*>(x) + (size_t)plane * HW4;
    v4f* dst = reinterpret_cast<v4f*>(y) + (size_t)plane * HW4;
    for (int j = blockIdx.x * kBlock + threadIdx.x; j < HW4; j += gridDim.x * kBlock) {
        const v4f v = src[j];
        v4f r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (OP == 0) r[e] = v[e] >= 0.f ? v[e] : a * v[e];
            else if constexpr (OP == 1) r[e] = __builtin_fmaf(b, v[e], a);
            else r[e] = (v[e] - a) * b;
        }
        dst[j] = r;
    }
}

// Copies one input's channel block of every image into its place in the concatenated tensor.
__global__ __launch_bounds__(kBlock) void concat_block_kernel(const float* __restrict__ x, float* __restrict__ y, size_t block,
                                                              size_t out_image, size_t out_offset) {
    const size_t img = blockIdx.y;
    for (size_t j = (size_t)blockIdx.x * kBlock + threadIdx.x; j < block; j += (size_t)gridDim.x * kBlock)
        y[img * out_image + out_offset + j] = x[img * block + j];
}

__global__ __launch_bounds__(kBlock) void concat_block_v4_kernel(const v4f* __restrict__ x, v4f* __restrict__ y, size_t block4,
                                                                 size_t out_image4, size_t out_offset4) {
    const size_t img = blockIdx.y;
    for (size_t j = (size_t)blockIdx.x * kBlock + threadIdx.x; j < block4; j += (size_t)gridDim.x * kBlock)
        y[img * out_image4 + out_offset4 + j] = x[img * block4 + j];
}

// Channel concatenation of NHWC half blobs (every channel count a multiple of 8): a thread moves one 16-byte vector of
// one output pixel; `first[i]` is the first output channel of input i.
struct ConcatNhwcArgs {
    const uint16_t* src[8];
    int first[9];  // first[n_inputs] = total channels
    int n_inputs;
};
__global__ __launch_bounds__(kBlock) void concat_nhwc_f16_kernel(ConcatNhwcArgs a, uint16_t* __restrict__ y, size_t total8) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total8) return;
    const int vecs = a.first[a.n_inputs] / 8;
    const int v = (int)(i % vecs);
    const size_t pix = i / vecs;
    const int c = v * 8;
    int k = 0;
#pragma unroll
    for (int j = 1; j < 8; ++j)
        if (j < a.n_inputs && c >= a.first[j]) k = j;
    const int ck = a.first[k + 1] - a.first[k];
    reinterpret_cast<v4i*>(y)[i] = *reinterpret_cast<const v4i*>(a.src[k] + pix * ck + (c - a.first[k]));
}

// Concat (or a single blob) with the BatchNorm layer and the activation layer behind it applied on the way: the values are
// those the layers produce one after the other (each stores halves, so the value is rounded to half between them).
// UOP: -1 no activation, else unary_value's operation. p0 == nullptr: no BatchNorm.
// V: 16-byte vectors (eight channels) per thread.
template <int UOP, int V>
__global__ __launch_bounds__(kBlock) void concat_affine_unary_nhwc_f16_kernel(ConcatNhwcArgs a, uint16_t* __restrict__ y, size_t total,
                                                                              const float* __restrict__ p0, const float* __restrict__ p1,
                                                                              float alpha, float beta) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int channels = a.first[a.n_inputs];
    const int per_pixel = channels / (8 * V);
    int part;
    size_t pix;
    if (total <= 0xFFFFFFFFull) {  // 32-bit division where it will do
        const unsigned p32 = (unsigned)i / (unsigned)per_pixel;
        part = (int)((unsigned)i - p32 * (unsigned)per_pixel);
        pix = p32;
    } else {
        part = (int)(i % per_pixel);
        pix = i / per_pixel;
    }
    const int c = part * 8 * V;
    int k = 0;
    for (int j = 1; j < a.n_inputs; ++j)
        if (c >= a.first[j]) k = j;
    const int ck = a.first[k + 1] - a.first[k];
    const v4i* src = reinterpret_cast<const v4i*>(a.src[k] + pix * ck + (c - a.first[k]));
    v4i* dst = reinterpret_cast<v4i*>(y + pix * channels + c);
#pragma unroll
    for (int u = 0; u < V; ++u) {
        v8f v = __builtin_convertvector(__builtin_bit_cast(v8h, src[u]), v8f);
        if (p0) {
            // eight consecutive parameters of each array: 16-byte aligned where the arrays are (device allocations)
            const v4f a0 = *reinterpret_cast<const v4f*>(p0 + c + 8 * u), a1 = *reinterpret_cast<const v4f*>(p0 + c + 8 * u + 4);
            const v4f b0 = *reinterpret_cast<const v4f*>(p1 + c + 8 * u), b1 = *reinterpret_cast<const v4f*>(p1 + c + 8 * u + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] = channel_value<1>(v[e], a0[e], b0[e]);
                v[e + 4] = channel_value<1>(v[e + 4], a1[e], b1[e]);
            }
            if constexpr (UOP >= 0) v = __builtin_convertvector(__builtin_convertvector(v, v8h), v8f);
        }
        if constexpr (UOP >= 0) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = unary_value<UOP>(v[e], alpha, beta);
        }
        dst[u] = __builtin_bit_cast(v4i, __builtin_convertvector(v, v8h));
    }
}

// The float32 NHWC form of the kernel above for the int8 executor: channel blocks of up to eight float32 NHWC tensors
// (each with its own channel stride) are laid side by side, then BatchNorm and the activation layer as the float32
// layers compute them (no rounding between them), and the result leaves as a float32 NHWC tensor and / or as the int8
// tensor the convolutions that read it would make of it (q8(v * fs)). A thread moves four channels of one pixel.
struct ConcatNhwcF32Args {
    const float* src[8];
    int first[9];   // first[n_inputs] = total channels
    int stride[8];  // channel stride of each input, in elements
    int n_inputs;
};
// V: vectors of four channels per thread. V == 4 (every input's channel count and the output stride multiples of 16): the
// thread's index arithmetic and input selection are shared by 16 channels and the int8 result leaves as one 16-byte store
// -- the kernel is bound by its vector instructions, not by memory.
template <int UOP, int V>
__global__ __launch_bounds__(kBlock) void concat_affine_unary_nhwc_f32_kernel(ConcatNhwcF32Args a, float* __restrict__ y_f,
                                                                              int8_t* __restrict__ y_q, int out_stride, float fs,
                                                                              size_t total, const float* __restrict__ p0,
                                                                              const float* __restrict__ p1, float alpha, float beta) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int per_pixel = out_stride / (4 * V);
    int part;
    size_t pix;
    if (total <= 0xFFFFFFFFull) {  // 32-bit division where it will do
        const unsigned p32 = (unsigned)i / (unsigned)per_pixel;
        part = (int)((unsigned)i - p32 * (unsigned)per_pixel);
        pix = p32;
    } else {
        part = (int)(i % per_pixel);
        pix = i / per_pixel;
    }
    const int c = part * 4 * V;
    v4f v[V];
#pragma unroll
    for (int u = 0; u < V; ++u) v[u] = v4f{0.f, 0.f, 0.f, 0.f};
    if (c < a.first[a.n_inputs]) {  // pad channels of the output hold zeros
        int k = 0;
        for (int j = 1; j < a.n_inputs; ++j)
            if (c >= a.first[j]) k = j;
        const float* src = a.src[k] + pix * a.stride[k] + (c - a.first[k]);
#pragma unroll
        for (int u = 0; u < V; ++u) v[u] = reinterpret_cast<const v4f*>(src)[u];
        if (p0) {
#pragma unroll
            for (int u = 0; u < V; ++u) {
                const v4f a0 = *reinterpret_cast<const v4f*>(p0 + c + 4 * u), b0 = *reinterpret_cast<const v4f*>(p1 + c + 4 * u);
#pragma unroll
                for (int e = 0; e < 4; ++e) v[u][e] = channel_value<1>(v[u][e], a0[e], b0[e]);
            }
        }
        if constexpr (UOP >= 0) {
#pragma unroll
            for (int u = 0; u < V; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e) v[u][e] = unary_value<UOP>(v[u][e], alpha, beta);
        }
    }
    if (y_f) {
#pragma unroll
        for (int u = 0; u < V; ++u) reinterpret_cast<v4f*>(y_f + pix * out_stride + c)[u] = v[u];
    }
    if (y_q) {
        uint32_t w[V];
#pragma unroll
        for (int u = 0; u < V; ++u) {
            w[u] = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) w[u] |= (uint32_t)(exhip_q8(v[u][e] * fs) & 0xff) << (8 * e);
        }
        if constexpr (V == 4) *reinterpret_cast<v4i*>(y_q + pix * out_stride + c) = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
        else *reinterpret_cast<uint32_t*>(y_q + pix * out_stride + c) = w[0];
    }
}

// Nearest-neighbour resize of an NHWC half blob (channels a multiple of 8), the index rule of the NCHW kernel below.
__global__ __launch_bounds__(kBlock) void interp_nearest_nhwc_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                                         int H, int W, int C8, int OH, int OW, float hs, float ws,
                                                                         size_t total8) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total8) return;
    const int v = (int)(i % C8);
    size_t t = i / C8;
    const int ox = (int)(t % OW);
    t /= OW;
    const int oy = (int)(t % OH);
    const size_t n = t / OH;
    int iy = (int)(oy * hs), ix = (int)(ox * ws);
    iy = iy > H - 1 ? H - 1 : iy;
    ix = ix > W - 1 ? W - 1 : ix;
    reinterpret_cast<v4i*>(y)[i] = reinterpret_cast<const v4i*>(x)[((n * H + iy) * W + ix) * C8 + v];
}

// One direction of a stride-1 "same" max pooling on NHWC half storage (window K, padding K / 2, taps outside the image
// do not count): the K x K maximum is the maximum over rows of the maxima over columns, so two launches of 2K taps
// replace K * K. ALONG_W: the window runs along x, else along y.
template <int K, bool ALONG_W>
__global__ __launch_bounds__(kBlock) void maxpool_same_1d_nhwc_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                                          int H, int W, int C8, size_t total8) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total8) return;
    const int v = (int)(i % C8);
    size_t t = i / C8;
    const int ox = (int)(t % W);
    t /= W;
    const int oy = (int)(t % H);
    const size_t n = t / H;
    const _Float16 ninf = -__builtin_inff16();
    v8h best = {ninf, ninf, ninf, ninf, ninf, ninf, ninf, ninf};
#pragma unroll
    for (int d = -(K / 2); d <= K / 2; ++d) {
        const int iy = ALONG_W ? oy : oy + d, ix = ALONG_W ? ox + d : ox;
        if ((unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W)
            best = __builtin_elementwise_max(best, __builtin_bit_cast(v8h, reinterpret_cast<const v4i*>(x)[((n * H + iy) * W + ix) * C8 + v]));
    }
    reinterpret_cast<v4i*>(y)[i] = __builtin_bit_cast(v4i, best);
}

// Nearest-neighbour resize: in = min((int)(out * scale), size - 1), scale = size / (float)out_size.
__global__ __launch_bounds__(kBlock) void interp_nearest_kernel(const float* __restrict__ x, float* __restrict__ y, int H, int W,
                                                                int OH, int OW, float hs, float ws, size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int ox = (int)(i % OW);
    const size_t t = i / OW;
    const int oy = (int)(t % OH);
    const size_t plane = t / OH;
    int iy = (int)(oy * hs), ix = (int)(ox * ws);
    iy = iy > H - 1 ? H - 1 : iy;
    ix = ix > W - 1 ? W - 1 : ix;
    y[i] = x[(plane * H + iy) * W + ix];
}

// Space to depth of the YOLOv5 stem: out[n][g*C + c][i][j] = in[n][c][2i + g % 2][2j + g / 2], g < 4.
__global__ __launch_bounds__(kBlock) void focus_kernel(const float* __restrict__ x, float* __restrict__ y, int C, int H, int W,
                                                       size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int OH = H / 2, OW = W / 2;
    const int ox = (int)(i % OW);
    size_t t = i / OW;
    const int oy = (int)(t % OH);
    t /= OH;
    const int p = (int)(t % (4 * C));
    const size_t n = t / (4 * C);
    const int g = p / C, c = p % C;
    y[i] = x[((n * C + c) * H + 2 * oy + g % 2) * W + 2 * ox + g / 2];
}

// The front of an int8 detection network in one pass: the Input layer's (x - mean[c]) * scale[c], YoloV5Focus (above) and
// the first convolution's quantizer q8(v * fs), from the float32 NCHW image to int8 NHWC pixels of 32 bytes (4 C channels,
// the rest zero). A thread makes one output pixel from two neighbouring columns of two rows of each plane.
struct FrontArgs {
    float mean[4], scale[4];
};
template <int C>
__global__ __launch_bounds__(kBlock) void input_focus_quantize_kernel(const float* __restrict__ x, int8_t* __restrict__ y, int H, int W,
                                                                      FrontArgs a, float fs, size_t total) {
    static_assert(4 * C <= 16, "one 16-byte vector of channels");
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int OH = H / 2, OW = W / 2;
    const int ox = (int)(i % OW);
    size_t t = i / OW;
    const int oy = (int)(t % OH);
    const size_t n = t / OH;
    uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < C; ++c) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const float* src = x + ((n * C + c) * H + 2 * oy + r) * W + 2 * ox;
            const float v0 = src[0], v1 = src[1];
            // channel g * C + c holds row parity g % 2 and column parity g / 2
            const int p0 = r * C + c, p1 = (r + 2) * C + c;
            const int q0 = exhip_q8(((v0 - a.mean[c]) * a.scale[c]) * fs), q1 = exhip_q8(((v1 - a.mean[c]) * a.scale[c]) * fs);
            w[p0 >> 2] |= (uint32_t)(q0 & 0xff) << (8 * (p0 & 3));
            w[p1 >> 2] |= (uint32_t)(q1 & 0xff) << (8 * (p1 & 3));
        }
    }
    v4i* dst = reinterpret_cast<v4i*>(y + i * 32);
    dst[0] = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    dst[1] = v4i{0, 0, 0, 0};
}

// A detection head's Reshape + Transpose on the convolution's float32 NHWC result: y[n][g][pixel][j] = x[n][pixel][g * J + j]
// (G groups of J channels: the anchors and their values). blockIdx.y = n * G + g; one value per thread, reads and writes
// run along j; 32-bit index arithmetic with one division.
__global__ __launch_bounds__(kBlock) void nhwc_f32_to_grouped_kernel(const float* __restrict__ x, float* __restrict__ y, unsigned HW, unsigned G,
                                                                     unsigned J, unsigned stride, unsigned per_plane) {
    const unsigned i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= per_plane) return;
    const unsigned plane = blockIdx.y, n = plane / G, g = plane - n * G;
    const unsigned pix = i / J, j = i - pix * J;
    y[(size_t)plane * per_plane + i] = x[((size_t)n * HW + pix) * stride + g * J + j];
}
// The same, four consecutive results per thread (planes a multiple of four values long): one 16-byte store
__global__ __launch_bounds__(kBlock) void nhwc_f32_to_grouped_x4_kernel(const float* __restrict__ x, float* __restrict__ y, unsigned HW, unsigned G,
                                                                        unsigned J, unsigned stride, unsigned per_plane4) {
    const unsigned i4 = blockIdx.x * kBlock + threadIdx.x;
    if (i4 >= per_plane4) return;
    const unsigned plane = blockIdx.y, n = plane / G, g = plane - n * G;
    unsigned pix = (i4 * 4) / J, j = i4 * 4 - pix * J;
    const float* src = x + ((size_t)n * HW + pix) * stride + g * J;
    v4f o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        o[e] = src[j];
        if (++j == J) {  // on to the next pixel
            j = 0;
            src += stride;
        }
    }
    reinterpret_cast<v4f*>(y + (size_t)plane * per_plane4 * 4)[i4] = o;
}

// Four neighbouring outputs of a row per thread (output rows a multiple of four long): one 16-byte store
__global__ __launch_bounds__(kBlock) void interp_nearest_x4_kernel(const float* __restrict__ x, float* __restrict__ y, int H, int W,
                                                                   int OH, int OW4, float hs, float ws, size_t total4) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total4) return;
    const int q = (int)(i % OW4);
    const size_t t = i / OW4;
    const int oy = (int)(t % OH);
    const size_t plane = t / OH;
    int iy = (int)(oy * hs);
    iy = iy > H - 1 ? H - 1 : iy;
    const float* row = x + (plane * H + iy) * W;
    v4f o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        int ix = (int)((4 * q + e) * ws);
        ix = ix > W - 1 ? W - 1 : ix;
        o[e] = row[ix];
    }
    reinterpret_cast<v4f*>(y)[i] = o;
}

// Eight neighbouring inputs of a row per thread (rows a multiple of eight long): the even columns go to one output
// plane and the odd ones to another, 16 bytes each
__global__ __launch_bounds__(kBlock) void focus_x8_kernel(const float* __restrict__ x, float* __restrict__ y, int C, int H, int W,
                                                          size_t total8) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total8) return;
    const int W8 = W / 8, OH = H / 2, OW = W / 2;
    const int q = (int)(i % W8);
    size_t t = i / W8;
    const int iy = (int)(t % (2 * OH));
    t /= 2 * OH;
    const int c = (int)(t % C);
    const size_t n = t / C;
    const v4f* src = reinterpret_cast<const v4f*>(x + ((n * C + c) * H + iy) * W + 8 * q);
    const v4f a = src[0], b = src[1];
    const v4f even = {a[0], a[2], b[0], b[2]}, odd = {a[1], a[3], b[1], b[3]};
    const int g = iy & 1;  // g % 2 selects the row parity, g / 2 the column parity
    float* dst = y + ((n * 4 * C + c) * OH + iy / 2) * OW + 4 * q;
    *reinterpret_cast<v4f*>(dst + (size_t)g * C * OH * OW) = even;
    *reinterpret_cast<v4f*>(dst + (size_t)(g + 2) * C * OH * OW) = odd;
}

// The same on half storage (values are only moved): sixteen neighbouring inputs of a row per thread, 16 bytes to each
// of the two output planes; rows of any other length take one output per thread.
__global__ __launch_bounds__(kBlock) void focus_f16_x16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y, int C, int H, int W,
                                                               size_t total16) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total16) return;
    const int W16 = W / 16, OH = H / 2, OW = W / 2;
    const int q = (int)(i % W16);
    size_t t = i / W16;
    const int iy = (int)(t % (2 * OH));
    t /= 2 * OH;
    const int c = (int)(t % C);
    const size_t n = t / C;
    const v4i* src = reinterpret_cast<const v4i*>(x + ((n * C + c) * H + iy) * W + 16 * q);
    const v4i a = src[0], b = src[1];
    v4i even, odd;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const unsigned lo = (unsigned)(e < 2 ? a[2 * e] : b[2 * e - 4]), hi = (unsigned)(e < 2 ? a[2 * e + 1] : b[2 * e - 3]);
        even[e] = (int)((lo & 0xffffu) | (hi << 16));
        odd[e] = (int)((lo >> 16) | (hi & 0xffff0000u));
    }
    const int g = iy & 1;
    uint16_t* dst = y + ((n * 4 * C + c) * OH + iy / 2) * OW + 8 * q;
    *reinterpret_cast<v4i*>(dst + (size_t)g * C * OH * OW) = even;
    *reinterpret_cast<v4i*>(dst + (size_t)(g + 2) * C * OH * OW) = odd;
}
__global__ __launch_bounds__(kBlock) void focus_f16_kernel(const uint16_t* __restrict__ x, uint16_t* __restrict__ y, int C, int H, int W,
                                                           size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int OH = H / 2, OW = W / 2;
    const int ox = (int)(i % OW);
    size_t t = i / OW;
    const int oy = (int)(t % OH);
    t /= OH;
    const int p = (int)(t % (4 * C));
    const size_t n = t / (4 * C);
    const int g = p / C, c = p % C;
    y[i] = x[((n * C + c) * H + 2 * oy + g % 2) * W + 2 * ox + g / 2];
}

// Softmax over the channels of every (image, position) of an NCHW tensor: a thread owns one position and walks the
// channels three times (maximum, exponentials and their sum, quotient); neighbouring threads read neighbouring
// positions, so every access is coalesced.
__global__ __launch_bounds__(kBlock) void softmax_channels_kernel(const float* __restrict__ x, float* __restrict__ y, int C, int HW,
                                                                  size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const size_t img = i / HW;
    const int k = (int)(i - img * HW);
    const float* in = x + img * C * HW + k;
    float* out = y + img * C * HW + k;
    float m = in[0];
    for (int j = 1; j < C; ++j) {
        const float v = in[(size_t)j * HW];
        m = m < v ? v : m;
    }
    float sum = 0.f;
    for (int j = 0; j < C; ++j) {
        const float e = expf(in[(size_t)j * HW] - m);
        out[(size_t)j * HW] = e;
        sum += e;
    }
    for (int j = 0; j < C; ++j) out[(size_t)j * HW] = out[(size_t)j * HW] / sum;
}

// The same for at most CMAX channels: a position's values stay in registers between the three walks, so every value
// is read once and written once (same operations in the same order: same results).
template <int CMAX>
__global__ __launch_bounds__(kBlock) void softmax_channels_reg_kernel(const float* __restrict__ x, float* __restrict__ y, int C, int HW,
                                                                      size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const size_t img = i / HW;
    const int k = (int)(i - img * HW);
    const float* in = x + img * C * HW + k;
    float* out = y + img * C * HW + k;
    float v[CMAX];
#pragma unroll
    for (int j = 0; j < CMAX; ++j) v[j] = j < C ? in[(size_t)j * HW] : 0.f;
    float m = v[0];
#pragma unroll
    for (int j = 1; j < CMAX; ++j)
        if (j < C) m = m < v[j] ? v[j] : m;
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < CMAX; ++j) {
        if (j < C) {
            v[j] = expf(v[j] - m);
            sum += v[j];
        }
    }
#pragma unroll
    for (int j = 0; j < CMAX; ++j)
        if (j < C) out[(size_t)j * HW] = v[j] / sum;
}

// Rows and columns of every plane change places, through a 32 x 32 LDS tile so that both sides are coalesced.
template <typename T>
__global__ __launch_bounds__(kBlock) void transpose_hw_kernel(const T* __restrict__ x, T* __restrict__ y, int H, int W) {
    __shared__ T tile[32][33];
    const size_t plane = blockIdx.z;
    const int x0 = blockIdx.x * 32, y0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    const T* in = x + plane * H * W;
    T* out = y + plane * H * W;
#pragma unroll
    for (int r = ty; r < 32; r += 8)
        if (y0 + r < H && x0 + tx < W) tile[r][tx] = in[(size_t)(y0 + r) * W + x0 + tx];
    __syncthreads();
#pragma unroll
    for (int r = ty; r < 32; r += 8)
        if (x0 + r < W && y0 + tx < H) out[(size_t)(x0 + r) * H + y0 + tx] = tile[tx][r];
}

// Transposed convolution by gathering (NCHW float32, group 1, dilation 1): output (k, oy, ox) sums, over the taps
// (r, q) whose input pixel ((oy + pt - r) / sh, (ox + pl - q) / sw) exists, the products over the input channels.
// Weights [C][K][kh][kw]. One thread per output element; the layers that use it are small upsampling heads.
__global__ __launch_bounds__(kBlock) void deconv2d_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                              const float* __restrict__ bias, float* __restrict__ y, int C, int H,
                                                              int W, int K, int KH, int KW, int SH, int SW, int PT, int PL, int OH,
                                                              int OW, size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int ox = (int)(i % OW);
    size_t t = i / OW;
    const int oy = (int)(t % OH);
    t /= OH;
    const int k = (int)(t % K);
    const size_t n = t / K;
    float acc = 0.f;
    for (int r = 0; r < KH; ++r) {
        const int ty = oy + PT - r;
        if (ty < 0 || ty % SH) continue;
        const int iy = ty / SH;
        if (iy >= H) continue;
        for (int q = 0; q < KW; ++q) {
            const int tx = ox + PL - q;
            if (tx < 0 || tx % SW) continue;
            const int ix = tx / SW;
            if (ix >= W) continue;
            const float* xp = x + ((n * C) * H + iy) * W + ix;
            const float* wp = w + ((size_t)k * KH + r) * KW + q;
            for (int c = 0; c < C; ++c) acc = __builtin_fmaf(xp[(size_t)c * H * W], wp[(size_t)c * K * KH * KW], acc);
        }
    }
    y[i] = bias ? acc + bias[k] : acc;
}

// a + b (+ ReLU), four floats per thread where the arrays allow it
__global__ __launch_bounds__(kBlock) void add_f32_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                         float* __restrict__ y, size_t n4, size_t count, int relu) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n4) {
        const v4f va = reinterpret_cast<const v4f*>(a)[i];
        v4f r = va;
        if (b) {
            const v4f vb = reinterpret_cast<const v4f*>(b)[i];
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = va[e] + vb[e];
        }
        if (relu) {
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = (0.f > r[e]) ? 0.f : r[e];
        }
        reinterpret_cast<v4f*>(y)[i] = r;
    } else {
        const size_t j = n4 * 4 + (i - n4);
        if (j < count) {
            float r = b ? a[j] + b[j] : a[j];
            if (relu) r = (0.f > r) ? 0.f : r;
            y[j] = r;
        }
    }
}

// The same on half storage (float sum, rounded once), eight values per thread over the aligned body
__global__ __launch_bounds__(kBlock) void add_f16_kernel(const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
                                                         uint16_t* __restrict__ y, size_t n8, size_t count, int relu) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n8) {
        v8f r = __builtin_convertvector(__builtin_bit_cast(v8h, reinterpret_cast<const v4i*>(a)[i]), v8f);
        if (b) r += __builtin_convertvector(__builtin_bit_cast(v8h, reinterpret_cast<const v4i*>(b)[i]), v8f);
        if (relu) {
#pragma unroll
            for (int e = 0; e < 8; ++e) r[e] = (0.f > r[e]) ? 0.f : r[e];
        }
        reinterpret_cast<v4i*>(y)[i] = __builtin_bit_cast(v4i, __builtin_convertvector(r, v8h));
    } else {
        const size_t j = n8 * 8 + (i - n8);
        if (j >= count) return;
        float r = exhip_h2f(a[j]);
        if (b) r += exhip_h2f(b[j]);
        if (relu) r = (0.f > r) ? 0.f : r;
        y[j] = exhip_f2h(r);
    }
}

// ---------------------------------------------------------------------------------------------
// Inner product: one wave per output neuron, up to 8 batch rows at a time, float4 loads along k.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void innerproduct_f32_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                  const float* __restrict__ bias, float* __restrict__ y, int m,
                                                                  int n_out, int k_in) {
    const int lane = threadIdx.x & 63;
    const int j = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (j >= n_out) return;
    const float* wr = w + (size_t)j * k_in;
    const bool vec = (k_in % 4 == 0);
    for (int m0 = blockIdx.y * 8; m0 < m; m0 += gridDim.y * 8) {  // groups of eight batch rows across blockIdx.y
        float acc[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) acc[r] = 0.f;
        if (vec) {
            for (int k = lane * 4; k < k_in; k += 256) {
                const v4f wv = *reinterpret_cast<const v4f*>(wr + k);
#pragma unroll
                for (int r = 0; r < 8; ++r)
                    if (m0 + r < m) {
                        const v4f xv = *reinterpret_cast<const v4f*>(x + (size_t)(m0 + r) * k_in + k);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[r] = __builtin_fmaf(xv[e], wv[e], acc[r]);
                    }
            }
        } else {
            for (int k = lane; k < k_in; k += 64) {
                const float wv = wr[k];
#pragma unroll
                for (int r = 0; r < 8; ++r)
                    if (m0 + r < m) acc[r] = __builtin_fmaf(x[(size_t)(m0 + r) * k_in + k], wv, acc[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            float v = acc[r];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
            if (lane == 0 && m0 + r < m) y[(size_t)(m0 + r) * n_out + j] = v + (bias ? bias[j] : 0.f);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Convolution straight from the definition on NCHW f32 (any geometry, groups). One thread per output.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void conv_direct_kernel(const float* __restrict__ x, const float* __restrict__ wf,
                                                             const int8_t* __restrict__ wq, float fs,
                                                             const float* __restrict__ scale, const float* __restrict__ bias,
                                                             float* __restrict__ y, int C, int H, int W, int K, int OH, int OW,
                                                             int kh, int kw, int sh, int sw, int pt, int pl, int groups,
                                                             int act, size_t total) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= total) return;
    const int ox = (int)(i % OW);
    size_t t = i / OW;
    const int oy = (int)(t % OH);
    t /= OH;
    const int k = (int)(t % K);
    const size_t n = t / K;
    const int cg = C / groups, g = k / (K / groups);
    float accf = 0.f;
    int acci = 0;
    for (int c = 0; c < cg; ++c) {
        const float* in = x + (n * C + g * cg + c) * H * W;
        for (int a = 0; a < kh; ++a) {
            const int iy = oy * sh - pt + a;
            if (iy < 0 || iy >= H) continue;
            for (int b = 0; b < kw; ++b) {
                const int ix = ox * sw - pl + b;
                if (ix < 0 || ix >= W) continue;
                const size_t wi = (((size_t)k * cg + c) * kh + a) * kw + b;
                const float xv = in[(size_t)iy * W + ix];
                if (wq) acci += exhip_q8(xv * fs) * (int)wq[wi];
                else accf = __builtin_fmaf(xv, wf[wi], accf);
            }
        }
    }
    float v;
    if (wq) v = __builtin_fmaf((float)acci, scale[k], bias ? bias[k] : 0.f);
    else v = accf + (bias ? bias[k] : 0.f);
    y[i] = exhip_act(v, act);
}

}  // namespace

// ================================ C ABI ================================

#define REQ_CTX(name) EXHIP_REQUIRE(ctx, name ": NULL ctx")

template <int MODE>
static int launch_to_nhwc(exhip_ctx* ctx, const void* x, void* y, int n, int c, int h, int w, int c_stride, float fs,
                          const float* fs_pc) {
    EXHIP_REQUIRE(x && y, "layout conversion: NULL tensor");
    EXHIP_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0 && c_stride >= c, "layout conversion: bad shape");
    dim3 grid((h * w + 63) / 64, n);
    hipLaunchKernelGGL(nchw_to_nhwc_kernel<MODE>, grid, dim3(kBlock), 0, ctx->stream,
                       (const typename Conv<MODE>::in_t*)x, (typename Conv<MODE>::out_t*)y, c, h * w, c_stride, fs, fs_pc,
                       (h * w) % 4 == 0 && (uintptr_t)x % 16 == 0 ? 1 : 0);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_quantize_nchw_f32_to_nhwc_i8(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, float fs,
                                                  const float* fs_pc, int c_stride, int8_t* y) {
    REQ_CTX("exhip_quantize_nchw_f32_to_nhwc_i8");
    if (c_stride == 4 && c <= 4) {
        EXHIP_REQUIRE(x && y && n > 0 && h > 0 && w > 0, "quantize: bad argument");
        if ((h * w) % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0) {
            dim3 grid4(blocks_for((size_t)h * w / 4), n);
            hipLaunchKernelGGL(quantize_nchw_to_nhwc4_x4_kernel, grid4, dim3(kBlock), 0, ctx->stream, x, (int4*)y, c, h * w / 4, fs, fs_pc);
            EXHIP_LAUNCH_CHECK();
            return 0;
        }
        dim3 grid(blocks_for((size_t)h * w), n);
        hipLaunchKernelGGL(quantize_nchw_to_nhwc4_kernel, grid, dim3(kBlock), 0, ctx->stream, x, (int*)y, c, h * w, fs, fs_pc);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    return launch_to_nhwc<0>(ctx, x, y, n, c, h, w, c_stride, fs, fs_pc);
}
extern "C" int exhip_nchw_f32_to_nhwc_f32(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, int cs, float* y) {
    REQ_CTX("exhip_nchw_f32_to_nhwc_f32");
    return launch_to_nhwc<1>(ctx, x, y, n, c, h, w, cs, 0.f, nullptr);
}
extern "C" int exhip_nchw_f32_to_nhwc_f16(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, int cs, uint16_t* y) {
    REQ_CTX("exhip_nchw_f32_to_nhwc_f16");
    return launch_to_nhwc<2>(ctx, x, y, n, c, h, w, cs, 0.f, nullptr);
}
extern "C" int exhip_nchw_f16_to_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, int n, int c, int h, int w, int cs, uint16_t* y) {
    REQ_CTX("exhip_nchw_f16_to_nhwc_f16");
    if (cs == 4 && c >= 1 && c <= 4 && x && y && n > 0 && n <= 65535 && h > 0 && w > 0 && ((size_t)h * w) % 8 == 0 && (uintptr_t)x % 16 == 0 &&
        (uintptr_t)y % 16 == 0) {
        const int hw8 = (int)((size_t)h * w / 8);
        hipLaunchKernelGGL(nchw_f16_to_nhwc4_x8_kernel, dim3(blocks_for((size_t)hw8), n), dim3(kBlock), 0, ctx->stream, x,
                           reinterpret_cast<v4i*>(y), c, hw8);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    return launch_to_nhwc<3>(ctx, x, y, n, c, h, w, cs, 0.f, nullptr);
}

template <typename T> static size_t c_stride_bytes(int cs) { return (size_t)cs * sizeof(T); }

template <int MODE, typename Tin, typename Tout>
static int launch_to_nchw(exhip_ctx* ctx, const Tin* x, Tout* y, int n, int c, int h, int w, int cs) {
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && h > 0 && w > 0 && cs >= c, "layout conversion: bad argument");
    if ((size_t)c_stride_bytes<Tin>(cs) % 16 == 0 && (uintptr_t)x % 16 == 0 && (size_t)h * w >= 64 && n <= 65535) {
        hipLaunchKernelGGL((nhwc_to_nchw_tiled_kernel<MODE, Tin, Tout>), dim3((h * w + 63) / 64, n), dim3(kBlock), 0, ctx->stream,
                           x, y, c, h * w, cs);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    const size_t total = (size_t)n * c * h * w;
    hipLaunchKernelGGL((nhwc_to_nchw_kernel<MODE, Tin, Tout>), dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, c,
                       h * w, cs, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}
extern "C" int exhip_nhwc_f32_to_nchw_f32(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, int cs, float* y) {
    REQ_CTX("exhip_nhwc_f32_to_nchw_f32");
    return launch_to_nchw<0>(ctx, x, y, n, c, h, w, cs);
}
extern "C" int exhip_nhwc_f16_to_nchw_f32(exhip_ctx* ctx, const uint16_t* x, int n, int c, int h, int w, int cs, float* y) {
    REQ_CTX("exhip_nhwc_f16_to_nchw_f32");
    return launch_to_nchw<1>(ctx, x, y, n, c, h, w, cs);
}
extern "C" int exhip_nhwc_f16_to_nchw_f16(exhip_ctx* ctx, const uint16_t* x, int n, int c, int h, int w, int cs, uint16_t* y) {
    REQ_CTX("exhip_nhwc_f16_to_nchw_f16");
    return launch_to_nchw<2>(ctx, x, y, n, c, h, w, cs);
}

extern "C" int exhip_f32_to_f16(exhip_ctx* ctx, const float* x, uint16_t* y, size_t count) {
    REQ_CTX("exhip_f32_to_f16");
    EXHIP_REQUIRE((x && y) || !count, "exhip_f32_to_f16: NULL tensor");
    if (!count) return 0;
    const size_t n8 = ((uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0) ? count / 8 : 0;
    hipLaunchKernelGGL(f32_to_f16_kernel, dim3(blocks_for(n8 + (count - n8 * 8))), dim3(kBlock), 0, ctx->stream, x, y, n8, count);
    EXHIP_LAUNCH_CHECK();
    return 0;
}
extern "C" int exhip_f16_to_f32(exhip_ctx* ctx, const uint16_t* x, float* y, size_t count) {
    REQ_CTX("exhip_f16_to_f32");
    EXHIP_REQUIRE((x && y) || !count, "exhip_f16_to_f32: NULL tensor");
    if (!count) return 0;
    const size_t n8 = ((uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0) ? count / 8 : 0;
    hipLaunchKernelGGL(f16_to_f32_kernel, dim3(blocks_for(n8 + (count - n8 * 8))), dim3(kBlock), 0, ctx->stream, x, y, n8, count);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

static int dw_out(int h, int w, int stride, int pt, int pb, int pl, int pr, int* oh, int* ow) {
    EXHIP_REQUIRE(stride == 1 || stride == 2, "dwconv3x3: stride %d not supported", stride);
    EXHIP_REQUIRE(h + pt + pb >= 3 && w + pl + pr >= 3, "dwconv3x3: input smaller than the kernel");
    *oh = (h + pt + pb - 3) / stride + 1;
    *ow = (w + pl + pr - 3) / stride + 1;
    return 0;
}

static int dw_nchw_f32(exhip_ctx* ctx, const float* x, const float* w9, const float* bias, float* y, int n, int c, int h, int w,
                       int stride, int pt, int pb, int pl, int pr, int act, const float* slope, int slope_shared) {
    REQ_CTX("exhip_dwconv3x3_nchw_f32");
    EXHIP_REQUIRE(x && w9 && y && n > 0 && c > 0, "exhip_dwconv3x3_nchw_f32: bad argument");
    int oh, ow;
    int rc = dw_out(h, w, stride, pt, pb, pl, pr, &oh, &ow);
    if (rc) return rc;
    const size_t x_bytes = (size_t)n * c * h * w * 4, y_bytes = (size_t)n * c * oh * ow * 4;
    const size_t desc_limit = (size_t)1 << 30;
    if ((stride == 1 || stride == 2) && (act == 0 || act == 1 || act == 3) && (pl == 0 || pl == 1) && w % 4 == 0 &&
        (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 && x_bytes <= desc_limit &&
        y_bytes <= desc_limit) {
        const int strips = (ow + 3) / 4;
        const size_t per_band = (size_t)n * c * strips;
        const size_t want = (size_t)256 * 8 * 64;
        // about eight rows to a band (measured at 32x64x160x160: 5 to 10 rows 65 % of the HBM peak, 16 rows 61 %, 20 and more 59 %)
        int bands = (int)std::min<size_t>((size_t)oh, std::max<size_t>((oh + 7) / 8, (want + per_band - 1) / per_band));
        const int env_rows = g_exhip_options.dw_band_rows;
        int band_rows = (oh + bands - 1) / bands;
        if (env_rows > 0) band_rows = std::min(env_rows, oh);
        bands = (oh + band_rows - 1) / band_rows;
        const size_t total = per_band * bands;
#define EXHIP_DW_STRIP(S, A)                                                                                                     \
    do {                                                                                                                         \
        if (pl == 0)                                                                                                             \
            hipLaunchKernelGGL((dwconv3x3_nchw_f32_strip_kernel<S, A, 0>), dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, \
                               w9, bias, y, c, h, w, oh, ow, pt, band_rows, bands, strips, (unsigned)x_bytes, (unsigned)y_bytes,  \
                               total, slope, slope_shared);                                                                      \
        else                                                                                                                     \
            hipLaunchKernelGGL((dwconv3x3_nchw_f32_strip_kernel<S, A, 1>), dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, \
                               w9, bias, y, c, h, w, oh, ow, pt, band_rows, bands, strips, (unsigned)x_bytes, (unsigned)y_bytes,  \
                               total, slope, slope_shared);                                                                      \
    } while (0)
        if (stride == 1) {
            if (slope) EXHIP_DW_STRIP(1, kDwPrelu);
            else if (act == 0) EXHIP_DW_STRIP(1, 0);
            else if (act == 1) EXHIP_DW_STRIP(1, 1);
            else EXHIP_DW_STRIP(1, 3);
        } else {
            if (slope) EXHIP_DW_STRIP(2, kDwPrelu);
            else if (act == 0) EXHIP_DW_STRIP(2, 0);
            else if (act == 1) EXHIP_DW_STRIP(2, 1);
            else EXHIP_DW_STRIP(2, 3);
        }
#undef EXHIP_DW_STRIP
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    if (slope) {
        exhip_set_error("exhip_dwconv3x3_nchw_f32_prelu: this shape runs the general kernel, which has no PReLU epilogue");
        return EXHIP_ERR_UNSUPPORTED;
    }
    const size_t total = (size_t)n * c * oh * ow;
    hipLaunchKernelGGL(dwconv3x3_nchw_f32_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, w9, bias, y, c, h, w,
                       oh, ow, stride, pt, pl, act, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_dwconv3x3_nchw_f32(exhip_ctx* ctx, const float* x, const float* w9, const float* bias, float* y, int n,
                                        int c, int h, int w, int stride, int pt, int pb, int pl, int pr, int act) {
    return dw_nchw_f32(ctx, x, w9, bias, y, n, c, h, w, stride, pt, pb, pl, pr, act, nullptr, 0);
}

extern "C" int exhip_dwconv3x3_nchw_f32_prelu(exhip_ctx* ctx, const float* x, const float* w9, const float* bias,
                                              const float* slope, int slope_shared, float* y, int n, int c, int h, int w,
                                              int stride, int pt, int pb, int pl, int pr) {
    EXHIP_REQUIRE(slope, "exhip_dwconv3x3_nchw_f32_prelu: NULL slopes");
    return dw_nchw_f32(ctx, x, w9, bias, y, n, c, h, w, stride, pt, pb, pl, pr, 0, slope, slope_shared);
}

static int dw_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, const float* w9, const float* bias, uint16_t* y, int n, int c, int h,
                       int w, int cs, int stride, int pt, int pb, int pl, int pr, int act, const float* slope,
                       int slope_shared) {
    REQ_CTX("exhip_dwconv3x3_nhwc_f16");
    EXHIP_REQUIRE(x && w9 && y && n > 0 && c > 0 && cs >= c && cs % 8 == 0, "exhip_dwconv3x3_nhwc_f16: bad argument (c_stride %% 8)");
    int oh, ow;
    int rc = dw_out(h, w, stride, pt, pb, pl, pr, &oh, &ow);
    if (rc) return rc;
    const size_t x_bytes = (size_t)n * h * w * cs * 2, y_bytes = (size_t)n * oh * ow * cs * 2;
    const size_t desc_limit = (size_t)1 << 30;
    if ((stride == 1 || stride == 2) && (act == 0 || act == 1 || act == 3) && x_bytes <= desc_limit && y_bytes <= desc_limit) {
        // bands of output rows: about fourteen rows each (the per-thread set-up and the two halo rows are worth several
        // rows of work), shorter where that would leave fewer than fourteen waves for every compute unit, never under
        // seven rows (measured at 64x128x56x56: 7 rows beat 4, 10, 14 and 28 at both strides)
        // stride 2: strips of two pixels (five input columns a row); three pixels (seven columns) sit at the register
        // limit of four waves per SIMD, spill with the PReLU epilogue, and measured slower without it
        const int px = stride == 1 ? 4 : 2;
        const int strips = (ow + px - 1) / px;
        const size_t per_band = (size_t)n * strips * (cs / 4);
        const int env_rows = g_exhip_options.dw_band_rows;
        const size_t want = (size_t)256 * 14 * 64;
        int bands = (int)std::min<size_t>((size_t)std::max(1, oh / 7), std::max<size_t>((oh + 13) / 14, (want + per_band - 1) / per_band));
        int band_rows = (oh + bands - 1) / bands;
        if (env_rows > 0) band_rows = std::min(env_rows, oh);
        bands = (oh + band_rows - 1) / band_rows;
        const size_t total = per_band * bands;
#define EXHIP_DW_STRIP(S, P, A)                                                                                          \
    hipLaunchKernelGGL((dwconv3x3_nhwc_f16_strip_kernel<S, P, A>), dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, \
                       x, w9, bias, y, c, h, w, cs, oh, ow, pt, pl, band_rows, bands, strips, (unsigned)x_bytes,        \
                       (unsigned)y_bytes, total, slope, slope_shared)
        if (stride == 1) {
            if (slope) EXHIP_DW_STRIP(1, 4, kDwPrelu);
            else if (act == 0) EXHIP_DW_STRIP(1, 4, 0);
            else if (act == 1) EXHIP_DW_STRIP(1, 4, 1);
            else EXHIP_DW_STRIP(1, 4, 3);
        } else {
            if (slope) EXHIP_DW_STRIP(2, 2, kDwPrelu);
            else if (act == 0) EXHIP_DW_STRIP(2, 2, 0);
            else if (act == 1) EXHIP_DW_STRIP(2, 2, 1);
            else EXHIP_DW_STRIP(2, 2, 3);
        }
#undef EXHIP_DW_STRIP
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    if (slope) {
        exhip_set_error("exhip_dwconv3x3_nhwc_f16_prelu: this shape runs the general kernel, which has no PReLU epilogue");
        return EXHIP_ERR_UNSUPPORTED;
    }
    const size_t total = (size_t)n * oh * ow * (cs / 8);
    hipLaunchKernelGGL(dwconv3x3_nhwc_f16_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, w9, bias, y, c, h, w,
                       cs, oh, ow, stride, pt, pl, act, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_dwconv3x3_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, const float* w9, const float* bias, uint16_t* y,
                                        int n, int c, int h, int w, int cs, int stride, int pt, int pb, int pl, int pr,
                                        int act) {
    return dw_nhwc_f16(ctx, x, w9, bias, y, n, c, h, w, cs, stride, pt, pb, pl, pr, act, nullptr, 0);
}

extern "C" int exhip_dwconv3x3_nhwc_f16_prelu(exhip_ctx* ctx, const uint16_t* x, const float* w9, const float* bias,
                                              const float* slope, int slope_shared, uint16_t* y, int n, int c, int h, int w,
                                              int cs, int stride, int pt, int pb, int pl, int pr) {
    EXHIP_REQUIRE(slope, "exhip_dwconv3x3_nhwc_f16_prelu: NULL slopes");
    return dw_nhwc_f16(ctx, x, w9, bias, y, n, c, h, w, cs, stride, pt, pb, pl, pr, 0, slope, slope_shared);
}

extern "C" int exhip_dw_dequant_weights(exhip_ctx* ctx, const int8_t* w, const float* ws, float* wf, int k, int per_group) {
    REQ_CTX("exhip_dw_dequant_weights");
    EXHIP_REQUIRE(w && ws && wf && k > 0 && per_group > 0, "exhip_dw_dequant_weights: bad argument");
    hipLaunchKernelGGL(dw_dequant_kernel, dim3(blocks_for((size_t)k * per_group)), dim3(kBlock), 0, ctx->stream, w, ws, wf, k,
                       per_group);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_pool_out_hw(int h, int w, int kh, int kw, int sh, int sw, int pt, int pb, int pl, int pr, int pad_mode,
                                 int* oh, int* ow) {
    EXHIP_REQUIRE(oh && ow && sh > 0 && sw > 0, "exhip_pool_out_hw: bad argument");
    EXHIP_REQUIRE(pad_mode == 0 || pad_mode == 1, "exhip_pool_out_hw: pad_mode %d", pad_mode);
    // float quotient then ceil / floor, as src/Excalibur/operation_pooling.cpp:103-121
    const float qh = (float)(h + pt + pb - kh) / sh, qw = (float)(w + pl + pr - kw) / sw;
    *oh = (int)(pad_mode == 0 ? ceilf(qh) : floorf(qh)) + 1;
    *ow = (int)(pad_mode == 0 ? ceilf(qw) : floorf(qw)) + 1;
    return 0;
}

extern "C" int exhip_pool2d_nchw_f32(exhip_ctx* ctx, const float* x, float* y, int n, int c, int h, int w, int oh, int ow,
                                     int type, int kh, int kw, int sh, int sw, int pt, int pb, int pl, int pr,
                                     int include_pad) {
    REQ_CTX("exhip_pool2d_nchw_f32");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && oh > 0 && ow > 0 && kh > 0 && kw > 0, "exhip_pool2d_nchw_f32: bad argument");
    EXHIP_REQUIRE(type == 0 || type == 1, "exhip_pool2d_nchw_f32: unknown pooling type %d", type);
    const bool same_window = type == 0 && kh == kw && (kh == 5 || kh == 9 || kh == 13) && sh == 1 && sw == 1 && pt == kh / 2 &&
                             pb == kh / 2 && pl == kh / 2 && pr == kh / 2 && oh == h && ow == w && (long long)n * c <= 65535;
    if (same_window) {
        const dim3 grid((w + 31) / 32, (h + 31) / 32, n * c);
        if (kh == 5) hipLaunchKernelGGL((maxpool_same_nchw_f32_kernel<5>), grid, dim3(kBlock), 0, ctx->stream, x, y, h, w);
        else if (kh == 9) hipLaunchKernelGGL((maxpool_same_nchw_f32_kernel<9>), grid, dim3(kBlock), 0, ctx->stream, x, y, h, w);
        else hipLaunchKernelGGL((maxpool_same_nchw_f32_kernel<13>), grid, dim3(kBlock), 0, ctx->stream, x, y, h, w);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    if (type == 1 && oh == 1 && ow == 1 && kh == h && kw == w && pt == 0 && pb == 0 && pl == 0 && pr == 0 && h * w >= 64) {
        // the whole plane in one window: a wave per plane instead of one thread walking it
        const size_t planes = (size_t)n * c;
        hipLaunchKernelGGL(global_avgpool_nchw_f32_kernel, dim3((unsigned)((planes + kBlock / 64 - 1) / (kBlock / 64))), dim3(kBlock), 0,
                           ctx->stream, x, y, h * w, planes);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    const bool strip_window = kh == kw && (kh == 2 || kh == 3) && sh == 2 && sw == 2 && pl >= 0 && pl <= 1 && pt >= 0 &&
                              w % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0;
    if (strip_window) {
        const int strips = (ow + 3) / 4;
        // maximum: two output rows per thread (five input rows instead of six: the windows share one); the averages keep
        // one row per thread
        const int rows = type == 0 ? 2 : 1;
        const int row_blocks = (oh + rows - 1) / rows;
        const size_t threads = (size_t)n * c * row_blocks * strips;
#define EXHIP_POOL_STRIP(K, T, R)                                                                                                  \
    do {                                                                                                                           \
        if (pl == 0)                                                                                                               \
            hipLaunchKernelGGL((pool_s2_nchw_f32_strip_kernel<K, T, R, 0>), dim3(blocks_for(threads)), dim3(kBlock), 0, ctx->stream, \
                               x, y, h, w, oh, ow, pt, pb, pr, include_pad, strips, row_blocks, threads);                          \
        else                                                                                                                       \
            hipLaunchKernelGGL((pool_s2_nchw_f32_strip_kernel<K, T, R, 1>), dim3(blocks_for(threads)), dim3(kBlock), 0, ctx->stream, \
                               x, y, h, w, oh, ow, pt, pb, pr, include_pad, strips, row_blocks, threads);                          \
    } while (0)
        if (kh == 2 && type == 0) EXHIP_POOL_STRIP(2, 0, 2);
        else if (kh == 2) EXHIP_POOL_STRIP(2, 1, 1);
        else if (type == 0) EXHIP_POOL_STRIP(3, 0, 2);
        else EXHIP_POOL_STRIP(3, 1, 1);
#undef EXHIP_POOL_STRIP
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    const size_t total = (size_t)n * c * oh * ow;
    hipLaunchKernelGGL(pool2d_nchw_f32_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, h, w, oh, ow, type,
                       kh, kw, sh, sw, pt, pb, pl, pr, include_pad, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_maxpool2d_nhwc_f32(exhip_ctx* ctx, const float* x, float* y, int8_t* y_i8, float fs_out, int n, int c,
                                        int h, int w, int cs, int oh, int ow, int kh, int kw, int sh, int sw, int pt, int pl) {
    REQ_CTX("exhip_maxpool2d_nhwc_f32");
    EXHIP_REQUIRE(x && (y || y_i8) && n > 0 && c > 0 && cs >= c && cs % 4 == 0, "exhip_maxpool2d_nhwc_f32: bad argument");
    if (kh == 3 && kw == 3 && sh == 2 && sw == 2 && pt >= 0 && pl >= 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0 &&
        (!y || (reinterpret_cast<uintptr_t>(y) & 15) == 0)) {
        const size_t threads = (size_t)n * ((oh + 1) / 2) * ((ow + 1) / 2) * (cs / 4);
        hipLaunchKernelGGL(maxpool3x3s2_nhwc_f32_block_kernel, dim3(blocks_for(threads)), dim3(kBlock), 0, ctx->stream, x, y, y_i8,
                           fs_out, h, w, cs, oh, ow, pt, pl, threads);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    const size_t total = (size_t)n * oh * ow * (cs / 4);
    hipLaunchKernelGGL(maxpool_nhwc_f32_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, y_i8, fs_out, h, w,
                       cs, oh, ow, kh, kw, sh, sw, pt, pl, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_maxpool2d_nhwc_i8(exhip_ctx* ctx, const int8_t* x, int8_t* y, int n, int c, int h, int w, int cs, int oh, int ow,
                                       int kh, int kw, int sh, int sw, int pt, int pl) {
    REQ_CTX("exhip_maxpool2d_nhwc_i8");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && cs >= c && cs % 16 == 0 && h > 0 && w > 0 && oh > 0 && ow > 0 && kh > 0 && kw > 0 && sh > 0 && sw > 0 &&
                      pt >= 0 && pl >= 0 && pt < kh && pl < kw,
                  "exhip_maxpool2d_nhwc_i8: bad argument");
    EXHIP_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0, "exhip_maxpool2d_nhwc_i8: tensors must be 16-byte aligned");
    // every window holds at least one pixel of the image
    EXHIP_REQUIRE((oh - 1) * sh - pt < h && (ow - 1) * sw - pl < w, "exhip_maxpool2d_nhwc_i8: output %dx%d does not fit input %dx%d", oh, ow, h, w);
    const size_t total = (size_t)n * oh * ow * (cs / 16);
    hipLaunchKernelGGL(maxpool_nhwc_i8_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, h, w, cs, oh, ow, kh, kw, sh, sw, pt, pl,
                       total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_maxpool_same_pyramid_nhwc_i8(exhip_ctx* ctx, const int8_t* x, int8_t* y1, int8_t* y2, int8_t* y3, int n, int c, int h, int w,
                                                  int cs, int k) {
    REQ_CTX("exhip_maxpool_same_pyramid_nhwc_i8");
    EXHIP_REQUIRE(x && y1 && (y2 || !y3) && n > 0 && c > 0 && cs >= c && cs % 16 == 0 && h > 0 && w > 0 && k > 0 && (k & 1), "exhip_maxpool_same_pyramid_nhwc_i8: bad argument");
    EXHIP_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y1) | reinterpret_cast<uintptr_t>(y2) | reinterpret_cast<uintptr_t>(y3)) & 15) == 0,
                  "exhip_maxpool_same_pyramid_nhwc_i8: tensors must be 16-byte aligned");
    if ((long long)h * w <= kPyrPixels && n <= 65535) {
        hipLaunchKernelGGL(maxpool_pyramid_nhwc_i8_kernel, dim3((unsigned)(cs / 16), (unsigned)n), dim3(kBlock), 0, ctx->stream, x, y1, y2, y3, h, w, cs, k);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    // a map that does not fit the group's LDS: level by level through the window kernel
    const int8_t* src = x;
    int8_t* const outs[3] = {y1, y2, y3};
    for (int level = 0; level < 3 && outs[level]; ++level) {
        const int rc = exhip_maxpool2d_nhwc_i8(ctx, src, outs[level], n, c, h, w, cs, h, w, k, k, 1, 1, k / 2, k / 2);
        if (rc) return rc;
        src = outs[level];
    }
    return 0;
}

extern "C" int exhip_pool2d_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int h, int w, int cs,
                                     int oh, int ow, int type, int kh, int kw, int sh, int sw, int pt, int pb, int pl,
                                     int pr, int include_pad) {
    REQ_CTX("exhip_pool2d_nhwc_f16");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && cs >= c && cs % 8 == 0, "exhip_pool2d_nhwc_f16: bad argument");
    EXHIP_REQUIRE(type == 0 || type == 1, "exhip_pool2d_nhwc_f16: unknown pooling type %d", type);
    const size_t total = (size_t)n * oh * ow * (cs / 8);
    if (type == 0 && kh == kw && sh == sw && sh == 2 && (kh == 2 || kh == 3) && pt >= 0 && pl >= 0 && pt < kh && pl < kw &&
        (oh - 1) * 2 - pt < h && (ow - 1) * 2 - pl < w) {
        if (kh == 3) {
            const size_t threads = (size_t)n * ((oh + 1) / 2) * ((ow + 1) / 2) * (cs / 8);
            hipLaunchKernelGGL(maxpool3x3s2_nhwc_f16_block_kernel, dim3(blocks_for(threads)), dim3(kBlock), 0, ctx->stream, x, y, h, w,
                               cs, oh, ow, pt, pl, threads);
        } else
            hipLaunchKernelGGL((maxpool_nhwc_f16_window_kernel<2, 2>), dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, h,
                               w, cs, oh, ow, pt, pl, total);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    if (type == 1 && oh == 1 && ow == 1 && kh == h && kw == w && pt == 0 && pb == 0 && pl == 0 && pr == 0 && h * w >= 16) {
        // the whole plane in one window: parallel partial sums instead of one thread walking the plane
        int G = 32;
        while (G > 1 && (cs / 8) % G != 0) G >>= 1;
        const int slabs = (cs / 8) / G;
        hipLaunchKernelGGL(global_avgpool_nhwc_f16_kernel, dim3(n * slabs), dim3(kBlock), 0, ctx->stream, x, y, h * w, cs, G, slabs);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    hipLaunchKernelGGL(pool2d_nhwc_f16_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, h, w, cs, oh, ow,
                       type, kh, kw, sh, sw, pt, pb, pl, pr, include_pad, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_eltwise_f32(exhip_ctx* ctx, const float* const* inputs, int n_inputs, const float* coeffs, int type,
                                 float* y, size_t count) {
    REQ_CTX("exhip_eltwise_f32");
    EXHIP_REQUIRE(inputs && y, "exhip_eltwise_f32: NULL tensor");
    EXHIP_REQUIRE(n_inputs >= 2 && n_inputs <= 8, "exhip_eltwise_f32: %d inputs (2..8 supported)", n_inputs);
    EXHIP_REQUIRE(type >= 0 && type <= 2, "exhip_eltwise_f32: unknown elementwise operation %d", type);
    if (!count) return 0;
    EltArgs a;
    a.n = n_inputs;
    for (int i = 0; i < n_inputs; ++i) {
        EXHIP_REQUIRE(inputs[i], "exhip_eltwise_f32: input %d is NULL", i);
        a.in[i] = inputs[i];
        a.coeff[i] = coeffs ? coeffs[i] : 1.0f;
    }
    bool aligned = (uintptr_t)y % 16 == 0;
    for (int i = 0; i < n_inputs; ++i) aligned = aligned && (uintptr_t)inputs[i] % 16 == 0;
    if (aligned) {
        const size_t body = count - count % 8;
        const dim3 grid(blocks_for(body / 4 + count % 8));
        if (type == 0) hipLaunchKernelGGL((eltwise_f32_v4_kernel<0>), grid, dim3(kBlock), 0, ctx->stream, a, y, count, body);
        else if (type == 1) hipLaunchKernelGGL((eltwise_f32_v4_kernel<1>), grid, dim3(kBlock), 0, ctx->stream, a, y, count, body);
        else hipLaunchKernelGGL((eltwise_f32_v4_kernel<2>), grid, dim3(kBlock), 0, ctx->stream, a, y, count, body);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    hipLaunchKernelGGL(eltwise_f32_kernel, dim3(blocks_for(count)), dim3(kBlock), 0, ctx->stream, a, type, y, count,
                       count - count % 8);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

static int launch_add_f32(exhip_ctx* ctx, const float* a, const float* b, float* y, size_t count, int relu) {
    if (!count) return 0;
    const bool aligned = ((uintptr_t)a % 16 == 0) && ((uintptr_t)y % 16 == 0) && (!b || (uintptr_t)b % 16 == 0);
    const size_t n4 = aligned ? count / 4 : 0;
    const size_t threads = n4 + (count - n4 * 4);
    hipLaunchKernelGGL(add_f32_kernel, dim3(blocks_for(threads)), dim3(kBlock), 0, ctx->stream, a, b, y, n4, count, relu);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_add_f32(exhip_ctx* ctx, const float* a, const float* b, float* y, size_t count, int relu) {
    REQ_CTX("exhip_add_f32");
    EXHIP_REQUIRE((a && b && y) || !count, "exhip_add_f32: NULL tensor");
    return launch_add_f32(ctx, a, b, y, count, relu);
}
extern "C" int exhip_relu_f32(exhip_ctx* ctx, const float* x, float* y, size_t count) {
    REQ_CTX("exhip_relu_f32");
    EXHIP_REQUIRE((x && y) || !count, "exhip_relu_f32: NULL tensor");
    return launch_add_f32(ctx, x, nullptr, y, count, 1);
}
extern "C" int exhip_add_f16(exhip_ctx* ctx, const uint16_t* a, const uint16_t* b, uint16_t* y, size_t count, int relu) {
    REQ_CTX("exhip_add_f16");
    EXHIP_REQUIRE((a && b && y) || !count, "exhip_add_f16: NULL tensor");
    if (!count) return 0;
    const size_t n8 = ((uintptr_t)a % 16 == 0 && (uintptr_t)b % 16 == 0 && (uintptr_t)y % 16 == 0) ? count / 8 : 0;
    hipLaunchKernelGGL(add_f16_kernel, dim3(blocks_for(n8 + (count - n8 * 8))), dim3(kBlock), 0, ctx->stream, a, b, y, n8, count, relu);
    EXHIP_LAUNCH_CHECK();
    return 0;
}
extern "C" int exhip_relu_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, size_t count) {
    REQ_CTX("exhip_relu_f16");
    EXHIP_REQUIRE((x && y) || !count, "exhip_relu_f16: NULL tensor");
    if (!count) return 0;
    const size_t n8 = ((uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0) ? count / 8 : 0;
    hipLaunchKernelGGL(add_f16_kernel, dim3(blocks_for(n8 + (count - n8 * 8))), dim3(kBlock), 0, ctx->stream, x, (const uint16_t*)nullptr, y, n8, count, 1);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_innerproduct_f32(exhip_ctx* ctx, const float* x, const float* w, const float* bias, float* y, int m,
                                      int n_out, int k_in) {
    REQ_CTX("exhip_innerproduct_f32");
    EXHIP_REQUIRE(x && w && y && m > 0 && n_out > 0 && k_in > 0, "exhip_innerproduct_f32: bad argument");
    const unsigned row_groups = (unsigned)std::min((m + 7) / 8, 1024);
    hipLaunchKernelGGL(innerproduct_f32_kernel, dim3((n_out + 3) / 4, row_groups), dim3(kBlock), 0, ctx->stream, x, w, bias, y, m, n_out, k_in);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_conv2d_direct_nchw(exhip_ctx* ctx, const exhip_conv_desc* d, int groups, const float* x, const float* wf,
                                        const int8_t* wq, float fs, const float* scale, const float* bias, float* y) {
    REQ_CTX("exhip_conv2d_direct_nchw");
    EXHIP_REQUIRE(d && x && y && (wf || wq), "exhip_conv2d_direct_nchw: NULL argument");
    EXHIP_REQUIRE(!wq || scale, "exhip_conv2d_direct_nchw: int8 weights need scales");
    EXHIP_REQUIRE(groups > 0 && d->c % groups == 0 && d->k % groups == 0, "exhip_conv2d_direct_nchw: channels not divisible by groups");
    EXHIP_REQUIRE(d->sh > 0 && d->sw > 0 && d->kh > 0 && d->kw > 0, "exhip_conv2d_direct_nchw: bad kernel/stride");
    const int oh = (d->h + d->pt + d->pb - d->kh) / d->sh + 1, ow = (d->w + d->pl + d->pr - d->kw) / d->sw + 1;
    EXHIP_REQUIRE(oh > 0 && ow > 0, "exhip_conv2d_direct_nchw: empty output");
    const size_t total = (size_t)d->n * d->k * oh * ow;
    hipLaunchKernelGGL(conv_direct_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, wf, wq, fs, scale, bias, y,
                       d->c, d->h, d->w, d->k, oh, ow, d->kh, d->kw, d->sh, d->sw, d->pt, d->pl, groups, d->act, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

// ---- activation / glue layers ----
template <int OP>
static int launch_unary(exhip_ctx* ctx, const float* x, float* y, size_t count, float alpha, float beta) {
    if (!count) return 0;
    const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0);
    const size_t n4 = aligned ? count / 4 : 0;
    const size_t threads = n4 + (count - n4 * 4);
    hipLaunchKernelGGL((unary_f32_kernel<OP>), dim3(blocks_for(threads)), dim3(kBlock), 0, ctx->stream, x, y, n4, count, alpha, beta);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_unary_f32(exhip_ctx* ctx, int op, const float* x, float* y, size_t count, float alpha, float beta) {
    REQ_CTX("exhip_unary_f32");
    EXHIP_REQUIRE((x && y) || !count, "exhip_unary_f32: NULL tensor");
    switch (op) {
    case EXHIP_UNARY_HARDSWISH: return launch_unary<0>(ctx, x, y, count, alpha, beta);
    case EXHIP_UNARY_LEAKYRELU: return launch_unary<1>(ctx, x, y, count, alpha, beta);
    case EXHIP_UNARY_SIGMOID: return launch_unary<2>(ctx, x, y, count, alpha, beta);
    case EXHIP_UNARY_HARDSIGMOID: return launch_unary<3>(ctx, x, y, count, alpha, beta);
    case EXHIP_UNARY_CLIP: return launch_unary<4>(ctx, x, y, count, alpha, beta);
    default: exhip_set_error("exhip_unary_f32: unknown op %d", op); return EXHIP_ERR_ARG;
    }
}

template <int OP>
static int launch_unary_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, size_t count, float alpha, float beta) {
    if (!count) return 0;
    const bool aligned = ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0);
    const size_t n8 = aligned ? count / 8 : 0;
    const size_t threads = n8 + (count - n8 * 8);
    hipLaunchKernelGGL((unary_f16_kernel<OP>), dim3(blocks_for(threads)), dim3(kBlock), 0, ctx->stream, x, y, n8, count, alpha, beta);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_unary_f16(exhip_ctx* ctx, int op, const uint16_t* x, uint16_t* y, size_t count, float alpha, float beta) {
    REQ_CTX("exhip_unary_f16");
    EXHIP_REQUIRE((x && y) || !count, "exhip_unary_f16: NULL tensor");
    switch (op) {
    case EXHIP_UNARY_HARDSWISH: return launch_unary_f16<0>(ctx, x, y, count, alpha, beta);
    case EXHIP_UNARY_LEAKYRELU: return launch_unary_f16<1>(ctx, x, y, count, alpha, beta);
    case EXHIP_UNARY_SIGMOID: return launch_unary_f16<2>(ctx, x, y, count, alpha, beta);
    case EXHIP_UNARY_HARDSIGMOID: return launch_unary_f16<3>(ctx, x, y, count, alpha, beta);
    case EXHIP_UNARY_CLIP: return launch_unary_f16<4>(ctx, x, y, count, alpha, beta);
    default: exhip_set_error("exhip_unary_f16: unknown op %d", op); return EXHIP_ERR_ARG;
    }
}

template <int OP>
static void launch_channelwise_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int hw, const float* p0,
                                   const float* p1, int shared) {
    const bool vec = hw % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0;
    unsigned bx = blocks_for((size_t)(vec ? hw / 8 : hw));
    if (bx > 64) bx = 64;
    const dim3 grid(bx, (unsigned)(n * c));
    if (vec) hipLaunchKernelGGL((channelwise_f16_kernel<OP, 8>), grid, dim3(kBlock), 0, ctx->stream, x, y, c, hw, p0, p1, shared);
    else hipLaunchKernelGGL((channelwise_f16_kernel<OP, 1>), grid, dim3(kBlock), 0, ctx->stream, x, y, c, hw, p0, p1, shared);
}

extern "C" int exhip_channelwise_f16(exhip_ctx* ctx, int op, const uint16_t* x, uint16_t* y, int n, int c, int hw, const float* p0,
                                     const float* p1, int shared) {
    REQ_CTX("exhip_channelwise_f16");
    EXHIP_REQUIRE(x && y && p0 && n > 0 && c > 0 && hw > 0, "exhip_channelwise_f16: bad argument");
    EXHIP_REQUIRE(op == EXHIP_CHANNEL_PRELU || p1, "exhip_channelwise_f16: this op needs two parameter arrays");
    EXHIP_REQUIRE(c <= 65535, "exhip_channelwise_f16: more than 65535 channels");
    EXHIP_REQUIRE(op == EXHIP_CHANNEL_PRELU || op == EXHIP_CHANNEL_BATCHNORM || op == EXHIP_CHANNEL_INPUT,
                  "exhip_channelwise_f16: unknown op %d", op);
    // one block row per (image, channel) plane, at most 65535 rows to a launch: whole images per launch
    const int per_launch = 65535 / c;
    for (int n0 = 0; n0 < n; n0 += per_launch) {
        const int nn = std::min(per_launch, n - n0);
        const size_t off = (size_t)n0 * c * hw;
        if (op == EXHIP_CHANNEL_PRELU) launch_channelwise_f16<0>(ctx, x + off, y + off, nn, c, hw, p0, p1, shared);
        else if (op == EXHIP_CHANNEL_BATCHNORM) launch_channelwise_f16<1>(ctx, x + off, y + off, nn, c, hw, p0, p1, 0);
        else launch_channelwise_f16<2>(ctx, x + off, y + off, nn, c, hw, p0, p1, 0);
        EXHIP_LAUNCH_CHECK();
    }
    return 0;
}

extern "C" int exhip_concat_channels_nhwc_f16(exhip_ctx* ctx, const uint16_t* const* inputs, const int* channels, int n_inputs,
                                              size_t pixels, uint16_t* y) {
    REQ_CTX("exhip_concat_channels_nhwc_f16");
    EXHIP_REQUIRE(inputs && channels && y && n_inputs >= 1 && n_inputs <= 8 && pixels > 0, "exhip_concat_channels_nhwc_f16: bad argument");
    ConcatNhwcArgs a = {};
    a.n_inputs = n_inputs;
    int total = 0;
    for (int i = 0; i < n_inputs; ++i) {
        EXHIP_REQUIRE(inputs[i] && channels[i] > 0 && channels[i] % 8 == 0 && (reinterpret_cast<uintptr_t>(inputs[i]) & 15) == 0,
                      "exhip_concat_channels_nhwc_f16: input %d needs a multiple of 8 channels and 16-byte alignment", i);
        a.src[i] = inputs[i];
        a.first[i] = total;
        total += channels[i];
    }
    a.first[n_inputs] = total;
    EXHIP_REQUIRE((reinterpret_cast<uintptr_t>(y) & 15) == 0, "exhip_concat_channels_nhwc_f16: output must be 16-byte aligned");
    const size_t total8 = pixels * (size_t)(total / 8);
    hipLaunchKernelGGL(concat_nhwc_f16_kernel, dim3(blocks_for(total8)), dim3(kBlock), 0, ctx->stream, a, y, total8);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_concat_batchnorm_unary_nhwc_f16(exhip_ctx* ctx, const uint16_t* const* inputs, const int* channels, int n_inputs,
                                                     size_t pixels, const float* bn_a, const float* bn_b, int unary_op, float alpha,
                                                     float beta, uint16_t* y) {
    REQ_CTX("exhip_concat_batchnorm_unary_nhwc_f16");
    EXHIP_REQUIRE(inputs && channels && y && n_inputs >= 1 && n_inputs <= 8 && pixels > 0, "exhip_concat_batchnorm_unary_nhwc_f16: bad argument");
    EXHIP_REQUIRE((bn_a == nullptr) == (bn_b == nullptr), "exhip_concat_batchnorm_unary_nhwc_f16: BatchNorm needs both parameter arrays");
    ConcatNhwcArgs a = {};
    a.n_inputs = n_inputs;
    int total = 0;
    for (int i = 0; i < n_inputs; ++i) {
        EXHIP_REQUIRE(inputs[i] && channels[i] > 0 && channels[i] % 8 == 0 && (reinterpret_cast<uintptr_t>(inputs[i]) & 15) == 0,
                      "exhip_concat_batchnorm_unary_nhwc_f16: input %d needs a multiple of 8 channels and 16-byte alignment", i);
        a.src[i] = inputs[i];
        a.first[i] = total;
        total += channels[i];
    }
    a.first[n_inputs] = total;
    EXHIP_REQUIRE((reinterpret_cast<uintptr_t>(y) & 15) == 0, "exhip_concat_batchnorm_unary_nhwc_f16: output must be 16-byte aligned");
    EXHIP_REQUIRE(!bn_a || ((reinterpret_cast<uintptr_t>(bn_a) | reinterpret_cast<uintptr_t>(bn_b)) & 15) == 0,
                  "exhip_concat_batchnorm_unary_nhwc_f16: BatchNorm parameters must be 16-byte aligned");
    // one vector per thread: two (the float32 kernel's gain) measured slower on halves, 104 against 90 us at 2 x 32x64x160x160
    const size_t threads = pixels * (size_t)(total / 8);
    const dim3 grid(blocks_for(threads)), block(kBlock);
#define EXHIP_CAU(UOP) hipLaunchKernelGGL((concat_affine_unary_nhwc_f16_kernel<UOP, 1>), grid, block, 0, ctx->stream, a, y, threads, bn_a, bn_b, alpha, beta)
    switch (unary_op) {
    case -1: EXHIP_CAU(-1); break;
    case EXHIP_UNARY_HARDSWISH: EXHIP_CAU(0); break;
    case EXHIP_UNARY_LEAKYRELU: EXHIP_CAU(1); break;
    case EXHIP_UNARY_HARDSIGMOID: EXHIP_CAU(3); break;
    case EXHIP_UNARY_CLIP: EXHIP_CAU(4); break;
    default: exhip_set_error("exhip_concat_batchnorm_unary_nhwc_f16: activation %d is not one this kernel applies", unary_op); return EXHIP_ERR_ARG;
    }
#undef EXHIP_CAU
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_concat_batchnorm_unary_nhwc_f32(exhip_ctx* ctx, const float* const* inputs, const int* channels, const int* strides,
                                                     int n_inputs, size_t pixels, const float* bn_a, const float* bn_b, int unary_op,
                                                     float alpha, float beta, int out_stride, float* y_f32, int8_t* y_i8, float fs_out) {
    REQ_CTX("exhip_concat_batchnorm_unary_nhwc_f32");
    EXHIP_REQUIRE(inputs && channels && strides && (y_f32 || y_i8) && n_inputs >= 1 && n_inputs <= 8 && pixels > 0,
                  "exhip_concat_batchnorm_unary_nhwc_f32: bad argument");
    EXHIP_REQUIRE((bn_a == nullptr) == (bn_b == nullptr), "exhip_concat_batchnorm_unary_nhwc_f32: BatchNorm needs both parameter arrays");
    ConcatNhwcF32Args a = {};
    a.n_inputs = n_inputs;
    int total = 0;
    for (int i = 0; i < n_inputs; ++i) {
        EXHIP_REQUIRE(inputs[i] && channels[i] > 0 && channels[i] % 4 == 0 && strides[i] >= channels[i] && strides[i] % 4 == 0 &&
                          (reinterpret_cast<uintptr_t>(inputs[i]) & 15) == 0,
                      "exhip_concat_batchnorm_unary_nhwc_f32: input %d needs channels and a stride that are multiples of 4 and 16-byte alignment", i);
        a.src[i] = inputs[i];
        a.first[i] = total;
        a.stride[i] = strides[i];
        total += channels[i];
    }
    a.first[n_inputs] = total;
    EXHIP_REQUIRE(out_stride >= total && out_stride % 4 == 0, "exhip_concat_batchnorm_unary_nhwc_f32: output stride %d for %d channels", out_stride, total);
    EXHIP_REQUIRE(!y_f32 || (reinterpret_cast<uintptr_t>(y_f32) & 15) == 0, "exhip_concat_batchnorm_unary_nhwc_f32: float output must be 16-byte aligned");
    EXHIP_REQUIRE(!y_i8 || (reinterpret_cast<uintptr_t>(y_i8) & 3) == 0, "exhip_concat_batchnorm_unary_nhwc_f32: int8 output must be 4-byte aligned");
    EXHIP_REQUIRE(!bn_a || ((reinterpret_cast<uintptr_t>(bn_a) | reinterpret_cast<uintptr_t>(bn_b)) & 15) == 0,
                  "exhip_concat_batchnorm_unary_nhwc_f32: BatchNorm parameters must be 16-byte aligned");
    bool wide = out_stride % 16 == 0 && (!y_i8 || (reinterpret_cast<uintptr_t>(y_i8) & 15) == 0);
    for (int i = 0; i < n_inputs; ++i) wide = wide && channels[i] % 16 == 0;
    const size_t threads = pixels * (size_t)(out_stride / (wide ? 16 : 4));
    const dim3 grid(blocks_for(threads)), block(kBlock);
#define EXHIP_CAU32(UOP)                                                                                                                      \
    do {                                                                                                                                      \
        if (wide)                                                                                                                             \
            hipLaunchKernelGGL((concat_affine_unary_nhwc_f32_kernel<UOP, 4>), grid, block, 0, ctx->stream, a, y_f32, y_i8, out_stride, fs_out, \
                               threads, bn_a, bn_b, alpha, beta);                                                                              \
        else                                                                                                                                  \
            hipLaunchKernelGGL((concat_affine_unary_nhwc_f32_kernel<UOP, 1>), grid, block, 0, ctx->stream, a, y_f32, y_i8, out_stride, fs_out, \
                               threads, bn_a, bn_b, alpha, beta);                                                                              \
    } while (0)
    switch (unary_op) {
    case -1: EXHIP_CAU32(-1); break;
    case EXHIP_UNARY_HARDSWISH: EXHIP_CAU32(0); break;
    case EXHIP_UNARY_LEAKYRELU: EXHIP_CAU32(1); break;
    case EXHIP_UNARY_HARDSIGMOID: EXHIP_CAU32(3); break;
    case EXHIP_UNARY_CLIP: EXHIP_CAU32(4); break;
    default: exhip_set_error("exhip_concat_batchnorm_unary_nhwc_f32: activation %d is not one this kernel applies", unary_op); return EXHIP_ERR_ARG;
    }
#undef EXHIP_CAU32
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_interp_nearest_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int h, int w, int oh,
                                             int ow) {
    REQ_CTX("exhip_interp_nearest_nhwc_f16");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && c % 8 == 0 && h > 0 && w > 0 && oh > 0 && ow > 0, "exhip_interp_nearest_nhwc_f16: bad argument");
    EXHIP_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0,
                  "exhip_interp_nearest_nhwc_f16: tensors must be 16-byte aligned");
    const size_t total8 = (size_t)n * oh * ow * (c / 8);
    hipLaunchKernelGGL(interp_nearest_nhwc_f16_kernel, dim3(blocks_for(total8)), dim3(kBlock), 0, ctx->stream, x, y, h, w, c / 8, oh, ow,
                       h / (float)oh, w / (float)ow, total8);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_maxpool_same_nhwc_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* tmp, uint16_t* y, int n, int c, int h, int w,
                                           int k) {
    REQ_CTX("exhip_maxpool_same_nhwc_f16");
    EXHIP_REQUIRE(x && tmp && y && n > 0 && c > 0 && c % 8 == 0 && h > 0 && w > 0, "exhip_maxpool_same_nhwc_f16: bad argument");
    EXHIP_REQUIRE(k == 5 || k == 9 || k == 13, "exhip_maxpool_same_nhwc_f16: window %d (5, 9 or 13)", k);
    EXHIP_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(tmp) | reinterpret_cast<uintptr_t>(y)) & 15) == 0,
                  "exhip_maxpool_same_nhwc_f16: tensors must be 16-byte aligned");
    const size_t total8 = (size_t)n * h * w * (c / 8);
    const dim3 grid(blocks_for(total8)), block(kBlock);
#define EXHIP_SAME_POOL(K)                                                                                                   \
    do {                                                                                                                     \
        hipLaunchKernelGGL((maxpool_same_1d_nhwc_f16_kernel<K, true>), grid, block, 0, ctx->stream, x, tmp, h, w, c / 8, total8); \
        hipLaunchKernelGGL((maxpool_same_1d_nhwc_f16_kernel<K, false>), grid, block, 0, ctx->stream, tmp, y, h, w, c / 8, total8); \
    } while (0)
    if (k == 5) EXHIP_SAME_POOL(5);
    else if (k == 9) EXHIP_SAME_POOL(9);
    else EXHIP_SAME_POOL(13);
#undef EXHIP_SAME_POOL
    EXHIP_LAUNCH_CHECK();
    return 0;
}

// ---- the one entry point that allocates nothing ----
// The row pass of the separable pooling above needs an intermediate tensor of the input's size. For callers that cannot
// allocate device memory (code under graph capture, serving loops, harnesses that forbid hipMalloc) it lives in this
// file-scope device array: each GPU the library runs on holds its own copy until the process ends.
static constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// The array's name is only a host-side handle; its device address differs per GPU and is looked up once per device,
// with that device current (exhip_init does so), and kept here.
static constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kMaxDevices] = {};

int exhip_static_scratch_setup(int device) {
    EXHIP_REQUIRE(device >= 0 && device < kMaxDevices, "static scratch: device %d out of range", device);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device]) return 0;
    void* ptr = nullptr;
    EXHIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    EXHIP_REQUIRE(ptr != nullptr && (reinterpret_cast<uintptr_t>(ptr) & 255) == 0, "static scratch: bad device address %p", ptr);
    g_scratch_ptr[device] = ptr;
    return 0;
}

extern "C" size_t exhip_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int exhip_maxpool_same_nhwc_f16_static(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int h, int w, int k) {
    REQ_CTX("exhip_maxpool_same_nhwc_f16_static");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && c % 8 == 0 && h > 0 && w > 0, "exhip_maxpool_same_nhwc_f16_static: bad argument");
    const size_t bytes = (size_t)n * h * w * c * sizeof(uint16_t);
    EXHIP_REQUIRE(bytes <= kStaticScratchBytes,
                  "exhip_maxpool_same_nhwc_f16_static: the tensor has %zu bytes, the static scratch array holds %zu; use "
                  "exhip_maxpool_same_nhwc_f16 with a workspace of the caller's",
                  bytes, kStaticScratchBytes);
    EXHIP_REQUIRE(ctx->device >= 0 && ctx->device < kMaxDevices, "exhip_maxpool_same_nhwc_f16_static: device %d out of range", ctx->device);
    void* ptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        ptr = g_scratch_ptr[ctx->device];
    }
    EXHIP_REQUIRE(ptr != nullptr, "exhip_maxpool_same_nhwc_f16_static: device %d was not set up by exhip_init", ctx->device);
    // The row pass writes every element of the part of the array the column pass reads: nothing needs clearing.
    return exhip_maxpool_same_nhwc_f16(ctx, x, static_cast<uint16_t*>(ptr), y, n, c, h, w, k);
}

extern "C" int exhip_channelwise_nhwc_f16(exhip_ctx* ctx, int op, const uint16_t* x, uint16_t* y, size_t pixels, int c,
                                          const float* p0, const float* p1, int shared) {
    REQ_CTX("exhip_channelwise_nhwc_f16");
    EXHIP_REQUIRE(x && y && p0 && pixels > 0 && c > 0, "exhip_channelwise_nhwc_f16: bad argument");
    EXHIP_REQUIRE(c % 8 == 0, "exhip_channelwise_nhwc_f16: %d channels, need a multiple of 8", c);
    EXHIP_REQUIRE((reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0,
                  "exhip_channelwise_nhwc_f16: tensors must be 16-byte aligned");
    EXHIP_REQUIRE(op == EXHIP_CHANNEL_PRELU || p1, "exhip_channelwise_nhwc_f16: this op needs two parameter arrays");
    const size_t n8 = pixels * (size_t)c / 8;
    // about eight vectors per thread, in a launch whose thread count is a multiple of the channel groups
    const unsigned groups = (unsigned)c / 8;
    unsigned g = groups, r = kBlock;
    while (r) { const unsigned t = g % r; g = r; r = t; }           // g = gcd(groups, kBlock)
    const unsigned unit = groups / g;
    size_t blocks = (n8 + (size_t)kBlock * 8 - 1) / ((size_t)kBlock * 8);
    blocks = (blocks + unit - 1) / unit * unit;
    EXHIP_REQUIRE(blocks * kBlock < (1ull << 32), "exhip_channelwise_nhwc_f16: tensor too large");
    const bool vp = (reinterpret_cast<uintptr_t>(p0) & 15) == 0 && (reinterpret_cast<uintptr_t>(p1) & 15) == 0;
    const dim3 grid((unsigned)blocks);
#define EXHIP_CW_NHWC(OP, SH)                                                                                                 \
    if (vp) hipLaunchKernelGGL((channelwise_nhwc_f16_kernel<OP, true>), grid, dim3(kBlock), 0, ctx->stream, x, y, n8, groups, p0, p1, SH); \
    else hipLaunchKernelGGL((channelwise_nhwc_f16_kernel<OP, false>), grid, dim3(kBlock), 0, ctx->stream, x, y, n8, groups, p0, p1, SH)
    switch (op) {
    case EXHIP_CHANNEL_PRELU: EXHIP_CW_NHWC(0, shared); break;
    case EXHIP_CHANNEL_BATCHNORM: EXHIP_CW_NHWC(1, 0); break;
    case EXHIP_CHANNEL_INPUT: EXHIP_CW_NHWC(2, 0); break;
    default: exhip_set_error("exhip_channelwise_nhwc_f16: unknown op %d", op); return EXHIP_ERR_ARG;
    }
#undef EXHIP_CW_NHWC
    EXHIP_LAUNCH_CHECK();
    return 0;
}

static int channelwise_f32_launch(exhip_ctx* ctx, int op, const float* x, float* y, int n, int c, int hw, const float* p0,
                                  const float* p1, int shared);

extern "C" int exhip_channelwise_f32(exhip_ctx* ctx, int op, const float* x, float* y, int n, int c, int hw, const float* p0,
                                     const float* p1, int shared) {
    REQ_CTX("exhip_channelwise_f32");
    EXHIP_REQUIRE(x && y && p0 && n > 0 && c > 0 && hw > 0, "exhip_channelwise_f32: bad argument");
    EXHIP_REQUIRE(op == EXHIP_CHANNEL_PRELU || p1, "exhip_channelwise_f32: this op needs two parameter arrays");
    EXHIP_REQUIRE(c <= 65535, "exhip_channelwise_f32: more than 65535 channels");
    // one block row per (image, channel) plane, at most 65535 rows to a launch: whole images per launch
    const int per_launch = 65535 / c;
    for (int n0 = 0; n0 < n; n0 += per_launch) {
        const size_t off = (size_t)n0 * c * hw;
        const int rc = channelwise_f32_launch(ctx, op, x + off, y + off, std::min(per_launch, n - n0), c, hw, p0, p1, shared);
        if (rc) return rc;
    }
    return 0;
}

static int channelwise_f32_launch(exhip_ctx* ctx, int op, const float* x, float* y, int n, int c, int hw, const float* p0,
                                  const float* p1, int shared) {
    if (hw % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0) {
        unsigned bx4 = blocks_for((size_t)hw / 4);
        if (bx4 > 64) bx4 = 64;
        const dim3 grid4(bx4, (unsigned)(n * c));
        switch (op) {
        case EXHIP_CHANNEL_PRELU: hipLaunchKernelGGL((channelwise_f32_v4_kernel<0>), grid4, dim3(kBlock), 0, ctx->stream, x, y, c, hw / 4, p0, p1, shared); break;
        case EXHIP_CHANNEL_BATCHNORM: hipLaunchKernelGGL((channelwise_f32_v4_kernel<1>), grid4, dim3(kBlock), 0, ctx->stream, x, y, c, hw / 4, p0, p1, 0); break;
        case EXHIP_CHANNEL_INPUT: hipLaunchKernelGGL((channelwise_f32_v4_kernel<2>), grid4, dim3(kBlock), 0, ctx->stream, x, y, c, hw / 4, p0, p1, 0); break;
        default: exhip_set_error("exhip_channelwise_f32: unknown op %d", op); return EXHIP_ERR_ARG;
        }
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    unsigned bx = blocks_for((size_t)hw);
    if (bx > 64) bx = 64;
    const dim3 grid(bx, (unsigned)(n * c));
    switch (op) {
    case EXHIP_CHANNEL_PRELU: hipLaunchKernelGGL((channelwise_f32_kernel<0>), grid, dim3(kBlock), 0, ctx->stream, x, y, c, hw, p0, p1, shared); break;
    case EXHIP_CHANNEL_BATCHNORM: hipLaunchKernelGGL((channelwise_f32_kernel<1>), grid, dim3(kBlock), 0, ctx->stream, x, y, c, hw, p0, p1, 0); break;
    case EXHIP_CHANNEL_INPUT: hipLaunchKernelGGL((channelwise_f32_kernel<2>), grid, dim3(kBlock), 0, ctx->stream, x, y, c, hw, p0, p1, 0); break;
    default: exhip_set_error("exhip_channelwise_f32: unknown op %d", op); return EXHIP_ERR_ARG;
    }
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_concat_channels_f32(exhip_ctx* ctx, const float* const* inputs, const int* channels, int n_inputs, int n,
                                         int hw, float* y) {
    REQ_CTX("exhip_concat_channels_f32");
    EXHIP_REQUIRE(inputs && channels && y && n_inputs > 0 && n > 0 && hw > 0 && n <= 65535, "exhip_concat_channels_f32: bad argument");
    size_t total_c = 0;
    for (int i = 0; i < n_inputs; ++i) {
        EXHIP_REQUIRE(inputs[i] && channels[i] > 0, "exhip_concat_channels_f32: bad input %d", i);
        total_c += channels[i];
    }
    size_t off = 0;
    for (int i = 0; i < n_inputs; ++i) {
        const size_t block = (size_t)channels[i] * hw;
        if (block % 4 == 0 && off % 4 == 0 && (total_c * hw) % 4 == 0 && (uintptr_t)inputs[i] % 16 == 0 && (uintptr_t)y % 16 == 0) {
            unsigned bx4 = blocks_for(block / 4);
            if (bx4 > 1024) bx4 = 1024;
            hipLaunchKernelGGL(concat_block_v4_kernel, dim3(bx4, (unsigned)n), dim3(kBlock), 0, ctx->stream,
                               reinterpret_cast<const v4f*>(inputs[i]), reinterpret_cast<v4f*>(y), block / 4, total_c * hw / 4, off / 4);
            EXHIP_LAUNCH_CHECK();
            off += block;
            continue;
        }
        unsigned bx = blocks_for(block);
        if (bx > 1024) bx = 1024;
        hipLaunchKernelGGL(concat_block_kernel, dim3(bx, (unsigned)n), dim3(kBlock), 0, ctx->stream, inputs[i], y, block, total_c * hw, off);
        EXHIP_LAUNCH_CHECK();
        off += block;
    }
    return 0;
}

extern "C" int exhip_interp_nearest_f32(exhip_ctx* ctx, const float* x, float* y, int n, int c, int h, int w, int oh, int ow) {
    REQ_CTX("exhip_interp_nearest_f32");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && h > 0 && w > 0 && oh > 0 && ow > 0, "exhip_interp_nearest_f32: bad argument");
    if (ow % 4 == 0 && (uintptr_t)y % 16 == 0) {
        const size_t total4 = (size_t)n * c * oh * (ow / 4);
        hipLaunchKernelGGL(interp_nearest_x4_kernel, dim3(blocks_for(total4)), dim3(kBlock), 0, ctx->stream, x, y, h, w, oh, ow / 4,
                           h / (float)oh, w / (float)ow, total4);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    const size_t total = (size_t)n * c * oh * ow;
    hipLaunchKernelGGL(interp_nearest_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, h, w, oh, ow, h / (float)oh,
                       w / (float)ow, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_focus_f32(exhip_ctx* ctx, const float* x, float* y, int n, int c, int h, int w) {
    REQ_CTX("exhip_focus_f32");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && h > 1 && w > 1, "exhip_focus_f32: bad argument");
    if (w % 8 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0) {
        const size_t total8 = (size_t)n * c * (h / 2 * 2) * (w / 8);
        hipLaunchKernelGGL(focus_x8_kernel, dim3(blocks_for(total8)), dim3(kBlock), 0, ctx->stream, x, y, c, h, w, total8);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    const size_t total = (size_t)n * 4 * c * (h / 2) * (w / 2);
    hipLaunchKernelGGL(focus_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, c, h, w, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_input_focus_quantize_nchw_f32_to_nhwc_i8(exhip_ctx* ctx, const float* x, int n, int c, int h, int w, const float* means,
                                                              const float* scales, float fs, int c_stride, int8_t* y) {
    REQ_CTX("exhip_input_focus_quantize_nchw_f32_to_nhwc_i8");
    EXHIP_REQUIRE(x && y && means && scales && n > 0 && h > 1 && w > 1, "exhip_input_focus_quantize_nchw_f32_to_nhwc_i8: bad argument");
    if (c != 3 || c_stride != 32 || (h & 1) || (w & 1) || (reinterpret_cast<uintptr_t>(y) & 15) != 0) return EXHIP_ERR_UNSUPPORTED;
    FrontArgs a = {};
    for (int i = 0; i < c; ++i) { a.mean[i] = means[i]; a.scale[i] = scales[i]; }
    const size_t total = (size_t)n * (h / 2) * (w / 2);
    hipLaunchKernelGGL(input_focus_quantize_kernel<3>, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, h, w, a, fs, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_nhwc_f32_to_grouped_f32(exhip_ctx* ctx, const float* x, int n, int hw, int groups, int per_group, int c_stride, float* y) {
    REQ_CTX("exhip_nhwc_f32_to_grouped_f32");
    EXHIP_REQUIRE(x && y && n > 0 && hw > 0 && groups > 0 && per_group > 0 && c_stride >= groups * per_group,
                  "exhip_nhwc_f32_to_grouped_f32: bad argument");
    const long long per_plane = (long long)hw * per_group, planes = (long long)n * groups;
    EXHIP_REQUIRE(per_plane < (1ll << 31) && planes <= 65535, "exhip_nhwc_f32_to_grouped_f32: tensor too large");
    if (per_plane % 4 == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0)
        hipLaunchKernelGGL(nhwc_f32_to_grouped_x4_kernel, dim3((unsigned)((per_plane / 4 + kBlock - 1) / kBlock), (unsigned)planes), dim3(kBlock), 0,
                           ctx->stream, x, y, (unsigned)hw, (unsigned)groups, (unsigned)per_group, (unsigned)c_stride, (unsigned)(per_plane / 4));
    else
        hipLaunchKernelGGL(nhwc_f32_to_grouped_kernel, dim3((unsigned)((per_plane + kBlock - 1) / kBlock), (unsigned)planes), dim3(kBlock), 0,
                           ctx->stream, x, y, (unsigned)hw, (unsigned)groups, (unsigned)per_group, (unsigned)c_stride, (unsigned)per_plane);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

template <int OP, int MODE>
static int launch_binaryop(exhip_ctx* ctx, const float* big, const float* small, float* y, int n, int c, int hw, int small_n) {
    const bool vec = hw % 4 == 0 && (uintptr_t)big % 16 == 0 && (uintptr_t)y % 16 == 0;
    const size_t total = (size_t)n * c * (vec ? hw / 4 : hw);
    if (vec)
        hipLaunchKernelGGL((binaryop_f32_kernel<OP, MODE, 4>), dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, big, small, y, c,
                           hw, small_n, total);
    else
        hipLaunchKernelGGL((binaryop_f32_kernel<OP, MODE, 1>), dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, big, small, y, c,
                           hw, small_n, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}
template <int OP>
static int launch_binaryop_mode(exhip_ctx* ctx, int mode, const float* big, const float* small, float* y, int n, int c, int hw,
                                int small_n) {
    switch (mode) {
    case EXHIP_BINARY_EQUAL: return launch_binaryop<OP, 0>(ctx, big, small, y, n, c, hw, small_n);
    case EXHIP_BINARY_PER_IMAGE: return launch_binaryop<OP, 1>(ctx, big, small, y, n, c, hw, small_n);
    case EXHIP_BINARY_PER_CHANNEL: return launch_binaryop<OP, 2>(ctx, big, small, y, n, c, hw, small_n);
    case EXHIP_BINARY_PER_PIXEL: return launch_binaryop<OP, 3>(ctx, big, small, y, n, c, hw, small_n);
    default: exhip_set_error("exhip_binaryop_f32: unknown mode %d", mode); return EXHIP_ERR_ARG;
    }
}

extern "C" int exhip_binaryop_f32(exhip_ctx* ctx, int op, int mode, const float* large, const float* small, float* y, int n, int c,
                                  int hw, int small_n) {
    REQ_CTX("exhip_binaryop_f32");
    EXHIP_REQUIRE(large && small && y && n > 0 && c > 0 && hw > 0 && small_n > 0, "exhip_binaryop_f32: bad argument");
    EXHIP_REQUIRE(mode != EXHIP_BINARY_EQUAL || small_n == n, "exhip_binaryop_f32: equal shapes need equal batch sizes");
    switch (op) {
    case 0: return launch_binaryop_mode<0>(ctx, mode, large, small, y, n, c, hw, small_n);
    case 1: return launch_binaryop_mode<1>(ctx, mode, large, small, y, n, c, hw, small_n);
    case 2: return launch_binaryop_mode<2>(ctx, mode, large, small, y, n, c, hw, small_n);
    case 3: return launch_binaryop_mode<3>(ctx, mode, large, small, y, n, c, hw, small_n);
    default: exhip_set_error("exhip_binaryop_f32: unknown op %d (0 ADD, 1 SUB, 2 MUL, 3 DIV)", op); return EXHIP_ERR_ARG;
    }
}

extern "C" int exhip_softmax_channels_f32(exhip_ctx* ctx, const float* x, float* y, int n, int c, int hw) {
    REQ_CTX("exhip_softmax_channels_f32");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && hw > 0, "exhip_softmax_channels_f32: bad argument");
    const size_t total = (size_t)n * hw;
    if (c <= 32) hipLaunchKernelGGL(softmax_channels_reg_kernel<32>, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, c, hw, total);
    else hipLaunchKernelGGL(softmax_channels_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, c, hw, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_focus_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int n, int c, int h, int w) {
    REQ_CTX("exhip_focus_f16");
    EXHIP_REQUIRE(x && y && n > 0 && c > 0 && h > 1 && w > 1, "exhip_focus_f16: bad argument");
    if (w % 16 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0) {
        const size_t total16 = (size_t)n * c * (h / 2 * 2) * (w / 16);
        hipLaunchKernelGGL(focus_f16_x16_kernel, dim3(blocks_for(total16)), dim3(kBlock), 0, ctx->stream, x, y, c, h, w, total16);
        EXHIP_LAUNCH_CHECK();
        return 0;
    }
    const size_t total = (size_t)n * 4 * c * (h / 2) * (w / 2);
    hipLaunchKernelGGL(focus_f16_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, y, c, h, w, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_transpose_hw_f16(exhip_ctx* ctx, const uint16_t* x, uint16_t* y, int planes, int h, int w) {
    REQ_CTX("exhip_transpose_hw_f16");
    EXHIP_REQUIRE(x && y && planes > 0 && h > 0 && w > 0, "exhip_transpose_hw_f16: bad argument");
    EXHIP_REQUIRE(planes <= 65535 && (h + 31) / 32 <= 65535, "exhip_transpose_hw_f16: more than 65535 planes or row tiles");
    hipLaunchKernelGGL(transpose_hw_kernel<uint16_t>, dim3((w + 31) / 32, (h + 31) / 32, planes), dim3(kBlock), 0, ctx->stream, x, y, h, w);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_transpose_hw_f32(exhip_ctx* ctx, const float* x, float* y, int planes, int h, int w) {
    REQ_CTX("exhip_transpose_hw_f32");
    EXHIP_REQUIRE(x && y && planes > 0 && h > 0 && w > 0, "exhip_transpose_hw_f32: bad argument");
    EXHIP_REQUIRE(planes <= 65535 && (h + 31) / 32 <= 65535, "exhip_transpose_hw_f32: more than 65535 planes or row tiles");
    hipLaunchKernelGGL(transpose_hw_kernel<float>, dim3((w + 31) / 32, (h + 31) / 32, planes), dim3(kBlock), 0, ctx->stream, x, y, h, w);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

extern "C" int exhip_deconv2d_f32(exhip_ctx* ctx, const float* x, const float* w, const float* bias, float* y, int n, int c, int h,
                                  int wd, int k, int kh, int kw, int sh, int sw, int pt, int pb, int pl, int pr) {
    REQ_CTX("exhip_deconv2d_f32");
    EXHIP_REQUIRE(x && w && y && n > 0 && c > 0 && h > 0 && wd > 0 && k > 0 && kh > 0 && kw > 0 && sh > 0 && sw > 0,
                  "exhip_deconv2d_f32: bad argument");
    const int oh = (h - 1) * sh + kh - (pt + pb), ow = (wd - 1) * sw + kw - (pl + pr);
    EXHIP_REQUIRE(oh > 0 && ow > 0 && pt >= 0 && pl >= 0, "exhip_deconv2d_f32: empty output (%d x %d)", oh, ow);
    const size_t total = (size_t)n * k * oh * ow;
    hipLaunchKernelGGL(deconv2d_f32_kernel, dim3(blocks_for(total)), dim3(kBlock), 0, ctx->stream, x, w, bias, y, c, h, wd, k, kh, kw, sh,
                       sw, pt, pl, oh, ow, total);
    EXHIP_LAUNCH_CHECK();
    return 0;
}
