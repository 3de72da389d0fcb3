// The stem of an int8 network in one kernel: the input quantizer (float32 NCHW -> int8), the first convolution
// (<= 4 input channels, up to 8 taps per filter row, stride 2, 64-channel slabs) and the 3x3 stride-2 max pooling behind
// it, with float32 and / or requantized int8 NHWC results. Neither the quantized input nor the convolution's output
// reaches memory. References: src/Excalibur/operation_general_conv.cpp:584-720 (quantizer),
// src/Excalibur/operation_convolution.cpp:373-408 (int8 forward), src/Excalibur/operation_pooling.cpp:145-159 (MAX).
//
// A group of four waves is persistent and walks patches of MPH x MPW pooled pixels; a patch needs (2 MPH + 1) x (2 MPW + 1)
// convolution pixels, laid over a 16 x 16 grid of lanes (wave w holds grid rows 4 w .. 4 w + 3, a DPP row of 16 lanes is
// a grid row). Per patch:
//   * the float32 input tile of the NEXT patch is loaded into registers first, so it travels under this patch's work;
//   * the convolution is one MFMA k-step per filter row: a lane's B fragment is the 4 pixels x 4 channels starting at
//     its pixel's tap 0 or 4 (packed 4-byte pixels in LDS), the slab's whole filter stays in LDS for the group's life;
//   * pooling works on the int32 accumulators (the dequantization is monotone for scales >= 0, which the caller
//     asserts): the maximum over a window's three columns is taken between lanes (DPP row shifts), only the even columns
//     go to LDS, and the maximum over the three rows is taken from there by the threads that dequantize, requantize and
//     store the pooled pixels (16 consecutive threads per pixel: 256 / 64 contiguous bytes);
//   * the prefetched input is quantized into the other tile buffer.
#include <mutex>

#include "common.h"

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

namespace {

constexpr unsigned kRsrcWord3 = 0x00020000u;  // raw buffer: out-of-range loads return 0, stores are dropped
constexpr int kNP = 6;                        // tile pixels a thread stages: tiles of up to 1536 pixels
constexpr int kOob = 0x7FFFFF00;
constexpr unsigned kOobElem = 0x3FFFFF00u;
constexpr int kLowest = (int)0x80000000;
constexpr int kPoolPixB = 64 * 4 + 16;  // a pixel of the pooling buffer: 64 int32 channels and 16 bytes that spread neighbouring pixels over the banks

struct StemParams {
    const float* x;
    const char* wp;
    const float* scale;
    const float* bias;
    int8_t* y_q;
    float* y_f;
    int C, H, W, K, OH, OW, POH, POW;
    int PT, PL, ppt, ppl;
    int MPH, MPW, IH, IW;
    int tile_b, pool_b;
    int tiles_x, tiles_xy, n_ptiles, ktiles;
    unsigned magic_iw, magic_mpw, magic_tx, magic_txy;
    unsigned plane_bytes, out_elems;
    int adv_iy, adv_ix;  // 256 / IW, 256 % IW
    float fs_in, fs_out;
    int act, q_nonneg;
};

// n / d for n < 2^16 with magic = ceil(2^32 / d) as a 32-bit word: one multiply-high; d == 1 arrives as 0
__device__ __forceinline__ int fast_div(int n, unsigned magic) { return magic ? (int)__umulhi((unsigned)n, magic) : n; }

// the value the next lane of the same row of 16 lanes holds (DPP row_shl:1; 0 at the row's end)
__device__ __forceinline__ int right_neighbour(int v) { return __builtin_amdgcn_mov_dpp(v, 0x101, 0xF, 0xF, true); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t view(const void* base, unsigned range) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)range, kRsrcWord3);
}

template <int KH, int C>
__global__ __launch_bounds__(256, 3) void stem_conv_pool_kernel(const StemParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char* const lds_w = smem;                                   // [KH][2 channel tiles][64 lanes][16 B]
    char* const lds_tile = lds_w + KH * 2048;                   // two buffers of tile_b bytes: [IH][IW] 4-byte pixels
    char* const lds_pool = lds_tile + 2 * p.tile_b;             // [2 MPH + 1][MPW][64 channels] int32

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hh = lane >> 5, pc = lane & 15, pyw = (lane >> 4) & 1;
    // waits for this wave's LDS operations, then for the group. No memory fence: that would also wait for the next patch's
    // input, which is on its way to registers.
    auto barrier = [&]() { __asm__ volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    const int G = gridDim.x;
    int lb = blockIdx.x;
    if ((G & 7) == 0) lb = (lb & 7) * (G >> 3) + (lb >> 3);
    const int kt = __builtin_amdgcn_readfirstlane(lb % p.ktiles);
    const int pj = __builtin_amdgcn_readfirstlane(lb / p.ktiles);
    const int GP = G / p.ktiles;
    const int my_tiles = __builtin_amdgcn_readfirstlane((p.n_ptiles - pj + GP - 1) / GP);

    const int MPH = p.MPH, MPW = p.MPW, row_b = p.IW * 4;
    const int rows = 2 * MPH + 1, cols = 2 * MPW + 1;  // convolution pixels of a patch

    // ---- lane constants ----
    // The lane's two pixels (one per 32-pixel column block of the MFMA) are the even and the odd column 2 pc, 2 pc + 1 of
    // grid row 2 wave + pyw: a pooling window's three columns 2 j, 2 j + 1, 2 j + 2 are then this lane's two accumulator
    // tiles and the right neighbour's first.
    const int py = wave * 2 + pyw;
    int boff[2];
    {
        const int pyc = py < rows ? py : rows - 1;  // lanes past the patch compute a copy of its last row / column
#pragma unroll
        for (int nn = 0; nn < 2; ++nn) {
            const int px = 2 * pc + nn, pxc = px < cols ? px : cols - 1;
            boff[nn] = (2 * pyc) * row_b + (2 * pxc + 4 * hh) * 4;
        }
    }
    // staging: tile pixel v = tid + 256 i
    const int spare_off = p.IH * p.IW * 4;  // the 16 spare bytes behind a tile buffer's pixels
    int l_rel[kNP], l_yx[kNP], l_lds[kNP];
    {
        const int IW = p.IW, npix = p.IH * IW;
        int iy = fast_div(tid, p.magic_iw), ix = tid - iy * IW;
#pragma unroll
        for (int i = 0; i < kNP; ++i) {
            const bool ok = tid + 256 * i < npix;
            l_rel[i] = ok ? (iy * p.W + ix) * 4 : kOob;
            l_yx[i] = ok ? (iy | (ix << 16)) : -1;
            l_lds[i] = ok ? (iy * IW + ix) * 4 : spare_off;  // lanes past the tile write a spare word
            ix += p.adv_ix;
            iy += p.adv_iy;
            const int wrap = ix >= IW ? 1 : 0;
            ix -= wrap ? IW : 0;
            iy += wrap;
        }
    }
    // pooled outputs: item = (pooled pixel, four channels); a thread's items are tid + 256 k, all of the same four channels
    constexpr int kNI = 3;
    int it_src[kNI], it_rel[kNI], it_yx[kNI];
    {
        const int items = MPH * MPW * 16, g = tid & 15;
#pragma unroll
        for (int k = 0; k < kNI; ++k) {
            const int it = tid + 256 * k, q = it >> 4;
            const int i = fast_div(q, p.magic_mpw), j = q - i * MPW;
            const bool ok = it < items;
            it_src[k] = ok ? ((2 * i) * MPW + j) * kPoolPixB + g * 16 : -1;
            it_rel[k] = (i * p.POW + j) * p.K + g * 4;
            it_yx[k] = i | (j << 16);
        }
    }
    auto decode = [&](int t, int& n, int& ty, int& tx) {
        n = fast_div(t, p.magic_txy);
        const int r = t - n * p.tiles_xy;
        ty = fast_div(r, p.magic_tx);
        tx = r - ty * p.tiles_x;
    };

    // ---- input tile: float32 planes -> registers -> int8 pixels in LDS ----
    float xf[kNP][C];
    auto load_tile = [&](int n, int ty, int tx) {
        const int oy0 = 2 * ty * MPH - p.ppt, ox0 = 2 * tx * MPW - p.ppl;       // the patch's first convolution pixel
        const int iy0 = 2 * oy0 - p.PT, ix0 = 2 * ox0 - p.PL;                   // and the tile's first input pixel
        const bool interior = iy0 >= 0 && ix0 >= 0 && iy0 + p.IH <= p.H && ix0 + p.IW <= p.W;
        const int tile_base = (iy0 * p.W + ix0) * 4;
        int off[kNP];
#pragma unroll
        for (int i = 0; i < kNP; ++i) {
            if (interior) {
                off[i] = l_rel[i];
            } else {
                const int gy = iy0 + (l_yx[i] & 0xFFFF), gx = ix0 + (int)((unsigned)l_yx[i] >> 16);
                const bool in = ((unsigned)gy < (unsigned)p.H) & ((unsigned)gx < (unsigned)p.W);
                off[i] = in ? l_rel[i] + tile_base : kOob;
            }
        }
        const int vb = interior ? tile_base : 0;  // the part of the offset that is safe to put into the view's base
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const char* plane = reinterpret_cast<const char*>(p.x) + ((size_t)n * C + c) * p.plane_bytes + vb;
            const __amdgpu_buffer_rsrc_t r = view(plane, p.plane_bytes - (unsigned)vb);
#pragma unroll
            for (int i = 0; i < kNP; ++i) xf[i][c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off[i], 0, 0));
        }
    };
    auto quantize_tile = [&](char* dst) {
#pragma unroll
        for (int i = 0; i < kNP; ++i) {
            int pix = 0;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float t = xf[i][c] * p.fs_in;  // float32_to_int8: +-0.5, saturate, truncate
                const int q = (int)__builtin_amdgcn_fmed3f(t + __builtin_copysignf(0.5f, t), -128.f, 127.f);
                pix |= c == 3 ? (q << 24) : ((q & 0xff) << (8 * c));
            }
            *reinterpret_cast<int*>(dst + l_lds[i]) = pix;
        }
    };

    // ---- set-up: filter, scale and bias, first tile ----
    int n, ty, tx, pt = pj;
    decode(pt, n, ty, tx);
    load_tile(n, ty, tx);
    {
        const v4i* src = reinterpret_cast<const v4i*>(p.wp + (size_t)kt * (KH * 2048));
        for (int v = tid; v < KH * 128; v += 256) reinterpret_cast<v4i*>(lds_w)[v] = src[v];
    }
    v4f s4, b4;  // scale and bias of this thread's four output channels
    {
        const int ch = kt * 64 + (tid & 15) * 4;
        s4 = *reinterpret_cast<const v4f*>(p.scale + ch);
        b4 = p.bias ? *reinterpret_cast<const v4f*>(p.bias + ch) : v4f{0.f, 0.f, 0.f, 0.f};
    }
    quantize_tile(lds_tile);
    barrier();

    const __amdgpu_buffer_rsrc_t rq = view(p.y_q, p.out_elems);
    const __amdgpu_buffer_rsrc_t rf = view(p.y_f, p.out_elems * 4u);
    const bool has_f = p.y_f != nullptr, has_q = p.y_q != nullptr;
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    for (int done = 0; done < my_tiles; ++done) {
        const bool has_next = done + 1 < my_tiles;
        int n2 = n, ty2 = ty, tx2 = tx;
        if (has_next) {
            pt += GP;
            decode(pt, n2, ty2, tx2);
            load_tile(n2, ty2, tx2);
        }
        // ---- convolution: one k-step per filter row ----
        const char* const tile = lds_tile + (done & 1) * p.tile_b;
        v16i acc[2][2];
        v4i af[2][2], bf[2][2];
        auto fetch = [&](int buf, int r) {
#pragma unroll
            for (int m = 0; m < 2; ++m) af[buf][m] = *reinterpret_cast<const v4i*>(lds_w + (r * 2 + m) * 1024 + lane * 16);
            // the even column's four pixels start on a 16-byte boundary, the odd column's 8 bytes further
            bf[buf][0] = *reinterpret_cast<const v4i*>(tile + boff[0] + r * row_b);
            const char* a = tile + boff[1] + r * row_b;
            const v2i lo = *reinterpret_cast<const v2i*>(a), hi = *reinterpret_cast<const v2i*>(a + 8);
            bf[buf][1] = v4i{lo[0], lo[1], hi[0], hi[1]};
        };
        fetch(0, 0);
#pragma unroll
        for (int r = 0; r < KH; ++r) {
            if (r + 1 < KH) fetch((r + 1) & 1, r + 1);
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int nn = 0; nn < 2; ++nn)
                    acc[m][nn] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[r & 1][m], bf[r & 1][nn], r == 0 ? zero16 : acc[m][nn], 0, 0, 0);
        }
        // ---- pooling, columns: pixels outside the convolution's output drop out of every maximum ----
        const int oy0 = 2 * ty * MPH - p.ppt, ox0 = 2 * tx * MPW - p.ppl;
        const bool inside = oy0 >= 0 && ox0 >= 0 && oy0 + rows <= p.OH && ox0 + cols <= p.OW;
        if (!inside) {
            const bool yok = (unsigned)(oy0 + py) < (unsigned)p.OH;
#pragma unroll
            for (int nn = 0; nn < 2; ++nn) {
                const bool ok = yok & ((unsigned)(ox0 + 2 * pc + nn) < (unsigned)p.OW);
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[m][nn][e] = ok ? acc[m][nn][e] : kLowest;
            }
        }
        {
            // lanes outside the patch's pooled columns write a spare pixel behind the buffer (a branch per store costs more)
            const bool wr = pc < MPW && py < rows;
            char* const dst = lds_pool + (wr ? (py * MPW + pc) * kPoolPixB : rows * MPW * kPoolPixB) + hh * 64;
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    v4i h;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int even = acc[m][0][e4 * 4 + e], odd = acc[m][1][e4 * 4 + e];
                        const int next = right_neighbour(even);  // column 2 pc + 2 (anything at the row's end: not a writer)
                        const int t = even > odd ? even : odd;
                        h[e] = t > next ? t : next;
                    }
                    *reinterpret_cast<v4i*>(dst + (m * 32 + e4 * 4) * 4) = h;
                }
        }
        barrier();
        // ---- pooling, rows; dequantize, activate, requantize, store ----
        {
            const unsigned tile_elem = ((unsigned)(n * p.POH + ty * MPH) * (unsigned)p.POW + tx * MPW) * (unsigned)p.K + kt * 64;
            const int lim_y = p.POH - ty * MPH, lim_x = p.POW - tx * MPW;  // pooled pixels of the patch inside the image
#pragma unroll
            for (int k = 0; k < kNI; ++k) {
                if (it_src[k] < 0) continue;
                const char* src = lds_pool + it_src[k];
                v4i top = *reinterpret_cast<const v4i*>(src);
#pragma unroll
                for (int dr = 1; dr < 3; ++dr) {
                    const v4i t = *reinterpret_cast<const v4i*>(src + dr * MPW * kPoolPixB);
#pragma unroll
                    for (int e = 0; e < 4; ++e) top[e] = top[e] > t[e] ? top[e] : t[e];
                }
                v4f best;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = __builtin_fmaf((float)top[e], s4[e], b4[e]);
                    best[e] = p.act == 1 ? __builtin_fmaxf(v, 0.f) : v;
                }
                const bool ok = ((it_yx[k] & 0xFFFF) < lim_y) & ((int)((unsigned)it_yx[k] >> 16) < lim_x);
                const unsigned off = ok ? tile_elem + (unsigned)it_rel[k] : kOobElem;
                if (has_f) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, best), rf, (int)(off * 4u), 0, EXHIP_F32_STORE_AUX);
                if (has_q) {
                    int b[4], packed;
                    if (p.q_nonneg) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) b[e] = (int)__builtin_fminf(best[e] * p.fs_out + 0.5f, 127.f);
                        packed = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float t = best[e] * p.fs_out;
                            b[e] = (int)__builtin_amdgcn_fmed3f(t + __builtin_copysignf(0.5f, t), -128.f, 127.f);
                        }
                        packed = (b[0] & 0xff) | ((b[1] & 0xff) << 8) | ((b[2] & 0xff) << 16) | (b[3] << 24);
                    }
                    __builtin_amdgcn_raw_buffer_store_b32(packed, rq, (int)off, 0, 0);
                }
            }
        }
        if (has_next) quantize_tile(lds_tile + ((done + 1) & 1) * p.tile_b);
        n = n2; ty = ty2; tx = tx2;
        barrier();
    }
}

std::mutex g_attr_mutex;

template <int KH, int C>
int launch(exhip_ctx* ctx, const StemParams& p, int grid, int lds) {
    static unsigned long long attr_set = 0;
    auto kernel = stem_conv_pool_kernel<KH, C>;
    {
        std::lock_guard<std::mutex> lock(g_attr_mutex);
        const unsigned long long bit = 1ull << (ctx->device & 63);
        if (!(attr_set & bit)) {
            EXHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
            attr_set |= bit;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds, ctx->stream, p);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

}  // namespace

extern "C" int exhip_stem_f32_conv_i8_maxpool3x3s2(exhip_ctx* ctx, const exhip_conv_desc* d, int pool_pt, int pool_pl, int pool_oh,
                                                   int pool_ow, const float* x_nchw, float fs_in, const void* wp,
                                                   const float* scale, int scales_nonnegative, const float* bias, int8_t* y_i8,
                                                   float* y_f32_nhwc) {
    EXHIP_REQUIRE(ctx && d && x_nchw && wp && scale, "exhip_stem_f32_conv_i8_maxpool3x3s2: NULL argument");
    EXHIP_REQUIRE(y_i8 || y_f32_nhwc, "exhip_stem_f32_conv_i8_maxpool3x3s2: no output requested");
    if (!g_exhip_options.stem || !scales_nonnegative) return EXHIP_ERR_UNSUPPORTED;
    if (d->c < 3 || d->c > 4 || d->c_stride != 4 || d->kw > 8 || d->sh != 2 || d->sw != 2 || d->k % 64 != 0 || d->k_stride != d->k ||
        d->act > 1 || d->post_relu || d->post_op || d->post_bn_a || d->post_bn_b || d->exact_k || pool_pt < 0 || pool_pt > 1 || pool_pl < 0 || pool_pl > 1 ||
        !(d->kh == 7 || d->kh == 5 || d->kh == 3))
        return EXHIP_ERR_UNSUPPORTED;
    int oh = 0, ow = 0;
    int rc = exhip_conv_out_hw(d, &oh, &ow);
    if (rc) return rc;
    int tm = 0, packed = 0;
    rc = exhip_conv_packed_layout(d, EXHIP_I8, &tm, &packed);
    if (rc) return rc;
    if (tm != 64 || !packed) return EXHIP_ERR_UNSUPPORTED;  // the weights must be packed for 64-channel slabs of 4-byte pixels
    EXHIP_REQUIRE(pool_oh > 0 && pool_ow > 0 && 2 * (pool_oh - 1) - pool_pt < oh && 2 * (pool_ow - 1) - pool_pl < ow,
                  "stem: pooled size %dx%d does not fit a %dx%d convolution output", pool_oh, pool_ow, oh, ow);
    StemParams p = {};
    p.x = x_nchw; p.wp = (const char*)wp; p.scale = scale; p.bias = bias; p.y_q = y_i8; p.y_f = y_f32_nhwc;
    p.C = d->c; p.H = d->h; p.W = d->w; p.K = d->k; p.OH = oh; p.OW = ow; p.POH = pool_oh; p.POW = pool_ow;
    p.PT = d->pt; p.PL = d->pl; p.ppt = pool_pt; p.ppl = pool_pl;
    // a patch is at most 7 x 31 convolution pixels (the 8 x 32 lane grid less one row and column): 3 x 15 pooled pixels
    p.MPH = pool_oh < 3 ? pool_oh : 3;
    p.MPW = pool_ow < 15 ? pool_ow : 15;
    p.IH = (2 * p.MPH) * 2 + d->kh;   // rows 0 .. 2 MPH of the patch, KH filter rows each
    p.IW = (2 * p.MPW) * 2 + 8;       // columns 0 .. 2 MPW, eight taps each (taps past KW meet zero weights)
    if (p.IH * p.IW > kNP * 256) return EXHIP_ERR_UNSUPPORTED;
    p.tile_b = (p.IH * p.IW * 4 + 16 + 15) / 16 * 16;  // a fragment read may run 8 bytes past the last pixel it needs
    p.pool_b = ((2 * p.MPH + 1) * p.MPW + 1) * kPoolPixB;  // and one spare pixel
    p.tiles_x = (pool_ow + p.MPW - 1) / p.MPW;
    const int tiles_y = (pool_oh + p.MPH - 1) / p.MPH;
    p.tiles_xy = p.tiles_x * tiles_y;
    p.ktiles = d->k / 64;
    const long long n_ptiles = (long long)d->n * p.tiles_xy;
    const long long out_elems = (long long)d->n * pool_oh * pool_ow * d->k;
    if (n_ptiles >= 65536 || d->h >= 0x4000 || d->w >= 0x4000 || out_elems * 4 >= 0xFFFFF000ll || out_elems >= (long long)kOobElem ||
        (long long)d->h * d->w * 4 >= 0x7FFFFF00ll)
        return EXHIP_ERR_UNSUPPORTED;
    p.n_ptiles = (int)n_ptiles;
    auto magic = [](int v) { return (unsigned)(((1ull << 32) + v - 1) / v); };
    p.magic_iw = magic(p.IW); p.magic_mpw = magic(p.MPW); p.magic_tx = magic(p.tiles_x); p.magic_txy = magic(p.tiles_xy);
    p.plane_bytes = (unsigned)((size_t)d->h * d->w * 4);
    p.out_elems = (unsigned)out_elems;
    p.adv_iy = 256 / p.IW; p.adv_ix = 256 % p.IW;
    p.fs_in = fs_in; p.fs_out = d->fs_out;
    p.act = d->act; p.q_nonneg = d->fs_out > 0.f && d->act == 1;
    const int lds = d->kh * 2048 + 2 * p.tile_b + p.pool_b;  // 53536 bytes for a 7x7 filter: three groups per CU
    const long long total = n_ptiles * p.ktiles;
    long long G = total;
    if (total > 3 * 256) {
        const long long unit = 8ll * p.ktiles;
        G = 3 * 256 / unit * unit;
        if (G <= 0) G = p.ktiles;
    }
    if (g_exhip_options.lean_groups > 0 && G > (long long)g_exhip_options.lean_groups * p.ktiles) G = (long long)g_exhip_options.lean_groups * p.ktiles;
    if (g_exhip_options.debug_plan)
        fprintf(stderr, "stem %dx%dx%dx%d k%d %dx%d: pooled patch %dx%d, tile %dx%d, %lld groups for %lld patches, lds %d\n", d->n, d->c, d->h, d->w,
                d->k, d->kh, d->kw, p.MPH, p.MPW, p.IH, p.IW, G, total, lds);
    const bool c3 = d->c == 3;  // fewer channels run as four with zero planes' worth of weights: the loader reads c planes
    if (d->c != 3 && d->c != 4) return EXHIP_ERR_UNSUPPORTED;
    if (d->kh == 7) return c3 ? launch<7, 3>(ctx, p, (int)G, lds) : launch<7, 4>(ctx, p, (int)G, lds);
    if (d->kh == 5) return c3 ? launch<5, 3>(ctx, p, (int)G, lds) : launch<5, 4>(ctx, p, (int)G, lds);
    return c3 ? launch<3, 3>(ctx, p, (int)G, lds) : launch<3, 4>(ctx, p, (int)G, lds);
}
