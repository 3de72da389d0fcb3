// 3x3 stride-1 int8 convolution with the fused epilogue (dequantize, ReLU, float32 shortcut, float32 / int8 NHWC and
// float32 NCHW results): the layers that carry most of a ResNet-shaped int8 stack. Same implicit GEMM as
// conv_igemm.hip -- rows = 64 output channels, columns = a patch of up to 256 output pixels, v_mfma_i32_32x32x32_i8,
// every wave a 64 x 64 accumulator tile, operands from global memory straight into LDS -- but with everything the
// general kernel decides at run time fixed at compile time, so that a wave issues little besides its MFMAs:
//
//  * a group is persistent: it walks several patches of one 64-channel slab. Lane constants (fragment offsets, the
//    gather offsets of the staging loads relative to a patch's origin, output offsets) are computed once; per patch only
//    the border tests remain, and those only for patches that touch the image's border.
//  * the weight slices and the activation tiles of a group's whole run form one pipeline: what the next patch needs is
//    requested while the current one computes, so a patch boundary costs no refill.
//  * every wave issues the same, fixed number of staging loads per stage (a request without data gets a zero-length
//    buffer view), which makes every s_waitcnt an immediate.
//  * with 64 input channels the slab's whole filter (36 KiB) stays in LDS for the life of the group and a patch needs two
//    barriers in all.
//  * the epilogue works from registers: a lane holds 16 consecutive channels of a pixel per accumulator tile, and one
//    v_permlane32_swap per register pair turns the two half-waves' 64-byte runs into 32-byte pieces that two lanes
//    read or write side by side, so float32 tensors move as whole 32-byte sectors without an exchange through LDS.
//
// Arithmetic and rounding are the general kernel's (and so the reference's, src/Excalibur/operation_convolution.cpp:373-408,
// src/Primitives/simd_types.cpp:140-152): results are bit for bit the same.
#include <mutex>

#include "conv_i8_lean.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

namespace {

constexpr int kThreads = 256;
constexpr int kNAL = 7;                   // staging loads per thread for one activation tile (7 x 4 KiB)
constexpr int kActStride = 27 * 1024;     // LDS bytes of an activation tile buffer; the 28th KiB a request writes is a spare one
constexpr int kPixB = 80;                 // a staged pixel: a 64-byte channel chunk and 16 bytes that keep fragment reads off the same banks
constexpr int kWSlice = 3 * 2 * 2 * 1024; // weights of one filter row of one chunk: 3 taps x 2 k-steps x 2 channel tiles x 1 KiB
constexpr int kSbB = 512;                 // scale and bias of the slab's 64 channels
constexpr int kSpareB = 1024;
constexpr unsigned kRsrcWord3 = 0x00020000u;  // raw buffer: out-of-range loads return 0, stores are dropped
constexpr int kOob = 0x7FFFFF00;              // a byte offset past any tensor
constexpr unsigned kOobElem = 0x3FFFFF00u;    // an element offset whose byte offsets (x1, x4, + 255) lie past any accepted tensor

#ifndef EXHIP_STAMPS
#define EXHIP_STAMPS 0
#endif
constexpr bool kStamps = EXHIP_STAMPS != 0;
long long* g_lean_dbg = nullptr;

// E_HALF: the fp16 layer -- half operands (v_mfma_f32_32x32x16_f16 on the same bytes: a 64-byte chunk is 32 channels),
// float accumulators, the general kernel's fp16 epilogue with a half NHWC result (its switches are read from the
// parameters: E_RES / E_ACT / E_POST and post_op, residual_last).
enum { E_RES = 1, E_F = 2, E_Q = 4, E_NCHW = 8, E_ACT = 16, E_POST = 32, E_QNN = 64, E_HALF = 128 };

struct LeanParams {
    const char* x;
    const char* wp;
    const float* scale;
    const float* bias;
    const float* residual;
    int8_t* y_q;
    float* y_f;
    float* y_nchw;
    int H, W, K, OH, OW, PT, PL;
    int C_b, n_chunks;
    int PH, PW, IH, IW;
    int tiles_x, tiles_xy, ktiles, n_ptiles;
    unsigned img_bytes, out_elems;
    unsigned magic_iw, magic_pw, magic_tx, magic_txy;
    int adv_iy, adv_ix;  // (256 / 5) / IW, (256 / 5) % IW: how a thread's tile pixel advances from one staging load to the next
    float fs_out;
    int flags;
    // projection shortcut (kernels instantiated with PROJ): a 1x1 convolution of ds_x accumulated beside the 3x3 products
    const char* ds_x;
    const char* ds_wp;
    const float* ds_scale;
    const float* ds_bias;
    int ds_H, ds_W, ds_Cb, ds_chunks, ds_stride;
    unsigned ds_img_bytes;
    // fp16 layers (E_HALF): the activation layer behind the convolution and where the shortcut is added
    int post_op, residual_last;
    float post_alpha, post_beta;
    int stagger;     // persistent launches: a group whose waves sit in hardware wave slot s starts s * stagger * 64 cycles late
    long long* dbg;  // phase timestamps (builds with -DEXHIP_STAMPS=1 only)
};

// n / d for n < 2^16 with magic = ceil(2^32 / d) as a 32-bit word: one multiply-high; d == 1 arrives as 0
__device__ __forceinline__ int fast_div(int n, unsigned magic) { return magic ? (int)__umulhi((unsigned)n, magic) : n; }
__device__ __forceinline__ v4i lds_read16(const char* p) { return *reinterpret_cast<const v4i*>(p); }

// One 16-byte element per lane from a bounds-checked buffer view straight into LDS: lane l's data lands at
// lds_base + 16 * l (lds_base wave-uniform, in M0). Completion is counted by vmcnt like any other load.
__device__ __forceinline__ void async_load16(__amdgpu_buffer_rsrc_t rsrc, int voff, int soff, unsigned lds_base) {
    __asm__ volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(voff),
                     "s"(rsrc), "s"(__builtin_amdgcn_readfirstlane(soff))
                     : "m0");
}
// A buffer view whose base and range are pinned to scalar registers (the staging loads are inline assembly: the compiler
// cannot wrap them in the loop it would put around a view it keeps in vector registers).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t uniform_view(const char* base, int range) {
    const unsigned long long a = (unsigned long long)(uintptr_t)base;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char*>((uintptr_t)(((unsigned long long)hi << 32) | lo)), 0,
                                             __builtin_amdgcn_readfirstlane(range), kRsrcWord3);
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() { __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// WRES: the slab's whole filter is resident (one 64-byte chunk); otherwise weight slices rotate through NWB buffers and
// activation tiles through NAB. EPI >= 0: the epilogue's switches as compile-time constants; EPI < 0: read from p.flags.
// PROJ: the shortcut is a 1x1 convolution computed here (p.ds_*): its channel chunks follow the 3x3 layer's in every patch's
// run as stages of one tap, into accumulators of their own.
template <bool WRES, int NAB, int NWB, int EPI, bool PROJ = false>
__global__ __launch_bounds__(kThreads, (WRES || NAB == 2 || NWB == 3 || PROJ) ? 2 : 3) void conv3x3_i8_lean_kernel(const LeanParams p) {
    static_assert(!(PROJ && WRES), "the projection's chunks run in the streamed form");
    constexpr int NWS = WRES ? 3 : NWB;
    constexpr int A0 = NWS * kWSlice;
    constexpr int SB0 = A0 + NAB * kActStride;
    constexpr int SPARE0 = SB0 + (PROJ ? 2 * kSbB : kSbB);
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    float* const lds_sb = reinterpret_cast<float*>(smem + SB0);

    constexpr bool F16 = EPI >= 0 && (EPI & E_HALF) != 0;
    static_assert(!(F16 && PROJ), "the projection form is int8");
    using acc_t = std::conditional_t<F16, v16f, v16i>;
    const int flags = F16 ? p.flags : (EPI >= 0 ? EPI : p.flags);
    const bool has_res = flags & E_RES, has_f = flags & E_F, has_q = flags & E_Q, has_nchw = flags & E_NCHW;
    const bool act_relu = flags & E_ACT, post_relu = flags & E_POST, q_nonneg = flags & E_QNN;
    const bool q_only = q_nonneg && has_q && !has_res && !has_f && !has_nchw;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hh = lane >> 5;
    long long t_mfma = 0, t_wait = 0, t_bar = 0, t_epi = 0, t_gap = 0, t_mark = 0;
    auto now = [&]() -> long long { return kStamps && p.dbg ? (long long)clock64() : 0ll; };
    auto put = [&](int k, long long v) {
        if constexpr (kStamps)
            if (p.dbg && lane == 0) p.dbg[((size_t)blockIdx.x * 4 + wave) * 64 + k] = v;
    };
    put(0, now());
    if constexpr (kStamps) {
        put(16, __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | ((32 - 1) << 11)));   // HW_REG_HW_ID
        put(17, __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | ((32 - 1) << 11)));  // HW_REG_XCC_ID
    }
    int n_epi = 0;
    if (p.stagger > 0) {
        // Groups that share a CU start together and would reach their MFMA runs, waits and epilogues together, the matrix
        // pipes idle in between. The hardware wave slot (HW_ID bits 3:0) counts the waves a SIMD already holds: delaying a
        // group by its slot spreads the phases of a CU's groups over a patch's period.
        const int slot = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | ((4 - 1) << 11));  // HW_REG_HW_ID, offset 0, width 4
        for (int i = 0; i < slot * p.stagger; ++i) __builtin_amdgcn_s_sleep(1);
    }
    if constexpr (kStamps) put(10, (long long)wall_clock64());

    // ---- which patches this group walks: groups of one XCD (ids are dealt round-robin to the 8 XCDs) take neighbouring
    // patches, so that halos and the slabs of one patch meet in that XCD's L2 ----
    const int G = gridDim.x;
    int lb = blockIdx.x;
    if ((G & 7) == 0) lb = (lb & 7) * (G >> 3) + (lb >> 3);
    const int kt = __builtin_amdgcn_readfirstlane(lb % p.ktiles);
    const int pj = __builtin_amdgcn_readfirstlane(lb / p.ktiles);
    const int GP = G / p.ktiles;
    const int my_tiles = __builtin_amdgcn_readfirstlane((p.n_ptiles - pj + GP - 1) / GP);

    // ---- staging requests of weight slices ----
    const unsigned wave_slot = (unsigned)wave * 1024u;
    const int w_voff = tid * 16;
    const char* const wkt = p.wp + (size_t)kt * p.n_chunks * (3 * kWSlice);  // this slab's slices, in (chunk, filter row) order
    const int w_run_b = p.n_chunks * 3 * kWSlice;
    const int n_tot = p.n_chunks + (PROJ ? p.ds_chunks : 0);   // chunks of a patch's run: the 3x3 layer's, then the projection's
    int w_off = 0;                                  // next slice to request
    int w_left = my_tiles * n_tot * 3;              // slices of the whole run not requested yet
    // PROJ: behind the 3x3 layer's slices a patch's run takes three per projection chunk, to keep every stage's requests
    // alike: the chunk's one tap (4 KiB of the 1x1 layer's packed weights, slab kt) and two empty ones
    const char* const wkt_ds = PROJ ? p.ds_wp + (size_t)kt * p.ds_chunks * 4096 : nullptr;
    int w_ds = -1;                                  // >= 0: the next slice is number w_ds of the projection's
    auto request_w = [&](unsigned dst) {
        const char* src = wkt + w_off;
        int range = kWSlice;
        if constexpr (PROJ) {
            if (w_ds >= 0) {
                const int dc = w_ds / 3;
                src = wkt_ds + dc * 4096;
                range = w_ds == dc * 3 ? 4096 : 0;
            }
        }
        const __amdgpu_buffer_rsrc_t wr = uniform_view(src, w_left > 0 ? range : 0);
#pragma unroll
        for (int i = 0; i < 3; ++i) async_load16(wr, w_voff, i * 4096, dst + wave_slot + i * 4096);
        --w_left;
        if constexpr (PROJ) {
            if (w_ds >= 0) {
                if (++w_ds == p.ds_chunks * 3) w_ds = -1;
                return;
            }
        }
        w_off += kWSlice;
        if (w_off == w_run_b) {
            w_off = 0;
            if constexpr (PROJ) w_ds = 0;
        }
    };
    // the first slices go out before anything else: their latency covers the set-up below
    if constexpr (WRES) {
        for (int r = 0; r < 3; ++r) request_w(lds0 + r * kWSlice);
    } else {
        request_w(lds0);
    }

    // ---- lane constants ----
    // staging: slot v = tid + 256 * i of a tile is 16 bytes of pixel v / 5, part v % 5 (part 4 is the padding)
    int a_rel[kNAL], a_yx[kNAL], a_off[kNAL];
    {
        const int IW = p.IW, npix = p.IH * IW, W = p.W, cb = p.C_b;
        int pix = fast_div(tid, 0x33333334u), part = tid - pix * 5;
        int iy = fast_div(pix, p.magic_iw), ix = pix - iy * IW;
#pragma unroll
        for (int i = 0; i < kNAL; ++i) {
            const bool ok = (pix < npix) & (part < 4);
            a_rel[i] = ok ? (iy * W + ix) * cb + part * 16 : kOob;
            a_yx[i] = ok ? (iy | (ix << 16)) : -1;
            part += 1;
            const int carry = part >= 5 ? 1 : 0;
            part -= carry ? 5 : 0;
            pix += 51 + carry;
            ix += p.adv_ix + carry;
            iy += p.adv_iy;
            const int wrap = ix >= IW ? 1 : 0;
            ix -= wrap ? IW : 0;
            iy += wrap;
        }
    }
    // the lane's two pixels (one per 32-pixel column block of its wave): fragment offset in a tile, position in the patch
    // (its position in the output is worked out again in every epilogue: a dozen instructions instead of six registers
    // held through the MFMA stages)
    int boff[2];
    auto patch_pixel = [&](int nn, int& py, int& px) -> bool {
        int pp = (wave * 2 + nn) * 32 + (lane & 31);
        const bool ok = pp < p.PH * p.PW;
        pp = ok ? pp : 0;
        py = fast_div(pp, p.magic_pw);
        px = pp - py * p.PW;
        return ok;
    };
#pragma unroll
    for (int nn = 0; nn < 2; ++nn) {
        int py, px;
        patch_pixel(nn, py, px);
        boff[nn] = py * (p.IW * kPixB) + px * kPixB + hh * 16;
    }
    const int row_b = p.IW * kPixB;
    const int img_px = p.OH * p.OW;

    acc_t acc[2][2];
    acc_t acc_ds[2][2];  // PROJ: the projection's products
    auto clear_acc = [&]() {
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int nn = 0; nn < 2; ++nn)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[m][nn][e] = 0;
                    if constexpr (PROJ) acc_ds[m][nn][e] = 0;
                }
    };

    // ---- patch bookkeeping (all wave-uniform) ----
    auto decode = [&](int t, int& n, int& oy0, int& ox0) {
        n = fast_div(t, p.magic_txy);
        const int r = t - n * p.tiles_xy;
        const int ty = fast_div(r, p.magic_tx), tx = r - ty * p.tiles_x;
        oy0 = ty * p.PH;
        ox0 = tx * p.PW;
    };
    // gather offsets of a patch's staging loads; returns what goes into the buffer view's base instead
    const int part0 = tid - fast_div(tid, 0x33333334u) * 5;   // the 16-byte part of a pixel this thread's first slot holds
    auto part_of = [&](int i) {
        int part = part0 + i;
        part -= part >= 5 ? 5 : 0;
        part -= part >= 5 ? 5 : 0;
        return part;
    };
    auto set_offsets = [&](int oy0, int ox0) -> int {
        const int iy0 = oy0 - p.PT, ix0 = ox0 - p.PL;
        if constexpr (PROJ) {
            // two accumulator sets leave no registers for the patch-relative offsets: made from the pixel positions
#pragma unroll
            for (int i = 0; i < kNAL; ++i) {
                const int gy = iy0 + (a_yx[i] & 0xFFFF), gx = ix0 + (int)((unsigned)a_yx[i] >> 16);
                const bool in = ((unsigned)gy < (unsigned)p.H) & ((unsigned)gx < (unsigned)p.W);
                a_off[i] = in ? (gy * p.W + gx) * p.C_b + part_of(i) * 16 : kOob;
            }
            return 0;
        }
        const int tile_base = (iy0 * p.W + ix0) * p.C_b;
        const bool interior = iy0 >= 0 && ix0 >= 0 && iy0 + p.IH <= p.H && ix0 + p.IW <= p.W;
        if (interior) {
#pragma unroll
            for (int i = 0; i < kNAL; ++i) a_off[i] = a_rel[i];
            return tile_base;
        }
#pragma unroll
        for (int i = 0; i < kNAL; ++i) {
            const int gy = iy0 + (a_yx[i] & 0xFFFF), gx = ix0 + (int)((unsigned)a_yx[i] >> 16);
            const bool in = ((unsigned)gy < (unsigned)p.H) & ((unsigned)gx < (unsigned)p.W);
            a_off[i] = in ? a_rel[i] + tile_base : kOob;
        }
        return 0;
    };

    // ---- staging requests of tiles (the weight requests stand above the lane constants) ----
    auto request_a = [&](const char* img, int base, int cc, bool valid, unsigned dst) {
        const int off = base + cc * 64;
        const __amdgpu_buffer_rsrc_t xr = uniform_view(img + off, valid ? (int)p.img_bytes - off : 0);
#pragma unroll
        for (int i = 0; i < kNAL; ++i) {
            unsigned d = dst + wave_slot + i * 4096;
            if (i == kNAL - 1) d = wave == 3 ? lds0 + SPARE0 : d;  // the KiB past the buffer
            async_load16(xr, a_off[i], 0, d);
        }
    };
    // PROJ: chunk dc of the projection's input under the patch at (oy0, ox0) of image n, in the 3x3 layer's tile geometry
    // (tile pixel (y, x) is the pixel under output (oy0 - PT + y, ox0 - PL + x)): the tap reads where the 3x3 layer's
    // centre tap does
    auto request_ds = [&](int n, int oy0, int ox0, int dc, unsigned dst) {
        const int off0 = dc * 64;
        const __amdgpu_buffer_rsrc_t xr = uniform_view(p.ds_x + (size_t)n * p.ds_img_bytes + off0, (int)p.ds_img_bytes - off0);
        const int y0 = (oy0 - p.PT) * p.ds_stride, x0 = (ox0 - p.PL) * p.ds_stride;
#pragma unroll
        for (int i = 0; i < kNAL; ++i) {
            unsigned d = dst + wave_slot + i * 4096;
            if (i == kNAL - 1) d = wave == 3 ? lds0 + SPARE0 : d;
            const int part = part_of(i);
            const int gy = y0 + (a_yx[i] & 0xFFFF) * p.ds_stride, gx = x0 + (int)((unsigned)a_yx[i] >> 16) * p.ds_stride;
            const bool in = (a_yx[i] >= 0) & ((unsigned)gy < (unsigned)p.ds_H) & ((unsigned)gx < (unsigned)p.ds_W);
            async_load16(xr, in ? (gy * p.ds_W + gx) * p.ds_Cb + part * 16 : kOob, 0, d);
        }
    };

    // ---- MFMAs of filter rows: k-steps in (tap, channel half) order, fragments fetched one step ahead ----
    v4i af[2][2], bf[2][2];
    auto compute = [&](int buf) {
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int nn = 0; nn < 2; ++nn) {
                if constexpr (F16)
                    acc[m][nn] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, af[buf][m]), __builtin_bit_cast(v8h, bf[buf][nn]),
                                                                        acc[m][nn], 0, 0, 0);
                else
                    acc[m][nn] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[buf][m], bf[buf][nn], acc[m][nn], 0, 0, 0);
            }
    };
    auto fetch = [&](int buf, const char* wrow, const char* a0, const char* a1, int s) {
        af[buf][0] = lds_read16(wrow + s * 2048);
        af[buf][1] = lds_read16(wrow + s * 2048 + 1024);
        bf[buf][0] = lds_read16(a0 + (s >> 1) * kPixB + (s & 1) * 32);
        bf[buf][1] = lds_read16(a1 + (s >> 1) * kPixB + (s & 1) * 32);
    };
    // NR filter rows whose weights lie kWSlice apart from wrow on and whose tile rows lie row_b apart from a0 / a1 on;
    // `requests` runs once, behind the first k-step's MFMAs
    auto mfma_rows = [&](auto nr_t, const char* wrow, const char* a0, const char* a1, auto&& requests) {
        constexpr int NR = decltype(nr_t)::value;
        fetch(0, wrow, a0, a1, 0);
#pragma unroll
        for (int r = 0; r < NR; ++r) {
#pragma unroll
            for (int s = 0; s < 6; ++s) {
                const int k = r * 6 + s;
                if (s + 1 < 6) fetch((k + 1) & 1, wrow + r * kWSlice, a0 + r * row_b, a1 + r * row_b, s + 1);
                else if (r + 1 < NR) fetch((k + 1) & 1, wrow + (r + 1) * kWSlice, a0 + (r + 1) * row_b, a1 + (r + 1) * row_b, 0);
                // keep this order: the next k-step's fragment reads go out before this k-step's MFMAs
                __builtin_amdgcn_sched_barrier(0);
                compute(k & 1);
                __builtin_amdgcn_sched_barrier(0);
                if (k == 0) requests();
            }
        }
    };
    // PROJ: a projection chunk's two k-steps, on the pixels the 3x3 layer's centre tap reads
    auto mfma_ds = [&](const char* wrow, const char* a0c, const char* a1c) {
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            af[s][0] = lds_read16(wrow + s * 2048);
            af[s][1] = lds_read16(wrow + s * 2048 + 1024);
            bf[s][0] = lds_read16(a0c + s * 32);
            bf[s][1] = lds_read16(a1c + s * 32);
        }
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int nn = 0; nn < 2; ++nn)
                    if constexpr (!F16) acc_ds[m][nn] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[s][m], bf[s][nn], acc_ds[m][nn], 0, 0, 0);
    };
    constexpr std::integral_constant<int, 1> one_row{};
    constexpr std::integral_constant<int, 3> three_rows{};

    // ---- epilogue of one patch, from registers ----
    const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(p.y_q, 0, (int)p.out_elems, kRsrcWord3);
    const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc(p.y_f, 0, (int)(p.out_elems * 4u), kRsrcWord3);
    const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.residual), 0, (int)(p.out_elems * 4u), kRsrcWord3);
    const __amdgpu_buffer_rsrc_t rn = __builtin_amdgcn_make_buffer_rsrc(p.y_nchw, 0, (int)(p.out_elems * 4u), kRsrcWord3);
    // 32-byte pieces of a pixel's 32 channels in the order the register pairs hold them after the half-wave swap
    auto piece = [](int j) { return j == 0 ? 0 : j == 1 ? 64 : j == 2 ? 32 : 96; };
    auto epilogue = [&](int n, int oy0, int ox0) {
        const bool full = oy0 + p.PH <= p.OH && ox0 + p.PW <= p.OW;
        const unsigned obase = ((unsigned)n * (unsigned)img_px + (unsigned)(oy0 * p.OW + ox0)) * (unsigned)p.K + (unsigned)(kt * 64);
        if constexpr (F16) {
            // The general kernel's fp16 epilogue (conv_igemm.hip) on 16 consecutive channels of a pixel per block: bias,
            // ReLU, the shortcut added to the value rounded to half (in front of or behind the activation layer), the
            // activation layer on the rounded half, one rounding; 64-byte runs from lanes (p, p + 1) of both half-waves.
            // Every wave issues the same eight stores and, with a shortcut, eight loads, whatever its pixels: what lies
            // outside the image goes to an offset the buffer view drops.
            const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(p.y_q, 0, (int)(p.out_elems * 2u), kRsrcWord3);
            const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.residual), 0, (int)(p.out_elems * 2u), kRsrcWord3);
            const bool odd = lane & 1;
#pragma unroll
            for (int nn = 0; nn < 2; ++nn) {
                int py, px;
                const bool in_patch = patch_pixel(nn, py, px);
                const bool valid = in_patch & (full | ((oy0 + py < p.OH) & (ox0 + px < p.OW)));
                const unsigned mine = valid ? (obase + (unsigned)((py * p.OW + px) * p.K)) * 2u : (unsigned)kOob;
                const unsigned other = (unsigned)lane_neighbour((int)mine);
                const unsigned even_b = odd ? other : mine, odd_b = odd ? mine : other;
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    const int cb = (m * 32 + hh * 16) * 2;  // byte offset of the lane's 16 channels in the pixel's slab
                    v4i r0 = {0, 0, 0, 0}, r1 = {0, 0, 0, 0};
                    if (has_res) {
                        r0 = __builtin_amdgcn_raw_buffer_load_b128(rh, (int)mine + cb, 0, 0);
                        r1 = __builtin_amdgcn_raw_buffer_load_b128(rh, (int)mine + cb + 16, 0, 0);
                    }
                    float v[16];
#pragma unroll
                    for (int e = 0; e < 16; ++e) v[e] = acc[m][nn][e] + lds_sb[64 + m * 32 + hh * 16 + e];
                    if (act_relu) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) v[e] = (0.f > v[e]) ? 0.f : v[e];
                    }
                    auto add_shortcut = [&]() {
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const int word = e < 8 ? r0[e >> 1] : r1[(e - 8) >> 1];
                            v[e] = exhip_h2f(exhip_f2h(v[e])) + exhip_h2f((uint16_t)(((uint32_t)word >> ((e & 1) * 16)) & 0xffff));
                        }
                    };
                    if (has_res && !p.residual_last) add_shortcut();
                    if (post_relu) {
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            v[e] = exhip_h2f(exhip_f2h(v[e]));
                            v[e] = (0.f > v[e]) ? 0.f : v[e];
                        }
                    }
                    if (p.post_op) {
                        const float al = p.post_alpha, be = p.post_beta;
                        switch (p.post_op - 1) {
                        case EXHIP_UNARY_HARDSWISH:
#pragma unroll
                            for (int e = 0; e < 16; ++e) v[e] = unary_value<0>(exhip_h2f(exhip_f2h(v[e])), al, be);
                            break;
                        case EXHIP_UNARY_LEAKYRELU:
#pragma unroll
                            for (int e = 0; e < 16; ++e) v[e] = unary_value<1>(exhip_h2f(exhip_f2h(v[e])), al, be);
                            break;
                        case EXHIP_UNARY_HARDSIGMOID:
#pragma unroll
                            for (int e = 0; e < 16; ++e) v[e] = unary_value<3>(exhip_h2f(exhip_f2h(v[e])), al, be);
                            break;
                        default:
#pragma unroll
                            for (int e = 0; e < 16; ++e) v[e] = unary_value<4>(exhip_h2f(exhip_f2h(v[e])), al, be);
                            break;
                        }
                    }
                    if (has_res && p.residual_last) add_shortcut();
                    v4i o0, o1;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const uint32_t lo = exhip_f2h(v[2 * e]), hi = exhip_f2h(v[2 * e + 1]);
                        if (e < 4) o0[e] = (int)(lo | (hi << 16));
                        else o1[e - 4] = (int)(lo | (hi << 16));
                    }
                    pair_exchange4(o0, o1, odd);
                    __builtin_amdgcn_raw_buffer_store_b128(o0, ry, (int)even_b + cb + (odd ? 16 : 0), 0, 0);
                    __builtin_amdgcn_raw_buffer_store_b128(o1, ry, (int)odd_b + cb + (odd ? 16 : 0), 0, 0);
                }
            }
            return;
        }
        unsigned eoff[2], noff[2], feven[2], fodd[2];
        const bool odd_lane = lane & 1;
#pragma unroll
        for (int nn = 0; nn < 2; ++nn) {
            int py, px;
            const bool in_patch = patch_pixel(nn, py, px);
            const bool valid = in_patch & (full | ((oy0 + py < p.OH) & (ox0 + px < p.OW)));
            eoff[nn] = valid ? obase + (unsigned)((py * p.OW + px) * p.K) : kOobElem;
            if (has_f) {
                // float32 rows leave in 64-byte runs that a lane pair and its neighbour pair form: the even pixel's
                // runs in one store, the odd pixel's in the next
                const unsigned other = (unsigned)lane_neighbour((int)eoff[nn]);
                feven[nn] = (odd_lane ? other : eoff[nn]) * 4u + (odd_lane ? 32u : 0u) + hh * 16;
                fodd[nn] = (odd_lane ? eoff[nn] : other) * 4u + (odd_lane ? 32u : 0u) + hh * 16;
            }
            if (has_nchw) {
                const unsigned e = ((unsigned)n * (unsigned)p.K + (unsigned)(kt * 64 + hh * 16)) * (unsigned)img_px +
                                   (unsigned)((oy0 + py) * p.OW + ox0 + px);
                noff[nn] = valid ? e * 4u : (unsigned)kOob;
            }
        }
        // the shortcut's values first, so that all of them are in flight while the first are used
        v4i rs[2][2][4];
        if (has_res) {
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int nn = 0; nn < 2; ++nn)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        rs[m][nn][j] = __builtin_amdgcn_raw_buffer_load_b128(rr, (int)(eoff[nn] * 4u + hh * 16 + m * 128 + piece(j)), 0, 0);
        }
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            v4f s4[4], b4[4];
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                s4[e4] = *reinterpret_cast<const v4f*>(lds_sb + m * 32 + hh * 16 + e4 * 4);
                b4[e4] = *reinterpret_cast<const v4f*>(lds_sb + 64 + m * 32 + hh * 16 + e4 * 4);
            }
#pragma unroll
            for (int nn = 0; nn < 2; ++nn) {
                // two accumulator sets fill the register file: keep the scheduler from starting a block's reads and
                // conversions before the block in front of it is out
                if constexpr (PROJ) __builtin_amdgcn_sched_barrier(0);
                v4i q4;
                if (q_only) {
                    // int8 output only, ReLU last: q = trunc(max(v, 0) * fs + 0.5) capped at 127. With fs > 0 the maximum
                    // commutes with the product, and max(t, 0) + 0.5 == max(t + 0.5, 0.5) in float arithmetic (the sum is
                    // monotone in t), so one median does ReLU and saturation.
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4) {
                        int b[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float v = __builtin_fmaf((float)acc[m][nn][e4 * 4 + e], s4[e4][e], b4[e4][e]);
                            b[e] = (int)__builtin_amdgcn_fmed3f(v * p.fs_out + 0.5f, 0.5f, 127.f);
                        }
                        q4[e4] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                    }
                    __builtin_amdgcn_raw_buffer_store_b128(q4, rq, (int)(eoff[nn] + hh * 16 + m * 32), 0, 0);
                    continue;
                }
                v4i r4[4];
                if (has_res) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) r4[j] = rs[m][nn][j];
                    half_swap4(r4[0], r4[1]);
                    half_swap4(r4[2], r4[3]);
                }
                v4i o4[4];
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    v4f v;
                    if constexpr (PROJ) {  // read where used: the arrays above would not fit beside two accumulator sets
                        const v4f sc = *reinterpret_cast<const v4f*>(lds_sb + m * 32 + hh * 16 + e4 * 4);
                        const v4f bi = *reinterpret_cast<const v4f*>(lds_sb + 64 + m * 32 + hh * 16 + e4 * 4);
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf((float)acc[m][nn][e4 * 4 + e], sc[e], bi[e]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf((float)acc[m][nn][e4 * 4 + e], s4[e4][e], b4[e4][e]);
                    }
                    if (act_relu) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaxf(v[e], 0.f);
                    }
                    // the instantiation with run-time flags also takes the activation layer behind the convolution and the sum
                    // layer behind that one (a detection network's bottleneck)
                    const bool res_last = EPI < 0 && p.residual_last;
                    if (has_res && !res_last) {
                        const v4f rv = __builtin_bit_cast(v4f, r4[e4]);
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] += rv[e];
                    }
                    if constexpr (PROJ) {
                        // the value the 1x1 layer would have stored (no activation), added as the shortcut
                        const v4f sd = *reinterpret_cast<const v4f*>(lds_sb + 128 + m * 32 + hh * 16 + e4 * 4);
                        const v4f bd = *reinterpret_cast<const v4f*>(lds_sb + 192 + m * 32 + hh * 16 + e4 * 4);
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] += __builtin_fmaf((float)acc_ds[m][nn][e4 * 4 + e], sd[e], bd[e]);
                    }
                    if (post_relu) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaxf(v[e], 0.f);
                    }
                    if constexpr (EPI < 0) {
                        if (p.post_op) {
                            auto apply = [&](auto op) {
#pragma unroll
                                for (int e = 0; e < 4; ++e) v[e] = unary_value<decltype(op)::value>(v[e], p.post_alpha, p.post_beta);
                            };
                            switch (p.post_op - 1) {  // one switch per vector, not per value
                            case EXHIP_UNARY_HARDSWISH: apply(std::integral_constant<int, 0>{}); break;
                            case EXHIP_UNARY_LEAKYRELU: apply(std::integral_constant<int, 1>{}); break;
                            case EXHIP_UNARY_HARDSIGMOID: apply(std::integral_constant<int, 3>{}); break;
                            default: apply(std::integral_constant<int, 4>{}); break;
                            }
                        }
                        if (has_res && res_last) {
                            const v4f rv = __builtin_bit_cast(v4f, r4[e4]);
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] += rv[e];
                        }
                    }
                    o4[e4] = __builtin_bit_cast(v4i, v);
                    if (has_nchw) {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            __builtin_amdgcn_raw_buffer_store_b32(o4[e4][e], rn, (int)noff[nn], (m * 32 + e4 * 4 + e) * img_px * 4, 0);
                    }
                    if (has_q) {
                        // float32_to_int8(v * fs): product rounded first, then +-0.5, saturate, truncate. After a final
                        // ReLU every product is >= 0: the sign select and the lower clamp fall away.
                        int b[4];
                        if (q_nonneg) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) b[e] = (int)__builtin_fminf(v[e] * p.fs_out + 0.5f, 127.f);
                            q4[e4] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const float t = v[e] * p.fs_out;
                                b[e] = (int)__builtin_amdgcn_fmed3f(t + __builtin_copysignf(0.5f, t), -128.f, 127.f);
                            }
                            q4[e4] = (b[0] & 0xff) | ((b[1] & 0xff) << 8) | ((b[2] & 0xff) << 16) | (b[3] << 24);
                        }
                    }
                }
                if (has_f) {
                    // o4[0], o4[2]: channels 0-7 and 8-15 of the block's 32; o4[1], o4[3]: 16-23 and 24-31
                    half_swap4(o4[0], o4[1]);
                    half_swap4(o4[2], o4[3]);
                    pair_exchange4(o4[0], o4[2], odd_lane);
                    pair_exchange4(o4[1], o4[3], odd_lane);
                    __builtin_amdgcn_raw_buffer_store_b128(o4[0], rf, (int)(feven[nn] + m * 128), 0, EXHIP_F32_STORE_AUX);
                    __builtin_amdgcn_raw_buffer_store_b128(o4[1], rf, (int)(feven[nn] + m * 128 + 64), 0, EXHIP_F32_STORE_AUX);
                    __builtin_amdgcn_raw_buffer_store_b128(o4[2], rf, (int)(fodd[nn] + m * 128), 0, EXHIP_F32_STORE_AUX);
                    __builtin_amdgcn_raw_buffer_store_b128(o4[3], rf, (int)(fodd[nn] + m * 128 + 64), 0, EXHIP_F32_STORE_AUX);
                }
                if (has_q) __builtin_amdgcn_raw_buffer_store_b128(q4, rq, (int)(eoff[nn] + hh * 16 + m * 32), 0, 0);
            }
        }
    };
    // stores an epilogue issues (they stand behind the next tile's request in the wave's memory queue)
    constexpr int kEpiStores = EPI < 0 ? 64 : F16 ? 8 : ((EPI & E_F) ? 16 : 0) + ((EPI & E_Q) ? 4 : 0) + ((EPI & E_NCHW) ? 64 : 0);
    constexpr int kWaitBehindEpi = EPI < 0 ? 0 : (kEpiStores < 60 ? kEpiStores : 60);

    // ---- the run ----
    int n, oy0, ox0;                 // the patch being computed
    int pt = pj;
    decode(pt, n, oy0, ox0);
    const char* img = p.x + (size_t)n * p.img_bytes;   // image and view base of the next tile request
    int base = set_offsets(oy0, ox0);
    if (tid < 128) {
        const int ch = kt * 64 + (tid & 63);
        lds_sb[tid] = tid < 64 ? (F16 ? 1.f : p.scale[ch]) : (p.bias ? p.bias[ch] : 0.f);
    } else if (PROJ) {
        const int ch = kt * 64 + (tid & 63);
        lds_sb[tid] = tid < 192 ? p.ds_scale[ch] : (p.ds_bias ? p.ds_bias[ch] : 0.f);
    }
    clear_acc();

    if constexpr (WRES) {
        request_a(img, base, 0, true, lds0 + A0);
        put(1, now());
        wait_vmcnt<0>();
        __syncthreads();
        put(2, now());
        const char* const wrow = smem + lane * 16;
        const char* const a0 = smem + A0 + boff[0];
        const char* const a1 = smem + A0 + boff[1];
        for (int done = 0;;) {
            t_mark = now();
            mfma_rows(three_rows, wrow, a0, a1, []() {});
            { const long long t = now(); t_mfma += t - t_mark; t_mark = t; }
            __syncthreads();  // every wave has read the tile
            { const long long t = now(); t_bar += t - t_mark; t_mark = t; }
            const bool has_next = ++done < my_tiles;
            int nn_, ny, nx;
            if (has_next) {
                pt += GP;
                decode(pt, nn_, ny, nx);
                img = p.x + (size_t)nn_ * p.img_bytes;
                base = set_offsets(ny, nx);
                request_a(img, base, 0, true, lds0 + A0);
            }
            { const long long t = now(); t_gap += t - t_mark; t_mark = t; }
            if (kStamps && n_epi < 20) put(18 + 2 * n_epi, (long long)clock64());
            epilogue(n, oy0, ox0);
            if (kStamps && n_epi < 20) { put(19 + 2 * n_epi, (long long)clock64()); ++n_epi; }
            { const long long t = now(); t_epi += t - t_mark; t_mark = t; }
            if (!has_next) break;
            clear_acc();
            n = nn_; oy0 = ny; ox0 = nx;
            wait_vmcnt<kWaitBehindEpi>();
            { const long long t = now(); t_wait += t - t_mark; t_mark = t; }
            __syncthreads();
            { const long long t = now(); t_bar += t - t_mark; t_mark = t; }
        }
    } else {
        // waits at the end of a stage's MFMAs: the next stage's slice must have landed; what was requested behind it stays
        // in flight (the order of a stage's requests: its slice first, then the next chunk's tile)
        constexpr int kWait0 = (NWB == 3 ? 3 : 0) + (NAB == 2 ? kNAL : 0);
        constexpr int kWait1 = NWB == 3 ? 3 + (NAB == 2 ? kNAL : 0) : 0;
        constexpr int kWait2 = NWB == 3 ? 3 : 0;
        request_a(img, base, 0, true, lds0 + A0);
        if constexpr (NWB == 3) request_w(lds0 + kWSlice);
        put(1, now());
        wait_vmcnt<(NWB == 3 ? 3 : 0)>();
        __syncthreads();
        put(2, now());
        t_mark = now();
        int abuf = 0;   // tile buffer of the current chunk
        int wbuf = 0;   // NWB == 2: slice buffer of the current stage (with three buffers filter row r is in buffer r)
        int nn_ = n, ny = oy0, nx = ox0;
        for (int done = 0;;) {
            const bool has_next = done + 1 < my_tiles;
            for (int cc = 0; cc < n_tot; ++cc) {
                const bool last_cc = cc + 1 == n_tot;
                const bool proj_cc = PROJ && cc >= p.n_chunks;   // a chunk of the projection: one tap, in the first stage
                // what the next chunk's tile request asks for: the next chunk of this patch, or the next patch's first
                auto request_next_a = [&](unsigned dst) {
                    if (last_cc) {
                        if (has_next) {
                            pt += GP;
                            decode(pt, nn_, ny, nx);
                            img = p.x + (size_t)nn_ * p.img_bytes;
                            base = set_offsets(ny, nx);
                        }
                        request_a(img, base, 0, has_next, dst);
                    } else if (PROJ && cc + 1 >= p.n_chunks) {
                        request_ds(n, oy0, ox0, cc + 1 - p.n_chunks, dst);
                    } else {
                        request_a(img, base, cc + 1, true, dst);
                    }
                };
                // one stage: a filter row of a 3x3 chunk, or (first stage only) the tap of a projection chunk
                auto stage = [&](int r, const char* w, const char* a0r, const char* a1r, auto&& requests) {
                    if (!proj_cc) {
                        mfma_rows(one_row, w, a0r, a1r, requests);
                    } else {
                        if (r == 0) mfma_ds(w, a0r + row_b + kPixB, a1r + row_b + kPixB);
                        requests();
                    }
                };
                const char* const ab = smem + A0 + (NAB == 2 ? abuf * kActStride : 0);
                const char* const a0 = ab + boff[0];
                const char* const a1 = ab + boff[1];
                const unsigned a_other = lds0 + A0 + (NAB == 2 ? (1 - abuf) * kActStride : 0);
                if constexpr (NWB == 3) {
                    stage(0, smem + lane * 16, a0, a1, [&]() {
                        request_w(lds0 + 2 * kWSlice);
                        if constexpr (NAB == 2) request_next_a(a_other);
                    });
                    { const long long t = now(); t_mfma += t - t_mark; t_mark = t; }
                    wait_vmcnt<kWait0>();
                    { const long long t = now(); t_wait += t - t_mark; t_mark = t; }
                    __syncthreads();
                    { const long long t = now(); t_bar += t - t_mark; t_mark = t; }
                    stage(1, smem + kWSlice + lane * 16, a0 + row_b, a1 + row_b, [&]() { request_w(lds0); });
                    { const long long t = now(); t_mfma += t - t_mark; t_mark = t; }
                    wait_vmcnt<kWait1>();
                    { const long long t = now(); t_wait += t - t_mark; t_mark = t; }
                    __syncthreads();
                    { const long long t = now(); t_bar += t - t_mark; t_mark = t; }
                    stage(2, smem + 2 * kWSlice + lane * 16, a0 + 2 * row_b, a1 + 2 * row_b, [&]() { request_w(lds0 + kWSlice); });
                    { const long long t = now(); t_mfma += t - t_mark; t_mark = t; }
                    wait_vmcnt<kWait2>();
                    { const long long t = now(); t_wait += t - t_mark; t_mark = t; }
                    __syncthreads();
                    { const long long t = now(); t_bar += t - t_mark; t_mark = t; }
                } else {
                    stage(0, smem + wbuf * kWSlice + lane * 16, a0, a1, [&]() {
                        request_w(lds0 + (1 - wbuf) * kWSlice);
                        if constexpr (NAB == 2) request_next_a(a_other);
                    });
                    { const long long t = now(); t_mfma += t - t_mark; t_mark = t; }
                    wait_vmcnt<kWait0>();
                    { const long long t = now(); t_wait += t - t_mark; t_mark = t; }
                    __syncthreads();
                    { const long long t = now(); t_bar += t - t_mark; t_mark = t; }
                    wbuf = 1 - wbuf;
                    stage(1, smem + wbuf * kWSlice + lane * 16, a0 + row_b, a1 + row_b, [&]() { request_w(lds0 + (1 - wbuf) * kWSlice); });
                    { const long long t = now(); t_mfma += t - t_mark; t_mark = t; }
                    wait_vmcnt<kWait1>();
                    { const long long t = now(); t_wait += t - t_mark; t_mark = t; }
                    __syncthreads();
                    { const long long t = now(); t_bar += t - t_mark; t_mark = t; }
                    wbuf = 1 - wbuf;
                    stage(2, smem + wbuf * kWSlice + lane * 16, a0 + 2 * row_b, a1 + 2 * row_b,
                          [&]() { request_w(lds0 + (1 - wbuf) * kWSlice); });
                    { const long long t = now(); t_mfma += t - t_mark; t_mark = t; }
                    wait_vmcnt<kWait2>();
                    { const long long t = now(); t_wait += t - t_mark; t_mark = t; }
                    __syncthreads();
                    { const long long t = now(); t_bar += t - t_mark; t_mark = t; }
                    wbuf = 1 - wbuf;
                }
                if constexpr (NAB == 2) {
                    abuf = 1 - abuf;
                } else {
                    // a single tile buffer: refilled once every wave has left the chunk; between chunks the load is waited
                    // for in the open (the CU's other groups run meanwhile), behind a patch it lands under the epilogue
                    request_next_a(lds0 + A0);
                    if (!last_cc) {
                        wait_vmcnt<0>();
                        __syncthreads();
                    }
                    { const long long t = now(); t_gap += t - t_mark; t_mark = t; }
                }
            }
            if (kStamps && n_epi < 20) put(18 + 2 * n_epi, (long long)clock64());
            epilogue(n, oy0, ox0);
            if (kStamps && n_epi < 20) { put(19 + 2 * n_epi, (long long)clock64()); ++n_epi; }
            { const long long t = now(); t_epi += t - t_mark; t_mark = t; }
            if (!has_next) break;
            ++done;
            clear_acc();
            n = nn_; oy0 = ny; ox0 = nx;
            if constexpr (NAB == 1) {
                wait_vmcnt<kWaitBehindEpi>();
                __syncthreads();
                { const long long t = now(); t_gap += t - t_mark; t_mark = t; }
            }
        }
    }
    wait_vmcnt<0>();  // no staging load may land after the group's LDS has been given to another
    put(3, t_mfma); put(4, t_wait); put(5, t_bar); put(6, t_epi); put(7, t_gap); put(8, now()); put(9, my_tiles);
    if constexpr (kStamps) put(11, (long long)wall_clock64());
}

// ---- the same convolution with the work of a group split between two kinds of waves ----
// A group of eight waves owns a CU: waves 0-3 stage operands and run the MFMAs of a patch (a 64 x 64 accumulator tile each),
// then leave the accumulators in LDS; waves 4-7 take them from there one patch later and do everything that is not an
// MFMA -- dequantization, shortcut, ReLU, requantization, all traffic to and from the result tensors -- while the first
// four are already at the next patch. On every SIMD an MFMA wave and an epilogue wave run side by side, so the matrix
// pipe does not wait for vector work, and the shortcut's loads (requested a patch ahead) and the result stores have a
// memory queue of their own: the staging waits of the MFMA waves never stand behind them. The two kinds meet only at
// the stage barriers both execute in equal number. With one group per CU the whole LDS is the group's: three weight
// slice buffers (or the resident filter), two activation tile buffers, 64 KiB for the accumulators.
template <bool WRES, int EPI>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void conv3x3_i8_ws_kernel(const LeanParams p) {
    constexpr int A0 = 3 * kWSlice;
    constexpr int H0 = A0 + 2 * kActStride;          // accumulators on their way to the epilogue waves: 4 x 16 KiB
    constexpr int SB0 = H0 + 4 * 16384;
    constexpr int SPARE0 = SB0 + kSbB;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
    float* const lds_sb = reinterpret_cast<float*>(smem + SB0);

    const int flags = EPI >= 0 ? EPI : p.flags;
    const bool has_res = flags & E_RES, has_f = flags & E_F, has_q = flags & E_Q, has_nchw = flags & E_NCHW;
    const bool act_relu = flags & E_ACT, post_relu = flags & E_POST, q_nonneg = flags & E_QNN;
    const bool q_only = q_nonneg && has_q && !has_res && !has_f && !has_nchw;

    const int wave8 = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const bool mma_role = wave8 < 4;
    const int wave = wave8 & 3, lane = threadIdx.x & 63, tid = threadIdx.x & 255, hh = lane >> 5;

    // waits for this wave's LDS operations, then for the group: what was written before is visible behind it. No memory
    // fence: that would also wait for every global access in flight, which is what the epilogue waves must not do.
    long long t_mfma = 0, t_wait = 0, t_bar = 0, t_epi = 0, t_mark = 0;
    auto now = [&]() -> long long { return kStamps && p.dbg ? (long long)clock64() : 0ll; };
    auto put = [&](int k, long long v) {
        if constexpr (kStamps)
            if (p.dbg && lane == 0) p.dbg[((size_t)blockIdx.x * 8 + wave8) * 16 + k] = v;
    };
    auto lap = [&](long long& acc_t) {
        if constexpr (kStamps) { const long long t = now(); acc_t += t - t_mark; t_mark = t; }
    };
    put(0, now());
    if constexpr (kStamps) put(10, (long long)wall_clock64());
    auto barrier = [&]() {
        lap(t_mfma);
        __asm__ volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        lap(t_bar);
    };

    const int G = gridDim.x;
    int lb = blockIdx.x;
    if ((G & 7) == 0) lb = (lb & 7) * (G >> 3) + (lb >> 3);
    const int kt = __builtin_amdgcn_readfirstlane(lb % p.ktiles);
    const int pj = __builtin_amdgcn_readfirstlane(lb / p.ktiles);
    const int GP = G / p.ktiles;
    const int my_tiles = __builtin_amdgcn_readfirstlane((p.n_ptiles - pj + GP - 1) / GP);
    const int nst = WRES ? 2 : p.n_chunks * 3;   // barriers per patch
    const int row_b = p.IW * kPixB;
    const int img_px = p.OH * p.OW;

    auto decode = [&](int t, int& n, int& oy0, int& ox0) {
        n = fast_div(t, p.magic_txy);
        const int r = t - n * p.tiles_xy;
        const int ty = fast_div(r, p.magic_tx), tx = r - ty * p.tiles_x;
        oy0 = ty * p.PH;
        ox0 = tx * p.PW;
    };
    // the lane's two pixels (one per 32-pixel column block of its wave)
    int boff[2], o_rel[2], o_y[2], o_x[2];
#pragma unroll
    for (int nn = 0; nn < 2; ++nn) {
        int pp = (wave * 2 + nn) * 32 + (lane & 31);
        const bool ok = pp < p.PH * p.PW;
        pp = ok ? pp : 0;
        const int py = fast_div(pp, p.magic_pw), px = pp - py * p.PW;
        boff[nn] = py * row_b + px * kPixB + hh * 16;
        o_rel[nn] = (py * p.OW + px) * p.K;
        o_y[nn] = ok ? py : 0x4000;
        o_x[nn] = px;
    }
    char* const hand = smem + H0 + wave * 16384 + lane * 16;   // this wave pair's accumulators: 16 x 1 KiB

    if (mma_role) {
        // ================= staging and MFMAs =================
        int a_rel[kNAL], a_yx[kNAL], a_off[kNAL];
        {
            const int IW = p.IW, npix = p.IH * IW, W = p.W, cb = p.C_b;
            int pix = fast_div(tid, 0x33333334u), part = tid - pix * 5;
            int iy = fast_div(pix, p.magic_iw), ix = pix - iy * IW;
#pragma unroll
            for (int i = 0; i < kNAL; ++i) {
                const bool ok = (pix < npix) & (part < 4);
                a_rel[i] = ok ? (iy * W + ix) * cb + part * 16 : kOob;
                a_yx[i] = ok ? (iy | (ix << 16)) : -1;
                part += 1;
                const int carry = part >= 5 ? 1 : 0;
                part -= carry ? 5 : 0;
                pix += 51 + carry;
                ix += p.adv_ix + carry;
                iy += p.adv_iy;
                const int wrap = ix >= IW ? 1 : 0;
                ix -= wrap ? IW : 0;
                iy += wrap;
            }
        }
        auto set_offsets = [&](int oy0, int ox0) -> int {
            const int iy0 = oy0 - p.PT, ix0 = ox0 - p.PL;
            const int tile_base = (iy0 * p.W + ix0) * p.C_b;
            const bool interior = iy0 >= 0 && ix0 >= 0 && iy0 + p.IH <= p.H && ix0 + p.IW <= p.W;
            if (interior) {
#pragma unroll
                for (int i = 0; i < kNAL; ++i) a_off[i] = a_rel[i];
                return tile_base;
            }
#pragma unroll
            for (int i = 0; i < kNAL; ++i) {
                const int gy = iy0 + (a_yx[i] & 0xFFFF), gx = ix0 + (int)((unsigned)a_yx[i] >> 16);
                const bool in = ((unsigned)gy < (unsigned)p.H) & ((unsigned)gx < (unsigned)p.W);
                a_off[i] = in ? a_rel[i] + tile_base : kOob;
            }
            return 0;
        };
        const unsigned wave_slot = (unsigned)wave * 1024u;
        const int w_voff = tid * 16;
        const char* const wkt = p.wp + (size_t)kt * p.n_chunks * (3 * kWSlice);
        const int w_run_b = p.n_chunks * 3 * kWSlice;
        int w_off = 0;
        int w_left = my_tiles * p.n_chunks * 3;
        auto request_w = [&](unsigned dst) {
            const __amdgpu_buffer_rsrc_t wr = uniform_view(wkt + w_off, w_left > 0 ? kWSlice : 0);
#pragma unroll
            for (int i = 0; i < 3; ++i) async_load16(wr, w_voff, i * 4096, dst + wave_slot + i * 4096);
            --w_left;
            w_off += kWSlice;
            if (w_off == w_run_b) w_off = 0;
        };
        auto request_a = [&](const char* img, int base, int cc, bool valid, unsigned dst) {
            const int off = base + cc * 64;
            const __amdgpu_buffer_rsrc_t xr =
                uniform_view(img + off, valid ? (int)p.img_bytes - off : 0);
#pragma unroll
            for (int i = 0; i < kNAL; ++i) {
                unsigned d = dst + wave_slot + i * 4096;
                if (i == kNAL - 1) d = wave == 3 ? lds0 + SPARE0 : d;
                async_load16(xr, a_off[i], 0, d);
            }
        };
        v16i acc[2][2];
        auto clear_acc = [&]() {
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int nn = 0; nn < 2; ++nn)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[m][nn][e] = 0;
        };
        auto hand_over = [&]() {
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int nn = 0; nn < 2; ++nn)
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4)
                        *reinterpret_cast<v4i*>(hand + ((m * 2 + nn) * 4 + e4) * 1024) =
                            v4i{acc[m][nn][e4 * 4], acc[m][nn][e4 * 4 + 1], acc[m][nn][e4 * 4 + 2], acc[m][nn][e4 * 4 + 3]};
        };
        v4i af[2][2], bf[2][2];
        auto compute = [&](int buf) {
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int nn = 0; nn < 2; ++nn) acc[m][nn] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[buf][m], bf[buf][nn], acc[m][nn], 0, 0, 0);
        };
        auto fetch = [&](int buf, const char* wrow, const char* a0, const char* a1, int s) {
            af[buf][0] = lds_read16(wrow + s * 2048);
            af[buf][1] = lds_read16(wrow + s * 2048 + 1024);
            bf[buf][0] = lds_read16(a0 + (s >> 1) * kPixB + (s & 1) * 32);
            bf[buf][1] = lds_read16(a1 + (s >> 1) * kPixB + (s & 1) * 32);
        };
        auto mfma_rows = [&](auto nr_t, const char* wrow, const char* a0, const char* a1, auto&& requests) {
            constexpr int NR = decltype(nr_t)::value;
            fetch(0, wrow, a0, a1, 0);
#pragma unroll
            for (int r = 0; r < NR; ++r) {
#pragma unroll
                for (int s = 0; s < 6; ++s) {
                    const int k = r * 6 + s;
                    if (s + 1 < 6) fetch((k + 1) & 1, wrow + r * kWSlice, a0 + r * row_b, a1 + r * row_b, s + 1);
                    else if (r + 1 < NR) fetch((k + 1) & 1, wrow + (r + 1) * kWSlice, a0 + (r + 1) * row_b, a1 + (r + 1) * row_b, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    compute(k & 1);
                    __builtin_amdgcn_sched_barrier(0);
                    if (k == 0) requests();
                }
            }
        };
        constexpr std::integral_constant<int, 1> one_row{};
        constexpr std::integral_constant<int, 2> two_rows{};

        int n, oy0, ox0, pt = pj;
        decode(pt, n, oy0, ox0);
        const char* img = p.x + (size_t)n * p.img_bytes;
        int base = set_offsets(oy0, ox0);
        if (tid < 128) {
            const int ch = kt * 64 + (tid & 63);
            lds_sb[tid] = tid < 64 ? p.scale[ch] : (p.bias ? p.bias[ch] : 0.f);
        }
        clear_acc();
        int abuf = 0;
        // the next tile request: the next chunk of this patch, or the first chunk of the group's next patch
        auto request_next_a = [&](int cc, bool last_cc, bool has_next, unsigned dst) {
            if (last_cc) {
                if (has_next) {
                    pt += GP;
                    decode(pt, n, oy0, ox0);
                    img = p.x + (size_t)n * p.img_bytes;
                    base = set_offsets(oy0, ox0);
                }
                request_a(img, base, 0, has_next, dst);
            } else {
                request_a(img, base, cc + 1, true, dst);
            }
        };
        if constexpr (WRES) {
            request_a(img, base, 0, true, lds0 + A0);
            for (int r = 0; r < 3; ++r) request_w(lds0 + r * kWSlice);
            lap(t_mfma); wait_vmcnt<0>(); lap(t_wait);
            put(1, now());
            barrier();
            put(2, now());
            t_mark = now(); t_mfma = 0; t_bar = 0; t_wait = 0;
            for (int done = 0; done < my_tiles; ++done) {
                const bool has_next = done + 1 < my_tiles;
                const char* const ab = smem + A0 + abuf * kActStride;
                const unsigned a_other = lds0 + A0 + (1 - abuf) * kActStride;
                mfma_rows(one_row, smem + lane * 16, ab + boff[0], ab + boff[1], [&]() { request_next_a(0, true, has_next, a_other); });
                barrier();   // the epilogue waves have taken the previous patch's accumulators
                mfma_rows(two_rows, smem + kWSlice + lane * 16, ab + row_b + boff[0], ab + row_b + boff[1], []() {});
                hand_over();
                lap(t_mfma); wait_vmcnt<0>(); lap(t_wait);
                barrier();
                clear_acc();
                abuf = 1 - abuf;
            }
        } else {
            request_a(img, base, 0, true, lds0 + A0);
            request_w(lds0);
            request_w(lds0 + kWSlice);
            lap(t_mfma); wait_vmcnt<3>(); lap(t_wait);
            put(1, now());
            barrier();
            put(2, now());
            t_mark = now(); t_mfma = 0; t_bar = 0; t_wait = 0;
            for (int done = 0; done < my_tiles; ++done) {
                const bool has_next = done + 1 < my_tiles;
                for (int cc = 0; cc < p.n_chunks; ++cc) {
                    const bool last_cc = cc + 1 == p.n_chunks;
                    const char* const ab = smem + A0 + abuf * kActStride;
                    const char* const a0 = ab + boff[0];
                    const char* const a1 = ab + boff[1];
                    const unsigned a_other = lds0 + A0 + (1 - abuf) * kActStride;
                    mfma_rows(one_row, smem + lane * 16, a0, a1, [&]() {
                        request_w(lds0 + 2 * kWSlice);
                        request_next_a(cc, last_cc, has_next, a_other);
                    });
                    lap(t_mfma); wait_vmcnt<3 + kNAL>(); lap(t_wait);
                    barrier();
                    mfma_rows(one_row, smem + kWSlice + lane * 16, a0 + row_b, a1 + row_b, [&]() { request_w(lds0); });
                    lap(t_mfma); wait_vmcnt<3 + kNAL>(); lap(t_wait);
                    barrier();
                    mfma_rows(one_row, smem + 2 * kWSlice + lane * 16, a0 + 2 * row_b, a1 + 2 * row_b, [&]() { request_w(lds0 + kWSlice); });
                    if (last_cc) hand_over();
                    lap(t_mfma); wait_vmcnt<3>(); lap(t_wait);
                    barrier();
                    abuf = 1 - abuf;
                }
                clear_acc();
            }
        }
        wait_vmcnt<0>();  // no staging load may land after the group's LDS has been given to another
    } else {
        // ================= epilogues, one patch behind =================
        const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(p.y_q, 0, (int)p.out_elems, kRsrcWord3);
        const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc(p.y_f, 0, (int)(p.out_elems * 4u), kRsrcWord3);
        const __amdgpu_buffer_rsrc_t rr = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p.residual), 0, (int)(p.out_elems * 4u), kRsrcWord3);
        const __amdgpu_buffer_rsrc_t rn = __builtin_amdgcn_make_buffer_rsrc(p.y_nchw, 0, (int)(p.out_elems * 4u), kRsrcWord3);
        auto piece = [](int j) { return j == 0 ? 0 : j == 1 ? 64 : j == 2 ? 32 : 96; };
        // element offsets of the lane's two pixels in a patch's result tensors
        auto offsets = [&](int n, int oy0, int ox0, unsigned (&eoff)[2], unsigned (&noff)[2]) {
            const bool full = oy0 + p.PH <= p.OH && ox0 + p.PW <= p.OW;
            const unsigned obase = ((unsigned)n * (unsigned)img_px + (unsigned)(oy0 * p.OW + ox0)) * (unsigned)p.K + (unsigned)(kt * 64);
#pragma unroll
            for (int nn = 0; nn < 2; ++nn) {
                const bool valid = full ? o_y[nn] < 0x4000 : ((oy0 + o_y[nn] < p.OH) & (ox0 + o_x[nn] < p.OW));
                eoff[nn] = valid ? obase + (unsigned)o_rel[nn] : kOobElem;
                noff[nn] = 0;
                if (has_nchw) {
                    const unsigned e = ((unsigned)n * (unsigned)p.K + (unsigned)(kt * 64 + hh * 16)) * (unsigned)img_px +
                                       (unsigned)((oy0 + o_y[nn]) * p.OW + ox0 + o_x[nn]);
                    noff[nn] = valid ? e * 4u : (unsigned)kOob;
                }
            }
        };
        v4i rs[2][2][4];   // the shortcut's values of the patch whose epilogue comes next
        auto request_shortcut = [&](const unsigned (&eoff)[2]) {
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int nn = 0; nn < 2; ++nn)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        rs[m][nn][j] = __builtin_amdgcn_raw_buffer_load_b128(rr, (int)(eoff[nn] * 4u + hh * 16 + m * 128 + piece(j)), 0, 0);
        };
        // The accumulators taken over. With the resident filter all four tiles are read at once (the MFMA waves write the
        // next patch's before this patch's last blocks run); otherwise each block reads its own when its turn comes.
        v4i accq[WRES ? 4 : 1][4];
        auto take_over = [&](int b) {
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) accq[WRES ? b : 0][e4] = *reinterpret_cast<const v4i*>(hand + (b * 4 + e4) * 1024);
        };
        // one accumulator tile (32 channels x 32 pixels of the wave's 64 x 64)
        auto block = [&](auto m_t, auto nn_t, const unsigned (&eoff)[2], const unsigned (&noff)[2]) {
            constexpr int m = decltype(m_t)::value, nn = decltype(nn_t)::value;
            if constexpr (!WRES) take_over(m * 2 + nn);
            v4f s4[4], b4[4];
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                s4[e4] = *reinterpret_cast<const v4f*>(lds_sb + m * 32 + hh * 16 + e4 * 4);
                b4[e4] = *reinterpret_cast<const v4f*>(lds_sb + 64 + m * 32 + hh * 16 + e4 * 4);
            }
            v4i q4;
            if (q_only) {
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    int b[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float v = __builtin_fmaf((float)accq[WRES ? m * 2 + nn : 0][e4][e], s4[e4][e], b4[e4][e]);
                        b[e] = (int)__builtin_amdgcn_fmed3f(v * p.fs_out + 0.5f, 0.5f, 127.f);
                    }
                    q4[e4] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                }
                __builtin_amdgcn_raw_buffer_store_b128(q4, rq, (int)(eoff[nn] + hh * 16 + m * 32), 0, 0);
                return;
            }
            v4i r4[4];
            if (has_res) {
#pragma unroll
                for (int j = 0; j < 4; ++j) r4[j] = rs[m][nn][j];
                half_swap4(r4[0], r4[1]);
                half_swap4(r4[2], r4[3]);
            }
            v4i o4[4];
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                v4f v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf((float)accq[WRES ? m * 2 + nn : 0][e4][e], s4[e4][e], b4[e4][e]);
                if (act_relu) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaxf(v[e], 0.f);
                }
                if (has_res) {
                    const v4f rv = __builtin_bit_cast(v4f, r4[e4]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += rv[e];
                }
                if (post_relu) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaxf(v[e], 0.f);
                }
                o4[e4] = __builtin_bit_cast(v4i, v);
                if (has_nchw) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        __builtin_amdgcn_raw_buffer_store_b32(o4[e4][e], rn, (int)noff[nn], (m * 32 + e4 * 4 + e) * img_px * 4, 0);
                }
                if (has_q) {
                    int b[4];
                    if (q_nonneg) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) b[e] = (int)__builtin_fminf(v[e] * p.fs_out + 0.5f, 127.f);
                        q4[e4] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float t = v[e] * p.fs_out;
                            b[e] = (int)__builtin_amdgcn_fmed3f(t + __builtin_copysignf(0.5f, t), -128.f, 127.f);
                        }
                        q4[e4] = (b[0] & 0xff) | ((b[1] & 0xff) << 8) | ((b[2] & 0xff) << 16) | (b[3] << 24);
                    }
                }
            }
            if (has_f) {
                half_swap4(o4[0], o4[1]);
                half_swap4(o4[2], o4[3]);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    __builtin_amdgcn_raw_buffer_store_b128(o4[j], rf, (int)(eoff[nn] * 4u + hh * 16 + m * 128 + piece(j)), 0, 0);
            }
            if (has_q) __builtin_amdgcn_raw_buffer_store_b128(q4, rq, (int)(eoff[nn] + hh * 16 + m * 32), 0, 0);
        };
        constexpr std::integral_constant<int, 0> c0{};
        constexpr std::integral_constant<int, 1> c1{};
        auto block_i = [&](int b, const unsigned (&eoff)[2], const unsigned (&noff)[2]) {
            if (b == 0) block(c0, c0, eoff, noff);
            else if (b == 1) block(c0, c1, eoff, noff);
            else if (b == 2) block(c1, c0, eoff, noff);
            else block(c1, c1, eoff, noff);
        };
        // which of a patch's four blocks run before its barrier `s`: spread so that no step holds the MFMA waves up
        const int per_step = nst >= 4 ? 1 : 2;
        auto first_block = [&](int s) { return WRES ? (s == 0 ? 0 : 1) : s * per_step; };
        auto end_block = [&](int s) { const int e = WRES ? (s == 0 ? 1 : 4) : (s + 1) * per_step; return e < 4 ? e : 4; };

        unsigned e_prev[2] = {0, 0}, n_prev[2] = {0, 0};   // offsets of the patch whose accumulators are next
        unsigned e_cur[2], n_cur[2];
        int n, oy0, ox0, pt = pj;
        decode(pt, n, oy0, ox0);
        offsets(n, oy0, ox0, e_cur, n_cur);
        if (has_res) request_shortcut(e_cur);
        put(1, now());
        barrier();
        put(2, now());
        t_mark = now(); t_mfma = 0; t_bar = 0;
        for (int t = 0; t < my_tiles; ++t) {
            // during patch t's stages: the epilogue of patch t - 1 (offsets e_prev), then the request for patch t's shortcut
            for (int s = 0; s < nst; ++s) {
                if (t > 0) {
                    if constexpr (WRES) {
                        if (s == 0) {
#pragma unroll
                            for (int b = 0; b < 4; ++b) take_over(b);
                        }
                    }
                    const int b0 = first_block(s), b1 = end_block(s);
                    for (int b = b0; b < b1; ++b) block_i(b, e_prev, n_prev);
                    if (has_res && b0 < 4 && b1 == 4) request_shortcut(e_cur);
                }
                barrier();
            }
            e_prev[0] = e_cur[0]; e_prev[1] = e_cur[1]; n_prev[0] = n_cur[0]; n_prev[1] = n_cur[1];
            if (t + 1 < my_tiles) {
                pt += GP;
                decode(pt, n, oy0, ox0);
                offsets(n, oy0, ox0, e_cur, n_cur);
            }
        }
        if constexpr (WRES) {
#pragma unroll
            for (int b = 0; b < 4; ++b) take_over(b);
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) block_i(b, e_prev, n_prev);
    }
    lap(t_epi);
    put(3, t_mfma); put(4, t_wait); put(5, t_bar); put(6, t_epi); put(8, now()); put(9, my_tiles);
    if constexpr (kStamps) put(11, (long long)wall_clock64());
}

std::mutex g_attr_mutex;

template <bool WRES, int NAB, int NWB, int EPI, bool PROJ = false>
int launch(exhip_ctx* ctx, const LeanParams& p, int grid) {
    constexpr int lds = ((WRES ? 3 : NWB) * kWSlice) + NAB * kActStride + (PROJ ? 2 * kSbB : kSbB) + kSpareB;
    static unsigned long long attr_set = 0;
    auto kernel = conv3x3_i8_lean_kernel<WRES, NAB, NWB, EPI, PROJ>;
    {
        std::lock_guard<std::mutex> lock(g_attr_mutex);
        const unsigned long long bit = 1ull << (ctx->device & 63);
        if (!(attr_set & bit)) {
            EXHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            attr_set |= bit;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), lds, ctx->stream, p);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

template <bool WRES, int NAB, int NWB>
int launch_epi(exhip_ctx* ctx, const LeanParams& p, int grid) {
    if (p.post_op || p.residual_last) return launch<WRES, NAB, NWB, -1>(ctx, p, grid);  // only the run-time-flag form applies them
    switch (p.flags) {
    case E_Q | E_ACT | E_QNN: return launch<WRES, NAB, NWB, (E_Q | E_ACT | E_QNN)>(ctx, p, grid);
    case E_RES | E_F | E_Q | E_POST | E_QNN: return launch<WRES, NAB, NWB, (E_RES | E_F | E_Q | E_POST | E_QNN)>(ctx, p, grid);
    case E_RES | E_Q | E_POST | E_QNN: return launch<WRES, NAB, NWB, (E_RES | E_Q | E_POST | E_QNN)>(ctx, p, grid);  // a block's end read by int8 layers only
    case E_RES | E_NCHW | E_POST: return launch<WRES, NAB, NWB, (E_RES | E_NCHW | E_POST)>(ctx, p, grid);            // a network's last block
    default: return launch<WRES, NAB, NWB, -1>(ctx, p, grid);
    }
}

template <bool WRES, int EPI>
int launch_ws(exhip_ctx* ctx, const LeanParams& p, int grid) {
    constexpr int lds = 3 * kWSlice + 2 * kActStride + 4 * 16384 + kSbB + kSpareB;
    static unsigned long long attr_set = 0;
    auto kernel = conv3x3_i8_ws_kernel<WRES, EPI>;
    {
        std::lock_guard<std::mutex> lock(g_attr_mutex);
        const unsigned long long bit = 1ull << (ctx->device & 63);
        if (!(attr_set & bit)) {
            EXHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            attr_set |= bit;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(512), lds, ctx->stream, p);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

template <bool WRES>
int launch_ws_epi(exhip_ctx* ctx, const LeanParams& p, int grid) {
    switch (p.flags) {
    case E_Q | E_ACT | E_QNN: return launch_ws<WRES, (E_Q | E_ACT | E_QNN)>(ctx, p, grid);
    case E_RES | E_F | E_Q | E_POST | E_QNN: return launch_ws<WRES, (E_RES | E_F | E_Q | E_POST | E_QNN)>(ctx, p, grid);
    default: return launch_ws<WRES, -1>(ctx, p, grid);
    }
}

}  // namespace

#if EXHIP_STAMPS
// development builds only: where the kernel's waves leave their phase timestamps (16 words per wave), or NULL
extern "C" void exhip_dev_lean_stamps(void* device_buffer) { g_lean_dbg = (long long*)device_buffer; }
#endif

int exhip_conv3x3_i8_lean(exhip_ctx* ctx, const exhip_lean_geom& g, const int8_t* x, const void* wp, const float* scale,
                          const float* bias, const float* residual, int8_t* y_q, float* y_f, float* y_nchw,
                          const exhip_lean_proj* proj, const exhip_lean_f16_epilogue* post) {
    int mode = g_exhip_options.lean;
    if (mode == 0) return EXHIP_ERR_UNSUPPORTED;
    const bool with_post = post && (post->post_op || (post->residual_last && residual));
    if (with_post && (proj || mode == 3)) return EXHIP_ERR_UNSUPPORTED;
    if (post && post->post_op && (post->post_op < 1 || post->post_op > 1 + EXHIP_UNARY_CLIP || post->post_op == 1 + EXHIP_UNARY_SIGMOID))
        return EXHIP_ERR_UNSUPPORTED;
    if (proj) {
        // the projection's chunks ride along the persistent streamed form; the shortcut is computed, not read
        if (residual || y_nchw || !y_f || !y_q || !g.post_relu || g.act != 0 || !(g.fs_out > 0.f)) return EXHIP_ERR_UNSUPPORTED;
        if (!proj->x || !proj->wp || !proj->scale || proj->c_bytes % 64 != 0 || proj->c_bytes <= 0 || (proj->stride != 1 && proj->stride != 2) ||
            (proj->h - 1) / proj->stride + 1 != g.oh || (proj->w - 1) / proj->stride + 1 != g.ow || g.oh != g.h || g.ow != g.w ||
            proj->h >= 0x4000 || proj->w >= 0x4000 || (long long)proj->h * proj->w * proj->c_bytes >= 0x7FFFFF00ll)
            return EXHIP_ERR_UNSUPPORTED;
    }
    int cfg = g_exhip_options.lean_cfg;  // 0: one tile buffer, two slice buffers; 1: two and two; 2: one and three
    if (proj) {
        // two groups per CU (two accumulator sets fill the register file; what does not fit is reloaded where the one tile
        // buffer's refill is waited for anyway, which is why this form measured faster than two tile buffers)
        if (mode != 1 || cfg == 0) cfg = 2;
        mode = 1;
    }
    if (mode == 4) {
        // The form that measured fastest per layer class on the ResNet-18-shaped stack at 32 x 640 x 640: without a shortcut
        // the resident filter (64 channels) or one group per patch with three groups per CU, persistent groups with three
        // slice buffers from 512 channels on; with a shortcut see below.
        const int chunks = g.c_bytes / 64;
        if (!residual) {
            mode = chunks == 1 ? 1 : (chunks <= 4 ? 2 : 1);
            cfg = chunks <= 4 ? 0 : 2;
        } else if (chunks == 1 && !y_f && !y_nchw) {
            mode = 1;  // 64 channels, int8 result only (the block in front of a projection): the resident filter, 75 against 79 us
        } else {
            // float32 result next to the shortcut and at most 128 channels: the general kernel's three groups per CU keep
            // more of that traffic in flight. Otherwise one tile buffer and three slice buffers (128 channels, int8 result
            // only: 50 against 56 us in the general kernel; 256 channels: 38 against 39 us with two tile buffers).
            // On small maps (a detection network's 64-channel bottlenecks at 16 x 80 x 80: 27 against 34 us) the resident filter
            // wins with a float32 result as well.
            const bool small_map = chunks == 1 && (long long)g.n * g.oh * g.ow <= 262144;
            if (!small_map && chunks <= 2 && (y_f || y_nchw || chunks == 1)) return EXHIP_ERR_UNSUPPORTED;
            mode = 1;
            cfg = 2;
        }
    }
    const long long n_ptiles = (long long)g.n * g.tiles_y * g.tiles_x;
    const long long out_elems = (long long)g.n * g.oh * g.ow * g.k;
    if (g.c_bytes % 64 != 0 || g.k % 64 != 0 || g.ph * g.pw > 256 || g.ih * g.iw * kPixB + 16 > kActStride || n_ptiles >= 65536 ||
        g.h >= 0x4000 || g.w >= 0x4000 || g.ih >= 0x4000 || g.iw >= 0x4000 || g.ph >= 0x4000 || out_elems * 4 >= 0xFFFFF000ll ||
        out_elems >= (long long)kOobElem || (long long)g.h * g.w * g.c_bytes >= 0x7FFFFF00ll || g.act > 1 || g.ktiles != g.k / 64)
        return EXHIP_ERR_UNSUPPORTED;
    LeanParams p = {};
    p.x = (const char*)x; p.wp = (const char*)wp; p.scale = scale; p.bias = bias; p.residual = residual;
    p.y_q = y_q; p.y_f = y_f; p.y_nchw = y_nchw;
    p.H = g.h; p.W = g.w; p.K = g.k; p.OH = g.oh; p.OW = g.ow; p.PT = g.pt; p.PL = g.pl;
    p.C_b = g.c_bytes; p.n_chunks = g.c_bytes / 64;
    p.PH = g.ph; p.PW = g.pw; p.IH = g.ih; p.IW = g.iw;
    p.tiles_x = g.tiles_x; p.tiles_xy = g.tiles_x * g.tiles_y; p.ktiles = g.ktiles; p.n_ptiles = (int)n_ptiles;
    p.img_bytes = (unsigned)((size_t)g.h * g.w * g.c_bytes);
    p.out_elems = (unsigned)out_elems;
    auto magic = [](int d) { return (unsigned)(((1ull << 32) + d - 1) / d); };
    p.magic_iw = magic(g.iw); p.magic_pw = magic(g.pw); p.magic_tx = magic(g.tiles_x); p.magic_txy = magic(p.tiles_xy);
    p.adv_iy = 51 / g.iw; p.adv_ix = 51 % g.iw;
    p.fs_out = g.fs_out;
    p.dbg = g_lean_dbg;
    p.stagger = g_exhip_options.lean_stagger;
    if (proj) {
        p.ds_x = (const char*)proj->x; p.ds_wp = (const char*)proj->wp; p.ds_scale = proj->scale; p.ds_bias = proj->bias;
        p.ds_H = proj->h; p.ds_W = proj->w; p.ds_Cb = proj->c_bytes; p.ds_chunks = proj->c_bytes / 64; p.ds_stride = proj->stride;
        p.ds_img_bytes = (unsigned)((size_t)proj->h * proj->w * proj->c_bytes);
    }
    if (with_post) {
        p.post_op = post->post_op; p.post_alpha = post->post_alpha; p.post_beta = post->post_beta;
        p.residual_last = residual && post->residual_last;
    }
    const bool q_nonneg = g.fs_out > 0.f && !with_post && (g.post_relu || (g.act == 1 && !residual));
    p.flags = (residual ? E_RES : 0) | (y_f ? E_F : 0) | (y_q ? E_Q : 0) | (y_nchw ? E_NCHW : 0) | (g.act == 1 ? E_ACT : 0) |
              (g.post_relu ? E_POST : 0) | (q_nonneg ? E_QNN : 0);

    if (mode == 3) {
        // eight-wave groups, one per CU: MFMA waves and epilogue waves
        const long long total = n_ptiles * g.ktiles;
        long long G = total;
        if (total > 256) G = 256;   // 256 is a multiple of 8 x the slab counts this path meets
        if (G % g.ktiles != 0) G = G / g.ktiles * g.ktiles;
        if (G <= 0 || (G % 8 == 0 && (G / 8) % g.ktiles != 0 && G != total)) return EXHIP_ERR_UNSUPPORTED;
        if (g_exhip_options.lean_groups > 0 && G > (long long)g_exhip_options.lean_groups * g.ktiles)
            G = (long long)g_exhip_options.lean_groups * g.ktiles;
        if (g_exhip_options.debug_plan) fprintf(stderr, "  lean: wave-specialised, %lld groups for %lld tiles, flags %d\n", G, total, p.flags);
        if (p.n_chunks == 1 && g_exhip_options.lean_wres != 0) return launch_ws_epi<true>(ctx, p, (int)G);
        return launch_ws_epi<false>(ctx, p, (int)G);
    }
    // groups: as many as stay resident (persistent), or one per patch and slab (mode 2)
    const bool wres = p.n_chunks == 1 && g_exhip_options.lean_wres != 0 && !proj;
    const int per_cu = wres ? 2 : (cfg == 0 ? 3 : 2);
    const long long total = n_ptiles * g.ktiles;
    long long G = total;
    if (mode != 2 && total > per_cu * 256ll) {
        const long long unit = 8ll * g.ktiles;  // the XCD mapping and the slab of a group need whole units
        G = per_cu * 256ll / unit * unit;
        if (G <= 0) G = g.ktiles;
    }
    if (g_exhip_options.lean_groups > 0 && G > (long long)g_exhip_options.lean_groups * g.ktiles)
        G = (long long)g_exhip_options.lean_groups * g.ktiles;
    if (g_exhip_options.debug_plan)
        fprintf(stderr, "  lean: %s cfg %d, %lld groups for %lld tiles, flags %d\n", wres ? "resident filter" : "streamed filter", cfg, G, total,
                p.flags);
    if (proj) {
        constexpr int epi = E_F | E_Q | E_POST | E_QNN;
        if (p.flags != epi) return EXHIP_ERR_UNSUPPORTED;
        if (cfg == 1) return launch<false, 2, 2, epi, true>(ctx, p, (int)G);
        return launch<false, 1, 3, epi, true>(ctx, p, (int)G);
    }
    if (wres) return launch_epi<true, 1, 2>(ctx, p, (int)G);
    if (cfg == 1) return launch_epi<false, 2, 2>(ctx, p, (int)G);
    if (cfg == 2) return launch_epi<false, 1, 3>(ctx, p, (int)G);
    return launch_epi<false, 1, 2>(ctx, p, (int)G);
}

// The fp16 layer on the same kernel (E_HALF): half NHWC in, the general kernel's packed weights (64-channel slabs,
// 64-byte chunks = 32 channels), half NHWC out. Returns EXHIP_ERR_UNSUPPORTED outside what the kernel takes.
int exhip_conv3x3_f16_lean(exhip_ctx* ctx, const exhip_lean_geom& g, const exhip_lean_f16_epilogue& e, const uint16_t* x, const void* wp,
                           const float* bias, const uint16_t* residual, uint16_t* y) {
    if (g_exhip_options.lean == 0 || g_exhip_options.lean_f16 == 0) return EXHIP_ERR_UNSUPPORTED;
    const long long n_ptiles = (long long)g.n * g.tiles_y * g.tiles_x;
    const long long out_elems = (long long)g.n * g.oh * g.ow * g.k;
    if (g.c_bytes % 64 != 0 || g.k % 64 != 0 || g.ph * g.pw > 256 || g.ih * g.iw * kPixB + 16 > kActStride || n_ptiles >= 65536 ||
        g.h >= 0x4000 || g.w >= 0x4000 || g.ih >= 0x4000 || g.iw >= 0x4000 || g.ph >= 0x4000 || out_elems * 2 >= 0x7FFFF000ll ||
        (long long)g.h * g.w * g.c_bytes >= 0x7FFFFF00ll || g.act > 1 || g.ktiles != g.k / 64)
        return EXHIP_ERR_UNSUPPORTED;
    if (e.post_op && (e.post_op < 1 || e.post_op > 1 + EXHIP_UNARY_CLIP || e.post_op == 1 + EXHIP_UNARY_SIGMOID)) return EXHIP_ERR_UNSUPPORTED;
    LeanParams p = {};
    p.x = (const char*)x; p.wp = (const char*)wp; p.bias = bias; p.residual = reinterpret_cast<const float*>(residual);
    p.y_q = reinterpret_cast<int8_t*>(y);
    p.H = g.h; p.W = g.w; p.K = g.k; p.OH = g.oh; p.OW = g.ow; p.PT = g.pt; p.PL = g.pl;
    p.C_b = g.c_bytes; p.n_chunks = g.c_bytes / 64;
    p.PH = g.ph; p.PW = g.pw; p.IH = g.ih; p.IW = g.iw;
    p.tiles_x = g.tiles_x; p.tiles_xy = g.tiles_x * g.tiles_y; p.ktiles = g.ktiles; p.n_ptiles = (int)n_ptiles;
    p.img_bytes = (unsigned)((size_t)g.h * g.w * g.c_bytes);
    p.out_elems = (unsigned)out_elems;
    auto magic = [](int d) { return (unsigned)(((1ull << 32) + d - 1) / d); };
    p.magic_iw = magic(g.iw); p.magic_pw = magic(g.pw); p.magic_tx = magic(g.tiles_x); p.magic_txy = magic(p.tiles_xy);
    p.adv_iy = 51 / g.iw; p.adv_ix = 51 % g.iw;
    p.dbg = g_lean_dbg;
    p.post_op = e.post_op; p.post_alpha = e.post_alpha; p.post_beta = e.post_beta; p.residual_last = residual && e.residual_last;
    p.flags = E_HALF | (residual ? E_RES : 0) | (g.act == 1 ? E_ACT : 0) | (g.post_relu ? E_POST : 0);
    // the forms as for the int8 layers without a shortcut: the resident filter for one chunk, one group per patch up to
    // four chunks, persistent groups with three slice buffers beyond; lean_f16 = 2 / 3 / 4 pin the second / third / a
    // persistent two-slice form (tests)
    const int pin = g_exhip_options.lean_f16;
    const bool wres = p.n_chunks == 1 && g_exhip_options.lean_wres != 0 && pin == 1;
    const bool one_shot = pin == 2 || (pin == 1 && !wres && p.n_chunks <= 4);
    const bool three_slices = pin == 3 || (pin == 1 && !wres && !one_shot);
    const int per_cu = wres || three_slices ? 2 : 3;
    const long long total = n_ptiles * g.ktiles;
    long long G = total;
    if (!one_shot && total > per_cu * 256ll) {
        const long long unit = 8ll * g.ktiles;  // the XCD mapping and the slab of a group need whole units
        G = per_cu * 256ll / unit * unit;
        if (G <= 0) G = g.ktiles;
    }
    if (g_exhip_options.lean_groups > 0 && G > (long long)g_exhip_options.lean_groups * g.ktiles)
        G = (long long)g_exhip_options.lean_groups * g.ktiles;
    if (g_exhip_options.debug_plan)
        fprintf(stderr, "  lean fp16: %s, %lld groups for %lld tiles, flags %d\n",
                wres ? "resident filter" : one_shot ? "one group per patch" : three_slices ? "persistent, three slices" : "persistent, two slices", G,
                total, p.flags);
    if (wres) return launch<true, 1, 2, E_HALF>(ctx, p, (int)G);
    if (three_slices) return launch<false, 1, 3, E_HALF>(ctx, p, (int)G);
    return launch<false, 1, 2, E_HALF>(ctx, p, (int)G);
}
