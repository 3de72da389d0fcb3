// Dense convolution as an implicit GEMM on the gfx950 matrix cores.
//
// GEMM view: rows = output channels (the packed weights are the MFMA A operand), columns = output
// pixels (activations are the B operand), reduction = filter taps x input channels. One workgroup of
// 4 waves owns TM output channels x TN pixels of one image, where the pixels form a PH x PW patch so
// that the input halo is staged once in LDS and reused by every tap. The reduction walks "stages":
// (input-channel chunk, group of filter rows). Per stage the workgroup holds the weight slice for that
// chunk/rows in LDS, already in MFMA fragment order (the host packs it so), and per channel chunk the
// halo tile. The next stage's global loads are issued before the current stage's MFMAs and written to
// LDS afterwards.
//
// One k-step is 32 bytes of reduction per pixel: 32 int8 / 16 half / 8 float input channels of one
// tap ("generic" form), or, for first layers with <= 4 channels, one whole filter row of up to 8 (int8)
// or 4 (half) neighbouring pixels ("packed-row" form), which keeps the 7x7x3 stem from being padded
// out to 32 channels.
//
// MFMA 32x32 accumulator layout (verified on hardware): lane l, register i holds row
// 8*(i/4) + 4*(l/32) + i%4, column l%32. The host permutes the weight rows of each 32-channel tile so
// that a lane's 16 registers are 16 consecutive output channels of one pixel: NHWC stores are then
// 16-byte (int8) or 64-byte (f32) vectors.
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <type_traits>
#include <vector>

#include "common.h"
#include "conv_i8_lean.h"
#include "conv_pw.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

namespace {

constexpr int kMaxActVec = 12;   // loads per thread for one activation tile of one channel chunk (256-thread groups)
constexpr int kMaxWVec = 9;      // 16-byte weight vectors staged per thread and stage (256-thread groups)
constexpr int kMaxPackedPix = 8; // pixels staged per thread in packed-row form (256-thread groups)
constexpr unsigned kRsrcWord3 = 0x00020000u;  // raw buffer, 32-bit data format: out-of-range reads return 0
// per-wave LDS of the epilogue: a 32 x 64 float tile, a 32 x 64 int8 tile (rows padded by 16 bytes so that
// 16-byte accesses one row apart fall into different banks) and 32 pixel indices
constexpr int kEpiRowF = 64 * 4 + 16;
constexpr int kEpiRowQ = 64 + 16;
constexpr int kPoolRowB = 32 * 4 + 16;  // pooled epilogue: one tile pixel, 32 float32 channels + padding
constexpr int kEpiWaveBytes = 32 * kEpiRowF + 32 * kEpiRowQ + 128;
constexpr size_t kLdsLimit = 158 * 1024;  // dynamic LDS one group may use
constexpr size_t kLdsThird = 53 * 1024;   // at most this much each and three groups fit a CU's 160 KiB
constexpr size_t kLdsHalf = 80 * 1024;    // two groups per CU
constexpr long long kCUs = 256;           // compute units of the MI355X
constexpr int kSbBytes = 1024;  // LDS kept for per-channel scale and bias of the group's (at most 128) channels
// Phase timestamps (a development aid) are compiled in only with -DEXHIP_STAMPS=1: even as a never-taken branch
// they cost the stage loop scalar registers and a dozen instructions per stage.
#ifndef EXHIP_STAMPS
#define EXHIP_STAMPS 0
#endif
constexpr bool kStamps = EXHIP_STAMPS != 0;
constexpr unsigned kEpiInvalid = 0x3FFFFF00u;  // element offset whose byte offsets (x1, x4) lie past any accepted tensor

struct ConvParams {
    const char* x;
    const char* wp;
    const float* scale;
    const float* bias;
    const void* residual;
    void* y_q;       // i8: int8 NHWC ; f16: half NHWC ; f32: unused
    void* y_nhwc;    // f32 NHWC (i8 and f32 kernels)
    void* y_nchw;    // f32 NCHW
    void* y_nchw_h;  // half NCHW (f16 kernel)
    int32_t* acc_nchw;
    long long* dbg;  // optional phase timestamps (development aid), NULL in normal use
    int N, H, W, K, OH, OW;
    int KH, KWe, KS;          // filter rows, k-step groups per row (KW, or 1 packed), k-steps per chunk
    int S;                    // stride seen inside the staged tile
    int tile_step;            // input pixels between staged tile pixels (2 for 1x1 stride 2)
    int PT, PL;
    int cstride_b;            // bytes per input pixel
    int kstride;              // output channel stride (elements)
    int PH, PW, IH, IW;       // output patch and staged tile size in pixels
    int lds_pix_b, lds_row_b; // LDS bytes per tile pixel / row
    int lds_act_b;            // LDS bytes of one activation tile buffer
    int lds_w_b;              // LDS bytes of one weight stage buffer
    int act_bufs, w_bufs;     // 1, or 2 when consecutive chunks / stages alternate buffers
    int n_chunks, chunk_b;
    int RS, n_rg;             // filter rows per stage, stages per chunk
    int tiles_x, tiles_y, ktiles;
    int act, post_relu;
    int post_op;              // 0, or 1 + EXHIP_UNARY_*: the activation layer behind the convolution (general epilogue)
    int residual_last;        // the shortcut is added behind post_relu / post_op (general epilogue)
    float post_alpha, post_beta;
    const float* post_slope;  // post_op == EXHIP_POST_PRELU: slopes per output channel (one for all if post_slope_shared)
    int post_slope_shared;
    float fs_out;
    int b_align;              // alignment of B fragment reads in packed-row form (4, 8 or 16)
    unsigned img_bytes;       // bytes of one input image (buffer range for the bounds-checked loads)
    unsigned magic_iw, magic_pw; // ceil(2^32 / IW), ceil(2^32 / PW): exact quotients by one multiply-high for operands < 2^16
    unsigned magic_mpw;          // ceil(2^32 / MPW)
    int vp_shift;             // log2 of the 16-byte vectors per staged pixel
    int SL;                   // non-packed: 16-byte LDS slots per staged pixel (chunk / 16 + 1 padding slot)
    unsigned magic_sl;        // ceil(2^32 / SL)
    int adv_part, adv_pix;    // THREADS % SL, THREADS / SL: how (part, pixel) of a thread's slot advance per load
    int adv_iy, adv_ix;       // adv_pix / IW, adv_pix % IW: how the pixel's (row, column) advance
    int act_need_b;           // non-packed: bytes of one activation tile image in LDS (whole 16-byte slots)
    int epi_f;                // fused epilogue: the per-wave LDS tiles include the float32 one
    int epi_mode;             // which epilogue the launched kernel has (0 general, 1 fused, 2 pooled)
    int q_nonneg;             // fused epilogue: values reaching the quantizer are >= 0 (ReLU last, fs_out > 0)
    int tile_dy, tile_dx;     // output pixels between the origins of neighbouring patches (PH, PW unless pooled)
    int tile_oy, tile_ox;     // the first patch starts this many pixels before output pixel 0 (pooled form: the pool's padding)
    int MPH, MPW, POH, POW;   // pooled form: pooled pixels per patch and pooled image size
    // Split reduction (launches with too few tiles to fill the chip): `splits` groups share a tile, each reduces a run of
    // channel chunks and leaves its raw accumulators in split_acc; the group that arrives last at the tile's counter
    // adds the parts in split order and runs the epilogue. 1 = off.
    int splits;
    int* split_acc;           // [tile][split][16 vectors][THREADS][4] accumulator words (int32 or float bits)
    unsigned* split_count;    // [tile] arrivals, back to 0 when the tile is done
};

template <int DT> struct Acc { typedef v16i type; };
template <> struct Acc<EXHIP_F16> { typedef v16f type; };
template <> struct Acc<EXHIP_F32> { typedef v16f type; };

template <int DT>
__device__ __forceinline__ void mma(typename Acc<DT>::type& acc, const v4i& a, const v4i& b) {
    if constexpr (DT == EXHIP_I8) {
        acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc, 0, 0, 0);
    } else if constexpr (DT == EXHIP_F16) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), acc, 0, 0, 0);
    } else {
        const v4f af = __builtin_bit_cast(v4f, a), bf = __builtin_bit_cast(v4f, b);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af[e], bf[e], acc, 0, 0, 0);
    }
}

// n / d for n < 2^16 with magic = ceil(2^32 / d) as a 32-bit word: one multiply-high instead of an emulated division;
// d == 1 arrives as 0 (2^32 does not fit the word)
__device__ __forceinline__ int fast_div(int n, unsigned magic) { return magic ? (int)__umulhi((unsigned)n, magic) : n; }

__device__ __forceinline__ v4i lds_read16(const char* p) { return *reinterpret_cast<const v4i*>(p); }

__device__ __forceinline__ v4i lds_read16_unaligned(const char* p, int align) {
    v4i r;
    if (align >= 8) {
        const v2i lo = *reinterpret_cast<const v2i*>(p), hi = *reinterpret_cast<const v2i*>(p + 8);
        r[0] = lo[0]; r[1] = lo[1]; r[2] = hi[0]; r[3] = hi[1];
    } else {
        const int* q = reinterpret_cast<const int*>(p);
        r[0] = q[0]; r[1] = q[1]; r[2] = q[2]; r[3] = q[3];
    }
    return r;
}

// Orders a wave's LDS writes before its later LDS reads of other lanes' data. One wave runs in lockstep and
// the LDS serves a wave's accesses in issue order, so all that is needed is that the compiler keeps the
// order and that outstanding LDS operations have completed. A memory fence is deliberately not used: it would
// also wait for every outstanding global store, one full memory round trip per call.
__device__ __forceinline__ void wave_sync() {
    __asm__ volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
}

// sigmoid / mish evaluate double-precision transcendentals: kept out of line so the common epilogue stays small
__device__ __noinline__ float slow_activation(float v, int act) { return exhip_act(v, act); }

__device__ __forceinline__ float fast_activation(float v, int act) {
    if (act == 1) return (0.f > v) ? 0.f : v;
    if (act == 3) { const float d = (0.f > v) ? 0.f : v; return d <= 6.f ? d : 0.f; }
    return v;
}

// One 16-byte element per lane from a bounds-checked buffer view straight into LDS: lane l's data lands at
// lds_base + 16 * l (lds_base wave-uniform, in M0). Completion is counted by vmcnt like any other load.
__device__ __forceinline__ void async_load16(__amdgpu_buffer_rsrc_t rsrc, int voff, unsigned lds_base) {
    // no "memory" clobber: the LDS region written is not read before a later wait + barrier (which are
    // compiler barriers), and volatile keeps this ordered against them and against other loads of this kind
    __asm__ volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                     ::"s"(lds_base), "v"(voff), "s"(rsrc)
                     : "m0");
}

// Waits until at most `keep` of this wave's loads are in flight. The instruction takes an immediate, so a
// wave-uniform value selects one of seventeen waits (16 stands for "16 or more"): a computed jump into a table of
// (s_waitcnt, s_branch) pairs, eight bytes each. Written out by hand because the compiler turns the equivalent switch
// into a chain of some twenty-five scalar instructions and eight branches, once per stage of the convolution loop.
template <int N>
__device__ __forceinline__ void wait_vmcnt_imm() { __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
__device__ __forceinline__ void wait_vmcnt(int keep) {
    const int k = __builtin_amdgcn_readfirstlane(keep < 0 ? 0 : keep < 16 ? keep : 16);  // the jump must land inside the table
    int entry;
    __asm__ volatile(
        "s_getpc_b64 vcc\n\t"                    // address of the next instruction
        "s_lshl3_add_u32 %0, %1, 16\n\t"         // 8 * k + the 16 bytes from there to the table
        "s_add_u32 vcc_lo, vcc_lo, %0\n\t"
        "s_addc_u32 vcc_hi, vcc_hi, 0\n\t"
        "s_setpc_b64 vcc\n\t"
        "s_waitcnt vmcnt(0)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(1)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(2)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(3)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(4)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(5)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(6)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(7)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(8)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(9)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(10)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(11)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(12)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(13)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(14)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(15)\n\ts_branch .Lwait_done%=\n\t"
        "s_waitcnt vmcnt(16)\n"
        ".Lwait_done%=:"
        : "=&s"(entry)
        : "s"(k)
        : "vcc", "scc", "memory");
}

// The activation layer behind a convolution, applied in the convolution's epilogue to the values this layer would have
// stored: halves in the fp16 pipeline, so each value is rounded to half and widened again first. The sigmoid layer
// (double-precision exp) stays a layer of its own.
template <int OP, int DT>
__device__ __forceinline__ void post_activation_op(float (&v)[16], float alpha, float beta) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        float t = v[e];
        if constexpr (DT == EXHIP_F16) t = exhip_h2f(exhip_f2h(t));
        v[e] = unary_value<OP>(t, alpha, beta);
    }
}
template <int DT>
__device__ __forceinline__ void post_activation(float (&v)[16], int op, float alpha, float beta) {
    switch (op) {
    case EXHIP_UNARY_HARDSWISH: post_activation_op<0, DT>(v, alpha, beta); break;
    case EXHIP_UNARY_LEAKYRELU: post_activation_op<1, DT>(v, alpha, beta); break;
    case EXHIP_UNARY_HARDSIGMOID: post_activation_op<3, DT>(v, alpha, beta); break;
    default: post_activation_op<4, DT>(v, alpha, beta); break;
    }
}

// The same on four float32 values (the fused int8 epilogue works on vectors of four channels).
template <int OP>
__device__ __forceinline__ void post_activation4_op(v4f& v, float alpha, float beta) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = unary_value<OP>(v[e], alpha, beta);
}
// one switch per vector: a switch per value is a chain of wave-uniform branches around every operation
__device__ __forceinline__ void post_activation4(v4f& v, int op, float alpha, float beta) {
    switch (op) {
    case EXHIP_UNARY_HARDSWISH: post_activation4_op<0>(v, alpha, beta); break;
    case EXHIP_UNARY_LEAKYRELU: post_activation4_op<1>(v, alpha, beta); break;
    case EXHIP_UNARY_HARDSIGMOID: post_activation4_op<3>(v, alpha, beta); break;
    default: post_activation4_op<4>(v, alpha, beta); break;
    }
}

// KWE x KSC: the k-steps of one filter row (taps x 32-byte channel steps) when known at compile time, which
// turns every LDS fragment address of a row into an immediate offset; KWE == 0 keeps them as run-time values.
// LOWREG: held to 128 registers (a few spills) so that two 512-thread groups can share a CU.
template <int DT, int MT, int NT, int WM, int WN, bool PACKED, int EPI, int KWE, int KSC, bool LOWREG = false>
__global__ __launch_bounds__(64 * WM * WN, (MT * NT > 4 ? 1 : (LOWREG ? 4 : 2))) void conv_igemm_kernel(const ConvParams p) {
    constexpr int THREADS = 64 * WM * WN;
    constexpr int TM = 32 * MT * WM;
    // staging limits scale with the group size so that a 512-thread group needs half the registers
    constexpr int NAV = PACKED ? 1 : kMaxActVec * 256 / THREADS;  // asynchronous loads per thread and activation tile
    constexpr int NPP = PACKED ? kMaxPackedPix * 256 / THREADS : 1;
    constexpr int NWV = kMaxWVec * 256 / THREADS;
    typedef typename Acc<DT>::type acc_t;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // [scale, bias of this group's channels: 2 x 128 floats][activation buffers][weight buffers]
    float* const lds_sb = reinterpret_cast<float*>(smem);
    char* const lds_a0 = smem + kSbBytes;
    char* const lds_w0 = lds_a0 + p.act_bufs * p.lds_act_b;

    // wave-uniform values are pinned to scalar registers: a buffer resource built from a value the compiler keeps
    // in vector registers costs a serialising loop around every access
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    auto stamp = [&](int k) {
        if constexpr (kStamps)
            if (p.dbg && lane == 0) p.dbg[((size_t)blockIdx.x * (THREADS / 64) + wave) * 16 + k] = wall_clock64();
    };
    stamp(0);

    // Workgroup ids are dealt round-robin to the 8 XCDs; give each XCD one contiguous run of tiles so
    // that the channel tiles of a patch and its spatial neighbours share that XCD's L2.
    int bid = blockIdx.x;
    {
        const int per = gridDim.x >> 3;
        if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
    }
    // a split reduction's groups of one tile are neighbours in the grid
    const int sp = __builtin_amdgcn_readfirstlane(p.splits > 1 ? bid % p.splits : 0);
    if (p.splits > 1) bid /= p.splits;
    const int tile_id = bid;
    const int kt = __builtin_amdgcn_readfirstlane(bid % p.ktiles);
    int t = bid / p.ktiles;
    const int tx = __builtin_amdgcn_readfirstlane(t % p.tiles_x);
    t /= p.tiles_x;
    const int ty = __builtin_amdgcn_readfirstlane(t % p.tiles_y);
    const int n = __builtin_amdgcn_readfirstlane(t / p.tiles_y);
    const int oy0 = ty * p.tile_dy - p.tile_oy, ox0 = tx * p.tile_dx - p.tile_ox;
    const int iy0 = oy0 * p.S * p.tile_step - p.PT, ix0 = ox0 * p.S * p.tile_step - p.PL;

    // Bounds-checked buffer views: any offset at or past the range reads as zero, which is how halo
    // pixels outside the image and threads beyond the staged vector count are handled without branches.
    // The range check covers the per-lane offset only, so chunk and stage offsets go into the view's base.
    const char* const ximg = p.x + (size_t)n * p.img_bytes;

    // ---- staging plan (same for every chunk) ----
    // Non-packed form: operands travel from global memory straight into LDS (buffer loads with the LDS
    // modifier), no staging registers and no LDS store instructions. One such load moves 64 lanes x 16 bytes
    // to 1 KiB of consecutive LDS, so the LDS image of a tile is cut into 16-byte slots and slot v is fetched by
    // thread v % THREADS in its (v / THREADS)-th load. A pixel owns SL = chunk / 16 + 1 slots: its channel
    // chunk and one padding slot (the padding keeps the fragment reads of neighbouring pixels on different
    // banks); padding slots, halo pixels outside the image and slots past the tile get an offset beyond the
    // view's range and so are filled with zeros.
    // Packed form (first layer): 4- or 8-byte pixels through registers, as dword loads and LDS stores.
    int a_goff[PACKED ? NPP : NAV];
    int a_loff[PACKED ? NPP : 1];
    if constexpr (!PACKED) {
        // Slot tid + THREADS * i of the tile: its (pixel, part) and the pixel's (row, column) advance from one i to
        // the next by constants, so only the first needs divisions; all tests are evaluated without branches (a
        // branch per test costs more than the arithmetic it skips, and so do the re-fetches of the parameters a
        // branchy form makes).
        const int H = p.H, W = p.W, IW = p.IW, SL = p.SL, step = p.tile_step, cs_b = p.cstride_b, oob = (int)p.img_bytes;
        const int d_part = p.adv_part, d_pix = p.adv_pix, d_iy = p.adv_iy, d_ix = p.adv_ix;
        const int npix = p.IH * IW;
        int pix = fast_div(tid, p.magic_sl), part = tid - pix * SL;
        int iy = fast_div(pix, p.magic_iw), ix = pix - iy * IW;
#pragma unroll
        for (int i = 0; i < NAV; ++i) {
            // loads past the tile's last slot are never issued (the tile of a layer rarely needs all NAV): their two
            // dozen instructions are skipped as a whole, which a wave-uniform test per load does pay for
            if (i > 0 && i * THREADS * 16 >= p.act_need_b) {
                a_goff[i] = oob;
                continue;
            }
            const int gy = iy0 + iy * step, gx = ix0 + ix * step;
            const bool in_img = (pix < npix) & (part < SL - 1) & ((unsigned)gy < (unsigned)H) & ((unsigned)gx < (unsigned)W);
            const int off = (gy * W + gx) * cs_b + part * 16;
            a_goff[i] = in_img ? off : oob;
            part += d_part;
            const int carry = part >= SL ? 1 : 0;
            part -= carry ? SL : 0;
            pix += d_pix + carry;
            ix += d_ix + carry;
            iy += d_iy;
            const int wrap = ix >= IW ? 1 : 0;
            ix -= wrap ? IW : 0;
            iy += wrap;
        }
    } else {
        // the same without branches; pixel tid + THREADS * i advances by (adv_iy, adv_ix) per i
        const int H = p.H, W = p.W, IW = p.IW, cs_b = p.cstride_b, oob = (int)p.img_bytes, row_b = p.lds_row_b, pix_b = p.lds_pix_b;
        const int d_iy = p.adv_iy, d_ix = p.adv_ix;
        const int npix = p.IH * IW;
        int iy = fast_div(tid, p.magic_iw), ix = tid - iy * IW;
#pragma unroll
        for (int i = 0; i < NPP; ++i) {
            if (i > 0 && THREADS * i >= npix) {  // past the tile for every thread: skipped as a whole
                a_loff[i] = -1;
                a_goff[i] = oob;
                continue;
            }
            const int gy = iy0 + iy, gx = ix0 + ix;
            const bool in_tile = tid + THREADS * i < npix;
            const bool in_img = in_tile & ((unsigned)gy < (unsigned)H) & ((unsigned)gx < (unsigned)W);
            a_loff[i] = in_tile ? iy * row_b + ix * pix_b : -1;
            a_goff[i] = in_img ? (gy * W + gx) * cs_b : oob;
            ix += d_ix;
            iy += d_iy;
            const int wrap = ix >= IW ? 1 : 0;
            ix -= wrap ? IW : 0;
            iy += wrap;
        }
    }

    // per-lane B fragment offsets inside the tile and the lane's pixels
    int boff[NT];
    int pvalid = 0;
    int ppy[NT], ppx[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        int pp = (wn * NT + j) * 32 + (lane & 31);
        const bool ok = pp < p.PH * p.PW;
        pp = ok ? pp : 0;
        const int py = fast_div(pp, p.magic_pw), px = pp - py * p.PW;
        ppy[j] = py;
        ppx[j] = px;
        if (ok && (unsigned)(oy0 + py) < (unsigned)p.OH && (unsigned)(ox0 + px) < (unsigned)p.OW) pvalid |= 1 << j;
        boff[j] = py * p.S * p.lds_row_b + px * p.S * p.lds_pix_b + (lane >> 5) * 16;
    }
    const int aoff = wm * MT * 1024 + lane * 16;

    acc_t acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const int row_w_b = p.KWe * p.KS * (TM / 32) * 1024;  // packed weight bytes of one filter row
    // this group's run of channel chunks: all of them, or its share of a split reduction
    const int chunk0 = __builtin_amdgcn_readfirstlane(p.splits > 1 ? sp * p.n_chunks / p.splits : 0);
    const int my_chunks = __builtin_amdgcn_readfirstlane(p.splits > 1 ? (sp + 1) * p.n_chunks / p.splits - chunk0 : p.n_chunks);
    const int n_stages = my_chunks * p.n_rg;
    const char* const wkt = p.wp + ((size_t)kt * p.n_chunks + chunk0) * p.KH * row_w_b;
    auto stage_rows = [&](int rg) { const int r0 = rg * p.RS; return (p.KH - r0 < p.RS ? p.KH - r0 : p.RS); };
    // (chunk, row group) of the stage `by` stages after (cc, rg), without dividing
    auto stage_after = [&](int cc, int rg, int by, int& cc_out, int& rg_out) {
        for (int i = 0; i < by; ++i)
            if (++rg == p.n_rg) { rg = 0; ++cc; }
        cc_out = cc;
        rg_out = rg;
    };

    // ---- the MFMAs of one stage: k-steps in (row, tap, channel) order, fragments fetched one step ahead ----
    // wl: this wave's first weight fragment of the stage; al: the stage's first filter row in the activation tile;
    // nrows: filter rows in the stage
    auto mfma_stage = [&](const char* wl, const char* al, int nrows, auto&& after_first_row) {
        constexpr int NFB = 2;  // fragment buffers: the fetch of k-step s + 1 runs under the MFMAs of k-step s
        v4i af[NFB][MT], bf[NFB][NT];
        auto compute = [&](int buf) {
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int nn = 0; nn < NT; ++nn) mma<DT>(acc[m][nn], af[buf][m], bf[buf][nn]);
        };
        if constexpr (KWE > 0) {
            constexpr int NS = KWE * KSC;             // k-steps per filter row
            constexpr int STEPB = (TM / 32) * 1024;   // weight bytes per k-step
            constexpr int PIXB = PACKED ? 0 : KSC * 32 + 16;
            const char* ar[NT];
#pragma unroll
            for (int nn = 0; nn < NT; ++nn) ar[nn] = al + boff[nn];
            auto fetch_at = [&](int buf, const char* wrow, const char* const (&arow)[NT], int s_) {
                const int q_ = s_ / KSC, j_ = s_ % KSC;
#pragma unroll
                for (int m = 0; m < MT; ++m) af[buf][m] = lds_read16(wrow + s_ * STEPB + m * 1024);
#pragma unroll
                for (int nn = 0; nn < NT; ++nn) {
                    if constexpr (PACKED) bf[buf][nn] = lds_read16_unaligned(arow[nn], p.b_align);
                    else bf[buf][nn] = lds_read16(arow[nn] + q_ * PIXB + j_ * 32);
                }
            };
            {
                // One filter row, entered with k-step 0 already in buffer P0; leaves the next row's k-step 0 in
                // buffer (P0 + NS) & 1 when there is a next row. The callback runs once, between the first row
                // and the rest.
                auto row = [&](auto p0, bool has_next) {
                    constexpr int P0 = decltype(p0)::value;
                    const char* nr[NT];
#pragma unroll
                    for (int nn = 0; nn < NT; ++nn) nr[nn] = ar[nn] + p.lds_row_b;
#pragma unroll
                    for (int s_ = 0; s_ < NS; ++s_) {
                        if (s_ + 1 < NS) fetch_at((P0 + s_ + 1) & 1, wl, ar, s_ + 1);
                        else if (has_next) fetch_at((P0 + s_ + 1) & 1, wl + NS * STEPB, nr, 0);
                        // keep the order written here: the next k-step's fragment reads go out before this k-step's
                        // MFMAs and are waited for after them (left alone, the scheduler sinks the reads to their uses)
                        __builtin_amdgcn_sched_barrier(0);
                        compute((P0 + s_) & 1);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    wl += NS * STEPB;
#pragma unroll
                    for (int nn = 0; nn < NT; ++nn) ar[nn] = nr[nn];
                };
                fetch_at(0, wl, ar, 0);
                if constexpr (NS % 2 == 0) {
                    row(std::integral_constant<int, 0>{}, nrows > 1);
                    after_first_row();
                    for (int r = 1; r < nrows; ++r) row(std::integral_constant<int, 0>{}, r + 1 < nrows);
                } else {
                    row(std::integral_constant<int, 0>{}, nrows > 1);
                    after_first_row();
                    int r = 1;
                    for (; r + 1 < nrows; r += 2) {
                        row(std::integral_constant<int, 1>{}, true);
                        row(std::integral_constant<int, 0>{}, r + 2 < nrows);
                    }
                    if (r < nrows) row(std::integral_constant<int, 1>{}, false);
                }
            }
        } else {
            const int nk = nrows * p.KWe * p.KS;
            int q = 0, j = 0;          // tap column and channel k-step of the fragments being fetched
            int koff = 0;              // their byte offset inside the activation tile
            auto fetch = [&](int buf) {
#pragma unroll
                for (int m = 0; m < MT; ++m) af[buf][m] = lds_read16(wl + m * 1024);
#pragma unroll
                for (int nn = 0; nn < NT; ++nn) {
                    if constexpr (PACKED) bf[buf][nn] = lds_read16_unaligned(al + koff + boff[nn], p.b_align);
                    else bf[buf][nn] = lds_read16(al + koff + boff[nn]);
                }
                wl += (TM / 32) * 1024;
                // advance (j, q, row) and the tile offset
                if (++j == p.KS) {
                    j = 0;
                    koff += p.lds_pix_b - (p.KS - 1) * 32;
                    if (++q == p.KWe) {
                        q = 0;
                        koff += p.lds_row_b - p.KWe * p.lds_pix_b;
                    }
                } else {
                    koff += 32;
                }
            };
            fetch(0);
            after_first_row();
            int it = 0;
            for (; it + 2 <= nk - 1; it += 2) {
                fetch(1);
                compute(0);
                fetch(0);
                compute(1);
            }
            // 1 or 2 k-steps left; buffer 0 holds step `it`
            if (it + 1 < nk) {
                fetch(1);
                compute(0);
                compute(1);
            } else {
                compute(0);
            }
        }
    };

    stamp(1);
    // Per-channel scale and bias of this group's channels go to LDS for the epilogue. The load is issued here, ahead of
    // the staging requests, and its value is stored behind the wait for the first stage's operands (loads return in
    // order, so it has arrived by then): a wait here would put a whole memory round trip in front of the first request.
    float sb_value = 0.f;
    if constexpr (EPI >= 1) {
        if (tid < 2 * TM) {
            const int ch = kt * TM + (tid < TM ? tid : tid - TM);
            if (ch < p.K) sb_value = tid < TM ? p.scale[ch] : (p.bias ? p.bias[ch] : 0.f);
        }
    }
    auto publish_scale_bias = [&]() {
        if constexpr (EPI >= 1) {
            if (tid < 2 * TM) {
                lds_sb[(tid < TM ? 0 : 128) + (tid < TM ? tid : tid - TM)] = sb_value;
                if constexpr (EPI == 2) {
                    // pooled form: does any channel have a negative scale? (wave 0 holds all 64 scales; slot 64 is spare)
                    if (tid < TM) {
                        const unsigned long long neg = __ballot(__builtin_bit_cast(int, sb_value) < 0);
                        if (tid == 0) reinterpret_cast<int*>(lds_sb)[64] = neg != 0ull;
                    }
                }
            }
        }
    };

    if constexpr (!PACKED) {
        // ---- asynchronous pipeline ----
        // Weights of the stage `dist` stages ahead and the activation tile of the next chunk are requested while a
        // stage runs; weights rotate through up to three LDS buffers, activation tiles through two. The loads are
        // inline assembly the compiler does not track, so the waits are explicit: wave-uniform counters hold how
        // many loads this wave has issued after the last load of (a) the next stage's weights, (b) the weights
        // after those, (c) the next chunk's tile; the wait before the stage-end barrier lets exactly that many
        // stay in flight. A wave issues one load per 1 KiB piece of a tile or slice that starts inside the data.
        // All per-stage addresses are running values advanced by additions: a stage is short (24 MFMAs per wave
        // in a 3x3 layer), so scalar bookkeeping counts.
        const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
        const unsigned wave_slot = (unsigned)wave * 1024u;
        auto pieces = [&](int need_b) {
            const int left = need_b - wave * 1024;
            return left <= 0 ? 0 : (left + THREADS * 16 - 1) / (THREADS * 16);
        };
        const int w_stage_b = p.RS * row_w_b;  // one stage's weight slice, in memory and in LDS (RS divides KH)
        const int nal = pieces(p.act_need_b), nwl = pieces(w_stage_b);
        const int dist = p.w_bufs - 1;
        int after_w[2] = {0, 0}, after_act = 0;

        const char* w_src = wkt;                   // slice of the next stage to request (stages lie in request order)
        int w_req_left = n_stages;                 // stages not requested yet
        const unsigned w_lds0 = lds_base + kSbBytes + p.act_bufs * p.lds_act_b + wave_slot;
        const unsigned w_lds_end = w_lds0 + p.w_bufs * p.lds_w_b;
        unsigned w_dst = w_lds0;                   // where that slice goes
        auto request_w = [&](int slot) {
            if (w_req_left > 0) {
                // a view of exactly the slice: lanes past its end read zeros
                const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(w_src), 0, w_stage_b, kRsrcWord3);
                for (int i = 0; i < nwl; ++i) async_load16(wr, (tid + THREADS * i) * 16, w_dst + i * (THREADS * 16));
                after_w[0] += nwl; after_w[1] += nwl; after_act += nwl;
                after_w[slot] = 0;
                --w_req_left;
                w_src += w_stage_b;
                w_dst += p.lds_w_b;
                if (w_dst == w_lds_end) w_dst = w_lds0;
            }
        };
        const char* a_src = ximg + chunk0 * p.chunk_b;  // channel chunk of the next tile to request
        int a_range = (int)p.img_bytes - chunk0 * p.chunk_b;
        int a_req_left = my_chunks;
        unsigned a_dst = lds_base + kSbBytes + wave_slot;
        const unsigned a_flip = p.act_bufs > 1 ? (unsigned)p.lds_act_b : 0u;  // the two tile buffers alternate
        bool a_odd = false;
        auto request_a = [&]() {
            const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(a_src), 0, a_range, kRsrcWord3);
#pragma unroll
            for (int i = 0; i < NAV; ++i)
                if (i < nal) async_load16(xr, a_goff[i], a_dst + i * (THREADS * 16));
            after_w[0] += nal; after_w[1] += nal; after_act = 0;
            --a_req_left;
            a_src += p.chunk_b;
            a_range -= p.chunk_b;
            a_dst = a_odd ? a_dst - a_flip : a_dst + a_flip;
            a_odd = !a_odd;
        };
        request_a();
        request_w(0);
        if (dist == 2) request_w(0);
        stamp(2);
        wait_vmcnt(dist == 2 ? nwl : 0);
        publish_scale_bias();
        stamp(3);
        __syncthreads();
        stamp(4);
        const char* w_cur = lds_w0 + aoff;         // this wave's fragments in the current stage's buffer
        const char* const w_cur_end = w_cur + p.w_bufs * p.lds_w_b;
        const char* a_cur = lds_a0;                // current tile, first filter row of the current stage
        const int a_stage_b = p.RS * p.lds_row_b;
        bool cur_odd = false;
        // One stage. first_rg / next_chunk: it is the first / last stage of its channel chunk; nrows: its filter rows.
        // The three arrive as compile-time constants from the drivers below where the layer's shape fixes them: a stage
        // is two dozen MFMAs per wave, and every wave-uniform test the compiler can drop from it counts.
        auto stage = [&](int st, auto first_rg_t, auto next_chunk_t, auto nrows_t) {
            const bool first_rg = first_rg_t, next_chunk = next_chunk_t;
            const int nrows = nrows_t;
            const bool more = st + 1 < n_stages;
            // With one tile buffer the next chunk's tile can only be requested once every wave has left this chunk's
            // last stage (below); with two it is requested during the chunk's first stage.
            const bool want_a = p.act_bufs > 1 && first_rg && a_req_left > 0;
            // The requests go out after the stage's first filter row has been issued: their issue cost then
            // overlaps with MFMAs already in the pipe instead of standing in front of them. The request needed
            // sooner goes first, so that the wait below can leave the other in flight.
            auto requests = [&]() {
                if (want_a && next_chunk && dist == 2) request_a();
                if (dist > 0) request_w(dist - 1);
                if (want_a && !(next_chunk && dist == 2)) request_a();
            };
            long long t0 = 0, t1 = 0, t2 = 0;
            if (kStamps && p.dbg) t0 = wall_clock64();
            mfma_stage(w_cur, a_cur, nrows, requests);
            if (kStamps && p.dbg) t1 = wall_clock64();
            if (more) wait_vmcnt(next_chunk && after_act < after_w[0] ? after_act : after_w[0]);
            if (kStamps && p.dbg) t2 = wall_clock64();
            __syncthreads();
            if (kStamps && p.dbg && lane == 0) {
                const long long t3 = wall_clock64();
                long long* d = p.dbg + ((size_t)blockIdx.x * (THREADS / 64) + wave) * 16;
                d[9] += t1 - t0;
                d[10] += t2 - t1;
                d[11] += t3 - t2;
            }
            if (p.act_bufs == 1 && next_chunk && more) {
                // single tile buffer: refill it now and wait for it in the open; the other groups of the CU (this layout
                // is chosen where it lets a third one in) run meanwhile
                request_a();
                wait_vmcnt(0);
                __syncthreads();
            }
            after_w[0] = after_w[1];
            w_cur += p.lds_w_b;
            if (w_cur == w_cur_end) w_cur = lds_w0 + aoff;
            if (next_chunk) {
                a_cur = lds_a0 + (cur_odd ? 0 : a_flip);
                cur_odd = !cur_odd;
            } else {
                a_cur += a_stage_b;
            }
        };
        constexpr std::true_type yes{};
        constexpr std::false_type no{};
        constexpr std::integral_constant<int, 1> one_row{};
        bool done = false;
        if constexpr (EPI == 1 && KWE > 0) {
            if (p.n_rg == 3 && p.RS == 1) {  // three filter rows, one per stage (the 3x3 layers)
                for (int st = 0; st < n_stages; st += 3) {
                    stage(st, yes, no, one_row);
                    stage(st + 1, no, no, one_row);
                    stage(st + 2, no, yes, one_row);
                }
                done = true;
            } else if (p.n_rg == 1) {        // one stage per chunk (1x1 layers, 3x3 with all rows in a stage)
                for (int st = 0; st < n_stages; ++st) stage(st, yes, yes, p.RS);
                done = true;
            }
        }
        if (!done) {
            int rg = 0;
            for (int st = 0; st < n_stages; ++st) {
                const bool next_chunk = rg + 1 == p.n_rg;
                stage(st, rg == 0, next_chunk, p.RS);
                rg = next_chunk ? 0 : rg + 1;
            }
        }
    } else {
        // ---- register-staged pipeline (packed first-layer form) ----
        // Weights of stage st travel in set (st & 1); with DEEP the set of stage st + 2 is requested at the start
        // of stage st, so every load has one whole stage to land before it is needed.
        constexpr bool DEEP = THREADS == 512;
        int a_reg_p[NPP][2];
        v4i w_set0[NWV], w_set1[DEEP ? NWV : 1];
        auto load_act = [&]() {
            const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(ximg), 0, (int)p.img_bytes, kRsrcWord3);
#pragma unroll
            for (int i = 0; i < NPP; ++i) {
                a_reg_p[i][0] = __builtin_amdgcn_raw_buffer_load_b32(xr, a_goff[i], 0, 0);
                a_reg_p[i][1] = p.cstride_b == 8 ? __builtin_amdgcn_raw_buffer_load_b32(xr, a_goff[i] + 4, 0, 0) : 0;
            }
        };
        auto store_act = [&](char* dst) {
#pragma unroll
            for (int i = 0; i < NPP; ++i)
                if (a_loff[i] >= 0) {
                    *reinterpret_cast<int*>(dst + a_loff[i]) = a_reg_p[i][0];
                    if (p.cstride_b == 8) *reinterpret_cast<int*>(dst + a_loff[i] + 4) = a_reg_p[i][1];
                }
        };
        auto load_w = [&](int cc, int rg, auto& regs, bool valid) {
            // a view of exactly this stage's slice: lanes past its end read zeros; an invalid request gets a
            // zero-length view, so that every stage issues the same number of loads
            const __amdgpu_buffer_rsrc_t wr = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<char*>(wkt + (size_t)(cc * p.KH + rg * p.RS) * row_w_b), 0, valid ? stage_rows(rg) * row_w_b : 0, kRsrcWord3);
#pragma unroll
            for (int i = 0; i < NWV; ++i) regs[i] = __builtin_amdgcn_raw_buffer_load_b128(wr, (tid + THREADS * i) * 16, 0, 0);
        };
        auto store_w = [&](char* dst, auto& regs) {
#pragma unroll
            for (int i = 0; i < NWV; ++i) {
                const int v = (tid + THREADS * i) * 16;
                if (v < p.lds_w_b) *reinterpret_cast<v4i*>(dst + v) = regs[i];
            }
        };
        // One stage: request what later stages need, run the MFMAs of this one from LDS, then publish the next
        // stage's weights into the other LDS buffer. `mine` is the register set this stage's weights came in
        // (free again), `next` the set holding stage st + 1. The packed form has one channel chunk, so the
        // activation tile is staged once, before the first stage.
        auto run_stage = [&](int st, int cc, int rg, auto& mine, auto& next) {
            const bool more = st + 1 < n_stages;
            if constexpr (DEEP) {
                int c2, r2;
                stage_after(cc, rg, 2, c2, r2);
                load_w(c2, r2, mine, st + 2 < n_stages);
            } else {
                if (more) {
                    int c1, r1;
                    stage_after(cc, rg, 1, c1, r1);
                    load_w(c1, r1, next, true);
                }
            }
            mfma_stage(lds_w0 + (st & (p.w_bufs - 1)) * p.lds_w_b + aoff, lds_a0 + rg * p.RS * p.lds_row_b, stage_rows(rg), []() {});
            if (more) store_w(lds_w0 + ((st + 1) & (p.w_bufs - 1)) * p.lds_w_b, next);
            __syncthreads();
        };
        load_act();
        load_w(0, 0, w_set0, true);
        if constexpr (DEEP) {
            int c1, r1;
            stage_after(0, 0, 1, c1, r1);
            load_w(c1, r1, w_set1, n_stages > 1);
        }
        stamp(2);
        store_act(lds_a0);
        store_w(lds_w0, w_set0);
        publish_scale_bias();
        stamp(3);
        __syncthreads();
        stamp(4);
        int cc = 0, rg = 0;
        if constexpr (DEEP) {
            for (int st = 0; st < n_stages; st += 2) {
                run_stage(st, cc, rg, w_set0, w_set1);
                stage_after(cc, rg, 1, cc, rg);
                if (st + 1 < n_stages) {
                    run_stage(st + 1, cc, rg, w_set1, w_set0);
                    stage_after(cc, rg, 1, cc, rg);
                }
            }
        } else {
            for (int st = 0; st < n_stages; ++st) {
                run_stage(st, cc, rg, w_set0, w_set0);
                stage_after(cc, rg, 1, cc, rg);
            }
        }
    }

    stamp(5);
    if (p.splits > 1) {
        // every group leaves its accumulators (a lane's 64 words as 16 vectors, lanes contiguous per vector); the one
        // that finds the tile's counter at splits - 1 is the last: it adds the parts in split order, so the result
        // does not depend on who came last, and goes on to the epilogue
        // (the counter's value travels through the first word of the staging area: the loop ended with a barrier, so
        // nobody reads that area any more, and the epilogue's tiles are written only after this exchange)
        volatile unsigned* const arrived = reinterpret_cast<volatile unsigned*>(smem + kSbBytes);
        // The parts travel with the cache policy of device-scope atomic accesses (sc0 sc1: stores are written through,
        // loads are not served from a cache that another XCD's stores cannot reach), so that no fence has to write back
        // or invalidate a whole L2: all that is needed is that a group's stores have completed before its arrival counts.
        constexpr int kDeviceCoherent = 1 | 16;  // sc0 | sc1
        const unsigned part_b = 16u * THREADS * 16u;  // bytes of one group's part
        const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
            reinterpret_cast<char*>(p.split_acc) + (size_t)tile_id * p.splits * part_b, 0, (int)(p.splits * part_b), kRsrcWord3);
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    v4i v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const auto a = acc[i][j][e4 * 4 + e];  // a scalar copy: a bit cast of a vector element reads element 0
                        v[e] = __builtin_bit_cast(int, a);
                    }
                    __builtin_amdgcn_raw_buffer_store_b128(v, rs, (int)(((((i * NT + j) * 4 + e4) * THREADS) + tid) * 16u), (int)(sp * part_b),
                                                           kDeviceCoherent);
                }
        __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (tid == 0) *arrived = atomicAdd(p.split_count + tile_id, 1u);
        __syncthreads();
        const unsigned before_me = *arrived;
        __syncthreads();  // everyone has read the word before the epilogue reuses the area
        if (before_me != (unsigned)(p.splits - 1)) return;
        if (tid == 0) p.split_count[tile_id] = 0;  // ready for the next launch (launches on one stream run in order)
        for (int q = 0; q < p.splits; ++q) {
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < NT; ++j)
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4) {
                        const v4i v = __builtin_amdgcn_raw_buffer_load_b128(rs, (int)(((((i * NT + j) * 4 + e4) * THREADS) + tid) * 16u),
                                                                            (int)(q * part_b), kDeviceCoherent);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            typedef decltype(acc[i][j][0] + acc[i][j][0]) elem_t;
                            const int word = v[e];
                            const elem_t x = __builtin_bit_cast(elem_t, word);
                            acc[i][j][e4 * 4 + e] = q == 0 ? x : acc[i][j][e4 * 4 + e] + x;
                        }
                    }
        }
    }
    // ---- epilogue ----
    // A lane holds, per accumulator tile, 16 consecutive output channels of one pixel.
    const int img_px = p.OH * p.OW;
    if constexpr (EPI == 1) {
        // Fused int8 form (K a multiple of 64, channel stride == K): optional f32 NHWC shortcut input, optional
        // f32 NHWC and int8 NHWC outputs. A lane's own NHWC vectors lie a whole pixel apart from its neighbours',
        // so the three tensors go through a per-wave LDS tile of 32 pixels x 64 channels: lanes exchange rows
        // there and global memory sees 256 / 64 contiguous bytes per pixel. All global accesses are
        // bounds-checked buffer operations: a pixel outside the image gets an offset past the range, its
        // loads return 0 and its stores are dropped, so no lane-divergent branch is needed.
        // the staging buffers are free: the loop ended with a barrier. The float32 tile exists only when a
        // float32 tensor is read or written (the launch sizes the LDS accordingly).
        const int tile_f_b = p.epi_f ? 32 * kEpiRowF : 0;
        char* const epi = smem + kSbBytes + wave * (tile_f_b + 32 * kEpiRowQ + 128);
        char* const tile_f = epi;                       // [32 px][64 ch f32 + 16 B]
        char* const tile_q = epi + tile_f_b;            // [32 px][64 ch i8 + 16 B]
        unsigned* const table = reinterpret_cast<unsigned*>(epi + tile_f_b + 32 * kEpiRowQ);  // element offset per tile pixel
        const int chb = kt * TM + wm * 64;              // first channel of this wave's 64-channel slab
        const int px_l = lane & 31, hh = lane >> 5;
        const bool has_res = p.residual != nullptr, has_f = p.y_nhwc != nullptr, has_q = p.y_q != nullptr;
        const unsigned bytes_q = (unsigned)p.N * (unsigned)img_px * (unsigned)p.K;
        const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(p.y_q, 0, (int)bytes_q, kRsrcWord3);
        const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc(p.y_nhwc, 0, (int)(bytes_q * 4u), kRsrcWord3);
        const __amdgpu_buffer_rsrc_t rr =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.residual), 0, (int)(bytes_q * 4u), kRsrcWord3);
        const bool has_nchw = p.y_nchw != nullptr;
        const __amdgpu_buffer_rsrc_t rn = __builtin_amdgcn_make_buffer_rsrc(p.y_nchw, 0, (int)(bytes_q * 4u), kRsrcWord3);
        const int nt_run = chb < p.K ? NT : 0;  // a wave whose slab lies past the last channel has nothing to write
        // K a multiple of 32 only: the last slab holds 32 channels. Its rows in the tiles keep the 64-channel layout; the
        // pieces of a row past the last channel are not stored (they would land in the next pixel's row).
        const int live_ch = p.K - chb;
        const float act_floor = p.act == 1 ? 0.f : -__builtin_inff(), post_floor = p.post_relu ? 0.f : -__builtin_inff();
        const bool q_only = p.q_nonneg && has_q && !has_res && !has_f && !has_nchw;
#pragma unroll
        for (int nn = 0; nn < NT; ++nn) {
            if (nn >= nt_run) break;
            const bool valid = (pvalid >> nn) & 1;
            const unsigned pix = (unsigned)n * img_px + (oy0 + ppy[nn]) * p.OW + ox0 + ppx[nn];
            if (lane < 32) table[lane] = valid ? pix * (unsigned)p.K + chb : kEpiInvalid;
            const unsigned nchw0 = ((unsigned)n * (unsigned)p.K + chb) * (unsigned)img_px + (oy0 + ppy[nn]) * p.OW + ox0 + ppx[nn];
            wave_sync();
            if (has_res) {
                // offsets first, then all loads, then all LDS writes: the table lives in the same LDS as the tile,
                // and reading it between the writes would serialise load, wait and write
                unsigned goff[8];
#pragma unroll
                for (int it = 0; it < 8; ++it) goff[it] = (table[(it * 64 + lane) >> 4] + (lane & 15) * 4) * 4u;
                v4i rv[8];
#pragma unroll
                for (int it = 0; it < 8; ++it) rv[it] = __builtin_amdgcn_raw_buffer_load_b128(rr, (int)goff[it], 0, 0);
#pragma unroll
                for (int it = 0; it < 8; ++it) {
                    const int idx = it * 64 + lane, tp = idx >> 4, part = idx & 15;
                    *reinterpret_cast<v4i*>(tile_f + tp * kEpiRowF + part * 16) = rv[it];
                }
                wave_sync();
            }
            if (nn == 0) stamp(6);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                if (m * 32 >= live_ch) continue;  // wave-uniform: the slab's second block has no channel
                const int ch0 = chb + m * 32 + hh * 16;
                char* const tf = tile_f + px_l * kEpiRowF + (m * 32 + hh * 16) * 4;
                v4i q4;
                if (q_only) {
                    // int8 output only, ReLU last: q = trunc(max(v, 0) * fs + 0.5) capped at 127. With fs > 0 the
                    // maximum commutes with the product, and max(t, 0) + 0.5 == max(t + 0.5, 0.5) in float
                    // arithmetic (the sum is monotone in t), so one median does ReLU and saturation.
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4) {
                        const v4f s4 = *reinterpret_cast<const v4f*>(lds_sb + (ch0 - kt * TM) + e4 * 4);
                        const v4f b4 = *reinterpret_cast<const v4f*>(lds_sb + 128 + (ch0 - kt * TM) + e4 * 4);
                        int b[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float v = __builtin_fmaf((float)acc[m][nn][e4 * 4 + e], s4[e], b4[e]);
                            b[e] = (int)__builtin_amdgcn_fmed3f(v * p.fs_out + 0.5f, 0.5f, 127.f);
                        }
                        q4[e4] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                    }
                    *reinterpret_cast<v4i*>(tile_q + px_l * kEpiRowQ + m * 32 + hh * 16) = q4;
                    continue;
                }
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    const v4f s4 = *reinterpret_cast<const v4f*>(lds_sb + (ch0 - kt * TM) + e4 * 4);
                    const v4f b4 = *reinterpret_cast<const v4f*>(lds_sb + 128 + (ch0 - kt * TM) + e4 * 4);
                    v4f v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf((float)acc[m][nn][e4 * 4 + e], s4[e], b4[e]);
                    // ReLU as a maximum with 0, no ReLU as a maximum with -inf: one instruction either way
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaxf(v[e], act_floor);
                    v4f rv = {0.f, 0.f, 0.f, 0.f};
                    if (has_res) rv = *reinterpret_cast<const v4f*>(tf + e4 * 16);
                    if (has_res && !p.residual_last) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] += rv[e];
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaxf(v[e], post_floor);
                    // the activation layer behind the convolution, and the sum layer behind that one
                    if (p.post_op) post_activation4(v, p.post_op - 1, p.post_alpha, p.post_beta);
                    if (has_res && p.residual_last) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] += rv[e];
                    }
                    if (has_f) *reinterpret_cast<v4f*>(tf + e4 * 16) = v;
                    if (has_nchw) {
                        // the reference's boundary layout, straight from the registers: lanes run along pixels, so
                        // each store writes runs of consecutive floats of one channel plane
                        const v4i vi = __builtin_bit_cast(v4i, v);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const unsigned off = (nchw0 + (unsigned)((m * 32 + hh * 16 + e4 * 4 + e) * img_px)) * 4u;
                            __builtin_amdgcn_raw_buffer_store_b32(vi[e], rn, valid ? (int)off : (int)0xFFFFFF00u, 0, 0);
                        }
                    }
                    // float32_to_int8(v * fs): product rounded first, then +-0.5, saturate, truncate. After a
                    // final ReLU every product is >= 0: the sign select and the lower clamp fall away.
                    int b[4];
                    if (p.q_nonneg) {
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
                if (has_q) *reinterpret_cast<v4i*>(tile_q + px_l * kEpiRowQ + m * 32 + hh * 16) = q4;
            }
            wave_sync();
            if (nn == 0) stamp(7);
            if (has_f) {
#pragma unroll
                for (int it = 0; it < 8; ++it) {
                    const int idx = it * 64 + lane, tp = idx >> 4, part = idx & 15;
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const v4i*>(tile_f + tp * kEpiRowF + part * 16), rf,
                                                           (int)(((part * 4 < live_ch ? table[tp] : kEpiInvalid) + part * 4) * 4u), 0,
                                                           EXHIP_F32_STORE_AUX);
                }
            }
            if (has_q) {
#pragma unroll
                for (int it = 0; it < 2; ++it) {
                    const int idx = it * 64 + lane, tp = idx >> 2, part = idx & 3;
                    __builtin_amdgcn_raw_buffer_store_b128(*reinterpret_cast<const v4i*>(tile_q + tp * kEpiRowQ + part * 16), rq,
                                                           (int)((part * 16 < live_ch ? table[tp] : kEpiInvalid) + part * 16), 0, 0);
                }
            }
            wave_sync();  // the tiles and the table are rewritten by the next column block
        }
    } else if constexpr (EPI == 2) {
        // Convolution followed by a 3x3 stride-2 max pool (int8 path, TM == 64): the patch is (2 MPH + 1) x (2 MPW + 1)
        // convolution pixels, written as float32 into an LDS tile [pixel][32 channels]; pixels outside the
        // convolution's output hold -inf, which is how the pool's own padding drops out of the maximum. After a
        // barrier the MPH x MPW pooled pixels are formed from the tile and leave as NHWC float32 and / or int8.
        static_assert(TM == 64, "pooled epilogue: one 64-channel slab per group");
        // One pass per 32-channel block (an accumulator tile row): half the LDS of a 64-channel tile, which lets
        // more groups share a CU.
        char* const pool = smem + kSbBytes;
        const int px_l = lane & 31, hh = lane >> 5;
        const int npatch = p.PH * p.PW;
        const float ninf = -__builtin_inff();
        const unsigned out_px = (unsigned)p.N * (unsigned)(p.POH * p.POW);
        const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(p.y_q, 0, (int)(out_px * (unsigned)p.K), kRsrcWord3);
        const __amdgpu_buffer_rsrc_t rf = __builtin_amdgcn_make_buffer_rsrc(p.y_nhwc, 0, (int)(out_px * (unsigned)p.K * 4u), kRsrcWord3);
        const bool has_f = p.y_nhwc != nullptr, has_q = p.y_q != nullptr;
        const int items = p.MPH * p.MPW * 8;  // 4-channel vectors of the pooled patch, per 32-channel block
        // With a scale >= 0 the dequantization fmaf((float)acc, scale, bias) and the ReLU are non-decreasing in acc, so the
        // maximum can be taken on the int32 accumulators and only the pooled pixels are dequantized: the same values
        // (the float of the largest accumulator is the largest float), a quarter of the conversions. The tile then
        // holds int32 and INT_MIN marks pixels outside the convolution's output. Any negative scale (never the case
        // for scales made as 1 / (ws * fs), but allowed) selects the float form.
        const bool int_pool = reinterpret_cast<const int*>(lds_sb)[64] == 0;  // written before the stage loop's barriers
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m > 0) __syncthreads();  // the previous block's tile has been read
#pragma unroll
            for (int nn = 0; nn < NT; ++nn) {
                const int pp = (wn * NT + nn) * 32 + px_l;
                if (int_pool) {
                    if (pp < npatch) {
                        char* const dst = pool + pp * kPoolRowB + hh * 64;
                        if ((pvalid >> nn) & 1) {
#pragma unroll
                            for (int e4 = 0; e4 < 4; ++e4)
                                *reinterpret_cast<v4i*>(dst + e4 * 16) =
                                    v4i{acc[m][nn][e4 * 4], acc[m][nn][e4 * 4 + 1], acc[m][nn][e4 * 4 + 2], acc[m][nn][e4 * 4 + 3]};
                        } else {
                            const int lowest = (int)0x80000000;
#pragma unroll
                            for (int e4 = 0; e4 < 4; ++e4) *reinterpret_cast<v4i*>(dst + e4 * 16) = v4i{lowest, lowest, lowest, lowest};
                        }
                    }
                    continue;
                }
                // median(v, lo, hi): a valid pixel gets max(v, 0) with ReLU (lo = 0, hi = +inf) or v without
                // (lo = -inf); a pixel outside the convolution's output gets -inf (lo = hi = -inf)
                const bool valid = (pvalid >> nn) & 1;
                const float hi = valid ? __builtin_inff() : ninf, lo = (valid && p.act == 1) ? 0.f : ninf;
                const int c0 = m * 32 + hh * 16;
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    const v4f s4 = *reinterpret_cast<const v4f*>(lds_sb + c0 + e4 * 4);
                    const v4f b4 = *reinterpret_cast<const v4f*>(lds_sb + 128 + c0 + e4 * 4);
                    v4f v;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        v[e] = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)acc[m][nn][e4 * 4 + e], s4[e], b4[e]), lo, hi);
                    if (pp < npatch) *reinterpret_cast<v4f*>(pool + pp * kPoolRowB + (hh * 16 + e4 * 4) * 4) = v;
                }
            }
            __syncthreads();
            if (m == 0) stamp(6);
            for (int i = tid; i < items; i += THREADS) {
                const int pq = i >> 3, part = i & 7;
                const int pyy = fast_div(pq, p.magic_mpw), pxx = pq - pyy * p.MPW;
                const int gy = ty * p.MPH + pyy, gx = tx * p.MPW + pxx;
                const char* w0 = pool + ((2 * pyy) * p.PW + 2 * pxx) * kPoolRowB + part * 16;
                v4f best;
                if (int_pool) {
                    v4i top = *reinterpret_cast<const v4i*>(w0);
#pragma unroll
                    for (int dr = 0; dr < 3; ++dr)
#pragma unroll
                        for (int dc = 0; dc < 3; ++dc) {
                            if (dr == 0 && dc == 0) continue;
                            const v4i t = *reinterpret_cast<const v4i*>(w0 + (dr * p.PW + dc) * kPoolRowB);
#pragma unroll
                            for (int e = 0; e < 4; ++e) top[e] = top[e] > t[e] ? top[e] : t[e];
                        }
                    const v4f s4 = *reinterpret_cast<const v4f*>(lds_sb + m * 32 + part * 4);
                    const v4f b4 = *reinterpret_cast<const v4f*>(lds_sb + 128 + m * 32 + part * 4);
                    const float floor = p.act == 1 ? 0.f : ninf;
#pragma unroll
                    for (int e = 0; e < 4; ++e) best[e] = __builtin_fmaxf(__builtin_fmaf((float)top[e], s4[e], b4[e]), floor);
                } else {
                    best = *reinterpret_cast<const v4f*>(w0);
#pragma unroll
                    for (int dr = 0; dr < 3; ++dr)
#pragma unroll
                        for (int dc = 0; dc < 3; ++dc) {
                            if (dr == 0 && dc == 0) continue;
                            const v4f t = *reinterpret_cast<const v4f*>(w0 + (dr * p.PW + dc) * kPoolRowB);
#pragma unroll
                            for (int e = 0; e < 4; ++e) best[e] = __builtin_fmaxf(best[e], t[e]);
                        }
                }
                const bool ok = gy < p.POH && gx < p.POW;
                const unsigned elem = ((unsigned)(n * p.POH + gy) * (unsigned)p.POW + gx) * (unsigned)p.K + kt * TM + m * 32 + part * 4;
                const unsigned off = ok ? elem : kEpiInvalid;
                if (has_f) __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, best), rf, (int)(off * 4u), 0, 0);
                if (has_q) {
                    int b[4], packed;
                    if (p.q_nonneg) {  // after ReLU every maximum is >= 0
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
    } else {
        // General form: every output kind, ragged channel counts, direct per-lane accesses.
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const int ch0 = kt * TM + (wm * MT + m) * 32 + (lane >> 5) * 16;
            if (ch0 >= p.kstride && ch0 >= p.K) continue;
            float sc[16], bi[16];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int ch = ch0 + e;
                sc[e] = (DT == EXHIP_I8 && ch < p.K) ? p.scale[ch] : 0.f;
                bi[e] = (p.bias && ch < p.K) ? p.bias[ch] : 0.f;
            }
#pragma unroll
            for (int nn = 0; nn < NT; ++nn) {
                if (!((pvalid >> nn) & 1)) continue;
                const int oy = oy0 + ppy[nn], ox = ox0 + ppx[nn];
                const size_t pix = (size_t)n * img_px + (size_t)oy * p.OW + ox;
                const size_t nchw0 = ((size_t)n * p.K + ch0) * img_px + (size_t)oy * p.OW + ox;
                float v[16];
                if constexpr (DT == EXHIP_I8) {
                    if (p.acc_nchw) {
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            if (ch0 + e < p.K) p.acc_nchw[nchw0 + (size_t)e * img_px] = acc[m][nn][e];
                    }
#pragma unroll
                    for (int e = 0; e < 16; ++e) v[e] = __builtin_fmaf((float)acc[m][nn][e], sc[e], bi[e]);
                } else {
#pragma unroll
                    for (int e = 0; e < 16; ++e) v[e] = acc[m][nn][e] + bi[e];
                }
                if (p.act >= 4) {
#pragma unroll 1
                    for (int e = 0; e < 16; ++e) v[e] = slow_activation(v[e], p.act);
                } else if (p.act) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) v[e] = fast_activation(v[e], p.act);
                }
                auto add_shortcut = [&]() {
                    if constexpr (DT == EXHIP_F16) {
                        // the add layer behind this one reads the stored (rounded) half
                        const uint16_t* r = reinterpret_cast<const uint16_t*>(p.residual) + pix * p.kstride + ch0;
                        if (ch0 + 16 <= p.K) {  // 32 aligned bytes: two loads
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
                    } else {
                        const float* r = reinterpret_cast<const float*>(p.residual) + pix * p.kstride + ch0;
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            if (ch0 + e < p.K) v[e] += r[e];
                    }
                };
                if (p.residual && !p.residual_last) add_shortcut();
                if (p.post_relu) {
                    // a ReLU layer reads what this layer stored: in the fp16 pipeline the rounded half (a tiny negative
                    // value is -0 there and stays -0)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        if constexpr (DT == EXHIP_F16) v[e] = exhip_h2f(exhip_f2h(v[e]));
                        v[e] = (0.f > v[e]) ? 0.f : v[e];
                    }
                }
                if (p.post_op == EXHIP_POST_PRELU) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        float t = v[e];
                        if constexpr (DT == EXHIP_F16) t = exhip_h2f(exhip_f2h(t));
                        const float slope = p.post_slope[p.post_slope_shared || ch0 + e >= p.K ? 0 : ch0 + e];
                        v[e] = t >= 0.f ? t : slope * t;
                    }
                } else if (p.post_op) {
                    post_activation<DT>(v, p.post_op - 1, p.post_alpha, p.post_beta);
                }
                if (p.residual && p.residual_last) add_shortcut();
#pragma unroll
                for (int e = 0; e < 16; ++e)
                    if (ch0 + e >= p.K) v[e] = 0.f;  // pad channels hold zeros
                if (p.y_nchw) {
                    float* y = reinterpret_cast<float*>(p.y_nchw) + nchw0;
#pragma unroll
                    for (int e = 0; e < 16; ++e)
                        if (ch0 + e < p.K) y[(size_t)e * img_px] = v[e];
                }
                const bool vec_ok = ch0 + 16 <= p.kstride;
                if constexpr (DT == EXHIP_F16) {
                    if (p.y_nchw_h) {
                        uint16_t* y = reinterpret_cast<uint16_t*>(p.y_nchw_h) + nchw0;
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            if (ch0 + e < p.K) y[(size_t)e * img_px] = exhip_f2h(v[e]);
                    }
                    if (p.y_q && vec_ok) {
                        v4i o[2];
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            const uint32_t lo = exhip_f2h(v[2 * e]), hi = exhip_f2h(v[2 * e + 1]);
                            o[e >> 2][e & 3] = (int)(lo | (hi << 16));
                        }
                        char* const yb = reinterpret_cast<char*>(p.y_q) + ch0 * 2;
                        if (__builtin_amdgcn_ballot_w64(true) == ~0ull && (size_t)p.N * img_px < (1u << 31)) {
                            // the whole wave stores: a lane's 32 bytes and its neighbour's trade halves, so that four
                            // lanes (p, p + 1 and the same two of the other half-wave) write 64 contiguous bytes of one
                            // pixel per instruction instead of four 16-byte pieces of two
                            const bool odd = lane & 1;
                            pair_exchange4(o[0], o[1], odd);
                            const unsigned mine = (unsigned)pix, other = (unsigned)lane_neighbour((int)mine);
                            const size_t even_pix = odd ? other : mine, odd_pix = odd ? mine : other;
                            const int sub = odd ? 16 : 0;
                            *reinterpret_cast<v4i*>(yb + even_pix * p.kstride * 2 + sub) = o[0];
                            *reinterpret_cast<v4i*>(yb + odd_pix * p.kstride * 2 + sub) = o[1];
                        } else {
                            v4i* y = reinterpret_cast<v4i*>(yb + pix * p.kstride * 2);
                            y[0] = o[0];
                            y[1] = o[1];
                        }
                    }
                } else {
                    if (p.y_nhwc) {
                        float* y = reinterpret_cast<float*>(p.y_nhwc) + pix * p.kstride + ch0;
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
                    if constexpr (DT == EXHIP_I8) {
                        if (p.y_q && vec_ok) {
                            v4i o;
#pragma unroll
                            for (int e4 = 0; e4 < 4; ++e4) {
                                uint32_t w = 0;
#pragma unroll
                                for (int e = 0; e < 4; ++e) w |= (uint32_t)(exhip_q8(v[e4 * 4 + e] * p.fs_out) & 0xff) << (8 * e);
                                o[e4] = (int)w;
                            }
                            *reinterpret_cast<v4i*>(reinterpret_cast<int8_t*>(p.y_q) + pix * p.kstride + ch0) = o;
                        }
                    }
                }
            }
        }
    }
    stamp(8);
}

// ---- host side: configuration search, packing, launch ----

inline int esize_of(int dt) { return dt == EXHIP_I8 ? 1 : dt == EXHIP_F16 ? 2 : 4; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Tile variants: output channels x pixels per workgroup, and its wave grid. Every wave owns a 64 x 64
// accumulator tile (MT = NT = 2): 128 bytes of LDS reads per MFMA-cycle per CU at full rate, within
// what the LDS delivers, at 64 accumulator registers so that two waves fit per SIMD.
struct Variant { int TM, TN, threads; };
const Variant kVariants[] = {
    {64, 256, 256},   // 0: waves 1 x 4
    {128, 256, 512},  // 1: waves 2 x 4
    {128, 128, 256},  // 2: waves 2 x 2
};
constexpr int kNumVariants = 3;

struct Plan {
    bool packed;
    int variant;
    int TM, TN, threads;
    int KWe, KS, chunk_b, n_chunks, RS, n_rg;
    int S, tile_step, PH, PW, IH, IW, lds_pix_b, lds_row_b, lds_act_b, lds_w_b, b_align;
    int act_bufs, w_bufs;
    int SL, act_need_b;
    int tiles_x, tiles_y, ktiles;
    int OH, OW;
    int MPH, MPW;  // pooled form: pooled pixels per patch (0 otherwise); the patch is then (2 MPH + 1) x (2 MPW + 1)
    bool two_per_cu = false;  // a 512-thread plan whose launch counts on two groups per CU (the 128-register kernel)
    size_t staging_bytes() const { return (size_t)act_bufs * lds_act_b + (size_t)w_bufs * lds_w_b; }
    // What the launch asks for: the staging buffers, reused by the epilogue's tiles. epi_wave_b: bytes of LDS
    // each wave's epilogue uses.
    size_t launch_lds_bytes(int epi_wave_b) const {
        const size_t epilogue = MPH ? (size_t)PH * PW * kPoolRowB : (size_t)(threads / 64) * epi_wave_b;
        return kSbBytes + (staging_bytes() > epilogue ? staging_bytes() : epilogue);
    }
    // What planning assumes: the largest epilogue, so that the plan (and with it the weight packing) does
    // not depend on which outputs a call asks for.
    size_t lds_bytes() const { return launch_lds_bytes(kEpiWaveBytes); }
};

// A 3x3 stride-2 max pool fused behind the convolution: its top / left padding and its output size.
struct PoolSpec { int pt, pl, oh, ow; };

int validate(const exhip_conv_desc* d, int dt) {
    EXHIP_REQUIRE(d, "conv: NULL descriptor");
    EXHIP_REQUIRE(d->n > 0 && d->c > 0 && d->h > 0 && d->w > 0 && d->k > 0, "conv: empty shape");
    EXHIP_REQUIRE(d->kh > 0 && d->kw > 0 && d->sh > 0 && d->sw > 0, "conv: bad kernel/stride");
    EXHIP_REQUIRE(d->sh == d->sw, "conv: MFMA path needs equal strides (got %dx%d)", d->sh, d->sw);
    EXHIP_REQUIRE(d->pt >= 0 && d->pb >= 0 && d->pl >= 0 && d->pr >= 0, "conv: negative padding");
    EXHIP_REQUIRE(d->h + d->pt + d->pb >= d->kh && d->w + d->pl + d->pr >= d->kw, "conv: kernel larger than padded input");
    EXHIP_REQUIRE(d->c_stride >= d->c, "conv: c_stride %d < c %d", d->c_stride, d->c);
    const int es = esize_of(dt), cb = d->c_stride * es;
    const bool packed_ok = (cb == 4 && dt == EXHIP_I8 && d->kw <= 8) || (cb == 8 && dt == EXHIP_F16 && d->kw <= 4);
    EXHIP_REQUIRE(cb % 32 == 0 || packed_ok, "conv: input pixel is %d bytes; need a multiple of 32 (or the packed first-layer form)", cb);
    EXHIP_REQUIRE((long long)d->h * d->w * cb < (1ll << 31), "conv: one input image exceeds 2 GiB");
    return 0;
}

// Picks the tile variant, patch shape and staging split for a layer. Maximises the share of issued
// MFMA work that is useful, subject to the per-thread staging limits and the LDS size.
int make_plan(const exhip_conv_desc* d, int dt, Plan* out, const PoolSpec* pool = nullptr) {
    int rc = validate(d, dt);
    if (rc) return rc;
    Plan best;
    double best_score = -1e30;
    bool found = false;
    const int es = esize_of(dt), cb = d->c_stride * es;
    const int OH = (d->h + d->pt + d->pb - d->kh) / d->sh + 1, OW = (d->w + d->pl + d->pr - d->kw) / d->sw + 1;
    const bool packed = cb < 32;
    const int force_variant = g_exhip_options.force_variant, force_chunk = g_exhip_options.force_chunk;
    const int force_rs = g_exhip_options.force_rs, force_abufs = g_exhip_options.force_abufs;
    // With launches of other streams on the GPU a launch's own rounds stop mattering (whatever it leaves idle is taken):
    // one more group per CU is then worth the exposed tile loads whenever it fits.
    const bool crowd = g_exhip_options.share_gpu != 0 && force_abufs == 0;
    for (int vc = 0; vc < 2 * kNumVariants; ++vc) {
        const int variant = vc >> 1, chunk_opt = (vc & 1) ? 32 : 64;
        if (force_variant >= 0 && !pool && !packed && variant != force_variant) continue;  // not the first-layer forms
        if (force_chunk > 0 && !packed && chunk_opt != force_chunk) continue;
        if (pool && variant != 0) continue;  // the pooled epilogue holds one 64-channel slab per group
        if (packed && chunk_opt == 64) continue;
        if (!packed && cb % chunk_opt != 0) continue;
        const int TM = kVariants[variant].TM, TN = kVariants[variant].TN;
        const int ktiles = ceil_div(d->k, TM);
        Plan p;
        p.packed = packed;
        p.variant = variant;
        p.TM = TM;
        p.TN = TN;
        p.threads = kVariants[variant].threads;
        p.OH = OH;
        p.OW = OW;
        p.ktiles = ktiles;
        if (packed) {
            p.KWe = 1; p.KS = 1; p.chunk_b = 32; p.n_chunks = 1;
        } else {
            p.KWe = d->kw;
            p.chunk_b = chunk_opt;
            p.KS = p.chunk_b / 32;
            p.n_chunks = cb / p.chunk_b;
        }
        p.tile_step = (d->kh == 1 && d->kw == 1) ? d->sh : 1;
        p.S = d->sh / p.tile_step;
        const int row_w_b = p.KWe * p.KS * (TM / 32) * 1024;
        const int group_b = p.threads * 16;  // bytes one load per thread moves
        p.act_need_b = 0;
        p.SL = p.chunk_b / 16 + 1;
        if (packed) {
            // register-staged weights: whole 16-byte vectors per thread
            const int w_budget = (kMaxWVec * 256 / p.threads) * group_b;
            p.RS = w_budget / row_w_b;
            if (p.RS < 1) continue;                  // one filter row does not fit
            if (p.RS > d->kh) p.RS = d->kh;
            p.n_rg = ceil_div(d->kh, p.RS);
            p.lds_w_b = p.RS * row_w_b;
            p.act_bufs = 1;
            p.w_bufs = p.n_rg > 1 ? 2 : 1;
        }
        // Non-packed form: filter rows per stage. A stage should hold at least six k-steps (less leaves the
        // barrier and the load requests a large share of the stage); among such splits the finest one is
        // tried first, because it lets the MFMA loop start on less data and needs the least LDS.
        int rs_order[16], n_rs = 0;
        if (!packed) {
            for (int rs = 1; rs <= d->kh && n_rs < 16; ++rs)
                if (d->kh % rs == 0 && rs * p.KWe * p.KS >= 6) rs_order[n_rs++] = rs;
            for (int rs = d->kh; rs >= 1 && n_rs < 16; --rs)
                if (d->kh % rs == 0 && rs * p.KWe * p.KS < 6) rs_order[n_rs++] = rs;
        }
        p.MPH = p.MPW = 0;
        // fills the patch-dependent fields; false when the patch exceeds a staging or LDS limit
        auto shape_patch = [&](int PH, int PW) {
            const long long wgs = (long long)d->n * ceil_div(pool ? pool->oh : OH, pool ? std::max(1, (PH - 1) / 2) : PH) *
                                  ceil_div(pool ? pool->ow : OW, pool ? std::max(1, (PW - 1) / 2) : PW) * ktiles;
            p.PH = PH;
            p.PW = PW;
            p.IH = (PH - 1) * p.S + d->kh;
            if (packed) {
                const int slots = 32 / cb;
                p.IW = (PW - 1) * p.S + slots;
                p.lds_pix_b = cb;
                p.lds_row_b = (p.IW * cb + 15) / 16 * 16;
                const int step = p.S * cb;
                p.b_align = step % 16 == 0 ? 16 : step % 8 == 0 ? 8 : 4;
                if (p.IH * p.IW > kMaxPackedPix * 256) return false;
            } else {
                p.IW = (PW - 1) * p.S + d->kw;
                p.lds_pix_b = p.chunk_b + 16;
                p.lds_row_b = p.IW * p.lds_pix_b;
                p.b_align = 16;
                // the tile image plus the 16 bytes a lane may read past its last pixel, in whole 1 KiB pieces (one
                // wave-wide load each)
                p.act_need_b = p.IH * p.lds_row_b + 16;
                p.lds_act_b = (p.act_need_b + 1023) / 1024 * 1024;
                if ((p.act_need_b + group_b - 1) / group_b > kMaxActVec * 256 / p.threads) return false;
                if (p.lds_act_b / 16 >= (1 << 16)) return false;  // slot numbers are divided by multiply-high
                p.act_bufs = p.n_chunks > 1 ? 2 : 1;
                for (int i = 0; i < n_rs; ++i) {
                    p.RS = rs_order[i];
                    if (force_rs > 0 && d->kh % force_rs == 0 && p.RS != force_rs) continue;
                    p.n_rg = d->kh / p.RS;
                    p.lds_w_b = p.RS * row_w_b;
                    const int n_stages = p.n_chunks * p.n_rg;
                    // three weight buffers (requests two stages ahead) unless two let one more group share the CU
                    p.w_bufs = n_stages < 3 ? n_stages : 3;
                    if (p.w_bufs == 3) {
                        const size_t with3 = p.lds_bytes();
                        p.w_bufs = 2;
                        const size_t with2 = p.lds_bytes();
                        const bool fits3 = with3 <= kLdsLimit;
                        if (fits3 && kLdsLimit / with2 <= kLdsLimit / with3) p.w_bufs = 3;
                    }
                    const size_t room = p.threads == 512 ? kLdsHalf : kLdsThird;   // 512-thread groups: two per CU at most
                    const long long per_cu = p.threads == 512 ? 2 : 3;
                    if (p.n_chunks > 1 && p.lds_bytes() > room) {
                        // A single tile buffer if that lets three groups share the CU and the launch has the groups to
                        // use the room: three per CU must need fewer rounds than two, by more than the 15 % a group
                        // loses to the tile's load latency, then in the open at every chunk boundary.
                        const long long r2 = (wgs + (per_cu - 1) * kCUs - 1) / ((per_cu - 1) * kCUs), r3 = (wgs + per_cu * kCUs - 1) / (per_cu * kCUs);
                        const int w_bufs_before = p.w_bufs;
                        p.act_bufs = 1;
                        if (p.lds_bytes() > room && p.w_bufs == 3) p.w_bufs = 2;
                        if (force_abufs == 2 || p.lds_bytes() > room || (force_abufs != 1 && !crowd && r3 * 115 >= r2 * 100)) {
                            p.act_bufs = 2;
                            p.w_bufs = w_bufs_before;
                        }
                    }
                    if (p.lds_bytes() <= kLdsLimit) return true;
                }
                return false;
            }
            // the tile plus the 16 bytes a lane may read past its last row's last pixel
            p.lds_act_b = (p.IH * p.lds_row_b + 16 + 63) / 64 * 64;
            return p.lds_bytes() <= kLdsLimit;
        };
        // small preferences: 64-byte chunks halve the number of stages; two independent 256-thread groups per
        // CU overlap each other's barriers and load waits, which one 512-thread group cannot; the 128-pixel
        // variant has the least reuse per staged byte
        // A strided window stages four input pixels per output pixel: there the 512-thread variant with 32-byte
        // chunks does best (twice the outputs per staged tile, and the tile still leaves room for the weights).
        const bool strided_window = !packed && dt == EXHIP_I8 && p.S == 2 && d->kh > 1;  // measured on int8 layers
        const double prefs = -(chunk_opt == 32 ? 0.004 : 0.0) - (variant == 1 ? 0.002 : 0.0) - (variant == 2 ? 0.02 : 0.0) +
                             (strided_window && variant == 1 && chunk_opt == 32 ? 0.3 : 0.0);
        auto consider = [&](double score) {
            if (!found || score > best_score) {
                best_score = score;
                best = p;
                found = true;
            }
        };
        if (pool) {
            for (int MPW = 1; 2 * MPW + 1 <= TN / 3 && MPW <= pool->ow; ++MPW) {
                int MPH = (TN / (2 * MPW + 1) - 1) / 2;
                if (MPH > pool->oh) MPH = pool->oh;
                if (MPH < 1) continue;
                p.MPH = MPH;
                p.MPW = MPW;
                if (!shape_patch(2 * MPH + 1, 2 * MPW + 1)) continue;
                p.tiles_y = ceil_div(pool->oh, MPH);
                p.tiles_x = ceil_div(pool->ow, MPW);
                // four convolution pixels per pooled pixel are the useful part of a patch
                const double useful = 4.0 * pool->oh * pool->ow;
                const double issued = (double)p.tiles_y * p.tiles_x * TN;
                consider(useful / issued + prefs);
            }
            continue;
        }
        for (int PW = 1; PW <= TN && PW <= OW; ++PW) {
            int PH = TN / PW;
            if (PH > OH) PH = OH;
            if (PH < 1) continue;
            if (!shape_patch(PH, PW)) continue;
            p.tiles_y = ceil_div(OH, PH);
            p.tiles_x = ceil_div(OW, PW);
            const double useful = (double)OH * OW * d->k;
            const double issued = (double)p.tiles_y * p.tiles_x * TN * ktiles * TM;
            // prefer square-ish patches (less halo) at equal utilisation
            const double halo = (double)p.IH * p.IW / ((double)PH * PW * p.S * p.S);
            consider(useful / issued - 0.01 * halo + prefs);
        }
    }
    if (!found) {
        exhip_set_error("conv: no tile configuration fits (kernel %dx%d, pixel bytes %d)", d->kh, d->kw, cb);
        return EXHIP_ERR_UNSUPPORTED;
    }
    *out = best;
    if (g_exhip_options.debug_plan)
        fprintf(stderr, "plan %dx%dx%dx%d k%d %dx%d s%d%s: variant %d chunk %d RS %d patch %dx%d tile %dx%d act %d B x%d w %d B x%d lds %zu\n", d->n,
                d->c, d->h, d->w, d->k, d->kh, d->kw, d->sh, pool ? " +pool" : "", best.variant, best.chunk_b, best.RS, best.PH, best.PW,
                best.IH, best.IW, best.lds_act_b, best.act_bufs, best.lds_w_b, best.w_bufs, best.lds_bytes());
    return 0;
}

// Per kernel: on which devices its dynamic LDS limit has been raised (bit i = device i), guarded by one mutex.
std::mutex g_attr_mutex;

template <typename K>
int launch_kernel(exhip_ctx* ctx, K kernel, unsigned long long* attr_set, const Plan& pl, const ConvParams& p, int grid) {
    // per-wave epilogue LDS: none in the general form, the int8 tile and offset table in the fused form, plus
    // the float32 tile when a float32 tensor is read or written
    const int epi_wave_b = p.epi_mode == 0 ? 0 : (p.epi_f ? kEpiWaveBytes : 32 * kEpiRowQ + 128);
    {
        std::lock_guard<std::mutex> lock(g_attr_mutex);
        const unsigned long long bit = 1ull << (ctx->device & 63);
        if (!(*attr_set & bit)) {  // raise the dynamic LDS limit once per kernel and device
            EXHIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            *attr_set |= bit;
        }
    }
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(pl.threads), pl.launch_lds_bytes(epi_wave_b), ctx->stream, p);
    EXHIP_LAUNCH_CHECK();
    return 0;
}

template <int DT, int NT, int WM, int WN, bool PACKED, int EPI, int KWE, int KSC>
int launch_inst(exhip_ctx* ctx, const Plan& pl, const ConvParams& p, int grid) {
    if constexpr (WM * WN == 8 && !PACKED && EPI == 1 && KWE == 3) {
        if (pl.two_per_cu) {
            static unsigned long long attr_low = 0;
            return launch_kernel(ctx, conv_igemm_kernel<DT, 2, NT, WM, WN, PACKED, EPI, KWE, KSC, true>, &attr_low, pl, p, grid);
        }
    }
    static unsigned long long attr = 0;
    return launch_kernel(ctx, conv_igemm_kernel<DT, 2, NT, WM, WN, PACKED, EPI, KWE, KSC>, &attr, pl, p, grid);
}

// The row shapes with compile-time fragment addresses: 3 taps x 64-byte chunks (3x3 layers), 1 tap x 64-byte
// chunks (1x1 layers), and the packed first-layer form (one 32-byte k-step per filter row). Anything else
// runs the run-time form.
template <int DT, int NT, int WM, int WN, bool PACKED, int EPI>
int launch_shape(exhip_ctx* ctx, const Plan& pl, const ConvParams& p, int grid) {
    if constexpr (PACKED) {
        return launch_inst<DT, NT, WM, WN, true, EPI, 1, 1>(ctx, pl, p, grid);
    } else {
        if (pl.KWe == 3 && pl.KS == 2) return launch_inst<DT, NT, WM, WN, false, EPI, 3, 2>(ctx, pl, p, grid);
        if (pl.KWe == 3 && pl.KS == 1) return launch_inst<DT, NT, WM, WN, false, EPI, 3, 1>(ctx, pl, p, grid);
        if (pl.KWe == 1 && pl.KS == 2) return launch_inst<DT, NT, WM, WN, false, EPI, 1, 2>(ctx, pl, p, grid);
        return launch_inst<DT, NT, WM, WN, false, EPI, 0, 0>(ctx, pl, p, grid);
    }
}

template <int DT, bool PACKED, int EPI>
int launch_variant(exhip_ctx* ctx, const Plan& pl, const ConvParams& p, int grid) {
    switch (pl.variant) {
    case 0: return launch_shape<DT, 2, 1, 4, PACKED, EPI>(ctx, pl, p, grid);
    case 1: return launch_shape<DT, 2, 2, 4, PACKED, EPI>(ctx, pl, p, grid);
    default: return launch_shape<DT, 2, 2, 2, PACKED, EPI>(ctx, pl, p, grid);
    }
}

// The plan assumes the largest epilogue so that the weight packing does not depend on a call's outputs; the number of
// staging buffers does not enter the packing, so a launch that knows its epilogue's LDS may trade the second tile
// buffer (and the third weight buffer) for one more group per CU, under make_plan's rule: the extra group must save
// more rounds than the exposed tile loads cost. `fused_3x3`: the launch runs the fused int8 epilogue on a 3-tap row
// shape, the instantiations whose 512-thread form is held to 128 registers and so may run two groups per CU.
void rebuffer(Plan& pl, const exhip_conv_desc* d, int epi_wave_b, bool fused_3x3) {
    const int force_abufs = g_exhip_options.force_abufs;
    if (pl.packed || pl.MPH || pl.n_chunks < 2 || pl.act_bufs == 1 || force_abufs == 2) return;
    const long long cap = pl.threads == 512 ? (fused_3x3 ? 2 : 1) : 3;
    auto groups = [&](const Plan& q) {
        const long long g = (long long)(160 * 1024 / q.launch_lds_bytes(epi_wave_b));
        return std::max(1ll, std::min(g, cap));
    };
    Plan one = pl;
    one.act_bufs = 1;
    if (groups(one) <= groups(pl) && one.w_bufs == 3) one.w_bufs = 2;
    const long long g_now = groups(pl), g_one = groups(one);
    if (g_one <= g_now) return;
    const long long wgs = (long long)d->n * pl.tiles_y * pl.tiles_x * pl.ktiles;
    const long long r_now = (wgs + g_now * kCUs - 1) / (g_now * kCUs), r_one = (wgs + g_one * kCUs - 1) / (g_one * kCUs);
    if (force_abufs == 1 || (g_exhip_options.share_gpu != 0 && force_abufs == 0) || r_one * 115 < r_now * 100) {
        pl = one;
        pl.two_per_cu = pl.threads == 512;
        if (g_exhip_options.debug_plan)
            fprintf(stderr, "  launch: act x%d w x%d, %lld groups per CU instead of %lld (%lld groups, LDS %zu)\n", pl.act_bufs, pl.w_bufs,
                    g_one, g_now, wgs, pl.launch_lds_bytes(epi_wave_b));
    }
}

// The fused int8 epilogue takes: int8 / float32 NHWC tensors (and the NCHW float32 one), whole 32-channel blocks, plain or
// ReLU activation, the activation layers of the general epilogue other than PReLU, the shortcut on either side of them.
inline bool fused_epilogue_ok(const exhip_conv_desc* d, const ConvParams& p, long long out_elems) {
    return !p.acc_nchw && d->post_op != EXHIP_POST_PRELU && d->k % 32 == 0 && d->k_stride == d->k && d->act <= 1 && out_elems * 4 < 0xFFFFF000ll &&
           out_elems < (long long)kEpiInvalid;
}

template <int DT>
int run_conv(exhip_ctx* ctx, const exhip_conv_desc* d, ConvParams p, const PoolSpec* pool = nullptr, const exhip_lean_proj* proj = nullptr) {
    EXHIP_REQUIRE(ctx, "conv: NULL ctx");
    // a BatchNorm in the epilogue and writes limited to the layer's own channels: int8 pointwise layers only (below)
    if ((d->post_bn_a || d->post_bn_b || d->exact_k) && (DT != EXHIP_I8 || pool || proj)) return EXHIP_ERR_UNSUPPORTED;
    Plan pl;
    int rc = make_plan(d, DT, &pl, pool);
    if (rc) return rc;
    if constexpr (DT == EXHIP_I8) {
        if (!pool) {
            const long long elems = (long long)d->n * pl.OH * pl.OW * d->k;
            const bool fused = fused_epilogue_ok(d, p, elems);
            const int epi_wave_b = !fused ? 0 : ((p.residual || p.y_nhwc) ? kEpiWaveBytes : 32 * kEpiRowQ + 128);
            rebuffer(pl, d, epi_wave_b, fused && pl.KWe == 3);
        }
    }
    EXHIP_REQUIRE(p.x && p.wp, "conv: NULL input or weights");
    EXHIP_REQUIRE(d->k_stride >= d->k || (!p.y_q && !p.y_nhwc && !p.residual), "conv: k_stride %d < k %d", d->k_stride, d->k);
    EXHIP_REQUIRE(!(p.y_q) || d->k_stride % 16 == 0, "conv: NHWC int8/half output needs k_stride %% 16 == 0");
    EXHIP_REQUIRE((!p.scale || (uintptr_t)p.scale % 16 == 0) && (!p.bias || (uintptr_t)p.bias % 16 == 0),
                  "conv: scale and bias arrays must be 16-byte aligned");
    EXHIP_REQUIRE((uintptr_t)p.x % 16 == 0 && (uintptr_t)p.wp % 16 == 0, "conv: input and weights must be 16-byte aligned");
    p.N = d->n; p.H = d->h; p.W = d->w; p.K = d->k; p.OH = pl.OH; p.OW = pl.OW;
    p.KH = d->kh; p.KWe = pl.KWe; p.KS = pl.KS; p.S = pl.S; p.tile_step = pl.tile_step;
    p.PT = d->pt; p.PL = d->pl;
    p.cstride_b = d->c_stride * esize_of(DT);
    p.kstride = d->k_stride;
    p.PH = pl.PH; p.PW = pl.PW; p.IH = pl.IH; p.IW = pl.IW;
    p.lds_pix_b = pl.lds_pix_b; p.lds_row_b = pl.lds_row_b; p.lds_act_b = pl.lds_act_b; p.lds_w_b = pl.lds_w_b;
    p.act_bufs = pl.act_bufs; p.w_bufs = pl.w_bufs;
    p.n_chunks = pl.n_chunks; p.chunk_b = pl.chunk_b; p.RS = pl.RS; p.n_rg = pl.n_rg;
    p.tiles_x = pl.tiles_x; p.tiles_y = pl.tiles_y; p.ktiles = pl.ktiles;
    p.act = d->act; p.post_relu = d->post_relu; p.fs_out = d->fs_out; p.b_align = pl.b_align;
    p.post_op = d->post_op; p.post_alpha = d->post_alpha; p.post_beta = d->post_beta;
    p.residual_last = d->residual_last && p.residual;
    p.post_slope = d->post_slope; p.post_slope_shared = d->post_slope_shared;
    EXHIP_REQUIRE((d->post_op >= 0 && d->post_op <= 1 + EXHIP_UNARY_CLIP && d->post_op != 1 + EXHIP_UNARY_SIGMOID) ||
                      (d->post_op == EXHIP_POST_PRELU && d->post_slope),
                  "conv: post_op %d is not an activation the epilogue applies", d->post_op);
    p.dbg = (kStamps && getenv("EXHIP_DEBUG_STAMPS")) ? (long long*)strtoull(getenv("EXHIP_DEBUG_STAMPS"), nullptr, 0) : nullptr;
    p.img_bytes = (unsigned)((size_t)d->h * d->w * p.cstride_b);
    p.magic_iw = (unsigned)(((1ull << 32) + pl.IW - 1) / pl.IW);
    p.magic_pw = (unsigned)(((1ull << 32) + pl.PW - 1) / pl.PW);
    p.vp_shift = pl.chunk_b == 64 ? 2 : 1;
    p.SL = pl.SL; p.act_need_b = pl.act_need_b;
    p.magic_sl = (unsigned)(((1ull << 32) + pl.SL - 1) / pl.SL);
    p.adv_part = pl.threads % pl.SL; p.adv_pix = pl.packed ? pl.threads : pl.threads / pl.SL;  // packed: a slot is a pixel
    p.adv_iy = p.adv_pix / pl.IW; p.adv_ix = p.adv_pix % pl.IW;
    p.tile_dy = pl.PH; p.tile_dx = pl.PW;
    if (pool) {
        p.MPH = pl.MPH; p.MPW = pl.MPW; p.POH = pool->oh; p.POW = pool->ow;
        p.tile_dy = 2 * pl.MPH; p.tile_dx = 2 * pl.MPW; p.tile_oy = pool->pt; p.tile_ox = pool->pl;
        p.magic_mpw = (unsigned)(((1ull << 32) + pl.MPW - 1) / pl.MPW);
    }
    EXHIP_REQUIRE((long long)d->n * pl.OH * pl.OW < (1ll << 31), "conv: more than 2^31 output pixels");
    const long long tiles = (long long)d->n * pl.tiles_y * pl.tiles_x * pl.ktiles;
    EXHIP_REQUIRE(tiles > 0 && tiles < (1ll << 31), "conv: grid too large");
    if constexpr (DT == EXHIP_F16) {
        // 3x3 stride-1 layers with only the NHWC result: the lean kernel takes them with the same packed weights, also where
        // this kernel would split the reduction of a small launch (measured faster down to 25 tiles; below 16 tiles the
        // split keeps more CUs busy). EXHIP_ERR_UNSUPPORTED leaves the layer to this kernel.
        const int min_chunks_ = (3 + pl.n_rg - 1) / pl.n_rg;
        const bool would_split = g_exhip_options.force_splits != 1 && pl.n_chunks / min_chunks_ >= 2 && kCUs / tiles >= 2;
        if ((tiles >= 16 || !would_split) && g_exhip_options.force_splits <= 1) {
            if (!pl.packed && !pool && d->kh == 3 && d->kw == 3 && d->sh == 1 && d->sw == 1 && pl.variant == 0 && pl.chunk_b == 64 &&
                pl.RS == 1 && p.cstride_b % 64 == 0 && d->k % 64 == 0 && d->k_stride == d->k && d->act <= 1 && p.y_q && !p.y_nchw_h && !p.y_nchw &&
                d->post_op != EXHIP_POST_PRELU) {
                exhip_lean_geom g = {};
                g.n = d->n; g.h = d->h; g.w = d->w; g.c_bytes = p.cstride_b; g.k = d->k; g.oh = pl.OH; g.ow = pl.OW;
                g.pt = d->pt; g.pl = d->pl; g.ph = pl.PH; g.pw = pl.PW; g.ih = pl.IH; g.iw = pl.IW;
                g.tiles_x = pl.tiles_x; g.tiles_y = pl.tiles_y; g.ktiles = pl.ktiles;
                g.act = d->act; g.post_relu = d->post_relu;
                const exhip_lean_f16_epilogue e = {d->post_op, d->post_alpha, d->post_beta, d->residual_last};
                rc = exhip_conv3x3_f16_lean(ctx, g, e, reinterpret_cast<const uint16_t*>(p.x), p.wp, p.bias, reinterpret_cast<const uint16_t*>(p.residual),
                                            reinterpret_cast<uint16_t*>(p.y_q));
                if (rc != EXHIP_ERR_UNSUPPORTED) return rc;
            }
        }
    }
    // A launch with too few tiles for the chip's 256 CUs (one image, deep layers) walks its whole reduction on a handful
    // of groups, one stage after the other. Such a launch splits each tile's channel chunks over several groups (at least
    // three stages each, which the loop's prologue counts on), up to about two groups per CU; the parts are added in a
    // fixed order, exactly for int32 and reproducibly for float.
    p.splits = 1;
    if (!pl.packed && !pool && g_exhip_options.force_splits != 1) {
        const int min_chunks = (3 + pl.n_rg - 1) / pl.n_rg;
        long long s = std::min<long long>(pl.n_chunks / min_chunks, kCUs / tiles);  // measured: no gain once every CU has a group
        s = std::min<long long>(s, 16);
        if (g_exhip_options.force_splits > 1) s = std::min<long long>(g_exhip_options.force_splits, pl.n_chunks / min_chunks);
        s = std::min<long long>(s, kSplitGroups / tiles);  // the scratch holds kSplitGroups groups' accumulators, whatever forces the split
        if (s >= 2) {
            const size_t acc_bytes = (size_t)tiles * s * pl.threads * 256;  // 64 words per lane
            rc = exhip_split_scratch(ctx, acc_bytes, (size_t)tiles, &p.split_acc, &p.split_count);
            if (rc) return rc;
            p.splits = (int)s;
        }
    }
    const long long grid = tiles * p.splits;
    EXHIP_REQUIRE(grid < (1ll << 31), "conv: grid too large");
    if constexpr (DT == EXHIP_I8) {
        if (pool) {
            const long long out_elems = (long long)d->n * pool->oh * pool->ow * d->k;
            EXHIP_REQUIRE(out_elems * 4 < 0xFFFFF000ll && out_elems < (long long)kEpiInvalid, "conv+pool: output tensor too large");
            p.epi_mode = 2;
            p.q_nonneg = d->fs_out > 0.f && d->act == 1;
            if (pl.packed) return launch_shape<DT, 2, 1, 4, true, 2>(ctx, pl, p, (int)grid);
            return launch_shape<DT, 2, 1, 4, false, 2>(ctx, pl, p, (int)grid);
        }
        if (!pl.packed && !proj && d->kh == 1 && d->kw == 1 && d->sh == 1 && d->sw == 1 && !d->pt && !d->pb && !d->pl && !d->pr && !p.acc_nchw &&
            !p.y_nchw && (p.y_q || p.y_nhwc)) {
            // a pointwise layer with NHWC results only: the kernel without staging takes it with the same packed weights;
            // EXHIP_ERR_UNSUPPORTED leaves it to this one
            exhip_pw_geom g = {};
            g.pixels = (long long)d->n * d->h * d->w; g.c_bytes = p.cstride_b; g.k = d->k; g.k_stride = d->k_stride;
            g.slab_blocks = pl.TM / 32; g.slabs = pl.ktiles;
            g.act = d->act; g.post_relu = d->post_relu; g.post_op = d->post_op; g.post_slope_shared = d->post_slope_shared;
            g.post_alpha = d->post_alpha; g.post_beta = d->post_beta; g.post_slope = d->post_slope; g.residual_last = d->residual_last;
            g.fs_out = d->fs_out;
            g.post_bn_a = d->post_bn_a; g.post_bn_b = d->post_bn_b; g.exact_k = d->exact_k;
            rc = exhip_conv1x1_i8_pw(ctx, g, reinterpret_cast<const int8_t*>(p.x), p.wp, p.scale, p.bias, reinterpret_cast<const float*>(p.residual),
                                     reinterpret_cast<int8_t*>(p.y_q), reinterpret_cast<float*>(p.y_nhwc));
            if (rc != EXHIP_ERR_UNSUPPORTED) return rc;
        }
        if (d->post_bn_a || d->post_bn_b || d->exact_k) return EXHIP_ERR_UNSUPPORTED;  // only the pointwise kernel has these
        if (!pl.packed && !proj && !p.acc_nchw && !p.y_nchw && (p.y_q || p.y_nhwc) && pl.KWe == d->kw) {
            // a layer with a filter on that kernel's tapped form, where it takes the layer
            exhip_pw_geom g = {};
            g.pixels = (long long)d->n * pl.OH * pl.OW; g.c_bytes = p.cstride_b; g.k = d->k; g.k_stride = d->k_stride;
            g.slab_blocks = pl.TM / 32; g.slabs = pl.ktiles;
            g.act = d->act; g.post_relu = d->post_relu; g.post_op = d->post_op; g.post_slope_shared = d->post_slope_shared;
            g.post_alpha = d->post_alpha; g.post_beta = d->post_beta; g.post_slope = d->post_slope; g.residual_last = d->residual_last;
            g.fs_out = d->fs_out;
            const exhip_pw_taps t = {d->n, d->h, d->w, pl.OH, pl.OW, d->kh, d->kw, d->sh, d->pt, d->pl, pl.n_chunks, pl.chunk_b};
            rc = exhip_conv1x1_i8_pw(ctx, g, reinterpret_cast<const int8_t*>(p.x), p.wp, p.scale, p.bias, reinterpret_cast<const float*>(p.residual),
                                     reinterpret_cast<int8_t*>(p.y_q), reinterpret_cast<float*>(p.y_nhwc), &t);
            if (rc != EXHIP_ERR_UNSUPPORTED) return rc;
        }
        // the fused epilogue: int8 / float32 NHWC tensors only, whole 64-channel slabs, plain or ReLU activation
        const long long out_elems = (long long)d->n * pl.OH * pl.OW * d->k;
        const bool fused = fused_epilogue_ok(d, p, out_elems);
        // (also where this kernel would split the reduction of a small launch, down to 16 tiles: as for the fp16 layers above)
        if (fused && (!proj || (!d->post_op && !d->residual_last)) && !pl.packed && (p.splits == 1 || (tiles >= 16 && g_exhip_options.force_splits <= 1)) && d->kh == 3 && d->kw == 3 && d->sh == 1 && pl.variant == 0 && pl.chunk_b == 64 && pl.RS == 1 &&
            p.cstride_b % 64 == 0) {
            // the lean kernel takes these layers with the same packed weights; EXHIP_ERR_UNSUPPORTED leaves them to this one
            exhip_lean_geom g = {};
            g.n = d->n; g.h = d->h; g.w = d->w; g.c_bytes = p.cstride_b; g.k = d->k; g.oh = pl.OH; g.ow = pl.OW;
            g.pt = d->pt; g.pl = d->pl; g.ph = pl.PH; g.pw = pl.PW; g.ih = pl.IH; g.iw = pl.IW;
            g.tiles_x = pl.tiles_x; g.tiles_y = pl.tiles_y; g.ktiles = pl.ktiles;
            g.act = d->act; g.post_relu = d->post_relu; g.fs_out = d->fs_out;
            const exhip_lean_f16_epilogue post = {d->post_op, d->post_alpha, d->post_beta, d->residual_last};
            rc = exhip_conv3x3_i8_lean(ctx, g, reinterpret_cast<const int8_t*>(p.x), p.wp, p.scale, p.bias, reinterpret_cast<const float*>(p.residual),
                                       reinterpret_cast<int8_t*>(p.y_q), reinterpret_cast<float*>(p.y_nhwc), reinterpret_cast<float*>(p.y_nchw), proj,
                                       &post);
            if (rc != EXHIP_ERR_UNSUPPORTED || proj) return rc;
        }
        if (proj) return EXHIP_ERR_UNSUPPORTED;  // only the lean kernel computes a projection beside its own products
        if (fused) {
            p.epi_mode = 1;
            p.epi_f = p.residual || p.y_nhwc;
            p.q_nonneg = d->fs_out > 0.f && !d->post_op && ((d->post_relu && !p.residual_last) || (d->act == 1 && !p.residual));
            if (pl.packed) return launch_variant<DT, true, 1>(ctx, pl, p, (int)grid);
            return launch_variant<DT, false, 1>(ctx, pl, p, (int)grid);
        }
    }
    if constexpr (DT == EXHIP_F16) {
        if (!pl.packed && !pool && d->kh == 1 && d->kw == 1 && d->sh == 1 && d->sw == 1 && !d->pt && !d->pb && !d->pl && !d->pr && p.y_q &&
            !p.y_nchw_h && !p.y_nchw) {
            // a pointwise layer with only the NHWC result: the kernel without staging takes it with the same packed weights;
            // EXHIP_ERR_UNSUPPORTED leaves it to this one
            exhip_pw_geom g = {};
            g.pixels = (long long)d->n * d->h * d->w; g.c_bytes = p.cstride_b; g.k = d->k; g.k_stride = d->k_stride;
            g.slab_blocks = pl.TM / 32; g.slabs = pl.ktiles;
            g.act = d->act; g.post_relu = d->post_relu; g.post_op = d->post_op; g.post_slope_shared = d->post_slope_shared;
            g.post_alpha = d->post_alpha; g.post_beta = d->post_beta; g.post_slope = d->post_slope; g.residual_last = d->residual_last;
            rc = exhip_conv1x1_f16_pw(ctx, g, reinterpret_cast<const uint16_t*>(p.x), p.wp, p.bias, reinterpret_cast<const uint16_t*>(p.residual),
                                      reinterpret_cast<uint16_t*>(p.y_q));
            if (rc != EXHIP_ERR_UNSUPPORTED) return rc;
        } else if (!pl.packed && !pool && p.y_q && !p.y_nchw_h && !p.y_nchw && pl.KWe == d->kw) {
            // a layer with a filter on that kernel's tapped form, where it takes the layer
            exhip_pw_geom g = {};
            g.pixels = (long long)d->n * pl.OH * pl.OW; g.c_bytes = p.cstride_b; g.k = d->k; g.k_stride = d->k_stride;
            g.slab_blocks = pl.TM / 32; g.slabs = pl.ktiles;
            g.act = d->act; g.post_relu = d->post_relu; g.post_op = d->post_op; g.post_slope_shared = d->post_slope_shared;
            g.post_alpha = d->post_alpha; g.post_beta = d->post_beta; g.post_slope = d->post_slope; g.residual_last = d->residual_last;
            const exhip_pw_taps t = {d->n, d->h, d->w, pl.OH, pl.OW, d->kh, d->kw, d->sh, d->pt, d->pl, pl.n_chunks, pl.chunk_b};
            rc = exhip_conv1x1_f16_pw(ctx, g, reinterpret_cast<const uint16_t*>(p.x), p.wp, p.bias, reinterpret_cast<const uint16_t*>(p.residual),
                                      reinterpret_cast<uint16_t*>(p.y_q), &t);
            if (rc != EXHIP_ERR_UNSUPPORTED) return rc;
        }
    }
    if (pl.packed) return launch_variant<DT, true, 0>(ctx, pl, p, (int)grid);
    return launch_variant<DT, false, 0>(ctx, pl, p, (int)grid);
}

template <typename T>
void pack_weights_t(const exhip_conv_desc* d, int dt, const Plan& pl, const T* w, char* out) {
    const int es = esize_of(dt), cb = d->c_stride * es;
    const int mts = pl.TM / 32;
    const int C = d->c, K = d->k, KH = d->kh, KW = d->kw;
    size_t o = 0;
    for (int kt = 0; kt < pl.ktiles; ++kt)
        for (int cc = 0; cc < pl.n_chunks; ++cc)
            for (int r = 0; r < KH; ++r)
                for (int q = 0; q < pl.KWe; ++q)
                    for (int j = 0; j < pl.KS; ++j)
                        for (int mt = 0; mt < mts; ++mt)
                            for (int lane = 0; lane < 64; ++lane) {
                                const int rr = lane % 32, h = lane / 32;
                                const int chan = ((rr / 4) % 2) * 16 + (rr / 8) * 4 + (rr % 4);
                                const int k = kt * pl.TM + mt * 32 + chan;
                                for (int e = 0; e < 16 / es; ++e, o += es) {
                                    T val = 0;
                                    if (pl.packed) {
                                        const int byte = h * 16 + e * es;
                                        const int slot = byte / cb, c = (byte % cb) / es;
                                        if (k < K && slot < KW && c < C) val = w[(((size_t)k * C + c) * KH + r) * KW + slot];
                                    } else {
                                        const int c = (cc * pl.chunk_b + j * 32 + h * 16) / es + e;
                                        if (k < K && c < C) val = w[(((size_t)k * C + c) * KH + r) * KW + q];
                                    }
                                    memcpy(out + o, &val, es);
                                }
                            }
}

}  // namespace

int exhip_conv_packed_layout(const exhip_conv_desc* d, int dtype, int* slab_channels, int* packed_form) {
    Plan pl;
    const int rc = make_plan(d, dtype, &pl);
    if (rc) return rc;
    *slab_channels = pl.TM;
    *packed_form = pl.packed ? 1 : 0;
    return 0;
}

extern "C" int exhip_conv_out_hw(const exhip_conv_desc* d, int* oh, int* ow) {
    EXHIP_REQUIRE(d && oh && ow, "exhip_conv_out_hw: NULL argument");
    EXHIP_REQUIRE(d->sh > 0 && d->sw > 0, "exhip_conv_out_hw: bad stride");
    *oh = (d->h + d->pt + d->pb - d->kh) / d->sh + 1;
    *ow = (d->w + d->pl + d->pr - d->kw) / d->sw + 1;
    return 0;
}

extern "C" size_t exhip_conv_packed_bytes(const exhip_conv_desc* d, int dtype) {
    Plan pl;
    if (dtype < 0 || dtype > 2 || make_plan(d, dtype, &pl)) return 0;
    return (size_t)pl.ktiles * pl.n_chunks * d->kh * pl.KWe * pl.KS * (pl.TM / 32) * 1024;
}

extern "C" int exhip_conv_pack_weights(const exhip_conv_desc* d, int dtype, const void* w, void* packed) {
    EXHIP_REQUIRE(w && packed, "exhip_conv_pack_weights: NULL argument");
    EXHIP_REQUIRE(dtype >= 0 && dtype <= 2, "exhip_conv_pack_weights: bad dtype %d", dtype);
    Plan pl;
    int rc = make_plan(d, dtype, &pl);
    if (rc) return rc;
    if (dtype == EXHIP_I8) pack_weights_t<int8_t>(d, dtype, pl, (const int8_t*)w, (char*)packed);
    else if (dtype == EXHIP_F16) pack_weights_t<uint16_t>(d, dtype, pl, (const uint16_t*)w, (char*)packed);
    else pack_weights_t<float>(d, dtype, pl, (const float*)w, (char*)packed);
    return 0;
}

extern "C" int exhip_conv2d_i8(exhip_ctx* ctx, const exhip_conv_desc* d, const int8_t* x, const void* wp,
                               const float* scale, const float* bias, const float* residual, int8_t* y_i8,
                               float* y_f32_nhwc, float* y_f32_nchw, int32_t* acc_nchw) {
    EXHIP_REQUIRE(scale, "exhip_conv2d_i8: NULL scale");
    EXHIP_REQUIRE(y_i8 || y_f32_nhwc || y_f32_nchw || acc_nchw, "exhip_conv2d_i8: no output requested");
    ConvParams p = {};
    p.x = (const char*)x; p.wp = (const char*)wp; p.scale = scale; p.bias = bias; p.residual = residual;
    p.y_q = y_i8; p.y_nhwc = y_f32_nhwc; p.y_nchw = y_f32_nchw; p.acc_nchw = acc_nchw;
    return run_conv<EXHIP_I8>(ctx, d, p);
}

// A residual block's second convolution with the block's projection shortcut computed in the same kernel: what
// exhip_conv2d_i8 would do for the 1x1 layer (float32 result, no activation) and then for the 3x3 layer with that result
// as `residual`, without the float32 tensor between them. EXHIP_ERR_UNSUPPORTED (and nothing launched) outside the
// shapes the lean kernel takes; the caller then issues the two calls.
extern "C" int exhip_conv2d_i8_projection(exhip_ctx* ctx, const exhip_conv_desc* d, const int8_t* x, const void* wp, const float* scale,
                                          const float* bias, const exhip_conv_desc* d_proj, const int8_t* x_proj, const void* wp_proj,
                                          const float* scale_proj, const float* bias_proj, int8_t* y_i8, float* y_f32_nhwc) {
    EXHIP_REQUIRE(d && d_proj && scale && scale_proj && x_proj && wp_proj, "exhip_conv2d_i8_projection: NULL argument");
    EXHIP_REQUIRE(y_i8 && y_f32_nhwc, "exhip_conv2d_i8_projection: both outputs are required");
    if (d->kh != 3 || d->kw != 3 || d->sh != 1 || d->sw != 1 || d->act != 0 || !d->post_relu || d->post_op || !(d->fs_out > 0.f) ||
        d->k % 64 != 0 || d->k_stride != d->k)
        return EXHIP_ERR_UNSUPPORTED;
    if (d_proj->kh != 1 || d_proj->kw != 1 || d_proj->sh != d_proj->sw || (d_proj->sh != 1 && d_proj->sh != 2) || d_proj->pt || d_proj->pb ||
        d_proj->pl || d_proj->pr || d_proj->act != 0 || d_proj->post_relu || d_proj->post_op || d_proj->k != d->k || d_proj->n != d->n ||
        d_proj->c_stride % 64 != 0 || d_proj->c_stride != d_proj->c)
        return EXHIP_ERR_UNSUPPORTED;
    // the 1x1 layer's packed weights must be the 64-channel-slab, 64-byte-chunk form: 4 KiB per slab and chunk
    Plan pp;
    int rc = make_plan(d_proj, EXHIP_I8, &pp);
    if (rc) return rc;
    if (pp.packed || pp.TM != 64 || pp.chunk_b != 64 || pp.KWe != 1 || pp.KS != 2 || pp.n_chunks != d_proj->c_stride / 64) return EXHIP_ERR_UNSUPPORTED;
    exhip_lean_proj proj = {};
    proj.x = x_proj; proj.wp = wp_proj; proj.scale = scale_proj; proj.bias = bias_proj;
    proj.h = d_proj->h; proj.w = d_proj->w; proj.c_bytes = d_proj->c_stride; proj.stride = d_proj->sh;
    ConvParams p = {};
    p.x = (const char*)x; p.wp = (const char*)wp; p.scale = scale; p.bias = bias;
    p.y_q = y_i8; p.y_nhwc = y_f32_nhwc;
    return run_conv<EXHIP_I8>(ctx, d, p, nullptr, &proj);
}

extern "C" int exhip_conv2d_i8_maxpool3x3s2(exhip_ctx* ctx, const exhip_conv_desc* d, int pool_pt, int pool_pl, int pool_oh,
                                            int pool_ow, const int8_t* x, const void* wp, const float* scale,
                                            const float* bias, int8_t* y_i8, float* y_f32_nhwc) {
    EXHIP_REQUIRE(d && scale, "exhip_conv2d_i8_maxpool3x3s2: NULL descriptor or scale");
    EXHIP_REQUIRE(y_i8 || y_f32_nhwc, "exhip_conv2d_i8_maxpool3x3s2: no output requested");
    EXHIP_REQUIRE(d->k % 64 == 0 && d->k_stride == d->k, "conv+pool: needs k %% 64 == 0 and k_stride == k (k %d, k_stride %d)", d->k, d->k_stride);
    EXHIP_REQUIRE(d->act <= 1 && !d->post_relu && !d->post_op, "conv+pool: activation must be none or ReLU");
    int oh = 0, ow = 0;
    int rc = exhip_conv_out_hw(d, &oh, &ow);
    if (rc) return rc;
    // every pooled window must hold at least one convolution pixel, as the reference's pooling guarantees
    EXHIP_REQUIRE(pool_pt >= 0 && pool_pt <= 1 && pool_pl >= 0 && pool_pl <= 1, "conv+pool: pool padding must be 0 or 1");
    EXHIP_REQUIRE(pool_oh > 0 && pool_ow > 0 && 2 * (pool_oh - 1) - pool_pt < oh && 2 * (pool_ow - 1) - pool_pl < ow,
                  "conv+pool: pooled size %dx%d does not fit a %dx%d convolution output", pool_oh, pool_ow, oh, ow);
    // same packed weights as exhip_conv2d_i8: the unpooled plan must use 64-channel slabs too
    Plan plain;
    rc = make_plan(d, EXHIP_I8, &plain);
    if (rc) return rc;
    if (plain.TM != 64) {
        exhip_set_error("conv+pool: this layer's weights are packed for %d-channel slabs", plain.TM);
        return EXHIP_ERR_UNSUPPORTED;
    }
    const PoolSpec pool = {pool_pt, pool_pl, pool_oh, pool_ow};
    Plan pooled;
    rc = make_plan(d, EXHIP_I8, &pooled, &pool);
    if (rc) return rc;
    if (pooled.chunk_b != plain.chunk_b || pooled.n_chunks != plain.n_chunks || pooled.KWe != plain.KWe || pooled.KS != plain.KS) {
        exhip_set_error("conv+pool: the pooled tiling needs a different weight packing than exhip_conv_pack_weights produced");
        return EXHIP_ERR_UNSUPPORTED;
    }
    ConvParams p = {};
    p.x = (const char*)x; p.wp = (const char*)wp; p.scale = scale; p.bias = bias;
    p.y_q = y_i8; p.y_nhwc = y_f32_nhwc;
    return run_conv<EXHIP_I8>(ctx, d, p, &pool);
}

extern "C" int exhip_conv2d_f16(exhip_ctx* ctx, const exhip_conv_desc* d, const uint16_t* x, const void* wp,
                                const float* bias, const uint16_t* residual, uint16_t* y_f16_nhwc,
                                uint16_t* y_f16_nchw, float* y_f32_nchw) {
    EXHIP_REQUIRE(y_f16_nhwc || y_f16_nchw || y_f32_nchw, "exhip_conv2d_f16: no output requested");
    ConvParams p = {};
    p.x = (const char*)x; p.wp = (const char*)wp; p.bias = bias; p.residual = residual;
    p.y_q = y_f16_nhwc; p.y_nchw_h = y_f16_nchw; p.y_nchw = y_f32_nchw;
    return run_conv<EXHIP_F16>(ctx, d, p);
}

extern "C" int exhip_conv2d_f32(exhip_ctx* ctx, const exhip_conv_desc* d, const float* x, const void* wp,
                                const float* bias, const float* residual, float* y_f32_nhwc, float* y_f32_nchw) {
    EXHIP_REQUIRE(y_f32_nhwc || y_f32_nchw, "exhip_conv2d_f32: no output requested");
    ConvParams p = {};
    p.x = (const char*)x; p.wp = (const char*)wp; p.bias = bias; p.residual = residual;
    p.y_nhwc = y_f32_nhwc; p.y_nchw = y_f32_nchw;
    return run_conv<EXHIP_F32>(ctx, d, p);
}
