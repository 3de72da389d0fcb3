// Shared declarations of the exhip library (HIP for gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/exhip.h"

struct exhip_ctx {
    int device;
    hipStream_t stream;
    // scratch of the convolution's split reduction, grown on demand and kept until the context is destroyed
    int* split_acc = nullptr;
    size_t split_acc_bytes = 0;
    unsigned* split_count = nullptr;
    size_t split_count_n = 0;
};

// The context's split-reduction scratch (partial accumulators, and one zeroed arrival counter per tile): allocated on first
// use at its fixed upper bound -- kSplitGroups groups per launch -- and never moved or grown afterwards; a request beyond
// the bound is an error (the planner clamps its splits to it).
constexpr int kSplitGroups = 256;
int exhip_split_scratch(exhip_ctx* ctx, size_t acc_bytes, size_t tiles, int** acc, unsigned** count);

void exhip_set_error(const char* fmt, ...);

// How exhip_conv_pack_weights lays this layer's weights out: output channels per slab, and whether it is the packed
// first-layer form (4- or 8-byte pixels, one k-step per filter row).
int exhip_conv_packed_layout(const exhip_conv_desc* d, int dtype, int* slab_channels, int* packed_form);

// Looks up, once per device and with that device current, the address of the static scratch array behind
// exhip_maxpool_same_nhwc_f16_static (defined beside that array).
int exhip_static_scratch_setup(int device);

#define EXHIP_CHECK(expr)                                                                          \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess) {                                                                    \
            exhip_set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(e_), __FILE__, __LINE__); \
            return (int)e_;                                                                        \
        }                                                                                          \
    } while (0)

#define EXHIP_REQUIRE(cond, ...)          \
    do {                                  \
        if (!(cond)) {                    \
            exhip_set_error(__VA_ARGS__); \
            return EXHIP_ERR_ARG;         \
        }                                 \
    } while (0)

// Kernel launch check: launch errors are reported at once, execution errors at the next sync.
#define EXHIP_LAUNCH_CHECK() EXHIP_CHECK(hipGetLastError())

// Switches for tests and development, set through exhip_set_option (never read from the environment): a test
// pins a plan choice to reach a code path small shapes would not take; zero / negative values mean "not set".
struct exhip_options {
    int force_variant = -1;  // tile variant of the convolution planner
    int force_chunk = 0;     // its channel chunk in bytes (32 / 64)
    int force_rs = 0;        // filter rows per stage
    int force_abufs = 0;     // activation tile buffers (1 / 2)
    int debug_plan = 0;      // one line per planned layer on stderr
    int dw_band_rows = 0;    // row-band height of the depthwise strip kernels
    int force_splits = 0;    // groups per tile of the convolution's split reduction (1 = never split)
    int share_gpu = 0;       // launches of several streams overlap: the planner then counts groups per CU, not rounds of one launch
    int lean = 4;            // 3x3 stride-1 int8 layers with the fused epilogue: 0 general kernel, 1 lean kernel with persistent groups, 2 lean, one
                             // group per patch, 3 lean with MFMA and epilogue waves, 4 the form measured fastest for the layer's class
    int lean_cfg = 0;        // its staging buffers for layers of more than 64 input channels: 0 one tile + two slices, 1 two + two, 2 one + three
    int lean_wres = 1;       // 64 input channels: keep the slab's whole filter in LDS (0: stream it like the deeper layers)
    int lean_stagger = 0;    // experiment: start delay per hardware wave slot, in units of 64 cycles
    int stem = 1;            // the stem (quantizer + first convolution + max pooling) as one kernel where the entry point offers it
    int lean_groups = 0;     // at most this many groups per 64-channel slab (tests: a few groups that walk many patches each)
    int lean_f16 = 1;        // 3x3 stride-1 fp16 layers with an NHWC result on the lean kernel: 0 never, 1 the form per layer class, 2 one group per
                             // patch, 3 persistent groups with three slice buffers, 4 persistent groups with two
    int direct = 1;          // layers with a filter, a stride or padding and NHWC results on the pointwise kernel's tapped form: 1 where it measured
                             // faster, 2 wherever it can run, 0 never
    int pw_tile = 0;         // that kernel's wave tile for more than 32 output channels: 0 = 32 pixels x 64 channels, 2 = 64 x 64 from 2048 waves on
    int pw = 1;              // 1x1 stride-1 fp16 layers with an NHWC result: 1 the pointwise kernel where it measured faster, 2 wherever it can run, 0 never
};
extern exhip_options g_exhip_options;

// Cache policy bits of the float32 result stores of the int8 kernels (the aux operand of the raw buffer store builtins).
#ifndef EXHIP_F32_STORE_AUX
#define EXHIP_F32_STORE_AUX 0
#endif

// ---- device helpers shared by the kernels ----
typedef int exhip_v4i __attribute__((ext_vector_type(4)));
// Stores reach full speed with runs of 64 contiguous bytes from neighbouring lanes (measured: 32-byte runs take twice as
// long), so two pixels in neighbouring lanes trade halves: afterwards `a` holds, in the even lane, its own a and, in the
// odd lane, the even lane's c; `c` holds the odd lane's a and, in the odd lane, its own c. (DPP quad_perm [1, 0, 3, 2].)
__device__ __forceinline__ int lane_neighbour(int v) { return __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true); }
__device__ __forceinline__ void pair_exchange4(exhip_v4i& a, exhip_v4i& c, bool odd) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int from_c = lane_neighbour(c[e]), from_a = lane_neighbour(a[e]);
        const int a2 = odd ? from_c : a[e], c2 = odd ? c[e] : from_a;
        a[e] = a2;
        c[e] = c2;
    }
}

// v_permlane32_swap: the upper half-wave of `a` changes places with the lower half-wave of `b`.
__device__ __forceinline__ void half_swap(int& a, int& b) {
    const auto r = __builtin_amdgcn_permlane32_swap((unsigned)a, (unsigned)b, false, false);
    a = (int)r[0];
    b = (int)r[1];
}
__device__ __forceinline__ void half_swap4(exhip_v4i& a, exhip_v4i& b) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        int x = a[e], y = b[e];
        half_swap(x, y);
        a[e] = x;
        b[e] = y;
    }
}

// float32_to_int8 of the reference (src/Primitives/simd_types.cpp:140-152): add +-0.5, saturate, truncate.
// Here: the +-0.5 by the value's sign bit, one conversion that truncates toward zero and saturates at the int32 range
// (NaN -> 0), and the saturation to [-128, 127] on the integer -- for every float the value of add, saturate, truncate
// (a sum beyond +-128 truncates to an integer beyond it, and -0.0 - 0.5 truncates to 0 like 0.0 + 0.5).
__device__ __forceinline__ int exhip_q8(float v) {
    int i;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(i) : "v"(v + __builtin_copysignf(0.5f, v)));
    i = i > 127 ? 127 : i;
    return i < -128 ? -128 : i;
}

// suffix_activation_cpu_f32 of the reference (src/Excalibur/operation_general_conv.cpp:127-272).
__device__ __forceinline__ float exhip_act(float v, int act) {
    switch (act) {
    case 1: return (0.f > v) ? 0.f : v;
    case 3: { float d = (0.f > v) ? 0.f : v; return d <= 6.f ? d : 0.f; }
    case 4: return (float)(1.0 / (1.0 + exp(-(double)v)));
    case 5: return (float)((double)v * tanh(log(1.0 + exp((double)v))));
    default: return v;
    }
}

__device__ __forceinline__ float exhip_h2f(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t exhip_f2h(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }

// One value of an elementwise activation. OP 0 HardSwish, 1 LeakyReLU, 2 sigmoid, 3 HardSigmoid, 4 Clip; the multiply-adds
// are fused where the CPU path's are (vector fmadd, and scalar expressions contracted by its compiler flags).
template <int OP>
__device__ __forceinline__ float unary_value(float x, float alpha, float beta) {
    if constexpr (OP == 0) {
        // clamp to [0, 1] as one median: NaN gives 0 as the two selects do (and the product below is NaN either way)
        return __builtin_amdgcn_fmed3f(__builtin_fmaf(x, alpha, beta), 0.f, 1.f) * x;
    } else if constexpr (OP == 1) {
        return x < 0.f ? alpha * x : x;
    } else if constexpr (OP == 2) {
        return (float)(1. / (1. + exp(-(double)x)));
    } else if constexpr (OP == 3) {
        return __builtin_amdgcn_fmed3f(__builtin_fmaf(alpha, x, beta), 0.f, 1.f);  // NaN -> 0 as with the two selects
    } else {
        const float t = beta < x ? beta : x;  // clip to [alpha, beta]
        return alpha < t ? t : alpha;
    }
}
