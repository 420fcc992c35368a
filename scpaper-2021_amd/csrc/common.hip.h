// Shared device/host helpers of the gfx950 kernels: vector types, wave64
// reductions, fp16 packing, status plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/et_abi.h"

namespace et {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

// ---- status -------------------------------------------------------------
void set_error(const char *fmt, ...);
int fail(int status, const char *fmt, ...);
int check_hip(hipError_t e, const char *what);

#define ET_REQUIRE(cond, status, ...) \
    do {                              \
        if (!(cond)) return ::et::fail(status, __VA_ARGS__); \
    } while (0)

#define ET_HIP(call)                                           \
    do {                                                       \
        int _s = ::et::check_hip((call), #call);               \
        if (_s != ET_OK) return _s;                            \
    } while (0)

inline hipStream_t as_stream(et_stream s) { return reinterpret_cast<hipStream_t>(s); }

// Checks the launch that was just issued (asynchronous errors surface later).
int check_launch(const char *kernel);

// ---- wave64 reductions ----------------------------------------------------
// Every lane ends with the total.  All 64 lanes must be active.  The 16 lanes of a
// DPP row are folded with cross-lane VALU operands (quad swaps, then row rotations
// by 4 and 8), which never touch the LDS crossbar; the four row totals are then read
// through scalar registers, in a fixed order, so the result is the same in every lane.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false);
    return __builtin_bit_cast(float, r);
}
constexpr int kDppQuadXor1 = 0xB1;  // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;  // quad_perm:[2,3,0,1]
constexpr int kDppRowRor4 = 0x124;  // row_ror:4
constexpr int kDppRowRor8 = 0x128;  // row_ror:8

__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move<kDppQuadXor1>(v);
    v += dpp_move<kDppQuadXor2>(v);
    v += dpp_move<kDppRowRor4>(v);
    v += dpp_move<kDppRowRor8>(v);
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<kDppQuadXor1>(v));
    v = fmaxf(v, dpp_move<kDppQuadXor2>(v));
    v = fmaxf(v, dpp_move<kDppRowRor4>(v));
    v = fmaxf(v, dpp_move<kDppRowRor8>(v));
    return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

// Butterflies across the four 16-lane rows of a wave (lane ^ 16, then lane ^ 32) with the gfx950
// row-swap instructions: v_permlane16_swap exchanges the odd rows of its first operand with the
// even rows of its second, v_permlane32_swap the upper half of the first with the lower half of
// the second.  Given the same value twice they return (this lane's row pair, the partner's), so
// one swap and one VALU operation make a butterfly step without the LDS crossbar a
// ds_bpermute-based shuffle goes through.  Every lane of a column (lane % 16) ends with the
// result over the column's four lanes.
__device__ __forceinline__ float rows_max(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float m = fmaxf(__builtin_bit_cast(float, (unsigned)a[0]), __builtin_bit_cast(float, (unsigned)a[1]));
    const unsigned w = __builtin_bit_cast(unsigned, m);
    auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return fmaxf(__builtin_bit_cast(float, (unsigned)b[0]), __builtin_bit_cast(float, (unsigned)b[1]));
}
__device__ __forceinline__ float rows_sum(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float m = __builtin_bit_cast(float, (unsigned)a[0]) + __builtin_bit_cast(float, (unsigned)a[1]);
    const unsigned w = __builtin_bit_cast(unsigned, m);
    auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return __builtin_bit_cast(float, (unsigned)b[0]) + __builtin_bit_cast(float, (unsigned)b[1]);
}

// tanh-form GELU, x*(0.5 + 0.5*tanh(x*(0.035677408*x^2 + 0.7978845608)))
// (the form the reference evaluates, Encoder/Encoder.cu:25-37).
__device__ __forceinline__ float gelu_tanh(float x) {
    // 0.5 + 0.5*tanh(u) = 1 - 1/(exp(2u) + 1), and exp(2u) = exp2(x*(c1*x^2 + c0)) with
    // 2*log2(e) folded into the polynomial: one exp2, one reciprocal, four multiply-adds.
    // exp2 overflow to +inf gives x, underflow to 0 gives 0.
    constexpr float k2log2e = 2.8853900817779268f;
    constexpr float c1 = 0.035677408136f * k2log2e, c0 = 0.7978845608028654f * k2log2e;
    const float e = __builtin_amdgcn_exp2f(x * (c1 * x * x + c0));
    return x - x * __builtin_amdgcn_rcpf(e + 1.0f);
}

__device__ __forceinline__ float apply_act(float x, int act) {
    if (act == ET_ACT_RELU) return x > 0.0f ? x : 0.0f;
    if (act == ET_ACT_GELU) return gelu_tanh(x);
    return x;
}

// ---- LayerNorm split between a producer and a consumer kernel ----------------
// The producer of a row (a Linear with the residual added in its epilogue) emits, per
// block-row group, the sum and the sum of squares of the values it stored; any consumer
// normalises with them.
constexpr int kMaxStatGroups = 16;  // block-row groups a RES producer may split a row over

// mean and reciprocal standard deviation of a row of H values from its partial sums,
// added in a fixed order (every consumer of the same sums gets the same bits).  All loads are
// issued before the first addition (index clamped, surplus selected away): a loop with a
// run-time trip count would wait for each load in turn.
// The two halves of row_stats: the requests (held in registers, so a kernel can put them ahead of
// larger loads and use them long after) and the sums.
__device__ __forceinline__ void row_stats_request(float2 (&p)[kMaxStatGroups], const float *st, int groups, int T, int tok) {
#pragma unroll
    for (int gi = 0; gi < kMaxStatGroups; gi++)
        p[gi] = *reinterpret_cast<const float2 *>(st + ((size_t)min(gi, groups - 1) * T + tok) * 2);
}
__device__ __forceinline__ float2 row_stats_finish(const float2 (&p)[kMaxStatGroups], int groups, int H, float eps) {
    // two halves in group order, then their sum: the order a consumer that deals the groups to
    // the two halves of a wave adds in, so that both get the same bits
    float s1 = 0.0f, s2 = 0.0f, u1 = 0.0f, u2 = 0.0f;
#pragma unroll
    for (int gi = 0; gi < kMaxStatGroups / 2; gi++) {
        s1 += gi < groups ? p[gi].x : 0.0f;
        s2 += gi < groups ? p[gi].y : 0.0f;
        u1 += gi + kMaxStatGroups / 2 < groups ? p[gi + kMaxStatGroups / 2].x : 0.0f;
        u2 += gi + kMaxStatGroups / 2 < groups ? p[gi + kMaxStatGroups / 2].y : 0.0f;
    }
    s1 += u1;
    s2 += u2;
    const float inv_h = 1.0f / (float)H;
    const float mean = s1 * inv_h;
    const float var = fmaxf(__builtin_fmaf(-mean, mean, s2 * inv_h), 0.0f);
    return float2{mean, rsqrtf(var + eps)};
}
__device__ __forceinline__ float2 row_stats(const float *st, int groups, int T, int tok, int H, float eps) {
    float2 p[kMaxStatGroups];
    row_stats_request(p, st, groups, T, tok);
    return row_stats_finish(p, groups, H, eps);
}

// one normalised value: the same two roundings wherever it is evaluated
__device__ __forceinline__ float norm_value(float v, float mean, float rstd, float gm, float bt) {
    return __builtin_fmaf((v - mean) * rstd, gm, bt);
}

}  // namespace et
