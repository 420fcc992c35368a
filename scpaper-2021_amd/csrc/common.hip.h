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
// Butterfly over the 64 lanes of a wavefront: every lane ends with the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
    return v;
}

// tanh-form GELU, x*(0.5 + 0.5*tanh(x*(0.035677408*x^2 + 0.7978845608)))
// (the form the reference evaluates, Encoder/Encoder.cu:25-37).
__device__ __forceinline__ float gelu_tanh(float x) {
    const float u = x * (0.035677408136f * x * x + 0.7978845608028654f);
    // tanh(u) = 1 - 2/(exp(2u)+1); exp overflow to +inf gives 1, underflow gives -1.
    const float t = 1.0f - 2.0f / (__expf(2.0f * u) + 1.0f);
    return x * (0.5f + 0.5f * t);
}

__device__ __forceinline__ float apply_act(float x, int act) {
    if (act == ET_ACT_RELU) return x > 0.0f ? x : 0.0f;
    if (act == ET_ACT_GELU) return gelu_tanh(x);
    return x;
}

}  // namespace et
