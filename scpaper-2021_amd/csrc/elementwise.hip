// Stand-alone activations and bias add (HBM-bound, 16-byte accesses).  The
// Linear kernels fuse these into their epilogues; these entry points exist for
// callers that keep the reference's separate act<>() / bias-map steps.
#include "common.hip.h"

namespace et {

enum { OP_GELU = 0, OP_RELU = 1 };

template <int OP>
__device__ __forceinline__ float unary(float x) {
    return OP == OP_GELU ? gelu_tanh(x) : (x > 0.0f ? x : 0.0f);
}

template <int OP>
__global__ __launch_bounds__(256) void unary_kernel(_Float16 *__restrict__ out,
                                                    const _Float16 *__restrict__ in, size_t n) {
    const size_t nvec = n / 8;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    if (aligned) {
        // four 16-byte loads in flight per lane before the first use
        constexpr int kU = 4;
        size_t v = i;
        for (; v + (kU - 1) * step < nvec; v += kU * step) {
            h8 x[kU];
#pragma unroll
            for (int u = 0; u < kU; u++) x[u] = reinterpret_cast<const h8 *>(in)[v + u * step];
#pragma unroll
            for (int u = 0; u < kU; u++) {
#pragma unroll
                for (int j = 0; j < 8; j++) x[u][j] = (_Float16)unary<OP>((float)x[u][j]);
                reinterpret_cast<h8 *>(out)[v + u * step] = x[u];
            }
        }
        for (; v < nvec; v += step) {
            h8 x = reinterpret_cast<const h8 *>(in)[v];
#pragma unroll
            for (int j = 0; j < 8; j++) x[j] = (_Float16)unary<OP>((float)x[j]);
            reinterpret_cast<h8 *>(out)[v] = x;
        }
        for (size_t e = nvec * 8 + i; e < n; e += step) out[e] = (_Float16)unary<OP>((float)in[e]);
    } else {
        for (size_t e = i; e < n; e += step) out[e] = (_Float16)unary<OP>((float)in[e]);
    }
}

__global__ __launch_bounds__(256) void bias_add_kernel(_Float16 *__restrict__ data,
                                                       const _Float16 *__restrict__ bias, int rows,
                                                       int cols) {
    // cols % 8 == 0: one thread handles 8 consecutive columns of one row.
    const int vec_per_row = cols >> 3;
    const size_t total = (size_t)rows * vec_per_row;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t v = blockIdx.x * (size_t)blockDim.x + threadIdx.x; v < total; v += step) {
        const int c = (int)(v % vec_per_row);
        h8 x = reinterpret_cast<h8 *>(data)[v];
        const h8 b = reinterpret_cast<const h8 *>(bias)[c];
#pragma unroll
        for (int j = 0; j < 8; j++) x[j] = (_Float16)((float)x[j] + (float)b[j]);
        reinterpret_cast<h8 *>(data)[v] = x;
    }
}

__global__ __launch_bounds__(256) void bias_add_scalar_kernel(_Float16 *__restrict__ data,
                                                              const _Float16 *__restrict__ bias,
                                                              int rows, int cols) {
    const size_t total = (size_t)rows * cols;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total; e += step)
        data[e] = (_Float16)((float)data[e] + (float)bias[e % cols]);
}

static inline unsigned ew_grid(size_t work_items) {
    size_t g = (work_items + 255) / 256;
    const size_t cap = 256u * 8u;
    return (unsigned)(g < 1 ? 1 : (g > cap ? cap : g));
}

}  // namespace et

using namespace et;

extern "C" {

int et_gelu_f16(et_f16 *out, const et_f16 *in, size_t n, et_stream stream) {
    ET_REQUIRE((out && in) || n == 0, ET_ERR_INVALID_ARG, "et_gelu_f16: NULL pointer");
    if (n == 0) return ET_OK;
    unary_kernel<OP_GELU><<<ew_grid(n / 8 + 1), 256, 0, as_stream(stream)>>>(
        reinterpret_cast<_Float16 *>(out), reinterpret_cast<const _Float16 *>(in), n);
    return check_launch("unary_kernel<gelu>");
}

int et_relu_f16(et_f16 *out, const et_f16 *in, size_t n, et_stream stream) {
    ET_REQUIRE((out && in) || n == 0, ET_ERR_INVALID_ARG, "et_relu_f16: NULL pointer");
    if (n == 0) return ET_OK;
    unary_kernel<OP_RELU><<<ew_grid(n / 8 + 1), 256, 0, as_stream(stream)>>>(
        reinterpret_cast<_Float16 *>(out), reinterpret_cast<const _Float16 *>(in), n);
    return check_launch("unary_kernel<relu>");
}

int et_bias_add_f16(et_f16 *data, const et_f16 *bias, int rows, int cols, et_stream stream) {
    ET_REQUIRE(data && bias, ET_ERR_INVALID_ARG, "et_bias_add_f16: NULL pointer");
    ET_REQUIRE(rows >= 0 && cols > 0, ET_ERR_INVALID_ARG, "et_bias_add_f16: rows=%d cols=%d", rows,
               cols);
    if (rows == 0) return ET_OK;
    const bool vec = cols % 8 == 0 &&
                     ((reinterpret_cast<uintptr_t>(data) | reinterpret_cast<uintptr_t>(bias)) & 15) == 0;
    if (vec) {
        bias_add_kernel<<<ew_grid((size_t)rows * (cols / 8)), 256, 0, as_stream(stream)>>>(
            reinterpret_cast<_Float16 *>(data), reinterpret_cast<const _Float16 *>(bias), rows, cols);
    } else {
        bias_add_scalar_kernel<<<ew_grid((size_t)rows * cols), 256, 0, as_stream(stream)>>>(
            reinterpret_cast<_Float16 *>(data), reinterpret_cast<const _Float16 *>(bias), rows, cols);
    }
    return check_launch("bias_add_kernel");
}

}  // extern "C"
