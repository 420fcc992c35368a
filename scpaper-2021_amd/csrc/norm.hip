// SkipLayerNorm / LayerNorm for gfx950: one wavefront owns one row, the row
// stays in registers between the statistics and the normalisation, so HBM sees
// each input once and the output once.  Statistics are fp32 (mean, then the
// centred second moment), wave64 butterfly reductions, no LDS.
#include "common.hip.h"

namespace et {

constexpr int kRowsPerBlock = 4;  // 4 waves of 64 lanes

__device__ __forceinline__ void unpack4(uint2 raw, float (&f)[4]) {
    const h2 lo = __builtin_bit_cast(h2, raw.x);
    const h2 hi = __builtin_bit_cast(h2, raw.y);
    f[0] = (float)lo[0];
    f[1] = (float)lo[1];
    f[2] = (float)hi[0];
    f[3] = (float)hi[1];
}

__device__ __forceinline__ uint2 pack4(const float (&f)[4]) {
    h2 lo, hi;
    lo[0] = (_Float16)f[0];
    lo[1] = (_Float16)f[1];
    hi[0] = (_Float16)f[2];
    hi[1] = (_Float16)f[3];
    uint2 raw;
    raw.x = __builtin_bit_cast(uint32_t, lo);
    raw.y = __builtin_bit_cast(uint32_t, hi);
    return raw;
}

// binary32 rows: a chunk is one float4
__device__ __forceinline__ void unpack4(float4 raw, float (&f)[4]) {
    f[0] = raw.x;
    f[1] = raw.y;
    f[2] = raw.z;
    f[3] = raw.w;
}
template <typename RAW> __device__ __forceinline__ RAW pack4_as(const float (&f)[4]);
template <> __device__ __forceinline__ uint2 pack4_as<uint2>(const float (&f)[4]) { return pack4(f); }
template <> __device__ __forceinline__ float4 pack4_as<float4>(const float (&f)[4]) {
    return float4{f[0], f[1], f[2], f[3]};
}
template <typename T> struct Chunk4;  // storage type of 4 consecutive elements
template <> struct Chunk4<_Float16> { using raw = uint2; };
template <> struct Chunk4<float> { using raw = float4; };

// NIT = number of 4-element chunks each lane owns: chunk c = lane + 64*i.
template <typename T, int NIT, bool SKIP>
__global__ __launch_bounds__(kWave *kRowsPerBlock) void layernorm_rows_kernel(
    T *__restrict__ out, const T *__restrict__ src, const T *__restrict__ skip,
    const T *__restrict__ gamma, const T *__restrict__ beta, int rows, int H, float eps) {
    using raw_t = typename Chunk4<T>::raw;
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int chunks = H >> 2;
    const raw_t *s = reinterpret_cast<const raw_t *>(src + (size_t)row * H);
    const raw_t *k = SKIP ? reinterpret_cast<const raw_t *>(skip + (size_t)row * H) : nullptr;

    // Every load of the row is issued before the first use, so src, skip, gamma and beta
    // arrive in one round trip.  The loads are unconditional (a chunk index past the row is
    // clamped onto the last chunk and its value ignored): loads under a branch end up in a
    // basic block of their own, where the compiler waits for each of them in turn.
    const raw_t *g = reinterpret_cast<const raw_t *>(gamma);
    const raw_t *b = reinterpret_cast<const raw_t *>(beta);
    // (Rows of more than 256 bytes per lane — binary32 rows wider than 4096 — would need more registers
    // than a lane has for that: there gamma and beta are loaded where they are used, a second round trip
    // that such a row hides behind its own length.)
    constexpr bool kLateAffine = sizeof(raw_t) * NIT > 256;
    constexpr int NAFF = kLateAffine ? 1 : NIT;
    raw_t rs[NIT], rk[SKIP ? NIT : 1], rg[NAFF], rb[NAFF];
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int c = min(lane + kWave * i, chunks - 1);
        rs[i] = s[c];
        if (SKIP) rk[i] = k[c];
        if (!kLateAffine) {
            rg[i] = g[c];
            rb[i] = b[c];
        }
    }

    // values past the row are selected away, not branched around: a branch would give the
    // compiler a block to sink the loads into
    float x[NIT][4];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const bool ok = lane + kWave * i < chunks;
        unpack4(rs[i], x[i]);
        if (SKIP) {
            float y[4];
            unpack4(rk[i], y);
#pragma unroll
            for (int j = 0; j < 4; j++) x[i][j] += y[j];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            x[i][j] = ok ? x[i][j] : 0.0f;
            sum += x[i][j];
        }
    }
    const float inv_h = 1.0f / (float)H;
    const float mean = wave_sum(sum) * inv_h;
    float sq = 0.0f;
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const bool ok = lane + kWave * i < chunks;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float d = ok ? x[i][j] - mean : 0.0f;
            sq += d * d;
        }
    }
    const float rstd = rsqrtf(wave_sum(sq) * inv_h + eps);

    raw_t *o = reinterpret_cast<raw_t *>(out + (size_t)row * H);
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int c = lane + kWave * i;
        if (c < chunks) {
            float gg[4], bb[4], y[4];
            unpack4(kLateAffine ? g[c] : rg[kLateAffine ? 0 : i], gg);
            unpack4(kLateAffine ? b[c] : rb[kLateAffine ? 0 : i], bb);
#pragma unroll
            for (int j = 0; j < 4; j++) y[j] = (x[i][j] - mean) * rstd * gg[j] + bb[j];
            o[c] = pack4_as<raw_t>(y);
        }
    }
}

// Mixed-precision SkipLayerNorm: the residual stream (src = a projection's fp32 output, skip = the
// fp32 residual) stays binary32 end to end; the result is written twice, as binary32 (the next
// residual) and rounded to binary16 (the operand the next projection's matrix cores read).
// gamma and beta are the model's binary16 parameters.  Same structure as layernorm_rows_kernel.
template <int NIT>
__global__ __launch_bounds__(kWave *kRowsPerBlock) void skip_layernorm_mixed_kernel(
    float *__restrict__ out32, _Float16 *__restrict__ out16, const float *__restrict__ src,
    const float *__restrict__ skip, const _Float16 *__restrict__ gamma, const _Float16 *__restrict__ beta,
    int rows, int H, float eps) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int chunks = H >> 2;
    const float4 *s = reinterpret_cast<const float4 *>(src + (size_t)row * H);
    const float4 *k = reinterpret_cast<const float4 *>(skip + (size_t)row * H);
    const uint2 *g = reinterpret_cast<const uint2 *>(gamma);
    const uint2 *b = reinterpret_cast<const uint2 *>(beta);
    float4 rs[NIT], rk[NIT];
    uint2 rg[NIT], rb[NIT];
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int c = min(lane + kWave * i, chunks - 1);
        rs[i] = s[c];
        rk[i] = k[c];
        rg[i] = g[c];
        rb[i] = b[c];
    }
    float x[NIT][4];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const bool ok = lane + kWave * i < chunks;
        float y[4];
        unpack4(rs[i], x[i]);
        unpack4(rk[i], y);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            x[i][j] = ok ? x[i][j] + y[j] : 0.0f;
            sum += x[i][j];
        }
    }
    const float inv_h = 1.0f / (float)H;
    const float mean = wave_sum(sum) * inv_h;
    float sq = 0.0f;
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const bool ok = lane + kWave * i < chunks;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float d = ok ? x[i][j] - mean : 0.0f;
            sq += d * d;
        }
    }
    const float rstd = rsqrtf(wave_sum(sq) * inv_h + eps);
    float4 *o32 = out32 ? reinterpret_cast<float4 *>(out32 + (size_t)row * H) : nullptr;
    uint2 *o16 = out16 ? reinterpret_cast<uint2 *>(out16 + (size_t)row * H) : nullptr;
#pragma unroll
    for (int i = 0; i < NIT; i++) {
        const int c = lane + kWave * i;
        if (c < chunks) {
            float gg[4], bb[4], y[4];
            unpack4(rg[i], gg);
            unpack4(rb[i], bb);
#pragma unroll
            for (int j = 0; j < 4; j++) y[j] = (x[i][j] - mean) * rstd * gg[j] + bb[j];
            if (o32) o32[c] = float4{y[0], y[1], y[2], y[3]};
            if (o16) o16[c] = pack4(y);
        }
    }
}

// out = normalisation of V + skip with the row statistics a producer kernel left behind: the
// stand-alone form of the NORM prologue of the tile-sparse Linear (same arithmetic, same bits).
__global__ __launch_bounds__(256) void norm_from_stats_kernel(_Float16 *__restrict__ out,
                                                              const _Float16 *__restrict__ V,
                                                              const _Float16 *__restrict__ skip,
                                                              const float *__restrict__ stats, int groups,
                                                              const _Float16 *__restrict__ gamma,
                                                              const _Float16 *__restrict__ beta, int rows,
                                                              int H, float eps) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float2 st = row_stats(stats, groups, rows, row, H, eps);
    const int vecs = H >> 3;
    const h8 *v = reinterpret_cast<const h8 *>(V + (size_t)row * H);
    const h8 *k = reinterpret_cast<const h8 *>(skip + (size_t)row * H);
    h8 *o = reinterpret_cast<h8 *>(out + (size_t)row * H);
    for (int c = lane; c < vecs; c += kWave) {
        const h8 x = v[c], s = k[c];
        const h8 gm = reinterpret_cast<const h8 *>(gamma)[c], bt = reinterpret_cast<const h8 *>(beta)[c];
        h8 y;
#pragma unroll
        for (int e = 0; e < 8; e++)
            y[e] = (_Float16)norm_value((float)x[e] + (float)s[e], st.x, st.y, (float)gm[e], (float)bt[e]);
        o[c] = y;
    }
}

// the same from a binary32 sum (no skip: the producer added it), binary32 and / or binary16 result
__global__ __launch_bounds__(256) void norm_from_stats_f32in_kernel(float *__restrict__ out32, _Float16 *__restrict__ out16,
                                                                    const float *__restrict__ V,
                                                                    const float *__restrict__ stats, int groups,
                                                                    const _Float16 *__restrict__ gamma,
                                                                    const _Float16 *__restrict__ beta, int rows, int H,
                                                                    float eps) {
    const int lane = threadIdx.x & (kWave - 1);
    const int row = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float2 st = row_stats(stats, groups, rows, row, H, eps);
    const int vecs = H >> 3;
    const f4 *v = reinterpret_cast<const f4 *>(V + (size_t)row * H);
    for (int c = lane; c < vecs; c += kWave) {
        const f4 lo = v[2 * c], hi = v[2 * c + 1];
        const h8 gm = reinterpret_cast<const h8 *>(gamma)[c], bt = reinterpret_cast<const h8 *>(beta)[c];
        f4 y0, y1;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            y0[e] = norm_value(lo[e], st.x, st.y, (float)gm[e], (float)bt[e]);
            y1[e] = norm_value(hi[e], st.x, st.y, (float)gm[4 + e], (float)bt[4 + e]);
        }
        if (out32) {
            f4 *o = reinterpret_cast<f4 *>(out32 + (size_t)row * H);
            o[2 * c] = y0;
            o[2 * c + 1] = y1;
        }
        if (out16)
            reinterpret_cast<h8 *>(out16 + (size_t)row * H)[c] =
                h8{(_Float16)y0[0], (_Float16)y0[1], (_Float16)y0[2], (_Float16)y0[3],
                   (_Float16)y1[0], (_Float16)y1[1], (_Float16)y1[2], (_Float16)y1[3]};
    }
}

template <bool SKIP, typename T>
static int launch_layernorm(T *out, const T *src, const T *skip, const T *gamma, const T *beta, int rows,
                            int H, float eps, hipStream_t stream) {
    const int chunks = H / 4;
    const int nit = (chunks + kWave - 1) / kWave;
    const dim3 grid((rows + kRowsPerBlock - 1) / kRowsPerBlock), block(kWave * kRowsPerBlock);
#define ET_LN_CASE(N)                                                                   \
    case N:                                                                             \
        layernorm_rows_kernel<T, N, SKIP><<<grid, block, 0, stream>>>(out, src, skip, gamma, \
                                                                   beta, rows, H, eps);  \
        break;
    switch (nit) {
        ET_LN_CASE(1) ET_LN_CASE(2) ET_LN_CASE(3) ET_LN_CASE(4)
        ET_LN_CASE(5) ET_LN_CASE(6) ET_LN_CASE(7) ET_LN_CASE(8)
        default:
            if (nit <= 16) {
                layernorm_rows_kernel<T, 16, SKIP><<<grid, block, 0, stream>>>(out, src, skip, gamma,
                                                                            beta, rows, H, eps);
            } else {
                layernorm_rows_kernel<T, 32, SKIP><<<grid, block, 0, stream>>>(out, src, skip, gamma,
                                                                            beta, rows, H, eps);
            }
    }
#undef ET_LN_CASE
    return check_launch("layernorm_rows_kernel");
}

static int launch_skip_layernorm_mixed(float *out32, _Float16 *out16, const float *src, const float *skip,
                                       const _Float16 *gamma, const _Float16 *beta, int rows, int H, float eps,
                                       hipStream_t stream) {
    const int chunks = H / 4;
    const int nit = (chunks + kWave - 1) / kWave;
    const dim3 grid((rows + kRowsPerBlock - 1) / kRowsPerBlock), block(kWave * kRowsPerBlock);
#define ET_LNM_CASE(N)                                                                                       \
    case N:                                                                                                  \
        skip_layernorm_mixed_kernel<N><<<grid, block, 0, stream>>>(out32, out16, src, skip, gamma, beta, rows, H, \
                                                                   eps);                                     \
        break;
    switch (nit) {
        ET_LNM_CASE(1) ET_LNM_CASE(2) ET_LNM_CASE(3) ET_LNM_CASE(4)
        ET_LNM_CASE(5) ET_LNM_CASE(6) ET_LNM_CASE(7) ET_LNM_CASE(8)
        default:
            if (nit <= 16) {
                skip_layernorm_mixed_kernel<16><<<grid, block, 0, stream>>>(out32, out16, src, skip, gamma, beta,
                                                                            rows, H, eps);
            } else {
                skip_layernorm_mixed_kernel<32><<<grid, block, 0, stream>>>(out32, out16, src, skip, gamma, beta,
                                                                            rows, H, eps);
            }
    }
#undef ET_LNM_CASE
    return check_launch("skip_layernorm_mixed_kernel");
}

static int check_ln_args(const char *fn, const void *out, const void *src, const void *gamma,
                         const void *beta, int rows, int H) {
    ET_REQUIRE(out && src && gamma && beta, ET_ERR_INVALID_ARG, "%s: NULL pointer", fn);
    ET_REQUIRE(rows >= 0 && H > 0, ET_ERR_INVALID_ARG, "%s: rows=%d H=%d", fn, rows, H);
    ET_REQUIRE(H % 4 == 0 && H <= 8192, ET_ERR_UNSUPPORTED,
               "%s: H=%d must be a multiple of 4 and at most 8192", fn, H);
    return ET_OK;
}

}  // namespace et

using namespace et;

extern "C" {

int et_skip_layernorm_f16(et_f16 *out, const et_f16 *src, const et_f16 *skip,
                          const et_f16 *gamma, const et_f16 *beta, int rows, int H, float eps,
                          et_stream stream) {
    int s = check_ln_args("et_skip_layernorm_f16", out, src, gamma, beta, rows, H);
    if (s != ET_OK) return s;
    ET_REQUIRE(skip != nullptr, ET_ERR_INVALID_ARG, "et_skip_layernorm_f16: skip is NULL");
    if (rows == 0) return ET_OK;
    return launch_layernorm<true>(
        reinterpret_cast<_Float16 *>(out), reinterpret_cast<const _Float16 *>(src),
        reinterpret_cast<const _Float16 *>(skip), reinterpret_cast<const _Float16 *>(gamma),
        reinterpret_cast<const _Float16 *>(beta), rows, H, eps, as_stream(stream));
}

int et_layernorm_f16(et_f16 *out, const et_f16 *src, const et_f16 *gamma, const et_f16 *beta,
                     int rows, int H, float eps, et_stream stream) {
    int s = check_ln_args("et_layernorm_f16", out, src, gamma, beta, rows, H);
    if (s != ET_OK) return s;
    if (rows == 0) return ET_OK;
    return launch_layernorm<false, _Float16>(
        reinterpret_cast<_Float16 *>(out), reinterpret_cast<const _Float16 *>(src), nullptr,
        reinterpret_cast<const _Float16 *>(gamma), reinterpret_cast<const _Float16 *>(beta), rows,
        H, eps, as_stream(stream));
}

int et_norm_from_stats_f16(et_f16 *out, const et_f16 *V, const et_f16 *skip, const float *stats, int stat_groups,
                           const et_f16 *gamma, const et_f16 *beta, int rows, int H, float eps,
                           et_stream stream) {
    ET_REQUIRE(out && V && skip && stats && gamma && beta, ET_ERR_INVALID_ARG, "et_norm_from_stats_f16: NULL pointer");
    ET_REQUIRE(rows >= 0 && H > 0, ET_ERR_INVALID_ARG, "et_norm_from_stats_f16: rows=%d H=%d", rows, H);
    ET_REQUIRE(stat_groups >= 1 && stat_groups <= kMaxStatGroups, ET_ERR_INVALID_ARG,
               "et_norm_from_stats_f16: stat_groups=%d must be in [1, %d]", stat_groups, kMaxStatGroups);
    ET_REQUIRE(H % 8 == 0, ET_ERR_UNSUPPORTED, "et_norm_from_stats_f16: H=%d must be a multiple of 8", H);
    if (rows == 0) return ET_OK;
    norm_from_stats_kernel<<<(rows + kRowsPerBlock - 1) / kRowsPerBlock, kWave * kRowsPerBlock, 0, as_stream(stream)>>>(
        reinterpret_cast<_Float16 *>(out), reinterpret_cast<const _Float16 *>(V),
        reinterpret_cast<const _Float16 *>(skip), stats, stat_groups,
        reinterpret_cast<const _Float16 *>(gamma), reinterpret_cast<const _Float16 *>(beta), rows, H, eps);
    return check_launch("norm_from_stats_kernel");
}

int et_norm_from_stats_f32in(float *out32, et_f16 *out16, const float *V, const float *stats, int stat_groups,
                             const et_f16 *gamma, const et_f16 *beta, int rows, int H, float eps, et_stream stream) {
    ET_REQUIRE((out32 || out16) && V && stats && gamma && beta, ET_ERR_INVALID_ARG,
               "et_norm_from_stats_f32in: NULL pointer");
    ET_REQUIRE(rows >= 0 && H > 0, ET_ERR_INVALID_ARG, "et_norm_from_stats_f32in: rows=%d H=%d", rows, H);
    ET_REQUIRE(stat_groups >= 1 && stat_groups <= kMaxStatGroups, ET_ERR_INVALID_ARG,
               "et_norm_from_stats_f32in: stat_groups=%d must be in [1, %d]", stat_groups, kMaxStatGroups);
    ET_REQUIRE(H % 8 == 0, ET_ERR_UNSUPPORTED, "et_norm_from_stats_f32in: H=%d must be a multiple of 8", H);
    if (rows == 0) return ET_OK;
    norm_from_stats_f32in_kernel<<<(rows + kRowsPerBlock - 1) / kRowsPerBlock, kWave * kRowsPerBlock, 0,
                                   as_stream(stream)>>>(out32, reinterpret_cast<_Float16 *>(out16), V, stats, stat_groups,
                                                        reinterpret_cast<const _Float16 *>(gamma),
                                                        reinterpret_cast<const _Float16 *>(beta), rows, H, eps);
    return check_launch("norm_from_stats_f32in_kernel");
}

int et_skip_layernorm_f32(float *out, const float *src, const float *skip, const float *gamma,
                          const float *beta, int rows, int H, float eps, et_stream stream) {
    int s = check_ln_args("et_skip_layernorm_f32", out, src, gamma, beta, rows, H);
    if (s != ET_OK) return s;
    ET_REQUIRE(skip != nullptr, ET_ERR_INVALID_ARG, "et_skip_layernorm_f32: skip is NULL");
    if (rows == 0) return ET_OK;
    return launch_layernorm<true>(out, src, skip, gamma, beta, rows, H, eps, as_stream(stream));
}

int et_layernorm_f32(float *out, const float *src, const float *gamma, const float *beta, int rows, int H,
                     float eps, et_stream stream) {
    int s = check_ln_args("et_layernorm_f32", out, src, gamma, beta, rows, H);
    if (s != ET_OK) return s;
    if (rows == 0) return ET_OK;
    return launch_layernorm<false, float>(out, src, nullptr, gamma, beta, rows, H, eps, as_stream(stream));
}

int et_skip_layernorm_mixed(float *out32, et_f16 *out16, const float *src, const float *skip,
                            const et_f16 *gamma, const et_f16 *beta, int rows, int H, float eps,
                            et_stream stream) {
    int s = check_ln_args("et_skip_layernorm_mixed", out32 ? (const void *)out32 : (const void *)out16, src, gamma,
                          beta, rows, H);
    if (s != ET_OK) return s;
    ET_REQUIRE(skip != nullptr, ET_ERR_INVALID_ARG, "et_skip_layernorm_mixed: skip is NULL");
    if (rows == 0) return ET_OK;
    return launch_skip_layernorm_mixed(out32, reinterpret_cast<_Float16 *>(out16), src, skip,
                                       reinterpret_cast<const _Float16 *>(gamma),
                                       reinterpret_cast<const _Float16 *>(beta), rows, H, eps, as_stream(stream));
}

}  // extern "C"
