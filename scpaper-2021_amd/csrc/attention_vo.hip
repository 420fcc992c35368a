// Attention forms whose probabilities go through memory:
//  * the pre-computed-VO attention of E.T. (FusedAttention): probabilities P are
//    written once as [rows x nh*S] and multiplied with the stacked VO matrix by
//    one MFMA GEMM per sequence;
//  * the unfused baseline (Norm_attn): P then a batched P*V GEMM per head.
// Also the Linear_VO projection (a strided-batched GEMM over heads sharing X).
#include <math.h>

#include "gemm.hip.h"

namespace et {

struct ProbsArgs {
    const _Float16 *Q, *K;
    _Float16 *P;           // [B*S][nh*S]
    const _Float16 *mask;  // [S x S] additive or nullptr
    const int32_t *lens;
    int ldq, ldk, ldp;
    int S, nh;
    float scale_log2e;
    int causal;
    int hd;  // head size, a multiple of 16; the kernel template is the next of 32, 64, 128
};

constexpr float kLog2e_ = 1.4426950408889634f;

// One wave = 16 query rows of one (sequence, head); all S <= 16*NKB scores stay
// in registers.  S^T = K Q^T as in the fused kernel: lane (r = lane%16,
// g = lane/16) holds query r against keys 16*kb + 4g..4g+3.  K fragments come
// straight from global memory (every wave of a head re-reads the same few KiB,
// which the L2 serves).
template <int HD, int NKB>
__global__ __launch_bounds__(256) void mha_probs_kernel(const ProbsArgs a) {
    constexpr int KS = HD / 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwave = blockDim.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int h = blockIdx.y, b = blockIdx.z;
    const int S = a.S;
    const size_t row0 = (size_t)b * S;
    const int qb = blockIdx.x * nwave + wave;
    if (qb * 16 >= S) return;  // no barriers in this kernel
    const int q = qb * 16 + r16;
    int klimit = S;
    if (a.lens) klimit = min(S, max(a.lens[b], 0));
    const int nkb = S >> 4;

    h8 qf[KS];
    {
        // columns [hd, HD) read as zero: no contribution to the scores
        const _Float16 *qp = a.Q + (row0 + q) * a.ldq + h * a.hd + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const bool live = 32 * ks + 8 * g < a.hd;
            qf[ks] = *reinterpret_cast<const h8 *>(qp + (live ? 32 * ks : 0));
            if (!live) qf[ks] = h8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }
    f4 sc[NKB];
    float m = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < NKB; kb++) {
        sc[kb] = f4{0.f, 0.f, 0.f, 0.f};
        if (kb < nkb) {
            if (kb * 16 < klimit) {
                const _Float16 *kp = a.K + (row0 + kb * 16 + r16) * a.ldk + h * a.hd + 8 * g;
#pragma unroll
                for (int ks = 0; ks < KS; ks++) {
                    // a dead column block multiplies the zeros of qf: any valid address will do
                    const h8 kf = *reinterpret_cast<const h8 *>(kp + (32 * ks + 8 * g < a.hd ? 32 * ks : 0));
                    sc[kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[ks], sc[kb], 0, 0, 0);
                }
            }
            const int key0 = kb * 16 + 4 * g;
            float mk[4] = {0.f, 0.f, 0.f, 0.f};
            if (a.mask) {
                const h4 mv = *reinterpret_cast<const h4 *>(a.mask + (size_t)q * S + key0);
#pragma unroll
                for (int j = 0; j < 4; j++) mk[j] = (float)mv[j] * kLog2e_;
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int key = key0 + j;
                float s = sc[kb][j] * a.scale_log2e + mk[j];
                if (key >= klimit || (a.causal && key > q)) s = -INFINITY;
                sc[kb][j] = s;
                m = fmaxf(m, s);
            }
        }
    }
    m = fmaxf(m, __shfl_xor(m, 16, kWave));
    m = fmaxf(m, __shfl_xor(m, 32, kWave));
    if (m == -INFINITY) m = 0.0f;
    float l = 0.0f;
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
        if (kb < nkb) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                sc[kb][j] = __builtin_amdgcn_exp2f(sc[kb][j] - m);  // raw v_exp_f32: tiny results flush to zero
                l += sc[kb][j];
            }
        }
    l += __shfl_xor(l, 16, kWave);
    l += __shfl_xor(l, 32, kWave);
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    _Float16 *pp = a.P + (row0 + q) * a.ldp + (size_t)h * S + 4 * g;
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
        if (kb < nkb) {
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = (_Float16)(sc[kb][j] * inv);
            *reinterpret_cast<h4 *>(pp + kb * 16) = o;
        }
}

template <int HD>
static int launch_probs_hd(const ProbsArgs &a, int B, hipStream_t stream) {
    const int qblocks = a.S / 16;
    const int nwave = qblocks >= 4 ? 4 : qblocks;
    const dim3 grid((qblocks + nwave - 1) / nwave, a.nh, B);
    if (a.S <= 128) mha_probs_kernel<HD, 8><<<grid, nwave * 64, 0, stream>>>(a);
    else if (a.S <= 256) mha_probs_kernel<HD, 16><<<grid, nwave * 64, 0, stream>>>(a);
    else mha_probs_kernel<HD, 32><<<grid, nwave * 64, 0, stream>>>(a);
    return check_launch("mha_probs_kernel");
}

static int launch_probs(const ProbsArgs &a, int B, int hd, hipStream_t stream) {
    if (hd <= 32) return launch_probs_hd<32>(a, B, stream);
    if (hd <= 64) return launch_probs_hd<64>(a, B, stream);
    return launch_probs_hd<128>(a, B, stream);
}

static int check_probs_shape(const char *fn, int B, int S, int nh, int hd, int flags) {
    ET_REQUIRE(B >= 0 && S > 0 && nh > 0 && hd > 0, ET_ERR_INVALID_ARG, "%s: B=%d S=%d nh=%d hd=%d", fn, B,
               S, nh, hd);
    ET_REQUIRE((flags & ~ET_MHA_CAUSAL) == 0, ET_ERR_INVALID_ARG, "%s: flags=%d", fn, flags);
    ET_REQUIRE(S % 16 == 0 && S <= 512, ET_ERR_UNSUPPORTED,
               "%s: S=%d must be a multiple of 16 and at most 512", fn, S);
    ET_REQUIRE(hd % 16 == 0 && hd <= 128, ET_ERR_UNSUPPORTED,
               "%s: head dim %d must be a multiple of 16, at most 128", fn, hd);
    ET_REQUIRE(B <= 65535 && nh <= 65535, ET_ERR_UNSUPPORTED, "%s: grid too large", fn);
    return ET_OK;
}

static inline const _Float16 *H(const et_f16 *p) { return reinterpret_cast<const _Float16 *>(p); }
static inline _Float16 *H(et_f16 *p) { return reinterpret_cast<_Float16 *>(p); }

// dst[h][n][k] = src[h][k][n]: the per-head weights of Linear_VO turned k-contiguous, once, at
// construction (32 x 32 tiles through LDS, both sides coalesced).
__global__ __launch_bounds__(256) void transpose_heads_kernel(_Float16 *__restrict__ dst,
                                                              const _Float16 *__restrict__ src, int Hk, int N) {
    __shared__ _Float16 tile[32][33];
    const size_t head = (size_t)blockIdx.z * Hk * N;
    const int k0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8)
        if (k0 + r < Hk && n0 + tx < N) tile[r][tx] = src[head + (size_t)(k0 + r) * N + n0 + tx];
    __syncthreads();
    for (int r = ty; r < 32; r += 8)
        if (n0 + r < N && k0 + tx < Hk) dst[head + (size_t)(n0 + r) * Hk + k0 + tx] = tile[tx][r];
}

}  // namespace et

using namespace et;

extern "C" {

int et_mha_probs_f16(const et_f16 *Q, const et_f16 *K, int ldq, int ldk, et_f16 *P, const et_f16 *mask,
                     const int32_t *lens, int B, int S, int nh, int hd, float scale, int flags,
                     et_stream stream) {
    ET_REQUIRE(Q && K && P, ET_ERR_INVALID_ARG, "et_mha_probs_f16: NULL pointer");
    int s = check_probs_shape("et_mha_probs_f16", B, S, nh, hd, flags);
    if (s != ET_OK) return s;
    ET_REQUIRE(ldq >= nh * hd && ldk >= nh * hd && ldq % 8 == 0 && ldk % 8 == 0, ET_ERR_INVALID_ARG,
               "et_mha_probs_f16: bad row strides %d %d", ldq, ldk);
    if (B == 0) return ET_OK;
    ProbsArgs a{H(Q), H(K), H(P), H(mask), lens, ldq, ldk, nh * S, S, nh, scale * kLog2e_,
                (flags & ET_MHA_CAUSAL) ? 1 : 0, hd};
    return launch_probs(a, B, hd, as_stream(stream));
}

int et_mha_unfused_f16(const et_f16 *Q, const et_f16 *K, const et_f16 *V, int ldq, int ldk, int ldv,
                       et_f16 *Z, int ldz, et_f16 *P, const et_f16 *mask, const int32_t *lens, int B,
                       int S, int nh, int hd, float scale, int flags, et_stream stream) {
    ET_REQUIRE(V && Z, ET_ERR_INVALID_ARG, "et_mha_unfused_f16: NULL pointer");
    int s = et_mha_probs_f16(Q, K, ldq, ldk, P, mask, lens, B, S, nh, hd, scale, flags, stream);
    if (s != ET_OK || B == 0) return s;
    ET_REQUIRE(ldv >= nh * hd && ldz >= nh * hd && ldv % 8 == 0 && ldz % 4 == 0, ET_ERR_INVALID_ARG,
               "et_mha_unfused_f16: bad row strides %d %d", ldv, ldz);
    // Z_h[b] (S x hd) = P_h[b] (S x S, row stride nh*S) * V_h[b] (S x hd, row stride ldv)
    GemmArgs g = gemm_args(H(P), H(V), H(Z), S, hd, S, nh * S, ldv, ldz);
    g.batch_inner = nh;
    g.sAo = (long long)S * nh * S;
    g.sAi = S;
    g.sBo = (long long)S * ldv;
    g.sBi = hd;
    g.sCo = (long long)S * ldz;
    g.sCi = hd;
    return launch_gemm(g, B * nh, false, as_stream(stream));
}

int et_linear_vo_f16(const et_f16 *W, const et_f16 *bias, const et_f16 *X, et_f16 *VO, int B, int S,
                     int H_, int N, int nh, et_stream stream) {
    ET_REQUIRE(W && X && VO, ET_ERR_INVALID_ARG, "et_linear_vo_f16: NULL pointer");
    ET_REQUIRE(B >= 0 && S > 0 && H_ > 0 && N > 0 && nh > 0, ET_ERR_INVALID_ARG,
               "et_linear_vo_f16: B=%d S=%d H=%d N=%d nh=%d", B, S, H_, N, nh);
    ET_REQUIRE(S % 16 == 0 && H_ % 16 == 0 && N % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_vo_f16: S=%d H=%d N=%d must be multiples of 16", S, H_, N);
    ET_REQUIRE((long long)B * nh <= 65535, ET_ERR_UNSUPPORTED, "et_linear_vo_f16: batch*nhead too large");
    if (B == 0) return ET_OK;
    // VO[b][h] (S x N) = X[b] (S x H) * W[h] (H x N) + bias[h]
    GemmArgs g = gemm_args(H(X), H(W), H(VO), S, N, H_, H_, N, N);
    g.batch_inner = nh;
    g.sAo = (long long)S * H_;
    g.sAi = 0;
    g.sBo = 0;
    g.sBi = (long long)H_ * N;
    g.sCo = (long long)nh * S * N;
    g.sCi = (long long)S * N;
    g.bias = H(bias);
    g.sBias_o = 0;
    g.sBias_i = N;
    return launch_gemm(g, B * nh, false, as_stream(stream));
}

int et_transpose_heads_f16(et_f16 *dst, const et_f16 *src, int nh, int H_, int N, et_stream stream) {
    ET_REQUIRE(dst && src && dst != src, ET_ERR_INVALID_ARG, "et_transpose_heads_f16: NULL or aliasing pointers");
    ET_REQUIRE(nh > 0 && nh <= 65535 && H_ > 0 && N > 0, ET_ERR_INVALID_ARG,
               "et_transpose_heads_f16: nh=%d H=%d N=%d", nh, H_, N);
    const dim3 grid((unsigned)((N + 31) / 32), (unsigned)((H_ + 31) / 32), (unsigned)nh);
    ET_REQUIRE(grid.y <= 65535, ET_ERR_UNSUPPORTED, "et_transpose_heads_f16: H=%d too large", H_);
    transpose_heads_kernel<<<grid, 256, 0, as_stream(stream)>>>(H(dst), H(src), H_, N);
    return check_launch("transpose_heads_kernel");
}

int et_linear_vo_t_f16(const et_f16 *Wt, const et_f16 *bias, const et_f16 *X, et_f16 *VO, int B, int S,
                       int H_, int N, int nh, et_stream stream) {
    ET_REQUIRE(Wt && X && VO, ET_ERR_INVALID_ARG, "et_linear_vo_t_f16: NULL pointer");
    ET_REQUIRE(B >= 0 && S > 0 && H_ > 0 && N > 0 && nh > 0, ET_ERR_INVALID_ARG,
               "et_linear_vo_t_f16: B=%d S=%d H=%d N=%d nh=%d", B, S, H_, N, nh);
    ET_REQUIRE(S % 16 == 0 && H_ % 16 == 0 && N % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_vo_t_f16: S=%d H=%d N=%d must be multiples of 16", S, H_, N);
    ET_REQUIRE((long long)B * nh <= 65535, ET_ERR_UNSUPPORTED, "et_linear_vo_t_f16: batch*nhead too large");
    if (B == 0) return ET_OK;
    // VO[b][h] (S x N) = X[b] (S x H) * Wt[h]^T (Wt[h] is N x H) + bias[h]
    GemmArgs g = gemm_args(H(X), H(Wt), H(VO), S, N, H_, H_, H_, N);
    g.batch_inner = nh;
    g.sAo = (long long)S * H_;
    g.sAi = 0;
    g.sBo = 0;
    g.sBi = (long long)N * H_;
    g.sCo = (long long)nh * S * N;
    g.sCi = (long long)S * N;
    g.bias = H(bias);
    g.sBias_o = 0;
    g.sBias_i = N;
    return launch_gemm(g, B * nh, true, as_stream(stream));
}

int et_linear_vo_keys_f16(const et_f16 *Wt, const et_f16 *X, et_f16 *VOt, int B, int S, int H_, int N, int nh,
                          et_stream stream) {
    ET_REQUIRE(Wt && X && VOt, ET_ERR_INVALID_ARG, "et_linear_vo_keys_f16: NULL pointer");
    ET_REQUIRE(B >= 0 && S > 0 && H_ > 0 && N > 0 && nh > 0, ET_ERR_INVALID_ARG,
               "et_linear_vo_keys_f16: B=%d S=%d H=%d N=%d nh=%d", B, S, H_, N, nh);
    ET_REQUIRE(S % 16 == 0 && H_ % 16 == 0 && N % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_vo_keys_f16: S=%d H=%d N=%d must be multiples of 16", S, H_, N);
    ET_REQUIRE((long long)B * nh <= 65535, ET_ERR_UNSUPPORTED, "et_linear_vo_keys_f16: batch*nhead too large");
    if (B == 0) return ET_OK;
    // VOt[b][h] (N x S) = Wt[h] (N x H) * X[b]^T (X[b] is S x H): the operands of et_linear_vo_t_f16 exchanged
    GemmArgs g = gemm_args(H(Wt), H(X), H(VOt), N, S, H_, H_, H_, S);
    g.batch_inner = nh;
    g.sAo = 0;
    g.sAi = (long long)N * H_;
    g.sBo = (long long)S * H_;
    g.sBi = 0;
    g.sCo = (long long)nh * N * S;
    g.sCi = (long long)N * S;
    return launch_gemm(g, B * nh, true, as_stream(stream));
}

int et_mha_vo_f16(const et_f16 *Q, const et_f16 *K, int ldq, int ldk, const et_f16 *VO, et_f16 *P,
                  et_f16 *out, const et_f16 *bias_o, const int32_t *col_scatter, const et_f16 *mask,
                  const int32_t *lens, int B, int S, int nh, int hd, int N, int out_width, float scale,
                  int flags, et_stream stream) {
    ET_REQUIRE(VO && out, ET_ERR_INVALID_ARG, "et_mha_vo_f16: NULL pointer");
    ET_REQUIRE(N > 0 && N % 16 == 0 && out_width >= N && out_width % 4 == 0, ET_ERR_INVALID_ARG,
               "et_mha_vo_f16: N=%d out_width=%d", N, out_width);
    ET_REQUIRE(col_scatter != nullptr || N == out_width, ET_ERR_INVALID_ARG,
               "et_mha_vo_f16: N < out_width needs the column list");
    int s = et_mha_probs_f16(Q, K, ldq, ldk, P, mask, lens, B, S, nh, hd, scale, flags, stream);
    if (s != ET_OK || B == 0) return s;
    hipStream_t st = as_stream(stream);
    if (col_scatter && N < out_width) {
        // columns no surviving VO column maps to carry the output bias alone
        s = et_fill_rows_bias_f16(out, bias_o, B * S, out_width, stream);
        if (s != ET_OK) return s;
    }
    // out[b] (S x N) = P[b] (S x nh*S) * VO[b] (nh*S x N) + bias_o
    GemmArgs g = gemm_args(H(P), H(VO), H(out), S, N, nh * S, nh * S, N, out_width);
    g.sAo = (long long)S * nh * S;
    g.sBo = (long long)nh * S * N;
    g.sCo = (long long)S * out_width;
    g.bias = H(bias_o);
    g.c_scatter = col_scatter;
    return launch_gemm(g, B, false, st);
}

}  // extern "C"
