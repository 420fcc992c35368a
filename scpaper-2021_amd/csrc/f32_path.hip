// fp32 twins of the dense Linear and the fused attention: every value is stored,
// multiplied and accumulated in binary32 (MFMA 16x16x4 f32 for the Linear, vector
// FMA for the attention core), so an encoder layer built from them agrees with a
// CPU fp32 forward to ~1e-5.  This is the verification path for dense fp32 models
// (the reference is fp16-only, Linear/Linear.h:9); the production path is fp16.
#include "common.hip.h"

namespace et {

// ---- dense Linear ---------------------------------------------------------------
// Y[T x out] = act(X[T x in] * W^T + b), W [out x in] row-major.  One workgroup of
// 4 waves computes a 64-token x 64-feature block; wave (wr, wc) owns tokens
// 32*wr.. and features 32*wc.. as 2x2 MFMA tiles.  The MFMA A operand is W and the B
// operand is X, so a lane ends with 4 consecutive output features of one token
// (one 16-byte store).
constexpr int kF32K = 64;       // k-values staged per step
constexpr int kF32Ld = kF32K + 1;  // LDS row stride in floats (odd: conflict-free column reads)

// TILE x TILE outputs per workgroup (64 or 32), a wave TILE/2 x TILE/2 of them.  The small
// tile is for problems that would leave compute units idle with the large one: the fp32 MFMA
// rate of the waves that run is what bounds a small problem.
// The pruned forms run the same kernel.  GATHER (column-pruned weight): W is [out x in] over the
// surviving input features and feature k of W multiplies X[:, in_id[k]].  OUT (row-pruned weight,
// W = its surviving rows): kOutScatter stores feature f in column out_id[f] of Y with bias[out_id[f]];
// kOutCompact stores it in column f with that same bias.  ldx and ldy are the row strides of X and Y.
constexpr int kOutPlain = 0, kOutScatter = 1, kOutCompact = 2;
struct LinearF32Args {
    const float *W, *bias, *X;
    float *Y;
    const int32_t *in_id, *out_id;
    int T, in, out, ldx, ldy;
};
template <int ACT, int TILE, bool GATHER, int OUT>
__global__ __launch_bounds__(256) void linear_dense_f32_kernel(const LinearF32Args a) {
    const float *__restrict__ W = a.W;
    const float *__restrict__ bias = a.bias;
    const float *__restrict__ X = a.X;
    float *__restrict__ Y = a.Y;
    const int T = a.T, in = a.in, out = a.out;
    constexpr int WB = TILE / 2;          // wave block
    constexpr int MI = WB / 16;           // 16 x 16 MFMA tiles per wave and dimension
    constexpr int TPR = 256 / TILE;       // staging threads per row
    constexpr int VPT = kF32K / 4 / TPR;  // float4 per thread, operand and step
    __shared__ float xs[TILE * kF32Ld];
    __shared__ float ws[TILE * kF32Ld];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wr = wave >> 1, wc = wave & 1;
    const int tok0 = blockIdx.y * TILE, f0 = blockIdx.x * TILE;
    const int r16 = lane & 15, kq = lane >> 4;

    // staging: thread -> (row, 4 consecutive k at sk, sk + 4 TPR, ...)
    const int srow = threadIdx.x / TPR, sk = (threadIdx.x % TPR) << 2;
    const bool x_ok = tok0 + srow < T, w_ok = f0 + srow < out;
    const float *xp = X + (size_t)(tok0 + (x_ok ? srow : 0)) * a.ldx;
    const float *wp = W + (size_t)(f0 + (w_ok ? srow : 0)) * in;
    const float4 zero4 = float4{0.0f, 0.0f, 0.0f, 0.0f};
    float4 xv[VPT], wv[VPT];
    // unconditional loads from clamped addresses and a select (a load under a branch is waited
    // for on the spot); `in` is a multiple of 16, so a group of 4 is inside or outside
    auto load_step = [&](int k0) {
#pragma unroll
        for (int j = 0; j < VPT; j++) {
            const int k = k0 + sk + 4 * TPR * j;
            const bool k_ok = k < in;
            if (GATHER) {
                const int4 id = *reinterpret_cast<const int4 *>(a.in_id + (k_ok ? k : 0));
                xv[j] = float4{xp[id.x], xp[id.y], xp[id.z], xp[id.w]};
            } else {
                xv[j] = *reinterpret_cast<const float4 *>(xp + (k_ok ? k : 0));
            }
            wv[j] = *reinterpret_cast<const float4 *>(wp + (k_ok ? k : 0));
            if (!(x_ok && k_ok)) xv[j] = zero4;
            if (!(w_ok && k_ok)) wv[j] = zero4;
        }
    };

    f4 acc[MI][MI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < MI; j++) acc[i][j] = f4{0.0f, 0.0f, 0.0f, 0.0f};

    load_step(0);
    for (int k0 = 0; k0 < in; k0 += kF32K) {
        __syncthreads();  // the previous step's reads are done
#pragma unroll
        for (int j = 0; j < VPT; j++) {
            float *xd = xs + srow * kF32Ld + sk + 4 * TPR * j, *wd = ws + srow * kF32Ld + sk + 4 * TPR * j;
            xd[0] = xv[j].x; xd[1] = xv[j].y; xd[2] = xv[j].z; xd[3] = xv[j].w;
            wd[0] = wv[j].x; wd[1] = wv[j].y; wd[2] = wv[j].z; wd[3] = wv[j].w;
        }
        __syncthreads();
        load_step(k0 + kF32K);  // the next step travels while this one is multiplied (past the end: zeros)
#pragma unroll
        for (int kk = 0; kk < kF32K; kk += 4) {
            float a[MI], b[MI];
#pragma unroll
            for (int i = 0; i < MI; i++) {
                a[i] = ws[(wc * WB + i * 16 + r16) * kF32Ld + kk + kq];  // A[m = feature][k]
                b[i] = xs[(wr * WB + i * 16 + r16) * kF32Ld + kk + kq];  // B[k][n = token]
            }
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < MI; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], b[i], acc[i][j], 0, 0, 0);
        }
    }
    // acc[i][j]: token tok0 + WB*wr + 16*i + r16, features f0 + WB*wc + 16*j + 4*kq .. +3
#pragma unroll
    for (int i = 0; i < MI; i++) {
        const int t = tok0 + wr * WB + i * 16 + r16;
        if (t >= T) continue;
#pragma unroll
        for (int j = 0; j < MI; j++) {
            const int f = f0 + wc * WB + j * 16 + kq * 4;
            if (f >= out) continue;  // out % 4 == 0: a group of 4 is inside or outside
            float4 o;
            float *po = reinterpret_cast<float *>(&o);
            int col[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                col[e] = OUT == kOutPlain ? f + e : a.out_id[f + e];
                float v = acc[i][j][e] + (bias ? bias[col[e]] : 0.0f);
                if (ACT == ET_ACT_RELU) v = v > 0.0f ? v : 0.0f;
                if (ACT == ET_ACT_GELU) v = gelu_tanh(v);
                po[e] = v;
            }
            if (OUT == kOutScatter) {
#pragma unroll
                for (int e = 0; e < 4; e++) Y[(size_t)t * a.ldy + col[e]] = po[e];
            } else {
                *reinterpret_cast<float4 *>(Y + (size_t)t * a.ldy + f) = o;
            }
        }
    }
}

// ---- fused attention ------------------------------------------------------------
// One workgroup = 16 queries of one head of one sequence.  The 16 x S strip of scores
// lives in LDS as fp32; K and V pass through LDS in blocks of 64 keys.  Thread
// (q = tid/16, c = tid%16) owns scores of keys c, c+16, .. of query q and output
// features c, c+16, .. of query q.
constexpr int kAttQ = 16;
constexpr int kAttKeys = 64;

struct MhaF32Args {
    const float *Q, *K, *V;
    float *Z;
    const float *mask;
    const int32_t *lens;
    int ldq, ldk, ldv, ldz;
    int B, S, nh, hd;
    float scale;
    int causal;
};

template <int HD>
__global__ __launch_bounds__(256) void mha_fused_f32_kernel(const MhaF32Args a) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float *qs = reinterpret_cast<float *>(smem_raw);  // [16][HD]
    float *kv = qs + kAttQ * HD;                       // [64][HD + 1]
    float *sc = kv + kAttKeys * (HD + 1);              // [16][S]
    const int q0 = blockIdx.x * kAttQ, h = blockIdx.y, b = blockIdx.z;
    const int q = threadIdx.x >> 4, c = threadIdx.x & 15;
    const int len = a.lens ? min(max(a.lens[b], 0), a.S) : a.S;
    const size_t row0 = (size_t)b * a.S;
    constexpr int kF = HD / 16;  // output features per thread

    // head sizes between the template sizes: columns [hd, HD) are staged as zero, not written
    const int hd = a.hd;
    float *zrow = a.Z + (row0 + q0 + q) * a.ldz + h * hd;
    if (len == 0) {  // a sequence without keys: zeros
#pragma unroll
        for (int i = 0; i < kF; i++)
            if (c + 16 * i < hd) zrow[c + 16 * i] = 0.0f;
        return;
    }
    for (int i = threadIdx.x; i < kAttQ * HD; i += 256) {
        const int r = i / HD, d = i - r * HD;
        qs[i] = d < hd ? a.Q[(row0 + q0 + r) * a.ldq + h * hd + d] * a.scale : 0.0f;
    }
    // keys this block of queries can see
    int kend = len;
    if (a.causal) kend = min(kend, q0 + kAttQ);
    const float ninf = -__builtin_inff();

    // ---- scores
    for (int kb = 0; kb < kend; kb += kAttKeys) {
        __syncthreads();
        for (int i = threadIdx.x; i < kAttKeys * HD; i += 256) {
            const int r = i / HD, d = i - r * HD;
            kv[r * (HD + 1) + d] = (kb + r < kend && d < hd) ? a.K[(row0 + kb + r) * a.ldk + h * hd + d] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < kAttKeys / 16; i++) {
            const int kl = c + 16 * i, key = kb + kl;
            if (key >= kend) continue;
            float s = 0.0f;
#pragma unroll 8
            for (int d = 0; d < HD; d++) s += qs[q * HD + d] * kv[kl * (HD + 1) + d];
            if (a.mask) s += a.mask[(size_t)(q0 + q) * a.S + key];
            if (a.causal && key > q0 + q) s = ninf;
            sc[q * a.S + key] = s;
        }
    }
    __syncthreads();
    // ---- softmax over keys [0, kend) of row q: 16 threads per row
    float m = ninf;
    for (int k = c; k < kend; k += 16) m = fmaxf(m, sc[q * a.S + k]);
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 16));
    float l = 0.0f;
    for (int k = c; k < kend; k += 16) {
        const float p = m == ninf ? 0.0f : __expf(sc[q * a.S + k] - m);
        sc[q * a.S + k] = p;
        l += p;
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) l += __shfl_xor(l, off, 16);

    // ---- Z = P V
    float acc[kF];
#pragma unroll
    for (int i = 0; i < kF; i++) acc[i] = 0.0f;
    for (int kb = 0; kb < kend; kb += kAttKeys) {
        __syncthreads();
        for (int i = threadIdx.x; i < kAttKeys * HD; i += 256) {
            const int r = i / HD, d = i - r * HD;
            kv[r * (HD + 1) + d] = (kb + r < kend && d < hd) ? a.V[(row0 + kb + r) * a.ldv + h * hd + d] : 0.0f;
        }
        __syncthreads();
        const int nk = min(kAttKeys, kend - kb);
        for (int k = 0; k < nk; k++) {
            const float p = sc[q * a.S + kb + k];
#pragma unroll
            for (int i = 0; i < kF; i++) acc[i] += p * kv[k * (HD + 1) + c + 16 * i];
        }
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
    for (int i = 0; i < kF; i++)
        if (c + 16 * i < hd) zrow[c + 16 * i] = acc[i] * inv;
}

template <int OP>
__global__ __launch_bounds__(256) void unary_f32_kernel(float *__restrict__ out, const float *__restrict__ in,
                                                        size_t n) {
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += step) {
        const float x = in[i];
        out[i] = OP == 0 ? gelu_tanh(x) : (x > 0.0f ? x : 0.0f);
    }
}

// Y[r][c] = act(bias[c]) (act(0) without a bias): the value of a pruned output feature.
__global__ __launch_bounds__(256) void fill_rows_bias_act_f32_kernel(float *__restrict__ Y,
                                                                     const float *__restrict__ bias, size_t n,
                                                                     int cols, int act) {
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += step)
        Y[i] = apply_act(bias ? bias[i % cols] : 0.0f, act);
}

}  // namespace et

using namespace et;

extern "C" {

// One launch of the Linear kernel in the form (gather, out mode, activation) names.
static int launch_linear_f32(const LinearF32Args &a, int act, bool gather, int out_mode, hipStream_t st) {
    // 64 x 64 tiles once they give every compute unit a workgroup, 32 x 32 below that
    const bool small = (long long)((a.out + 63) / 64) * ((a.T + 63) / 64) < 256;
    const int tile = small ? 32 : 64;
    const dim3 grid((a.out + tile - 1) / tile, (a.T + tile - 1) / tile);
#define ET_F32_FORM(ACTV, G, O)                                                       \
    {                                                                                 \
        if (small) linear_dense_f32_kernel<ACTV, 32, G, O><<<grid, 256, 0, st>>>(a);  \
        else linear_dense_f32_kernel<ACTV, 64, G, O><<<grid, 256, 0, st>>>(a);        \
    }
#define ET_F32_LINEAR(ACTV)                                                \
    {                                                                      \
        if (gather) ET_F32_FORM(ACTV, true, kOutPlain)                     \
        else if (out_mode == kOutScatter) ET_F32_FORM(ACTV, false, kOutScatter)  \
        else if (out_mode == kOutCompact) ET_F32_FORM(ACTV, false, kOutCompact)  \
        else ET_F32_FORM(ACTV, false, kOutPlain)                           \
    }
    switch (act) {
        case ET_ACT_RELU: ET_F32_LINEAR(ET_ACT_RELU) break;
        case ET_ACT_GELU: ET_F32_LINEAR(ET_ACT_GELU) break;
        default: ET_F32_LINEAR(ET_ACT_NONE) break;
    }
#undef ET_F32_LINEAR
#undef ET_F32_FORM
    return check_launch("linear_dense_f32_kernel");
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int et_linear_dense_f32(const float *W, const float *bias, const float *X, float *Y, int T, int in, int out,
                        int act, et_stream stream) {
    ET_REQUIRE(W && X && Y, ET_ERR_INVALID_ARG, "et_linear_dense_f32: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0, ET_ERR_INVALID_ARG, "et_linear_dense_f32: T=%d in=%d out=%d", T, in, out);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_dense_f32: act=%d", act);
    ET_REQUIRE(in % 16 == 0 && out % 4 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_dense_f32: in=%d must be a multiple of 16, out=%d of 4", in, out);
    ET_REQUIRE(aligned16(W) && aligned16(X) && aligned16(Y), ET_ERR_UNSUPPORTED,
               "et_linear_dense_f32: W, X and Y must be 16-byte aligned");
    if (T == 0) return ET_OK;
    const LinearF32Args a{W, bias, X, Y, nullptr, nullptr, T, in, out, in, out};
    return launch_linear_f32(a, act, false, kOutPlain, as_stream(stream));
}

int et_linear_rowpruned_f32(const float *rows, const int32_t *row_id, int nnz_row, const float *bias,
                            const float *X, float *Y, int T, int in, int out, int act, et_stream stream) {
    ET_REQUIRE(X && Y && (nnz_row == 0 || (rows && row_id)), ET_ERR_INVALID_ARG, "et_linear_rowpruned_f32: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0 && nnz_row >= 0 && nnz_row <= out, ET_ERR_INVALID_ARG,
               "et_linear_rowpruned_f32: T=%d in=%d out=%d nnz_row=%d", T, in, out, nnz_row);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_rowpruned_f32: act=%d", act);
    ET_REQUIRE(in % 16 == 0 && nnz_row % 4 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_rowpruned_f32: in=%d must be a multiple of 16, nnz_row=%d of 4", in, nnz_row);
    ET_REQUIRE(aligned16(rows) && aligned16(X), ET_ERR_UNSUPPORTED,
               "et_linear_rowpruned_f32: rows and X must be 16-byte aligned");
    if (T == 0) return ET_OK;
    hipStream_t st = as_stream(stream);
    // pruned features: act(bias) — every column is written first, the surviving ones again below
    const size_t n = (size_t)T * out;
    fill_rows_bias_act_f32_kernel<<<(unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536), 256, 0, st>>>(
        Y, bias, n, out, act);
    const int s = check_launch("fill_rows_bias_act_f32_kernel");
    if (s != ET_OK || nnz_row == 0) return s;
    const LinearF32Args a{rows, bias, X, Y, nullptr, row_id, T, in, nnz_row, in, out};
    return launch_linear_f32(a, act, false, kOutScatter, st);
}

int et_linear_rowpruned_compact_f32(const float *rows, const int32_t *row_id, int nnz_row, const float *bias,
                                    const float *X, float *Yc, int T, int in, et_stream stream) {
    ET_REQUIRE(rows && row_id && X && Yc, ET_ERR_INVALID_ARG, "et_linear_rowpruned_compact_f32: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && nnz_row > 0, ET_ERR_INVALID_ARG,
               "et_linear_rowpruned_compact_f32: T=%d in=%d nnz_row=%d", T, in, nnz_row);
    ET_REQUIRE(in % 16 == 0 && nnz_row % 4 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_rowpruned_compact_f32: in=%d must be a multiple of 16, nnz_row=%d of 4", in, nnz_row);
    ET_REQUIRE(aligned16(rows) && aligned16(X) && aligned16(Yc), ET_ERR_UNSUPPORTED,
               "et_linear_rowpruned_compact_f32: rows, X and Yc must be 16-byte aligned");
    if (T == 0) return ET_OK;
    const LinearF32Args a{rows, bias, X, Yc, nullptr, row_id, T, in, nnz_row, in, nnz_row};
    return launch_linear_f32(a, ET_ACT_NONE, false, bias ? kOutCompact : kOutPlain, as_stream(stream));
}

int et_linear_colpruned_f32(const float *cols, const int32_t *col_id, int nnz_col, const float *bias,
                            const float *X, float *Y, int T, int in, int out, int act, et_stream stream) {
    ET_REQUIRE(cols && col_id && X && Y, ET_ERR_INVALID_ARG, "et_linear_colpruned_f32: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0 && nnz_col > 0 && nnz_col <= in, ET_ERR_INVALID_ARG,
               "et_linear_colpruned_f32: T=%d in=%d out=%d nnz_col=%d", T, in, out, nnz_col);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_colpruned_f32: act=%d", act);
    ET_REQUIRE(nnz_col % 16 == 0 && out % 4 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_colpruned_f32: nnz_col=%d must be a multiple of 16, out=%d of 4", nnz_col, out);
    ET_REQUIRE(aligned16(cols) && aligned16(col_id) && aligned16(Y), ET_ERR_UNSUPPORTED,
               "et_linear_colpruned_f32: cols, col_id and Y must be 16-byte aligned");
    if (T == 0) return ET_OK;
    const LinearF32Args a{cols, bias, X, Y, col_id, nullptr, T, nnz_col, out, in, out};
    return launch_linear_f32(a, act, true, kOutPlain, as_stream(stream));
}

int et_mha_fused_f32(const float *Q, const float *K, const float *V, int ldq, int ldk, int ldv, float *Z, int ldz,
                     const float *mask, const int32_t *lens, int B, int S, int nh, int hd, float scale, int flags,
                     et_stream stream) {
    ET_REQUIRE(Q && K && V && Z, ET_ERR_INVALID_ARG, "et_mha_fused_f32: NULL pointer");
    ET_REQUIRE(B >= 0 && S > 0 && nh > 0, ET_ERR_INVALID_ARG, "et_mha_fused_f32: B=%d S=%d nh=%d", B, S, nh);
    ET_REQUIRE((flags & ~ET_MHA_CAUSAL) == 0, ET_ERR_INVALID_ARG, "et_mha_fused_f32: flags=%d", flags);
    ET_REQUIRE(S % 16 == 0 && hd > 0 && hd % 16 == 0 && hd <= 128, ET_ERR_UNSUPPORTED,
               "et_mha_fused_f32: S=%d and hd=%d must be multiples of 16, hd at most 128", S, hd);
    const int width = nh * hd;
    ET_REQUIRE(ldq >= width && ldk >= width && ldv >= width && ldz >= width, ET_ERR_INVALID_ARG,
               "et_mha_fused_f32: row strides must cover nh*hd=%d", width);
    const int hdt = hd <= 32 ? 32 : hd <= 64 ? 64 : 128;  // kernel template size
    const size_t lds = sizeof(float) * ((size_t)kAttQ * hdt + (size_t)kAttKeys * (hdt + 1) + (size_t)kAttQ * S);
    ET_REQUIRE(lds <= 160 * 1024, ET_ERR_UNSUPPORTED, "et_mha_fused_f32: S=%d does not fit the on-chip score strip", S);
    if (B == 0) return ET_OK;
    MhaF32Args a{Q, K, V, Z, mask, lens, ldq, ldk, ldv, ldz, B, S, nh, hd, scale, (flags & ET_MHA_CAUSAL) ? 1 : 0};
    const dim3 grid(S / kAttQ, nh, B);
    hipStream_t st = as_stream(stream);
#define ET_MHA32(HD)                                                                                         \
    {                                                                                                        \
        auto kern = mha_fused_f32_kernel<HD>;                                                                \
        if (lds > 64 * 1024)                                                                                 \
            ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                                 \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));               \
        kern<<<grid, 256, lds, st>>>(a);                                                                     \
    }
    if (hdt == 32) ET_MHA32(32) else if (hdt == 64) ET_MHA32(64) else ET_MHA32(128)
#undef ET_MHA32
    return check_launch("mha_fused_f32_kernel");
}

int et_gelu_f32(float *out, const float *in, size_t n, et_stream stream) {
    ET_REQUIRE((out && in) || n == 0, ET_ERR_INVALID_ARG, "et_gelu_f32: NULL pointer");
    if (n == 0) return ET_OK;
    size_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    unary_f32_kernel<0><<<(unsigned)blocks, 256, 0, as_stream(stream)>>>(out, in, n);
    return check_launch("unary_f32_kernel<gelu>");
}

int et_relu_f32(float *out, const float *in, size_t n, et_stream stream) {
    ET_REQUIRE((out && in) || n == 0, ET_ERR_INVALID_ARG, "et_relu_f32: NULL pointer");
    if (n == 0) return ET_OK;
    size_t blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    unary_f32_kernel<1><<<(unsigned)blocks, 256, 0, as_stream(stream)>>>(out, in, n);
    return check_launch("unary_f32_kernel<relu>");
}

}  // extern "C"
