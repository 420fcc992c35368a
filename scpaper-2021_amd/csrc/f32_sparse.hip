// binary32 twins of the Linear layers over the tile-sparse, 1x16 vector-sparse and CSR
// weight containers: values are stored, multiplied and accumulated in binary32
// (MFMA 16x16x4 f32 for the tile and vector forms, vector FMA for CSR).  They are the
// verification path of pruned fp32 models, as the dense twins are for dense ones; the
// reference's kernels are binary16 only (Linear/Linear.h:9).
//
// Operand feed shared by the tile and vector forms: v_mfma_f32_16x16x4_f32 contracts 4
// values of k per instruction, lane (r = lane % 16, q = lane / 16) supplying A[r][k_q] and
// B[k_q][r].  A sum over k does not care which k a lane brings as long as A and B bring the
// same one, so lane q holds k = 4q .. 4q+3 of a 16-wide cell (one 16-byte load per operand)
// and the cell takes four instructions, the j-th contracting k = {j, 4+j, 8+j, 12+j}.
#include "common.hip.h"

namespace et {

struct Bsr32Args {
    const int32_t *row_ptr, *col_idx;
    const float *tiles, *bias, *X;
    float *Y;
    int T, in, out, act;
};

__device__ __forceinline__ f4 mfma_cell_f32(const float4 w, const float4 x, f4 acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.x, x.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.y, x.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.z, x.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(w.w, x.w, acc, 0, 0, 0);
    return acc;
}

// lane (r, q) holds features f0 + 4q .. 4q+3 of token `tok`: bias, activation, one 16-byte store
__device__ __forceinline__ void store_cell_f32(float *Y, const float *bias, f4 acc, int tok, int T, int out,
                                               int f0, int act) {
    if (tok >= T) return;
    float4 o;
    float *po = reinterpret_cast<float *>(&o);
#pragma unroll
    for (int e = 0; e < 4; e++) po[e] = apply_act(acc[e] + (bias ? bias[f0 + e] : 0.0f), act);
    *reinterpret_cast<float4 *>(Y + (size_t)tok * out + f0) = o;
}

// ---- 16x16 tiles ----------------------------------------------------------------
// A wave owns one block-row (16 output features) and MT blocks of 16 tokens; the four
// waves of a workgroup take four neighbouring block-rows over the same tokens, so the rows
// of X they read are shared through the cache.  Tile t of the block-row: A = its 16 x 16
// weights (row = feature), B = X[tokens][16 col_idx[t] ..].
template <int MT>
__global__ __launch_bounds__(256) void bsr16_linear_f32_kernel(const Bsr32Args a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, q = lane >> 4;
    const int br = blockIdx.x * 4 + wave;
    if (br >= (a.out >> 4)) return;  // no workgroup barrier below
    const int tok0 = blockIdx.y * (MT * 16);
    const float *xrow[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) {
        const int tok = tok0 + m * 16 + r16;
        xrow[m] = a.X + (size_t)(tok < a.T ? tok : a.T - 1) * a.in + 4 * q;  // rows past the end: clamped, not stored
    }
    f4 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = f4{0.f, 0.f, 0.f, 0.f};
    const int ts = a.row_ptr[br], te = a.row_ptr[br + 1];
    const float *wp = a.tiles + (size_t)ts * 256 + r16 * 16 + 4 * q;
#pragma unroll 2
    for (int t = ts; t < te; t++, wp += 256) {
        const int c = a.col_idx[t];
        const float4 w = *reinterpret_cast<const float4 *>(wp);
#pragma unroll
        for (int m = 0; m < MT; m++)
            acc[m] = mfma_cell_f32(w, *reinterpret_cast<const float4 *>(xrow[m] + c * 16), acc[m]);
    }
#pragma unroll
    for (int m = 0; m < MT; m++)
        store_cell_f32(a.Y, a.bias, acc[m], tok0 + m * 16 + r16, a.T, a.out, br * 16 + 4 * q, a.act);
}

// ---- 1x16 vectors ---------------------------------------------------------------
struct V16F32Args {
    const int32_t *tile_idx, *row_idx;
    const float *data, *bias, *X;
    float *Y;
    int T, in, out, act;
};

constexpr int kV16F32Ld = 20;  // floats per row of the per-wave 16 x 16 weight cell (16-byte aligned rows)

// A wave owns one row-set and MT blocks of 16 tokens.  For each part that holds vectors it
// clears its private 16 x 16 cell in LDS, drops the vectors into the rows they name
// (row_idx % 16, at most 16 of them) and multiplies with the cell as the A operand.  LDS
// operations of one wave execute in issue order: clear, fill and read need no barrier.
template <int MT>
__global__ __launch_bounds__(256) void vec1x16_linear_f32_kernel(const V16F32Args a) {
    __shared__ __align__(16) float cells[4][16 * kV16F32Ld];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, q = lane >> 4;
    const int npart = a.in >> 4;
    const int rset = blockIdx.x * 4 + wave;
    if (rset >= (a.out >> 4)) return;  // no workgroup barrier below
    const int tok0 = blockIdx.y * (MT * 16);
    float *cell = cells[wave];
    const int32_t *cellp = a.tile_idx + (size_t)rset * (npart + 1);
    const float *xrow[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) {
        const int tok = tok0 + m * 16 + r16;
        xrow[m] = a.X + (size_t)(tok < a.T ? tok : a.T - 1) * a.in + 4 * q;
    }
    f4 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = f4{0.f, 0.f, 0.f, 0.f};
    const float4 zero4 = float4{0.f, 0.f, 0.f, 0.f};
    const int fill_vec = lane >> 2, fill_q = lane & 3;  // four lanes copy one vector
    for (int p = 0; p < npart; p++) {
        const int s = cellp[p], e = cellp[p + 1];
        if (e == s) continue;  // wave-uniform
        *reinterpret_cast<float4 *>(cell + fill_vec * kV16F32Ld + fill_q * 4) = zero4;
        const int idx = s + fill_vec;
        if (idx < e) {
            const int row = a.row_idx[idx] & 15;
            *reinterpret_cast<float4 *>(cell + row * kV16F32Ld + fill_q * 4) =
                *reinterpret_cast<const float4 *>(a.data + (size_t)idx * 16 + fill_q * 4);
        }
        const float4 w = *reinterpret_cast<const float4 *>(cell + r16 * kV16F32Ld + 4 * q);
#pragma unroll
        for (int m = 0; m < MT; m++)
            acc[m] = mfma_cell_f32(w, *reinterpret_cast<const float4 *>(xrow[m] + p * 16), acc[m]);
    }
#pragma unroll
    for (int m = 0; m < MT; m++)
        store_cell_f32(a.Y, a.bias, acc[m], tok0 + m * 16 + r16, a.T, a.out, rset * 16 + 4 * q, a.act);
}

// ---- CSR ------------------------------------------------------------------------
struct Csr32Args {
    const int32_t *indptr, *indices;
    const float *data, *bias, *X;
    float *Y;
    int T, in, out, act;
};

// A wave takes 16 tokens and four output features at a time: lane (tok = lane % 16,
// g = lane / 16) accumulates feature o0 + g of its token over that feature's non-zeros
// (index and value are the same for the 16 lanes of a feature; the rows of X come from
// the cache), then lane g == 0 collects the four results of its token into one 16-byte
// store.  Workgroup = 4 waves over the same tokens, 16 features a trip.
__global__ __launch_bounds__(256) void csr_linear_f32_kernel(const Csr32Args a, int rows_per_wg) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tokl = lane & 15, g = lane >> 4;
    const int tok = blockIdx.y * 16 + tokl;
    const bool tok_ok = tok < a.T;
    const float *xrow = a.X + (size_t)(tok_ok ? tok : 0) * a.in;
    const int o_begin = blockIdx.x * rows_per_wg;
    const int o_end = min(o_begin + rows_per_wg, a.out);
    for (int o0 = o_begin + wave * 4; o0 < o_end; o0 += 16) {  // out % 4 == 0: a group of four is whole
        const int o = o0 + g;
        const int ks = a.indptr[o], ke = a.indptr[o + 1];
        float acc = 0.0f;
        int k = ks;
        for (; k + 4 <= ke; k += 4) {  // four non-zeros a trip: their loads are issued together
            int idx[4];
            float val[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                idx[u] = a.indices[k + u];
                val[u] = a.data[k + u];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) acc = fmaf(val[u], xrow[idx[u]], acc);
        }
        for (; k < ke; k++) acc = fmaf(a.data[k], xrow[a.indices[k]], acc);
        acc = apply_act(acc + (a.bias ? a.bias[o] : 0.0f), a.act);
        const float v1 = __shfl(acc, tokl + 16, kWave);
        const float v2 = __shfl(acc, tokl + 32, kWave);
        const float v3 = __shfl(acc, tokl + 48, kWave);
        if (g == 0 && tok_ok) *reinterpret_cast<float4 *>(a.Y + (size_t)tok * a.out + o0) = float4{acc, v1, v2, v3};
    }
}

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// token blocks of 16 per wave: more of them reuse a weight cell more often, fewer give a
// small problem more workgroups
static inline int token_blocks(int T) { return T >= 2048 ? 4 : T >= 64 ? 2 : 1; }

}  // namespace et

using namespace et;

extern "C" {

int et_linear_bsr16_f32(const int32_t *row_ptr, const int32_t *col_idx, const float *tiles, const float *bias,
                        const float *X, float *Y, int T, int in, int out, int act, et_stream stream) {
    ET_REQUIRE(row_ptr && col_idx && tiles && X && Y, ET_ERR_INVALID_ARG, "et_linear_bsr16_f32: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0, ET_ERR_INVALID_ARG, "et_linear_bsr16_f32: T=%d in=%d out=%d", T, in, out);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_bsr16_f32: act=%d", act);
    ET_REQUIRE(in % 16 == 0 && out % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_f32: in=%d out=%d must be multiples of 16", in, out);
    ET_REQUIRE(aligned16(tiles) && aligned16(X) && aligned16(Y), ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_f32: tiles, X and Y must be 16-byte aligned");
    if (T == 0) return ET_OK;
    const Bsr32Args a{row_ptr, col_idx, tiles, bias, X, Y, T, in, out, act};
    const int mt = token_blocks(T);
    const dim3 grid((out / 16 + 3) / 4, (T + 16 * mt - 1) / (16 * mt));
    hipStream_t st = as_stream(stream);
    if (mt == 4) bsr16_linear_f32_kernel<4><<<grid, 256, 0, st>>>(a);
    else if (mt == 2) bsr16_linear_f32_kernel<2><<<grid, 256, 0, st>>>(a);
    else bsr16_linear_f32_kernel<1><<<grid, 256, 0, st>>>(a);
    return check_launch("bsr16_linear_f32_kernel");
}

int et_linear_vec1x16_f32(const int32_t *tile_idx, const int32_t *row_idx, const float *data, const float *bias,
                          const float *X, float *Y, int T, int in, int out, int act, et_stream stream) {
    ET_REQUIRE(tile_idx && row_idx && data && X && Y, ET_ERR_INVALID_ARG, "et_linear_vec1x16_f32: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0, ET_ERR_INVALID_ARG, "et_linear_vec1x16_f32: T=%d in=%d out=%d", T, in, out);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_vec1x16_f32: act=%d", act);
    ET_REQUIRE(in % 16 == 0 && out % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_vec1x16_f32: in=%d out=%d must be multiples of 16", in, out);
    ET_REQUIRE(aligned16(data) && aligned16(X) && aligned16(Y), ET_ERR_UNSUPPORTED,
               "et_linear_vec1x16_f32: data, X and Y must be 16-byte aligned");
    if (T == 0) return ET_OK;
    const V16F32Args a{tile_idx, row_idx, data, bias, X, Y, T, in, out, act};
    const int mt = token_blocks(T);
    const dim3 grid((out / 16 + 3) / 4, (T + 16 * mt - 1) / (16 * mt));
    hipStream_t st = as_stream(stream);
    if (mt == 4) vec1x16_linear_f32_kernel<4><<<grid, 256, 0, st>>>(a);
    else if (mt == 2) vec1x16_linear_f32_kernel<2><<<grid, 256, 0, st>>>(a);
    else vec1x16_linear_f32_kernel<1><<<grid, 256, 0, st>>>(a);
    return check_launch("vec1x16_linear_f32_kernel");
}

int et_linear_csr_f32(const int32_t *indptr, const int32_t *indices, const float *data, const float *bias,
                      const float *X, float *Y, int T, int in, int out, int act, et_stream stream) {
    ET_REQUIRE(indptr && indices && data && X && Y, ET_ERR_INVALID_ARG, "et_linear_csr_f32: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0, ET_ERR_INVALID_ARG, "et_linear_csr_f32: T=%d in=%d out=%d", T, in, out);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_csr_f32: act=%d", act);
    ET_REQUIRE(out % 4 == 0, ET_ERR_UNSUPPORTED, "et_linear_csr_f32: out=%d must be a multiple of 4", out);
    ET_REQUIRE(aligned16(Y), ET_ERR_UNSUPPORTED, "et_linear_csr_f32: Y must be 16-byte aligned");
    if (T == 0) return ET_OK;
    const Csr32Args a{indptr, indices, data, bias, X, Y, T, in, out, act};
    const int strips = (T + 15) / 16;
    int groups = (1024 + strips - 1) / strips;  // about 1024 workgroups, whole 16-feature groups each
    int rpw = (out + groups - 1) / groups;
    rpw = ((rpw + 15) / 16) * 16;
    const dim3 grid((out + rpw - 1) / rpw, strips);
    csr_linear_f32_kernel<<<grid, 256, 0, as_stream(stream)>>>(a, rpw);
    return check_launch("csr_linear_f32_kernel");
}

}  // extern "C"
