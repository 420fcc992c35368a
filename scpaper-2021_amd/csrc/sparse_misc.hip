// Linear layers over the two remaining weight containers:
//  * mat1x16 — 1x16 vector sparsity: MFMA on 16x16 weight tiles assembled in
//    LDS from the surviving 1x16 vectors of a (row-set, part) cell;
//  * csr_mat — unstructured CSR: scalar fp32 multiply-adds against a strip of
//    X held in LDS (no matrix-core shape exists for single-element sparsity).
#include "common.hip.h"

namespace et {

// ------------------------------------------------------------------ 1x16 ----
struct V16Args {
    const int32_t *tile_idx;  // [(out/16) * (npart + 1)] global vector offsets
    const int32_t *row_idx;   // [nvec] absolute output row of each vector
    const _Float16 *data;     // [nvec][16]
    const _Float16 *bias;
    const _Float16 *X;
    _Float16 *Y;
    int T, in, out, act;
};

constexpr int kV16Ld = 32 + 8;  // halfs per row of the per-wave 16x32 weight tile

// A wave owns one row-set (16 output features) and MT blocks of 16 tokens.  For
// each pair of parts (2 x 16 input columns) it clears its private 16x32 LDS
// tile, drops the surviving vectors of both cells into their rows (row_idx % 16),
// and feeds the tile as the MFMA A operand; X fragments come from global memory.
// LDS operations of one wave execute in issue order, so clear, fill and read
// need no barrier.
template <int MT>
__global__ __launch_bounds__(256) void vec1x16_linear_kernel(const V16Args a) {
    __shared__ __align__(16) _Float16 tiles[4][16 * kV16Ld];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, g = lane >> 4;
    const int npart = a.in >> 4;
    const int rset = blockIdx.x * 4 + wave;
    if (rset >= (a.out >> 4)) return;  // no workgroup barrier below
    const int tok0 = blockIdx.y * (MT * 16);
    _Float16 *tile = tiles[wave];
    const int32_t *cell = a.tile_idx + (size_t)rset * (npart + 1);
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    f4 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = f4{0.f, 0.f, 0.f, 0.f};

    const int fill_sel = lane >> 5;        // which part of the pair this lane fills
    const int fill_vec = (lane & 31) >> 1; // vector slot 0..15 inside the cell
    const int fill_half = lane & 1;        // which 8 of the vector's 16 weights

    for (int p = 0; p < npart; p += 2) {
        const int s0 = cell[p], e0 = cell[p + 1];
        const int e1 = (p + 1 < npart) ? cell[p + 2] : e0;
        if (e1 == s0) continue;  // both cells empty
        *reinterpret_cast<h8 *>(tile + (lane >> 2) * kV16Ld + (lane & 3) * 8) = zero8;
        {
            const int s = fill_sel ? e0 : s0;
            const int e = fill_sel ? e1 : e0;
            const int idx = s + fill_vec;
            if (idx < e) {
                const int row = a.row_idx[idx] & 15;
                *reinterpret_cast<h8 *>(tile + row * kV16Ld + fill_sel * 16 + fill_half * 8) =
                    *reinterpret_cast<const h8 *>(a.data + (size_t)idx * 16 + fill_half * 8);
            }
        }
        const h8 w = *reinterpret_cast<const h8 *>(tile + r16 * kV16Ld + g * 8);
        const int part = p + (g >> 1);
        const bool part_ok = part < npart;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const int tok = tok0 + m * 16 + r16;
            h8 x = zero8;
            if (tok < a.T && part_ok)
                x = *reinterpret_cast<const h8 *>(a.X + (size_t)tok * a.in + part * 16 + (g & 1) * 8);
            acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, x, acc[m], 0, 0, 0);
        }
    }
    const int f0 = rset * 16 + g * 4;
    float b[4] = {0.f, 0.f, 0.f, 0.f};
    if (a.bias) {
        const h4 bv = *reinterpret_cast<const h4 *>(a.bias + f0);
#pragma unroll
        for (int j = 0; j < 4; j++) b[j] = (float)bv[j];
    }
#pragma unroll
    for (int m = 0; m < MT; m++) {
        const int tok = tok0 + m * 16 + r16;
        if (tok >= a.T) continue;
        h4 o;
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = (_Float16)apply_act(acc[m][j] + b[j], a.act);
        *reinterpret_cast<h4 *>(a.Y + (size_t)tok * a.out + f0) = o;
    }
}

// Dense [out x in] image of a 1x16 weight.  One wave per (row-set, part) cell:
// it clears the cell's 16x16 block of W (two lanes per row, 16 bytes each),
// then the lanes that have a vector (two per vector) copy its halves to the
// row it names.  A wave's stores to one address complete in issue order.
__global__ __launch_bounds__(256) void vec1x16_expand_kernel(const int32_t *tile_idx, const int32_t *row_idx,
                                                             const _Float16 *data, _Float16 *W, int in,
                                                             int ncell) {
    const int lane = threadIdx.x & 63;
    const int cellno = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (cellno >= ncell) return;
    const int npart = in >> 4;
    const int rset = cellno / npart, part = cellno - rset * npart;
    const int32_t *cell = tile_idx + (size_t)rset * (npart + 1) + part;
    const int s = cell[0], e = cell[1];
    _Float16 *blk = W + (size_t)rset * 16 * in + part * 16;
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    if (lane < 32) *reinterpret_cast<h8 *>(blk + (size_t)(lane >> 1) * in + (lane & 1) * 8) = zero8;
    // a cell holds at most 16 vectors (one per row of the set); more would name a row twice
    for (int idx = s + (lane >> 1); idx < e; idx += 32) {
        const int row = row_idx[idx] & 15;
        *reinterpret_cast<h8 *>(blk + (size_t)row * in + (lane & 1) * 8) =
            *reinterpret_cast<const h8 *>(data + (size_t)idx * 16 + (lane & 1) * 8);
    }
}

// Dense image of a 16x16 BSR weight: one workgroup per block-row clears its 16 rows of W, then
// copies the block-row's tiles to their columns (thread t holds element t of every tile).  A
// position named twice keeps the later tile.
__global__ __launch_bounds__(256) void bsr16_expand_kernel(const int32_t *row_ptr, const int32_t *col_idx,
                                                           const _Float16 *tiles, _Float16 *W, int in) {
    const int rb = blockIdx.x;
    _Float16 *blk = W + (size_t)rb * 16 * in;
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int v = threadIdx.x; v < 2 * in; v += 256) reinterpret_cast<h8 *>(blk)[v] = zero8;  // 16 rows x in / 8 vectors
    __syncthreads();  // the zeros of other threads are ordered before this thread's tile elements
    const int lo = row_ptr[rb], hi = row_ptr[rb + 1];
    const int i = threadIdx.x >> 4, j = threadIdx.x & 15;
    for (int t = lo; t < hi; t++) blk[(size_t)i * in + col_idx[t] * 16 + j] = tiles[(size_t)t * 256 + threadIdx.x];
}

// ------------------------------------------------------------------- CSR ----
struct CsrArgs {
    const int32_t *indptr, *indices;
    const _Float16 *data;
    const _Float16 *bias;
    const _Float16 *X;
    _Float16 *Y;
    int T, in, out, act;
    int rows_per_wg;  // output features per workgroup (multiple of 16)
};

// A workgroup holds 16 token rows of X in LDS and walks a group of output
// features; a wave takes four features at a time: lane (tok = lane%16,
// g = lane/16) accumulates feature o0+g for token tok over that feature's
// non-zeros, then the four results of a token are collected into one lane and
// stored as 8 bytes.
template <bool STAGE>
__global__ __launch_bounds__(256) void csr_linear_kernel(const CsrArgs a) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    _Float16 *xs = reinterpret_cast<_Float16 *>(smem_raw);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tokl = lane & 15, g = lane >> 4;
    const int tok0 = blockIdx.y * 16;
    const int ld = a.in + 2;  // odd word stride: the 16 rows fall into distinct banks
    if (STAGE) {
        for (int e = threadIdx.x; e < 16 * a.in; e += blockDim.x) {
            const int r = e / a.in, c = e - r * a.in;
            xs[r * ld + c] = (tok0 + r < a.T) ? a.X[(size_t)(tok0 + r) * a.in + c] : (_Float16)0;
        }
        __syncthreads();
    }
    const int tok = tok0 + tokl;
    const bool tok_ok = tok < a.T;
    const _Float16 *xrow = STAGE ? xs + tokl * ld : a.X + (size_t)(tok_ok ? tok : 0) * a.in;
    const int o_begin = blockIdx.x * a.rows_per_wg;
    const int o_end = min(o_begin + a.rows_per_wg, a.out);
    for (int o0 = o_begin + wave * 4; o0 < o_end; o0 += 16) {
        const int o = o0 + g;
        float acc = 0.0f;
        if (o < o_end) {
            const int ks = a.indptr[o], ke = a.indptr[o + 1];
            // eight non-zeros per trip: their index and value loads are issued together instead
            // of one dependent chain per non-zero
            int k = ks;
            for (; k + 8 <= ke; k += 8) {
                int idx[8];
                _Float16 val[8];
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    idx[u] = a.indices[k + u];
                    val[u] = a.data[k + u];
                }
#pragma unroll
                for (int u = 0; u < 8; u++) acc += (float)val[u] * (float)xrow[idx[u]];
            }
            for (; k < ke; k++) acc += (float)a.data[k] * (float)xrow[a.indices[k]];
            if (a.bias) acc += (float)a.bias[o];
            acc = apply_act(acc, a.act);
        }
        // collect features o0..o0+3 of this token into the g == 0 lane
        const float v1 = __shfl(acc, tokl + 16, kWave);
        const float v2 = __shfl(acc, tokl + 32, kWave);
        const float v3 = __shfl(acc, tokl + 48, kWave);
        if (g == 0 && tok_ok) {
            if (o0 + 3 < o_end) {
                const h4 v = {(_Float16)acc, (_Float16)v1, (_Float16)v2, (_Float16)v3};
                *reinterpret_cast<h4 *>(a.Y + (size_t)tok * a.out + o0) = v;
            } else {
                const float vals[4] = {acc, v1, v2, v3};
                for (int j = 0; j < 4 && o0 + j < o_end; j++)
                    a.Y[(size_t)tok * a.out + o0 + j] = (_Float16)vals[j];
            }
        }
    }
}

static inline const _Float16 *H(const et_f16 *p) { return reinterpret_cast<const _Float16 *>(p); }
static inline _Float16 *H(et_f16 *p) { return reinterpret_cast<_Float16 *>(p); }

}  // namespace et

using namespace et;

extern "C" {

int et_vec1x16_to_dense_f16(const int32_t *tile_idx, const int32_t *row_idx, const et_f16 *data,
                            et_f16 *W, int in, int out, et_stream stream) {
    ET_REQUIRE(tile_idx && row_idx && data && W, ET_ERR_INVALID_ARG, "et_vec1x16_to_dense_f16: NULL pointer");
    ET_REQUIRE(in > 0 && out > 0 && in % 16 == 0 && out % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_vec1x16_to_dense_f16: in=%d out=%d must be positive multiples of 16", in, out);
    ET_REQUIRE((reinterpret_cast<uintptr_t>(W) & 15) == 0 && (reinterpret_cast<uintptr_t>(data) & 15) == 0,
               ET_ERR_UNSUPPORTED, "et_vec1x16_to_dense_f16: W and data must be 16-byte aligned");
    const long ncell = (long)(out / 16) * (in / 16);
    ET_REQUIRE(ncell <= 0x7fffffffL, ET_ERR_UNSUPPORTED, "et_vec1x16_to_dense_f16: %ld cells", ncell);
    vec1x16_expand_kernel<<<dim3((unsigned)((ncell + 3) / 4)), 256, 0, as_stream(stream)>>>(
        tile_idx, row_idx, H(data), H(W), in, (int)ncell);
    return check_launch("vec1x16_expand_kernel");
}

int et_bsr16_to_dense_f16(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, et_f16 *W, int in,
                          int out, et_stream stream) {
    ET_REQUIRE(row_ptr && col_idx && tiles && W, ET_ERR_INVALID_ARG, "et_bsr16_to_dense_f16: NULL pointer");
    ET_REQUIRE(in > 0 && out > 0 && in % 16 == 0 && out % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_bsr16_to_dense_f16: in=%d out=%d must be positive multiples of 16", in, out);
    ET_REQUIRE((reinterpret_cast<uintptr_t>(W) & 15) == 0, ET_ERR_UNSUPPORTED,
               "et_bsr16_to_dense_f16: W must be 16-byte aligned");
    bsr16_expand_kernel<<<dim3((unsigned)(out / 16)), 256, 0, as_stream(stream)>>>(row_ptr, col_idx, H(tiles), H(W), in);
    return check_launch("bsr16_expand_kernel");
}

int et_linear_vec1x16_f16(const int32_t *tile_idx, const int32_t *row_idx, const et_f16 *data,
                          const et_f16 *bias, const et_f16 *X, et_f16 *Y, int T, int in, int out,
                          int act, et_stream stream) {
    ET_REQUIRE(tile_idx && row_idx && data && X && Y, ET_ERR_INVALID_ARG, "et_linear_vec1x16_f16: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0, ET_ERR_INVALID_ARG, "et_linear_vec1x16_f16: T=%d in=%d out=%d", T,
               in, out);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_vec1x16_f16: act=%d",
               act);
    ET_REQUIRE(T % 16 == 0 && in % 16 == 0 && out % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_vec1x16_f16: T=%d in=%d out=%d must be multiples of 16", T, in, out);
    if (T == 0) return ET_OK;
    V16Args a{tile_idx, row_idx, H(data), H(bias), H(X), H(Y), T, in, out, act};
    const int rsets = out / 16;
    if (T >= 64) {
        vec1x16_linear_kernel<4><<<dim3((rsets + 3) / 4, (T + 63) / 64), 256, 0, as_stream(stream)>>>(a);
    } else {
        vec1x16_linear_kernel<1><<<dim3((rsets + 3) / 4, T / 16), 256, 0, as_stream(stream)>>>(a);
    }
    return check_launch("vec1x16_linear_kernel");
}

int et_linear_csr_f16(const int32_t *indptr, const int32_t *indices, const et_f16 *data,
                      const et_f16 *bias, const et_f16 *X, et_f16 *Y, int T, int in, int out, int act,
                      et_stream stream) {
    ET_REQUIRE(indptr && indices && data && X && Y, ET_ERR_INVALID_ARG, "et_linear_csr_f16: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0, ET_ERR_INVALID_ARG, "et_linear_csr_f16: T=%d in=%d out=%d", T, in,
               out);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_csr_f16: act=%d", act);
    ET_REQUIRE(out % 4 == 0, ET_ERR_UNSUPPORTED, "et_linear_csr_f16: out=%d must be a multiple of 4", out);
    if (T == 0) return ET_OK;
    CsrArgs a{indptr, indices, H(data), H(bias), H(X), H(Y), T, in, out, act, 0};
    const int strips = (T + 15) / 16;
    // about 1024 workgroups, whole 16-feature groups per workgroup
    int groups = (1024 + strips - 1) / strips;
    int rpw = (out + groups - 1) / groups;
    rpw = ((rpw + 15) / 16) * 16;
    a.rows_per_wg = rpw;
    const dim3 grid((out + rpw - 1) / rpw, strips);
    const size_t lds = (size_t)16 * (in + 2) * sizeof(_Float16);
    if (lds <= 160 * 1024) {
        if (lds > 64 * 1024) {
            static bool raised = false;  // more than 64 KB of dynamic LDS needs the attribute, once
            if (!raised) {
                ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(csr_linear_kernel<true>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
                raised = true;
            }
        }
        csr_linear_kernel<true><<<grid, 256, lds, as_stream(stream)>>>(a);
    } else {
        csr_linear_kernel<false><<<grid, 256, 0, as_stream(stream)>>>(a);
    }
    return check_launch("csr_linear_kernel");
}

}  // extern "C"
