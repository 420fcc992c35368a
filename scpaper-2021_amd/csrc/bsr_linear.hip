// Y[T x out] = act(X[T x in] * W^T + bias), W stored as 16x16 tiles (BSR over
// the [out x in] matrix, tile rows = output features) — gfx950 MFMA kernel.
//
// One workgroup owns a strip of MT*16 token rows and a contiguous group of
// block-rows of W.  The token strip of X is staged once in LDS (row stride
// padded by 16 bytes, so the 16 rows a fragment read touches fall in distinct
// banks) and every wave walks the tiles of its block-rows two at a time:
// v_mfma_f32_16x16x32_f16 contracts 32 values, i.e. tile t (k 0..15) and tile
// t+1 (k 16..31) of the same block-row in one instruction.  The reference tile
// layout [tile][out 16][in 16] is exactly the MFMA A-operand feed: lane
// (r = lane%16, g = lane/16) reads 8 consecutive halfs of row r of tile
// t + g/2 at offset 8*(g%2), so a tile pair is one contiguous 1 KiB wave load.
// The B operand is the matching 16-token x 16-feature block of X.  The
// accumulator of lane (r, g) is C[feature 4g..4g+3][token r]: four consecutive
// output features of one token, stored as one 8-byte write after bias and
// activation in fp32.
//
// Tile order inside a block-row is free (the sum commutes), as in the
// reference kernel (Linear/SPMM_tile.cu:277-283).
#include "common.hip.h"

namespace et {

struct BsrArgs {
    const int32_t *row_ptr;
    const int32_t *col_idx;
    const _Float16 *tiles;
    const _Float16 *bias;
    const _Float16 *X;
    _Float16 *Y;
    int T, in, out;
    int rows_per_wg;  // block-rows of W per workgroup
    int act;
};

constexpr int kLdsPad = 8;  // halfs

template <int MT, bool STAGE>
__global__ __launch_bounds__(512) void bsr16_linear_kernel(const BsrArgs a) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    _Float16 *xs = reinterpret_cast<_Float16 *>(smem_raw);

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nwave = blockDim.x >> 6;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int sel = g >> 1;         // which tile of the pair this lane feeds
    const int koff = (g & 1) << 3;  // offset of its 8 k-values inside the tile
    const int tok0 = blockIdx.y * (MT * 16);
    const int nbr = a.out >> 4;
    const int rb_begin = blockIdx.x * a.rows_per_wg;
    const int rb_end = min(rb_begin + a.rows_per_wg, nbr);
    const int lds_ld = a.in + kLdsPad;

    if (STAGE) {
        const int vec_per_row = a.in >> 3;
        const int total = MT * 16 * vec_per_row;
        for (int v = threadIdx.x; v < total; v += blockDim.x) {
            const int r = v / vec_per_row;
            const int c = v - r * vec_per_row;
            const int tok = tok0 + r;
            h8 val = {0, 0, 0, 0, 0, 0, 0, 0};
            if (tok < a.T) val = *reinterpret_cast<const h8 *>(a.X + (size_t)tok * a.in + c * 8);
            *reinterpret_cast<h8 *>(xs + r * lds_ld + c * 8) = val;
        }
        __syncthreads();
    }

    // per-lane base of the B-operand rows (token r16 of each 16-token block)
    const _Float16 *xrow[MT];
    bool tok_ok[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) {
        const int tok = tok0 + m * 16 + r16;
        tok_ok[m] = tok < a.T;
        if (STAGE) {
            xrow[m] = xs + (m * 16 + r16) * lds_ld + koff;
        } else {
            xrow[m] = a.X + (size_t)(tok_ok[m] ? tok : 0) * a.in + koff;
        }
    }
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    for (int rb = rb_begin + wave; rb < rb_end; rb += nwave) {
        f4 acc[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) acc[m] = f4{0.f, 0.f, 0.f, 0.f};

        const int t_begin = a.row_ptr[rb];
        const int t_end = a.row_ptr[rb + 1];
        const _Float16 *wbase = a.tiles + r16 * 16 + koff;

        // Software pipeline: operands of pair p+1 are in flight while pair p
        // is multiplied.
        int ti = t_begin + sel;
        bool ok = ti < t_end;
        h8 w_cur = zero8, x_cur[MT];
        {
            const int col = ok ? a.col_idx[ti] : 0;
            if (ok) w_cur = *reinterpret_cast<const h8 *>(wbase + (size_t)ti * 256);
#pragma unroll
            for (int m = 0; m < MT; m++) {
                x_cur[m] = *reinterpret_cast<const h8 *>(xrow[m] + col * 16);
                if (!ok || (!STAGE && !tok_ok[m])) x_cur[m] = zero8;
            }
        }
        for (int t = t_begin; t < t_end; t += 2) {
            const int tn = ti + 2;
            const bool okn = tn < t_end;
            h8 w_nxt = zero8, x_nxt[MT];
            {
                const int coln = okn ? a.col_idx[tn] : 0;
                if (okn) w_nxt = *reinterpret_cast<const h8 *>(wbase + (size_t)tn * 256);
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    x_nxt[m] = *reinterpret_cast<const h8 *>(xrow[m] + coln * 16);
                    if (!okn || (!STAGE && !tok_ok[m])) x_nxt[m] = zero8;
                }
            }
#pragma unroll
            for (int m = 0; m < MT; m++)
                acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w_cur, x_cur[m], acc[m], 0, 0, 0);
            w_cur = w_nxt;
#pragma unroll
            for (int m = 0; m < MT; m++) x_cur[m] = x_nxt[m];
            ti = tn;
        }

        // epilogue: lane holds features 16*rb + 4g .. +3 of token r16
        const int f0 = rb * 16 + g * 4;
        float b[4] = {0.f, 0.f, 0.f, 0.f};
        if (a.bias) {
            const h4 bv = *reinterpret_cast<const h4 *>(a.bias + f0);
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = (float)bv[j];
        }
#pragma unroll
        for (int m = 0; m < MT; m++) {
            if (!tok_ok[m]) continue;
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; j++) o[j] = (_Float16)apply_act(acc[m][j] + b[j], a.act);
            const int tok = tok0 + m * 16 + r16;
            *reinterpret_cast<h4 *>(a.Y + (size_t)tok * a.out + f0) = o;
        }
    }
}

struct BsrPlan {
    int mt;        // 16-token blocks per workgroup strip
    bool stage;    // X strip staged in LDS
    int threads;   // workgroup size
    int rows_per_wg;
    size_t lds;
};

// Launch geometry.  The strip is staged in LDS whenever MT*16 rows of X fit
// in the 160 KiB a workgroup may hold; the block-row group is sized so that
// the grid is a few workgroups per compute unit.
static BsrPlan plan_bsr(int T, int in, int out) {
    BsrPlan p;
    const size_t lds_cap = 160 * 1024;
    const size_t row_bytes = (size_t)(in + kLdsPad) * sizeof(_Float16);
    p.stage = true;
    if (T >= 64 && 64 * row_bytes <= lds_cap / 2) p.mt = 4;
    else if (T >= 32 && 32 * row_bytes <= lds_cap / 2) p.mt = 2;
    else if (16 * row_bytes <= lds_cap) p.mt = 1;
    else { p.mt = 4; p.stage = false; }
    p.lds = p.stage ? (size_t)p.mt * 16 * row_bytes : 0;
    p.threads = 256;
    const int nbr = out / 16;
    const int strips = (T + p.mt * 16 - 1) / (p.mt * 16);
    const int nwave = p.threads / 64;
    // aim for about 1024 workgroups, at least one block-row per wave
    int groups = (1024 + strips - 1) / strips;
    if (groups < 1) groups = 1;
    int rpw = (nbr + groups - 1) / groups;
    rpw = ((rpw + nwave - 1) / nwave) * nwave;
    if (rpw > nbr) rpw = nbr;
    if (rpw < 1) rpw = 1;
    p.rows_per_wg = rpw;
    return p;
}

template <int MT, bool STAGE>
static int launch_bsr(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    auto kernel = bsr16_linear_kernel<MT, STAGE>;
    if (p.lds > 64 * 1024) {
        static bool raised = false;  // per instantiation
        if (!raised) {
            ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            raised = true;
        }
    }
    const int nbr = args.out / 16;
    const dim3 grid((nbr + p.rows_per_wg - 1) / p.rows_per_wg,
                    (args.T + MT * 16 - 1) / (MT * 16));
    kernel<<<grid, p.threads, p.lds, stream>>>(args);
    return check_launch("bsr16_linear_kernel");
}

static int dispatch_bsr(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    if (p.stage) {
        switch (p.mt) {
            case 4: return launch_bsr<4, true>(args, p, stream);
            case 2: return launch_bsr<2, true>(args, p, stream);
            default: return launch_bsr<1, true>(args, p, stream);
        }
    }
    switch (p.mt) {
        case 4: return launch_bsr<4, false>(args, p, stream);
        case 2: return launch_bsr<2, false>(args, p, stream);
        default: return launch_bsr<1, false>(args, p, stream);
    }
}

}  // namespace et

using namespace et;

static int bsr_check(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles,
                     const et_f16 *X, et_f16 *Y, int T, int in, int out, int act) {
    ET_REQUIRE(row_ptr && col_idx && tiles && X && Y, ET_ERR_INVALID_ARG,
               "et_linear_bsr16_f16: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && out > 0, ET_ERR_INVALID_ARG,
               "et_linear_bsr16_f16: T=%d in=%d out=%d", T, in, out);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG,
               "et_linear_bsr16_f16: act=%d", act);
    ET_REQUIRE(T % 16 == 0 && in % 16 == 0 && out % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_f16: T=%d in=%d out=%d must be multiples of 16", T, in, out);
    return ET_OK;
}

extern "C" {

int et_linear_bsr16_f16(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles,
                        const et_f16 *bias, const et_f16 *X, et_f16 *Y, int T, int in, int out,
                        int act, et_stream stream) {
    int s = bsr_check(row_ptr, col_idx, tiles, X, Y, T, in, out, act);
    if (s != ET_OK) return s;
    if (T == 0) return ET_OK;
    BsrArgs args{row_ptr,
                 col_idx,
                 reinterpret_cast<const _Float16 *>(tiles),
                 reinterpret_cast<const _Float16 *>(bias),
                 reinterpret_cast<const _Float16 *>(X),
                 reinterpret_cast<_Float16 *>(Y),
                 T,
                 in,
                 out,
                 0,
                 act};
    BsrPlan p = plan_bsr(T, in, out);
    args.rows_per_wg = p.rows_per_wg;
    return dispatch_bsr(args, p, as_stream(stream));
}

// Tuning hook: same computation with an explicit launch geometry.  mt in
// {1,2,4}; stage selects the LDS-staged strip; threads a multiple of 64 up to
// 512.  Not part of the drop-in surface.
int et_linear_bsr16_f16_geom(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles,
                             const et_f16 *bias, const et_f16 *X, et_f16 *Y, int T, int in,
                             int out, int act, int mt, int stage, int threads, int rows_per_wg,
                             et_stream stream) {
    int s = bsr_check(row_ptr, col_idx, tiles, X, Y, T, in, out, act);
    if (s != ET_OK) return s;
    ET_REQUIRE((mt == 1 || mt == 2 || mt == 4) && threads >= 64 && threads <= 512 &&
                   threads % 64 == 0 && rows_per_wg >= 1,
               ET_ERR_INVALID_ARG, "et_linear_bsr16_f16_geom: mt=%d threads=%d rows_per_wg=%d", mt,
               threads, rows_per_wg);
    if (T == 0) return ET_OK;
    BsrPlan p;
    p.mt = mt;
    p.stage = stage != 0;
    p.threads = threads;
    p.rows_per_wg = rows_per_wg;
    p.lds = p.stage ? (size_t)mt * 16 * (in + kLdsPad) * sizeof(_Float16) : 0;
    ET_REQUIRE(p.lds <= 160 * 1024, ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_f16_geom: strip of %d rows x %d does not fit LDS", mt * 16, in);
    BsrArgs args{row_ptr,
                 col_idx,
                 reinterpret_cast<const _Float16 *>(tiles),
                 reinterpret_cast<const _Float16 *>(bias),
                 reinterpret_cast<const _Float16 *>(X),
                 reinterpret_cast<_Float16 *>(Y),
                 T,
                 in,
                 out,
                 rows_per_wg,
                 act};
    return dispatch_bsr(args, p, as_stream(stream));
}

}  // extern "C"
