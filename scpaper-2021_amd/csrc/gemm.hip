// Dense fp16 GEMM with fp32 accumulation for gfx950, and the Linear layers
// built on it (dense, row-pruned, column-pruned weights).
//
//   C[M x N] = A[M x K] * B^T   (B stored [N x K]: both operands K-contiguous,
//                                the natural MFMA feed)        trans_b = 1
//   C[M x N] = A[M x K] * B     (B stored [K x N]; the tile is transposed on
//                                its way into LDS)             trans_b = 0
//
// A workgroup of 4 waves (2 x 2) computes a (32*TM) x (32*TN) tile of C; each
// wave owns TM x TN accumulators of 16x16.  K is walked in steps of 64 through
// one LDS stage per operand (row stride padded by 16 bytes); the next stage is
// prefetched into registers while v_mfma_f32_16x16x32_f16 consumes the current
// one.  The MFMA A operand is fed from the B matrix and vice versa, so a lane
// ends with four consecutive columns of one row of C and stores 8 bytes.
//
// Optional fusions, all in the prologue/epilogue of the same kernel:
//   a_gather : column k of A is read from X[:, a_gather[k]]   (col_mat Linear:
//              replaces the reference's separate gather pass, Linear/SPMM_col.cu:8-23)
//   c_scatter: column n of the result is written to C[:, c_scatter[n]]
//              (row_mat Linear: replaces the scatter pass, Linear/SPMM_row.cu:14-30)
//   bias/act : y = act(acc + bias[column]) on the fp32 accumulator.
#include <atomic>
#include <mutex>

#include "gemm.hip.h"

namespace et {

constexpr int kBK = 64;
constexpr int kLdT = kBK + 8;  // halfs per LDS tile row

template <int TM, int TN, bool TRANS_B, bool GATHER>
__global__ __launch_bounds__(256) void gemm_f16_kernel(const GemmArgs g) {
    constexpr int BM = 32 * TM, BN = 32 * TN;
    constexpr int VA = BM * (kBK / 8) / 256;  // 16-byte vectors of the A stage per thread
    constexpr int VB = BN * (kBK / 8) / 256;
    __shared__ __align__(16) _Float16 As[BM * kLdT];
    __shared__ __align__(16) _Float16 Bs[BN * kLdT];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int r16 = lane & 15, grp = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const long long zo = blockIdx.z / g.batch_inner, zi = blockIdx.z % g.batch_inner;
    const _Float16 *A = g.A + zo * g.sAo + zi * g.sAi;
    const _Float16 *B = g.B + zo * g.sBo + zi * g.sBi;
    _Float16 *Cm = g.C + zo * g.sCo + zi * g.sCi;
    const _Float16 *bias = g.bias ? g.bias + zo * g.sBias_o + zi * g.sBias_i : nullptr;
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    f4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = f4{0.f, 0.f, 0.f, 0.f};

    h8 ra[VA], rb[VB];

    auto load_stage = [&](int k0) {
#pragma unroll
        for (int v = 0; v < VA; v++) {
            const int idx = tid + v * 256;
            const int r = idx >> 3, c = idx & 7;  // kBK/8 = 8 vectors per row
            const int m = m0 + r, k = k0 + c * 8;
            h8 val = zero8;
            if (m < g.M && k < g.K) {
                if (GATHER) {
#pragma unroll
                    for (int e = 0; e < 8; e++) val[e] = A[(size_t)m * g.lda + g.a_gather[k + e]];
                } else {
                    val = *reinterpret_cast<const h8 *>(A + (size_t)m * g.lda + k);
                }
            }
            ra[v] = val;
        }
#pragma unroll
        for (int v = 0; v < VB; v++) {
            const int idx = tid + v * 256;
            h8 val = zero8;
            if (TRANS_B) {
                const int r = idx >> 3, c = idx & 7;
                const int n = n0 + r, k = k0 + c * 8;
                if (n < g.N && k < g.K) val = *reinterpret_cast<const h8 *>(B + (size_t)n * g.ldb + k);
            } else {
                // B is [K x N]: vector = 8 consecutive n of one k
                constexpr int vec_per_k = BN / 8;
                const int kk = idx / vec_per_k, c = idx - kk * vec_per_k;
                const int k = k0 + kk, n = n0 + c * 8;
                if (k < g.K && n < g.N) val = *reinterpret_cast<const h8 *>(B + (size_t)k * g.ldb + n);
            }
            rb[v] = val;
        }
    };
    auto store_stage = [&]() {
#pragma unroll
        for (int v = 0; v < VA; v++) {
            const int idx = tid + v * 256;
            const int r = idx >> 3, c = idx & 7;
            *reinterpret_cast<h8 *>(As + r * kLdT + c * 8) = ra[v];
        }
#pragma unroll
        for (int v = 0; v < VB; v++) {
            const int idx = tid + v * 256;
            if (TRANS_B) {
                const int r = idx >> 3, c = idx & 7;
                *reinterpret_cast<h8 *>(Bs + r * kLdT + c * 8) = rb[v];
            } else {
                constexpr int vec_per_k = BN / 8;
                const int kk = idx / vec_per_k, c = idx - kk * vec_per_k;
#pragma unroll
                for (int e = 0; e < 8; e++) Bs[(c * 8 + e) * kLdT + kk] = rb[v][e];
            }
        }
    };

    load_stage(0);
    for (int k0 = 0; k0 < g.K; k0 += kBK) {
        __syncthreads();  // previous stage fully consumed
        store_stage();
        __syncthreads();
        if (k0 + kBK < g.K) load_stage(k0 + kBK);
#pragma unroll
        for (int ks = 0; ks < kBK / 32; ks++) {
            h8 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++)
                fa[i] = *reinterpret_cast<const h8 *>(As + ((wm * TM + i) * 16 + r16) * kLdT + ks * 32 + grp * 8);
#pragma unroll
            for (int j = 0; j < TN; j++)
                fb[j] = *reinterpret_cast<const h8 *>(Bs + ((wn * TN + j) * 16 + r16) * kLdT + ks * 32 + grp * 8);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
    }

    // epilogue: lane holds C[m = r16 of block i][n = 4*grp .. +3 of block j]
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + (wm * TM + i) * 16 + r16;
        if (m >= g.M) continue;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + (wn * TN + j) * 16 + grp * 4;
            if (n >= g.N) continue;
            if (g.c_scatter) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int col = g.c_scatter[n + e];
                    float y = acc[i][j][e];
                    if (bias) y += (float)bias[col];
                    Cm[(size_t)m * g.ldc + col] = (_Float16)apply_act(y, g.act);
                }
            } else {
                h4 o;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float y = acc[i][j][e];
                    if (bias) y += (float)bias[g.bias_idx ? g.bias_idx[n + e] : n + e];
                    o[e] = (_Float16)apply_act(y, g.act);
                }
                *reinterpret_cast<h4 *>(Cm + (size_t)m * g.ldc + n) = o;
            }
        }
    }
}

// Small results with a long K (one sequence through a pruned or dense Linear: 128 x 80 x 768):
// the tiled kernels would run a handful of workgroups, each stepping through K stage by stage —
// 12 dependent round trips for K = 768.  Here a workgroup owns one 16x16 tile of the result and
// its four waves split K between them; a wave requests all the rows of up to STEPS pieces of 64
// k-values before the first product, so the whole kernel is one or two memory round trips plus an
// LDS reduction of three partial tiles.  B is [N x K] (transposed form), no A-column gather; rows
// 16-byte aligned.  Every tile reads its 16 rows of A and of B in full, so this only pays while
// the tiles are few (used up to 1024 of them where the 64x64 tiling has fewer than 64 workgroups;
// 128 x 768 -> 80 / 384 / 768: 7.1 us tiled, 3.9 / 4.0 / 5.3 with fragments loaded straight from
// memory, 3.0 / 3.0 / 3.6 with whole rows; 256 x 768 -> 768: 7.5 -> 6.8 -> 4.4; 128 x 3072 -> 768:
// 18.6 -> 14.6 -> 7.7).  STEPS = 3 when that covers a wave's share of K: rows requested for
// pieces a wave does not have cost as much as real ones.
template <int STEPS>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const GemmArgs g) {
    // STEPS = pieces of 64 k-values (two MFMAs) a wave requests per round.  A wave loads whole rows
    // of its share — 8 rows x 128 bytes per instruction, the four lanes of a quad inside one cache
    // line — and turns each piece into fragments through 4 KB of LDS of its own (written as
    // loaded, read back in fragment order, 16-byte chunks XOR-swizzled by the row): a fragment
    // load straight from memory puts a quad of lanes on four rows and costs the memory pipeline
    // four times as much.  One wave's LDS instructions execute in order, so the piece is reused
    // without a barrier.
    constexpr int kPieces = STEPS;
    __shared__ f4 part[3][64];
    __shared__ __align__(16) _Float16 piece_lds[4][2][16 * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, grp = lane >> 4;
    const int row8 = lane >> 3, ch = lane & 7;  // place of this lane in a whole-row load
    const int ntn = g.N >> 4;
    const int tm = blockIdx.x / ntn, tn = blockIdx.x - tm * ntn;
    const long long zo = blockIdx.z / g.batch_inner, zi = blockIdx.z % g.batch_inner;
    const _Float16 *A = g.A + zo * g.sAo + zi * g.sAi + (size_t)(tm * 16 + row8) * g.lda;  // token rows row8 and row8 + 8
    const _Float16 *B = g.B + zo * g.sBo + zi * g.sBi + (size_t)(tn * 16 + row8) * g.ldb;  // feature rows likewise
    _Float16 *Cm = g.C + zo * g.sCo + zi * g.sCi;
    const _Float16 *bias = g.bias ? g.bias + zo * g.sBias_o + zi * g.sBias_i : nullptr;
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    _Float16 *pa = piece_lds[wave][0], *pb = piece_lds[wave][1];
    // places in a piece, in halfs: row * 64 + (chunk ^ (row & 7)) * 8
    const int w_at = row8 * 64 + ((ch ^ row8) * 8);  // rows row8 (+ 8 rows = + 512 halfs, same swizzle)
    int r_at[2];
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++) r_at[s2] = r16 * 64 + (((4 * s2 + grp) ^ (r16 & 7)) * 8);

    // pieces of this wave: [p_begin, p_end) of ceil(K / 64), a quarter each
    const int npieces = (g.K + 63) >> 6;
    const int per = (npieces + 3) >> 2;
    const int p_begin = wave * per, p_end = min(npieces, p_begin + per);
    f4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int p0 = p_begin; p0 < p_end; p0 += kPieces) {
        // unconditional loads from clamped addresses; values past K or past this wave's share
        // become zeros on their way into LDS (a load under a branch would be waited for on the spot)
        h8 ra[kPieces][2], rb[kPieces][2];
#pragma unroll
        for (int i = 0; i < kPieces; i++) {
            const int kc = min((p0 + i) * 64 + 8 * ch, g.K - 8);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                ra[i][h] = *reinterpret_cast<const h8 *>(A + (size_t)(8 * h) * g.lda + kc);
                rb[i][h] = *reinterpret_cast<const h8 *>(B + (size_t)(8 * h) * g.ldb + kc);
            }
        }
#pragma unroll
        for (int i = 0; i < kPieces; i++) {
            if (p0 + i < p_end) {  // wave-uniform
                const bool live = (p0 + i) * 64 + 8 * ch < g.K;
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    *reinterpret_cast<h8 *>(pa + w_at + h * 512) = live ? ra[i][h] : zero8;
                    *reinterpret_cast<h8 *>(pb + w_at + h * 512) = live ? rb[i][h] : zero8;
                }
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++) {
                    const h8 fa = *reinterpret_cast<const h8 *>(pa + r_at[s2]);
                    const h8 fb = *reinterpret_cast<const h8 *>(pb + r_at[s2]);
                    // features are the A operand: the lane ends with four consecutive features of its token
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb, fa, acc, 0, 0, 0);
                }
            }
        }
    }
    if (wave > 0) part[wave - 1][lane] = acc;
    __syncthreads();
    if (wave > 0) return;
    acc += part[0][lane] + part[1][lane] + part[2][lane];

    const int m = tm * 16 + r16, n = tn * 16 + 4 * grp;
    if (g.c_scatter) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int col = g.c_scatter[n + e];
            float y = acc[e];
            if (bias) y += (float)bias[col];
            Cm[(size_t)m * g.ldc + col] = (_Float16)apply_act(y, g.act);
        }
    } else {
        h4 o;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float y = acc[e];
            if (bias) y += (float)bias[g.bias_idx ? g.bias_idx[n + e] : n + e];
            o[e] = (_Float16)apply_act(y, g.act);
        }
        *reinterpret_cast<h4 *>(Cm + (size_t)m * g.ldc + n) = o;
    }
}

// The small-result kernel applies when the 64x64 tiling would leave most of the chip idle.  Up to
// 2048 tiles of 16 x 16 it beats the 64 x 64 tiles (512 x 768 -> 768: 6.1 against 7.3 us; 128 x 768
// -> 2304: 5.4 against 7.0), from about 2300 on it loses (256 x 768 -> 2304: 8.0 against 7.4).
static bool gemm_skinny_applies(const GemmArgs &g, int batch, bool trans_b) {
    const auto misaligned = [](const void *p, int a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0; };
    if (!trans_b || g.a_gather || batch < 1 || batch > 65535) return false;
    if (g.M <= 0 || g.M % 16 || g.N % 16 || g.K % 16 || g.K < 256) return false;
    if (g.lda % 8 || g.ldb % 8 || misaligned(g.A, 16) || misaligned(g.B, 16)) return false;
    if (!g.c_scatter && (g.ldc % 4 || misaligned(g.C, 8))) return false;
    if (batch > 1 && (((g.sAo | g.sAi | g.sBo | g.sBi) & 7) || ((g.sCo | g.sCi) & 3))) return false;
    const long long tiles64 = (long long)((g.M + 63) / 64) * ((g.N + 63) / 64) * batch;
    const long long tiles16 = (long long)(g.M / 16) * (g.N / 16);
    return tiles64 < 128 && tiles16 <= 2048;
}

// C[r][c] = act(bias[c]) for the columns a row-pruned weight does not produce.
__global__ __launch_bounds__(256) void bias_rows_kernel(_Float16 *__restrict__ C,
                                                        const _Float16 *__restrict__ bias, int rows,
                                                        int cols, int ldc, int act) {
    const size_t total = (size_t)rows * cols;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < total; e += step) {
        const int r = (int)(e / cols), c = (int)(e - (size_t)r * cols);
        const float b = bias ? (float)bias[c] : 0.0f;
        C[(size_t)r * ldc + c] = (_Float16)apply_act(b, act);
    }
}

// The same in 16-byte stores: a thread owns 8 consecutive columns (their values computed once)
// and walks down the rows of its block row-group.  cols and ldc multiples of 8, C 16-byte aligned.
__global__ __launch_bounds__(256) void bias_rows_vec_kernel(_Float16 *__restrict__ C,
                                                            const _Float16 *__restrict__ bias, int rows,
                                                            int cols, int ldc, int act, int rows_per_block) {
    const int chunk = blockIdx.x * blockDim.x + threadIdx.x;
    if (chunk * 8 >= cols) return;
    h8 v;
#pragma unroll
    for (int e = 0; e < 8; e++) v[e] = (_Float16)apply_act(bias ? (float)bias[chunk * 8 + e] : 0.0f, act);
    const int r0 = blockIdx.y * rows_per_block, r1 = min(rows, r0 + rows_per_block);
    for (int r = r0; r < r1; r++) *reinterpret_cast<h8 *>(C + (size_t)r * ldc + chunk * 8) = v;
}

static int launch_bias_rows(_Float16 *C, const _Float16 *bias, int rows, int cols, int ldc, int act,
                            hipStream_t st) {
    if (cols % 8 == 0 && ldc % 8 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0) {
        const int bx = (cols / 8 + 255) / 256;
        int rpb = (int)(((long long)rows * bx + 1023) / 1024);  // about 1024 blocks, at least 4 rows each
        if (rpb < 4) rpb = 4;
        const dim3 grid((unsigned)bx, (unsigned)((rows + rpb - 1) / rpb));
        bias_rows_vec_kernel<<<grid, 256, 0, st>>>(C, bias, rows, cols, ldc, act, rpb);
        return check_launch("bias_rows_vec_kernel");
    }
    const size_t total = (size_t)rows * cols;
    size_t blocks = (total + 255) / 256;
    if (blocks > 2048) blocks = 2048;
    bias_rows_kernel<<<(unsigned)blocks, 256, 0, st>>>(C, bias, rows, cols, ldc, act);
    return check_launch("bias_rows_kernel");
}

template <int TM, int TN>
static int launch_gemm_tile(const GemmArgs &g, int batch, bool trans_b, hipStream_t stream) {
    const dim3 grid((g.N + 32 * TN - 1) / (32 * TN), (g.M + 32 * TM - 1) / (32 * TM), batch);
    const bool gather = g.a_gather != nullptr;
    if (trans_b) {
        if (gather) gemm_f16_kernel<TM, TN, true, true><<<grid, 256, 0, stream>>>(g);
        else gemm_f16_kernel<TM, TN, true, false><<<grid, 256, 0, stream>>>(g);
    } else {
        if (gather) gemm_f16_kernel<TM, TN, false, true><<<grid, 256, 0, stream>>>(g);
        else gemm_f16_kernel<TM, TN, false, false><<<grid, 256, 0, stream>>>(g);
    }
    return check_launch("gemm_f16_kernel");
}

// The direct-to-LDS kernel where it applies; else this file's kernel, with 128x128 tiles once
// they still give a few hundred workgroups and 64x64 otherwise.
int launch_gemm(const GemmArgs &g, int batch, bool trans_b, hipStream_t stream) {
    if (gemm_skinny_applies(g, batch, trans_b)) {
        const dim3 grid((unsigned)((g.M / 16) * (g.N / 16)), 1, (unsigned)batch);
        if (g.K <= 3 * 4 * 64) gemm_skinny_kernel<3><<<grid, 256, 0, stream>>>(g);  // at most 3 pieces of 64 per wave
        else gemm_skinny_kernel<6><<<grid, 256, 0, stream>>>(g);
        return check_launch("gemm_skinny_kernel");
    }
    if (gemm_dma_applies(g, batch, trans_b)) return launch_gemm_dma(g, batch, trans_b, stream);
    const long long tiles128 = (long long)((g.M + 127) / 128) * ((g.N + 127) / 128) * batch;
    if (tiles128 >= 512) return launch_gemm_tile<4, 4>(g, batch, trans_b, stream);
    return launch_gemm_tile<2, 2>(g, batch, trans_b, stream);
}

static int check_gemm_shape(const char *fn, int M, int N, int K) {
    ET_REQUIRE(M >= 0 && N > 0 && K > 0, ET_ERR_INVALID_ARG, "%s: M=%d N=%d K=%d", fn, M, N, K);
    ET_REQUIRE(M % 16 == 0 && N % 16 == 0 && K % 16 == 0, ET_ERR_UNSUPPORTED,
               "%s: M=%d N=%d K=%d must be multiples of 16", fn, M, N, K);
    return ET_OK;
}

static inline const _Float16 *H(const et_f16 *p) { return reinterpret_cast<const _Float16 *>(p); }
static inline _Float16 *H(et_f16 *p) { return reinterpret_cast<_Float16 *>(p); }

// Column gather: dst[t][j] = X[t][col_id[j]], 8 gathered columns per lane (two 16-byte
// index loads, eight 2-byte reads inside one row of X, one 16-byte store) — the
// gather pass of the column-pruned Linear (Linear/SPMM_col.cu:25-39).
__global__ __launch_bounds__(256) void gather_cols_kernel(_Float16 *__restrict__ dst,
                                                          const _Float16 *__restrict__ X,
                                                          const int32_t *__restrict__ col_id, int T,
                                                          int in, int nnz) {
    const int per_row = nnz >> 3;
    const size_t total = (size_t)T * per_row;
    const size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t v = blockIdx.x * (size_t)blockDim.x + threadIdx.x; v < total; v += step) {
        const size_t t = v / per_row;
        const int c = (int)(v - t * per_row) * 8;
        const int4 i0 = *reinterpret_cast<const int4 *>(col_id + c);
        const int4 i1 = *reinterpret_cast<const int4 *>(col_id + c + 4);
        const _Float16 *row = X + t * (size_t)in;
        h8 o;
        o[0] = row[i0.x]; o[1] = row[i0.y]; o[2] = row[i0.z]; o[3] = row[i0.w];
        o[4] = row[i1.x]; o[5] = row[i1.y]; o[6] = row[i1.z]; o[7] = row[i1.w];
        *reinterpret_cast<h8 *>(dst + t * (size_t)nnz + c) = o;
    }
}

// The same through LDS: a workgroup stages R whole rows of X with 16-byte loads (a quad of lanes
// inside one cache line), then every lane picks its 8 columns out of LDS.  The 2-byte reads of the
// kernel above go to memory one by one, each quad of lanes on up to four cache lines of a row
// that the other waves are picking from at the same time.  R * in halfs of dynamic LDS.
__global__ __launch_bounds__(256) void gather_cols_staged_kernel(_Float16 *__restrict__ dst,
                                                                 const _Float16 *__restrict__ X,
                                                                 const int32_t *__restrict__ col_id, int T,
                                                                 int in, int nnz, int R) {
    extern __shared__ __align__(16) unsigned char gather_smem[];
    _Float16 *rows = reinterpret_cast<_Float16 *>(gather_smem);
    const int per_row = nnz >> 3, chunks = in >> 3;
    for (int r0 = blockIdx.x * R; r0 < T; r0 += gridDim.x * R) {
        const int nrow = min(R, T - r0);
        for (int i = threadIdx.x; i < nrow * chunks; i += 256)  // rows r0 .. r0 + nrow are contiguous in X
            reinterpret_cast<h8 *>(rows)[i] = reinterpret_cast<const h8 *>(X + (size_t)r0 * in)[i];
        __syncthreads();
        for (int v = threadIdx.x; v < nrow * per_row; v += 256) {
            const int r = v / per_row, c = (v - r * per_row) * 8;
            const int4 i0 = *reinterpret_cast<const int4 *>(col_id + c);
            const int4 i1 = *reinterpret_cast<const int4 *>(col_id + c + 4);
            const _Float16 *row = rows + r * in;
            h8 o;
            o[0] = row[i0.x]; o[1] = row[i0.y]; o[2] = row[i0.z]; o[3] = row[i0.w];
            o[4] = row[i1.x]; o[5] = row[i1.y]; o[6] = row[i1.z]; o[7] = row[i1.w];
            *reinterpret_cast<h8 *>(dst + (size_t)(r0 + r) * nnz + c) = o;
        }
        __syncthreads();
    }
}

}  // namespace et


// ---------------------------------------------------------------------------
// Scratch for the allocation-free column-pruned Linear: the gathered activations
// [T x nnz_col] live in this file-scope device array instead of a caller's or
// an allocated workspace.  Every GPU the library runs on holds its own copy at
// its own address until the process ends; the array's name below is only the
// host-side handle of the symbol, the device address comes from
// hipGetSymbolAddress, once per device, with that device current.
// ---------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;  // 8 MiB: e.g. 2048 rows x 2048 kept columns
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace et {

constexpr int kMaxDevices = 64;
static std::atomic<void *> g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (looked up on first use).
static int static_scratch(void **out) {
    int dev = -1;
    ET_HIP(hipGetDevice(&dev));
    ET_REQUIRE(dev >= 0 && dev < kMaxDevices, ET_ERR_UNSUPPORTED, "static scratch: device ordinal %d", dev);
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
        if (!p) {
            ET_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
            ET_REQUIRE(p != nullptr, ET_ERR_LAUNCH, "static scratch: hipGetSymbolAddress returned NULL");
            g_scratch_ptr[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return ET_OK;
}

}  // namespace et

using namespace et;

extern "C" {

int et_gemm_f16(const et_f16 *A, const et_f16 *B, et_f16 *C, int M, int N, int K, int lda, int ldb,
                int ldc, int trans_b, int batch, long long strideA, long long strideB,
                long long strideC, et_stream stream) {
    ET_REQUIRE(A && B && C, ET_ERR_INVALID_ARG, "et_gemm_f16: NULL pointer");
    int s = check_gemm_shape("et_gemm_f16", M, N, K);
    if (s != ET_OK) return s;
    ET_REQUIRE(batch >= 1 && batch <= 65535, ET_ERR_INVALID_ARG, "et_gemm_f16: batch=%d", batch);
    ET_REQUIRE(lda >= K && ldc >= N && ldb >= (trans_b ? K : N), ET_ERR_INVALID_ARG,
               "et_gemm_f16: leading dimensions (%d %d %d) too small", lda, ldb, ldc);
    ET_REQUIRE(lda % 8 == 0 && ldb % 8 == 0 && ldc % 4 == 0 && strideA % 8 == 0 && strideB % 8 == 0 &&
                   strideC % 4 == 0,
               ET_ERR_UNSUPPORTED, "et_gemm_f16: strides must keep 16-byte operand alignment");
    ET_REQUIRE(((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(C) & 7) == 0,
               ET_ERR_UNSUPPORTED, "et_gemm_f16: operands must be 16-byte aligned");
    if (M == 0) return ET_OK;
    GemmArgs g = gemm_args(H(A), H(B), H(C), M, N, K, lda, ldb, ldc);
    g.sAo = strideA;
    g.sBo = strideB;
    g.sCo = strideC;
    return launch_gemm(g, batch, trans_b != 0, as_stream(stream));
}

int et_linear_dense_f16(const et_f16 *W, const et_f16 *bias, const et_f16 *X, et_f16 *Y, int T,
                        int in, int out, int act, et_stream stream) {
    ET_REQUIRE(W && X && Y, ET_ERR_INVALID_ARG, "et_linear_dense_f16: NULL pointer");
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG,
               "et_linear_dense_f16: act=%d", act);
    int s = check_gemm_shape("et_linear_dense_f16", T, out, in);
    if (s != ET_OK) return s;
    if (T == 0) return ET_OK;
    GemmArgs g = gemm_args(H(X), H(W), H(Y), T, out, in, in, in, out);
    g.bias = H(bias);
    g.act = act;
    return launch_gemm(g, 1, true, as_stream(stream));
}

int et_linear_rowpruned_f16(const et_f16 *rows, const int32_t *row_id, int nnz_row,
                            const et_f16 *bias, const et_f16 *X, et_f16 *Y, int T, int in, int out,
                            int act, et_stream stream) {
    ET_REQUIRE(rows && row_id && X && Y, ET_ERR_INVALID_ARG, "et_linear_rowpruned_f16: NULL pointer");
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG,
               "et_linear_rowpruned_f16: act=%d", act);
    ET_REQUIRE(nnz_row >= 0 && nnz_row <= out, ET_ERR_INVALID_ARG,
               "et_linear_rowpruned_f16: nnz_row=%d out=%d", nnz_row, out);
    int s = check_gemm_shape("et_linear_rowpruned_f16", T, out, in);
    if (s != ET_OK) return s;
    ET_REQUIRE(nnz_row % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_linear_rowpruned_f16: nnz_row=%d must be a multiple of 16", nnz_row);
    if (T == 0) return ET_OK;
    hipStream_t st = as_stream(stream);
    if (nnz_row < out) {
        // pruned features carry the bias alone; live ones are overwritten below
        s = launch_bias_rows(H(Y), H(bias), T, out, out, act, st);
        if (s != ET_OK) return s;
    }
    if (nnz_row == 0) return ET_OK;
    GemmArgs g = gemm_args(H(X), H(rows), H(Y), T, nnz_row, in, in, in, out);
    g.bias = H(bias);
    g.c_scatter = row_id;
    g.act = act;
    return launch_gemm(g, 1, true, st);
}

int et_linear_rowpruned_compact_f16(const et_f16 *rows, const int32_t *row_id, int nnz_row,
                                    const et_f16 *bias, const et_f16 *X, et_f16 *Yc, int T, int in,
                                    et_stream stream) {
    ET_REQUIRE(rows && X && Yc, ET_ERR_INVALID_ARG, "et_linear_rowpruned_compact_f16: NULL pointer");
    ET_REQUIRE(bias == nullptr || row_id != nullptr, ET_ERR_INVALID_ARG,
               "et_linear_rowpruned_compact_f16: bias needs row_id");
    int s = check_gemm_shape("et_linear_rowpruned_compact_f16", T, nnz_row, in);
    if (s != ET_OK) return s;
    if (T == 0) return ET_OK;
    // Compact output: column j holds feature row_id[j]; its bias is bias[row_id[j]].
    GemmArgs g = gemm_args(H(X), H(rows), H(Yc), T, nnz_row, in, in, in, nnz_row);
    g.bias = H(bias);
    g.bias_idx = bias ? row_id : nullptr;
    return launch_gemm(g, 1, true, as_stream(stream));
}

int et_fill_rows_bias_f16(et_f16 *C, const et_f16 *bias, int rows, int cols, et_stream stream) {
    ET_REQUIRE(C != nullptr, ET_ERR_INVALID_ARG, "et_fill_rows_bias_f16: C is NULL");
    ET_REQUIRE(rows >= 0 && cols > 0, ET_ERR_INVALID_ARG, "et_fill_rows_bias_f16: rows=%d cols=%d", rows, cols);
    if (rows == 0) return ET_OK;
    return launch_bias_rows(H(C), H(bias), rows, cols, cols, ET_ACT_NONE, as_stream(stream));
}

int et_linear_colpruned_f16(const et_f16 *cols, const int32_t *col_id, int nnz_col,
                            const et_f16 *bias, const et_f16 *X, et_f16 *Y, int T, int in, int out,
                            int act, et_stream stream) {
    ET_REQUIRE(cols && col_id && X && Y, ET_ERR_INVALID_ARG, "et_linear_colpruned_f16: NULL pointer");
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG,
               "et_linear_colpruned_f16: act=%d", act);
    ET_REQUIRE(nnz_col >= 0 && nnz_col <= in, ET_ERR_INVALID_ARG,
               "et_linear_colpruned_f16: nnz_col=%d in=%d", nnz_col, in);
    ET_REQUIRE(in > 0 && T % 16 == 0 && out % 16 == 0 && nnz_col % 16 == 0 && T >= 0 && out > 0,
               ET_ERR_UNSUPPORTED,
               "et_linear_colpruned_f16: T=%d out=%d nnz_col=%d must be multiples of 16", T, out,
               nnz_col);
    if (T == 0) return ET_OK;
    hipStream_t st = as_stream(stream);
    if (nnz_col == 0) {
        return launch_bias_rows(H(Y), H(bias), T, out, out, act, st);
    }
    GemmArgs g = gemm_args(H(X), H(cols), H(Y), T, out, nnz_col, in, nnz_col, out);
    g.bias = H(bias);
    g.a_gather = col_id;
    g.act = act;
    return launch_gemm(g, 1, true, st);
}

int et_gather_cols_f16(et_f16 *dst, const et_f16 *X, const int32_t *col_id, int T, int in, int nnz_col,
                       et_stream stream) {
    ET_REQUIRE(dst && X && col_id, ET_ERR_INVALID_ARG, "et_gather_cols_f16: NULL pointer");
    ET_REQUIRE(T >= 0 && in > 0 && nnz_col >= 0, ET_ERR_INVALID_ARG, "et_gather_cols_f16: T=%d in=%d nnz_col=%d", T,
               in, nnz_col);
    ET_REQUIRE(nnz_col % 8 == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(col_id) & 15) == 0,
               ET_ERR_UNSUPPORTED, "et_gather_cols_f16: nnz_col=%d must be a multiple of 8, dst and col_id 16-byte aligned",
               nnz_col);
    const size_t total = (size_t)T * (nnz_col / 8);
    if (total == 0) return ET_OK;
    size_t blocks = (total + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    if (in % 8 == 0 && in <= 16384 && (reinterpret_cast<uintptr_t>(X) & 15) == 0) {
        // about 16 KB of rows a workgroup, so that several of them share a CU whatever the row length
        const int rows = std::max(1, std::min(8, 8192 / in));
        const unsigned groups = (unsigned)std::min<size_t>(((size_t)T + rows - 1) / rows, 2048);
        gather_cols_staged_kernel<<<groups, 256, (size_t)rows * in * sizeof(_Float16), as_stream(stream)>>>(
            H(dst), H(X), col_id, T, in, nnz_col, rows);
        return check_launch("gather_cols_staged_kernel");
    }
    gather_cols_kernel<<<(unsigned)blocks, 256, 0, as_stream(stream)>>>(H(dst), H(X), col_id, T, in, nnz_col);
    return check_launch("gather_cols_kernel");
}

int et_linear_colpruned_ws_f16(const et_f16 *cols, const int32_t *col_id, int nnz_col, const et_f16 *bias,
                               const et_f16 *X, et_f16 *Y, et_f16 *workspace, int T, int in, int out, int act,
                               et_stream stream) {
    ET_REQUIRE(workspace != nullptr, ET_ERR_INVALID_ARG, "et_linear_colpruned_ws_f16: workspace is NULL");
    if (nnz_col == 0 || T == 0)  // nothing to gather: bias and activation alone
        return et_linear_colpruned_f16(cols, col_id, nnz_col, bias, X, Y, T, in, out, act, stream);
    ET_REQUIRE(cols && col_id && X && Y, ET_ERR_INVALID_ARG, "et_linear_colpruned_ws_f16: NULL pointer");
    ET_REQUIRE(nnz_col > 0 && nnz_col <= in, ET_ERR_INVALID_ARG, "et_linear_colpruned_ws_f16: nnz_col=%d in=%d",
               nnz_col, in);
    int s = et_gather_cols_f16(workspace, X, col_id, T, in, nnz_col, stream);
    if (s != ET_OK) return s;
    return et_linear_dense_f16(cols, bias, workspace, Y, T, nnz_col, out, act, stream);
}

int et_linear_colpruned_static_f16(const et_f16 *cols, const int32_t *col_id, int nnz_col, const et_f16 *bias,
                                   const et_f16 *X, et_f16 *Y, int T, int in, int out, int act,
                                   et_stream stream) {
    ET_REQUIRE(T >= 0 && nnz_col >= 0, ET_ERR_INVALID_ARG, "et_linear_colpruned_static_f16: T=%d nnz_col=%d", T,
               nnz_col);
    const size_t need = (size_t)T * (size_t)nnz_col * sizeof(et_f16);
    ET_REQUIRE(need <= kStaticScratchBytes, ET_ERR_UNSUPPORTED,
               "et_linear_colpruned_static_f16: T x nnz_col = %d x %d needs %zu bytes of scratch, the built-in "
               "buffer holds %zu; use et_linear_colpruned_ws_f16 with a workspace of your own",
               T, nnz_col, need, kStaticScratchBytes);
    if (need == 0)  // nothing to gather, so no scratch and no address lookup: bias and activation alone
        return et_linear_colpruned_f16(cols, col_id, nnz_col, bias, X, Y, T, in, out, act, stream);
    void *ws = nullptr;
    int s = static_scratch(&ws);
    if (s != ET_OK) return s;
    // the gather overwrites every element of the [T x nnz_col] prefix it then reads: nothing to clear
    return et_linear_colpruned_ws_f16(cols, col_id, nnz_col, bias, X, Y, static_cast<et_f16 *>(ws), T, in, out,
                                      act, stream);
}

}  // extern "C"
