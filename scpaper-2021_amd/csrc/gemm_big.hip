// Large dense GEMM for gfx950: C[M x N] = act(A[M x K] * B^T + bias), A and B both
// K-contiguous (B stored [N x K]), M and N multiples of 256, K a multiple of 64.
//
// The 64x64-per-wave kernel in gemm.hip reads 1 byte of LDS per 32 flops, which at the
// MFMA peak is the whole bandwidth of the LDS port; it tops out near a third of the matrix
// peak.  Here a workgroup of 4 waves computes a 256 x 256 tile and each wave a 128 x 128
// block as 4 x 4 v_mfma_f32_32x32x16_f16 tiles, accumulators in 256 AGPR/VGPRs: 1 byte
// of LDS per 64 flops.  One wave per SIMD is resident, so the latencies are covered inside
// the wave: K advances in stages of 64 through two LDS buffers, the next stage is loaded
// straight from global memory into the idle buffer while the current one is multiplied
// (staging through registers and ds_write costs a third of the rate: the LDS port is then
// the bound), the fragment reads of the next K slice are issued ahead of the MFMAs that hide
// them, and the one workgroup barrier of a stage sits before its last K slice.
//
// The MFMA A operand is the B matrix (output features) and vice versa, so a lane ends with
// 4 consecutive features of one row of C per 8-row group of a tile; the epilogue transposes
// through LDS to store whole 256-byte row segments.
#include "gemm.hip.h"

namespace et {

constexpr int kBigTile = 256;            // rows of A and rows of B per workgroup
constexpr int kBigK = 64;                // K per stage: one 128-byte line of every row
constexpr int kBigXcds = 8;
constexpr int kSbM = 4, kSbN = 8;        // tile block one XCD works on at a time
constexpr size_t kBigLds = (size_t)2 * 2 * kBigTile * kBigK * sizeof(_Float16);  // 128 KB
// s_waitcnt immediate for vmcnt(0) alone on gfx9: vmcnt in bits 3:0 and 15:14, expcnt 6:4 and
// lgkmcnt 11:8 left at their maxima
constexpr int kWaitVm0 = 0x0F70;
#define ET_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define ET_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

typedef float f16v __attribute__((ext_vector_type(16)));

// IDX: the result columns are scattered (c_scatter) or their bias is gathered (bias_idx).
template <int ACT, bool IDX>
__global__ __launch_bounds__(256) void gemm_f16_big_kernel(const GemmArgs g) {
    extern __shared__ __align__(16) unsigned char big_smem[];
    _Float16 *As = reinterpret_cast<_Float16 *>(big_smem);  // [2][256][kBigK], chunks swizzled
    _Float16 *Bs = As + 2 * kBigTile * kBigK;                // [2][256][kBigK]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, kg = lane >> 5;
    // Workgroup id -> tile, XCD-aware.  Workgroups go to the 8 XCDs round-robin by id and each
    // XCD runs 32 of them at a time; those 32 are given a 4 x 8 block of tiles (4 panels of A,
    // 8 of B), so the XCD's L2 serves 12 panels to 32 workgroups instead of up to 64.
    const int tiles_m = g.M / kBigTile, tiles_n = g.N / kBigTile;
    const int nsbx = (tiles_n + kSbN - 1) / kSbN;
    const int xcd = blockIdx.x % kBigXcds, j = blockIdx.x / kBigXcds;
    const int gsb = (j / (kSbM * kSbN)) * kBigXcds + xcd, within = j % (kSbM * kSbN);
    const int ty = (gsb / nsbx) * kSbM + within / kSbN, tx = (gsb % nsbx) * kSbN + within % kSbN;
    if (ty >= tiles_m || tx >= tiles_n) return;  // padding of the block grid (whole workgroup)
    const int m0 = ty * kBigTile, n0 = tx * kBigTile;
    const _Float16 *A = g.A + (size_t)m0 * g.lda;
    const _Float16 *B = g.B + (size_t)n0 * g.ldb;

    f16v acc[4][4];  // [token tile][feature tile]
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // Stage loads go straight from global memory to LDS (global_load_lds_dwordx4): a wave
    // instruction fills 1 KB of consecutive LDS, 16 bytes per lane, from addresses the lanes
    // choose.  Here that is 8 rows of 128 bytes, 8 lanes a row (whole lines of the operand);
    // within the row the lane at position p fetches chunk p ^ swz(row), so that the fragment
    // reads below, 16 rows apart by one chunk column, spread over all banks with no padding.
    const int lrow = lane >> 3, lpos = lane & 7;
    auto load_stage = [&](int buf, int k0) {
#pragma unroll
        for (int v = 0; v < 8; v++) {
            const int r0 = wave * 64 + v * 8, r = r0 + lrow;
            const int c = lpos ^ ((r >> 1) & 7);
            __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(A + (size_t)r * g.lda + k0 + c * 8),
                                             ET_LDS_PTR(As + (buf * kBigTile + r0) * kBigK), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(B + (size_t)r * g.ldb + k0 + c * 8),
                                             ET_LDS_PTR(Bs + (buf * kBigTile + r0) * kBigK), 16, 0, 0);
        }
    };
    // fragments of one 16-wide K slice: 4 token tiles and 4 feature tiles of the wave's block.
    // Rows 128 wm + 32 i + l32: the swizzle term (row >> 1) & 7 depends on the lane only.
    struct Frag { h8 x[4], w[4]; };
    const int swz = (l32 >> 1) & 7;
    const _Float16 *a_rows = As + (wm * 128 + l32) * kBigK, *b_rows = Bs + (wn * 128 + l32) * kBigK;
    auto read_frag = [&](Frag &f, int buf, int ks) {
        const int off = buf * kBigTile * kBigK + (((ks * 2 + kg) ^ swz) * 8);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f.x[i] = *reinterpret_cast<const h8 *>(a_rows + off + i * 32 * kBigK);
            f.w[i] = *reinterpret_cast<const h8 *>(b_rows + off + i * 32 * kBigK);
        }
    };
    auto multiply = [&](const Frag &f) {
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.w[j], f.x[i], acc[i][j], 0, 0, 0);
    };

    const int nstage = g.K / kBigK;
    // Stage s is multiplied from LDS buffer s % 2.
    Frag f0, f1;
    load_stage(0, 0);
    __builtin_amdgcn_s_waitcnt(kWaitVm0);  // the data of a direct-to-LDS load is in LDS when vmcnt says so
    __syncthreads();
    read_frag(f0, 0, 0);
    // One stage, with the matrix pipe fed across the barrier: every K slice is read from LDS
    // while the one before it is multiplied, the first slice of the next stage included, so the
    // barrier of the stage sits before its last slice.  The loads of the next stage are issued at
    // the start of the stage into the other buffer (its last readers passed the previous
    // barrier) and waited for just before the barrier.  The load and fragment read of the last
    // stage, which has no successor, touch valid memory and are never used; the loop has a
    // single exit (a second one in the middle makes the register allocator copy the 256
    // accumulators).
    for (int s = 0; s < nstage; s++) {
        const int cur = s & 1, nxt = cur ^ 1;
        load_stage(nxt, min(s + 1, nstage - 1) * kBigK);
        read_frag(f1, cur, 1);
        multiply(f0);
        read_frag(f0, cur, 2);
        multiply(f1);
        read_frag(f1, cur, 3);
        multiply(f0);
        __builtin_amdgcn_s_waitcnt(kWaitVm0);
        __syncthreads();
        read_frag(f0, nxt, 0);
        multiply(f1);
    }
    __syncthreads();  // the staging LDS becomes the transposition buffer of the epilogue

    // Epilogue.  acc[i][j][e] is token 128 wm + 32 i + l32, feature 128 wn + 32 j + 8 (e / 4) +
    // 4 kg + e % 4 of the tile: a lane holds 4 consecutive features of one row, 32 rows per
    // instruction.  Each wave passes its 32 x 128 strip through its own LDS region and stores
    // rows of 256 contiguous bytes.
    constexpr int kEpLd = 128 + 8;
    _Float16 *ep = reinterpret_cast<_Float16 *>(big_smem) + wave * 32 * kEpLd;
    const int nbase = n0 + wn * 128;
    // unconditional loads (from B when there is no bias) and a select: a load under a branch
    // is waited for on the spot
    const bool has_bias = g.bias != nullptr;
    const int32_t *col_idx = g.c_scatter ? g.c_scatter : g.bias_idx;  // bias index of result column n
    h4 bias4[4][4];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int q = 0; q < 4; q++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int n = nbase + j * 32 + q * 8 + kg * 4 + e;
                _Float16 bv;
                if (IDX) {
                    const int bi = col_idx ? col_idx[n] : n;
                    bv = (has_bias ? g.bias : g.B)[has_bias ? bi : 0];
                } else {
                    bv = (has_bias ? g.bias : g.B)[n];
                }
                bias4[j][q][e] = has_bias ? bv : (_Float16)0.0f;
            }
    // the 8 output columns of the lane's 16-byte chunk of a stored row
    int scat[8];
    if (IDX) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int n = nbase + (lane % 16) * 8 + e;
            scat[e] = g.c_scatter ? g.c_scatter[n] : n;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                h4 o;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float y = acc[i][j][q * 4 + e] + (float)bias4[j][q][e];
                    if (ACT == ET_ACT_RELU) y = y > 0.0f ? y : 0.0f;
                    if (ACT == ET_ACT_GELU) y = gelu_tanh(y);
                    o[e] = (_Float16)y;
                }
                *reinterpret_cast<h4 *>(ep + l32 * kEpLd + j * 32 + q * 8 + kg * 4) = o;
            }
        __syncthreads();
#pragma unroll
        for (int v = 0; v < 8; v++) {
            const int idx = lane + v * 64, r = idx / 16, c = idx % 16;
            const h8 val = *reinterpret_cast<const h8 *>(ep + r * kEpLd + c * 8);
            _Float16 *crow = g.C + (size_t)(m0 + wm * 128 + i * 32 + r) * g.ldc;
            if (IDX) {
#pragma unroll
                for (int e = 0; e < 8; e++) crow[scat[e]] = val[e];
            } else {
                *reinterpret_cast<h8 *>(crow + nbase + c * 8) = val;
            }
        }
        __syncthreads();
    }
}

bool gemm_big_applies(const GemmArgs &g, int batch, bool trans_b) {
    return trans_b && batch == 1 && !g.a_gather && g.M % kBigTile == 0 &&
           g.N % kBigTile == 0 && g.K % kBigK == 0 &&
           (long long)(g.M / kBigTile) * (g.N / kBigTile) >= 256;
}

template <int ACT, bool IDX>
static int launch_big_variant(const GemmArgs &g, dim3 grid, hipStream_t stream) {
    auto kernel = gemm_f16_big_kernel<ACT, IDX>;
    static bool raised = false;  // 128 KB of dynamic LDS needs the attribute, once per kernel
    if (!raised) {
        ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)kBigLds));
        raised = true;
    }
    kernel<<<grid, 256, kBigLds, stream>>>(g);
    return check_launch("gemm_f16_big_kernel");
}

template <int ACT>
static int launch_big_act(const GemmArgs &g, dim3 grid, hipStream_t stream) {
    return (g.c_scatter || g.bias_idx) ? launch_big_variant<ACT, true>(g, grid, stream)
                                       : launch_big_variant<ACT, false>(g, grid, stream);
}

int launch_gemm_big(const GemmArgs &g, hipStream_t stream) {
    const int tiles_m = g.M / kBigTile, tiles_n = g.N / kBigTile;
    const int nsb = ((tiles_m + kSbM - 1) / kSbM) * ((tiles_n + kSbN - 1) / kSbN);
    const int rounds = (nsb + kBigXcds - 1) / kBigXcds;
    const dim3 grid((unsigned)(rounds * kBigXcds * kSbM * kSbN));
    switch (g.act) {
        case ET_ACT_RELU: return launch_big_act<ET_ACT_RELU>(g, grid, stream);
        case ET_ACT_GELU: return launch_big_act<ET_ACT_GELU>(g, grid, stream);
        default: return launch_big_act<ET_ACT_NONE>(g, grid, stream);
    }
}

}  // namespace et
