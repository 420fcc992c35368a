// Y[T x out] = act(X[T x in] * W^T + bias), W stored as 16x16 tiles (BSR over
// the [out x in] matrix, tile rows = output features) — gfx950 MFMA kernel.
//
// Work split.  One workgroup owns a strip of MT*16 token rows and a contiguous
// group of block-rows of W; its waves take those block-rows round-robin.  The
// strip of X is staged once in LDS (row stride padded by 16 bytes: the 16 rows
// a fragment read touches fall in distinct banks).  Workgroups are numbered so
// that all groups of one strip run on the same XCD (private L2).
//
// Matrix-core feed.  v_mfma_f32_16x16x32_f16 contracts 32 values, i.e. tile t
// (k 0..15) and tile t+1 (k 16..31) of one block-row in a single instruction —
// a "slot".  The reference tile layout [tile][out 16][in 16] is exactly the
// MFMA A-operand feed: lane (r = lane%16, g = lane/16) reads 8 consecutive
// halfs of row r of tile t + g/2 at offset 8*(g%2), so a slot is one contiguous
// 1 KiB wave load.  The B operand is the matching 16-token x 16-feature block
// of X from LDS.  The accumulator of lane (r, g) is C[feature 4g..4g+3][token r]:
// four consecutive output features of one token, stored as one 8-byte write
// after bias and activation in fp32.
//
// Latency and issue rate.  A global load costs on the order of a microsecond and
// a lone wave issues one vector instruction every few cycles, so the kernel keeps
// the per-slot instruction count minimal (one weight load and one index load with
// immediate offsets from per-row base pointers, one LDS read and one MFMA per
// 16-token block) and keeps loads in flight across rows: the row pointers of all
// rows of a wave are fetched with one load, and the weights, indices and bias of
// the next kNB - 1 row groups (up to kSlots slots each) are requested before the
// current one is multiplied.
//
// Tile order inside a block-row is free (the sum commutes), as in the
// reference kernel (Linear/SPMM_tile.cu:277-283).
#include "common.hip.h"
#include "../../include/et_tuning.h"

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
    // fused SkipLayerNorm prologue (LN kernels only): X = LN(ln_src + ln_skip)*gamma + beta is
    // formed while the strip is staged; the workgroups of block-row group 0 also write it to ln_out
    const _Float16 *ln_src, *ln_skip, *ln_gamma, *ln_beta;
    _Float16 *ln_out;
    float ln_eps;
    // NORM prologue (kFxNorm): X holds the output of a producer launched with kFxRes, ln_skip
    // the residual it was given and st_in its per-row partial sums [st_groups][T][2] (sum, sum
    // of squares of output + residual); the strip X + ln_skip is normalised with them,
    // ln_gamma, ln_beta and ln_eps on its way into LDS and the workgroups of block-row group 0
    // write the normalised rows to ln_out.  The sum is never rounded to fp16.
    const float *st_in;
    int st_groups;
    // RES epilogue (kFxRes): Y = X W^T + bias as usual, and st_out[group][token] = (sum, sum
    // of squares) of (Y as stored + resid) over the features of this workgroup.
    const _Float16 *resid;
    float *st_out;
    // binary32 result: when set, act(acc + bias) is stored here unrounded (16 bytes per lane)
    // and Y is not written — the mixed-precision layer keeps its residual stream in fp32
    float *Y32;
    // binary32 forms of the split normalisation (mixed-precision layer).  RES with kFxRes32: the sum
    // acc + bias + resid32 is stored unrounded to Y32 and the row sums are taken over it (Y, resid
    // unused).  NORM with kFxNorm32: the strip comes from X32 (that stored sum; ln_skip unused) and
    // the normalised rows go to ln_out32 and / or ln_out (either may be null), each vector written by
    // one of the strip's block-row groups.
    const float *resid32;
    const _Float16 *resid16;  // RES32: when set, the residual in binary16 (resid32 unused)
    const float *X32;
    float *ln_out32;
    // RES32: when rs_fin is set the residual is not read but formed, as the normalisation of
    // resid32 with these row statistics and affine vectors (what a consumer launched with
    // kFxNorm32 formed from the same data): the normalised rows then never have to be stored.
    const float *rs_fin;  // [T][2]: mean and rstd of every row of resid32, as a consumer left them in fin_out
    const _Float16 *rs_gamma, *rs_beta;
    // NORM32: when set, block-row group 0 stores mean and rstd of the rows of its strip here, [T][2]
    float *fin_out;
};

constexpr int kFxNorm = 1;
constexpr int kFxRes = 2;
constexpr int kFxNorm32 = 4;  // with kFxNorm: binary32 strip
constexpr int kFxRes32 = 8;   // with kFxRes: binary32 residual and result
constexpr int kFxRes16 = 32;  // with kFxRes32: the residual is read as binary16 (a kernel of its own, so that the
                              // 12-wave producer, at 168 registers, carries no second path)
constexpr int kFxWide = 16;   // plain kernel built for up to 12 waves (170 registers): two row groups in flight

constexpr int kXcds = 8;      // accelerator dies, each with a private L2
constexpr int kLdsPad = 8;    // halfs
constexpr int kSlots = 8;     // slots per row group held in registers
// Row groups a wave has requested ahead of the one it multiplies.  Inside a stack of layers every
// kernel starts on weights that have left the caches, and four groups in flight instead of two
// shorten a 12-layer forward by 3 % (the stand-alone kernel, whose weights stay in L2, gains 0-5 %).
// Five would spill (4 groups = 225 registers of the 256 that 8 waves per compute unit leave), and
// so would four in the kernels whose prologue normalises the strip: those keep two.
constexpr int kGroupsAhead = 4;
constexpr int kGroupsAheadNorm = 2;
constexpr int kStageU = 8;    // 16-byte strip vectors a thread keeps in flight
constexpr int kMaxWaveRows = 64;  // block-rows one wave can own (one lane each)

template <int ACT> __device__ __forceinline__ float act_fixed(float x) {
    if (ACT == ET_ACT_RELU) return x > 0.0f ? x : 0.0f;
    if (ACT == ET_ACT_GELU) return gelu_tanh(x);
    return x;
}

__device__ __forceinline__ int lane_read(int v, int lane) {
    return __builtin_amdgcn_readlane(v, lane);
}

// ACT is a template parameter: the epilogue carries no run-time branch and each
// fused activation is a separately named kernel in a profile.
template <int MT, bool STAGE, int ACT, int LN = 0, int FX = 0>
__global__ __launch_bounds__(((MT == 1 && (FX & kFxRes32) && !(FX & kFxRes16)) || (FX & (kFxNorm32 | kFxWide))) ? 768 : 512) void bsr16_linear_kernel(const BsrArgs a) {
    static_assert(!LN || STAGE, "the fused LayerNorm prologue writes the strip to LDS");
    static_assert(!(FX & kFxNorm) || (STAGE && !LN), "the NORM prologue writes the strip to LDS");
    constexpr bool NORM = (FX & kFxNorm) != 0;
    constexpr bool RES = (FX & kFxRes) != 0;
    constexpr bool NORM32 = (FX & kFxNorm32) != 0;
    static_assert(!NORM32 || NORM, "kFxNorm32 qualifies kFxNorm");
    constexpr bool RES32 = (FX & kFxRes32) != 0;
    static_assert(!RES32 || RES, "kFxRes32 qualifies kFxRes");
    // row groups resident per wave: four; two in the kernels whose prologue normalises fp16 strips
    // (four would spill) and in the forms built for 12 waves of at most two to four block-rows (the
    // consumer of a binary32 strip, the wide plain kernel); three with a binary32 residual in flight
    // per group
    constexpr bool WIDE = (FX & kFxWide) != 0;
    static_assert(!WIDE || (FX == kFxWide && !LN && MT <= 2), "the 12-wave form of the plain kernel");
    constexpr int kNB = (NORM32 || WIDE) ? 2 : RES32 ? 3 : (LN || NORM) ? kGroupsAheadNorm : kGroupsAhead;
    // 16-byte strip vectors a thread requests before it writes the first to LDS; binary32 vectors are
    // two loads each
    constexpr int kSU = NORM32 ? 4 : kStageU;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    _Float16 *xs = reinterpret_cast<_Float16 *>(smem_raw);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwave = blockDim.x >> 6;
    const int nthr = blockDim.x;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int sel = g >> 1;         // which tile of the slot this lane feeds
    const int koff = (g & 1) << 3;  // offset of its 8 k-values inside the tile
    // Workgroup id -> (token strip, block-row group), XCD-aware.  Workgroups are
    // handed to the 8 XCDs round-robin by linear id and each XCD has its own L2, so
    // strip s is pinned to XCD s % 8 and the groups of one strip follow each other on
    // that XCD: a strip of X is fetched into one L2 only and reused there.
    const int nbr = a.out >> 4;
    const int ngroups = (nbr + a.rows_per_wg - 1) / a.rows_per_wg;
    const int nstrips = (a.T + MT * 16 - 1) / (MT * 16);
    const int xcd = blockIdx.x % kXcds, k_in_xcd = blockIdx.x / kXcds;
    const int strip = xcd + kXcds * (k_in_xcd / ngroups);
    const int group = k_in_xcd % ngroups;
    if (strip >= nstrips) return;  // padding of the last round of strips (whole workgroup)
    const int tok0 = strip * (MT * 16);
    const int rb_begin = group * a.rows_per_wg;
    const int rb_end = min(rb_begin + a.rows_per_wg, nbr);
    const int lds_ld = a.in + kLdsPad;
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

    // ---- row pointers of this wave's block-rows: rows rb_begin + wave + nwave*i,
    // lane i holds [lo, hi) of row i (first in the load queue: loads return in
    // issue order and everything below depends on these few bytes)
    const int nrw = max(0, (rb_end - rb_begin - wave + nwave - 1) / nwave);
    int rp_lo = 0, rp_hi = 0;
    if (lane < nrw) {
        const int rb = rb_begin + wave + nwave * lane;
        rp_lo = a.row_ptr[rb];
        rp_hi = a.row_ptr[rb + 1];
    }

    // ---- NORM: the row sums (wave 0, a token per lane) and the affine vectors are requested ahead
    // of the strip.  Loads return in order: behind the strip they would keep the waves that
    // put them into LDS waiting for the whole strip before their weight requests go out.
    static_assert(!NORM || MT <= 2, "a half-wave of tokens");
    float2 st_part[NORM ? kMaxStatGroups / 2 : 1];  // lanes 0-31: groups 0-7 of token lane; lanes 32-63: groups 8-15
    h8 aff[NORM ? 2 : 1][2];  // gamma and beta vectors threadIdx.x and threadIdx.x + blockDim.x of the row
    if constexpr (NORM) {
        if (wave == 0) {
            const int tok = min(tok0 + (lane & 31), a.T - 1);
#pragma unroll
            for (int k = 0; k < kMaxStatGroups / 2; k++) {
                const int gi = min((lane >> 5) * (kMaxStatGroups / 2) + k, a.st_groups - 1);
                st_part[k] = *reinterpret_cast<const float2 *>(a.st_in + ((size_t)gi * a.T + tok) * 2);
            }
        }
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int c = min((int)threadIdx.x + k * nthr, (a.in >> 3) - 1);
            aff[k][0] = reinterpret_cast<const h8 *>(a.ln_gamma)[c];
            aff[k][1] = reinterpret_cast<const h8 *>(a.ln_beta)[c];
        }
    }

    // ---- strip copy, first batch: loads only.  X[tok0 .. tok0+MT*16) is one
    // contiguous block of global memory; only the LDS side has padded rows.
    const int vec_per_row = a.in >> 3;
    const int rows_here = min(MT * 16, a.T - tok0);
    const int total_vec = STAGE ? rows_here * vec_per_row : 0;
    const h8 *src = reinterpret_cast<const h8 *>(a.X + (size_t)tok0 * a.in);
    h8 sv[kSU];
    if (STAGE && !LN && !NORM32) {
        // unconditional loads, index clamped into the strip: a load under a branch gets a
        // basic block of its own and the register allocator's copies there make the wave
        // wait for it on the spot — a full memory round trip before the weight loads go out
#pragma unroll
        for (int u = 0; u < kSU; u++) sv[u] = src[min((int)threadIdx.x + u * nthr, total_vec - 1)];
    }
    constexpr bool SKIP16 = NORM && !NORM32;  // a binary16 skip strip is added
    const h8 *src_skip = SKIP16 ? reinterpret_cast<const h8 *>(a.ln_skip + (size_t)tok0 * a.in) : nullptr;
    h8 sk[SKIP16 ? kSU : 1];
    if (SKIP16) {
#pragma unroll
        for (int u = 0; u < kSU; u++) sk[u] = src_skip[min((int)threadIdx.x + u * nthr, total_vec - 1)];
    }
    // binary32 strip: a strip vector of 8 values is two 16-byte loads
    const f4 *src32 = NORM32 ? reinterpret_cast<const f4 *>(a.X32 + (size_t)tok0 * a.in) : nullptr;
    f4 s32[NORM32 ? kSU : 1][2];
    if (NORM32) {
#pragma unroll
        for (int u = 0; u < kSU; u++) {
            const int v = min((int)threadIdx.x + u * nthr, total_vec - 1);
            s32[u][0] = src32[2 * v];
            s32[u][1] = src32[2 * v + 1];
        }
    }
    // NORM: per-row (mean, rstd) and the affine vectors go to LDS behind the strip
    float2 *stat_lds = reinterpret_cast<float2 *>(xs + MT * 16 * lds_ld);
    _Float16 *gam_lds = reinterpret_cast<_Float16 *>(stat_lds + MT * 16);
    _Float16 *bet_lds = gam_lds + a.in;
    // Fused SkipLayerNorm: a wave normalises rows wave, wave+nwave, ... of the strip
    // (at most kLnRows of them); all their loads are issued here, one round trip.
    constexpr int kLnRows = LN ? MT * 16 / 8 : 1;        // rows per wave: LN kernels run 8 waves
    constexpr int kLnNit = LN ? LN : 1;                  // 4-element chunks per lane (LN = ceil(in / 256))
    uint2 ln_s[kLnRows][kLnNit], ln_k[kLnRows][kLnNit], ln_g[kLnNit], ln_b[kLnNit];
    const int ln_chunks = a.in >> 2;
    if (LN) {
        // unconditional loads (indices past the row or the strip are clamped and the values
        // selected away later): loads under a branch get a basic block of their own, where
        // the compiler waits for each in turn instead of once for all
#pragma unroll
        for (int i = 0; i < kLnNit; i++) {
            const int c = min(lane + 64 * i, ln_chunks - 1);
            ln_g[i] = reinterpret_cast<const uint2 *>(a.ln_gamma)[c];
            ln_b[i] = reinterpret_cast<const uint2 *>(a.ln_beta)[c];
        }
#pragma unroll
        for (int rr = 0; rr < kLnRows; rr++) {
            const int r = min(wave + 8 * rr, rows_here - 1);
            const uint2 *ps = reinterpret_cast<const uint2 *>(a.ln_src + (size_t)(tok0 + r) * a.in);
            const uint2 *pk = reinterpret_cast<const uint2 *>(a.ln_skip + (size_t)(tok0 + r) * a.in);
#pragma unroll
            for (int i = 0; i < kLnNit; i++) {
                const int c = min(lane + 64 * i, ln_chunks - 1);
                ln_s[rr][i] = ps[c];
                ln_k[rr][i] = pk[c];
            }
        }
    }

    // ---- row-group stream of this wave.  An item is up to kSlots slots of one
    // block-row; (it_row, it_part) is the next item to request.
    h8 w[kNB][kSlots];
    // column indices of an item's 2*kSlots tiles: one load, lane L holds that of tile L % 16
    int colv[kNB];
    h4 bias_v[kNB];
    // RES32: the residual of the block-row an item finishes (requested with the item, so that the
    // epilogue of the row does not wait for it), with the affine values of its four features
    f4 rsd[RES32 ? kNB : 1][MT];
    h4 rgm[RES32 ? kNB : 1], rbt[RES32 ? kNB : 1];
    auto load_resid = [&](int wave_row, f4 (&rs)[MT], h4 &gm, h4 &bt) {
        const int f0 = (rb_begin + wave + nwave * wave_row) * 16 + g * 4;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const int tok = min(tok0 + m * 16 + r16, a.T - 1);
            if constexpr ((FX & kFxRes16) != 0) {
                const h4 r = *reinterpret_cast<const h4 *>(a.resid16 + (size_t)tok * a.out + f0);
                rs[m] = f4{(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
            } else {
                rs[m] = *reinterpret_cast<const f4 *>(a.resid32 + (size_t)tok * a.out + f0);
            }
        }
        gm = bt = h4{0, 0, 0, 0};
        if (a.rs_fin) {
            gm = *reinterpret_cast<const h4 *>(a.rs_gamma + f0);
            bt = *reinterpret_cast<const h4 *>(a.rs_beta + f0);
        }
    };
    int g_row[kNB], g_nsl[kNB];  // resident items: wave row index (-1 = none), slots in the item
    bool g_last[kNB];            // item ends its block-row
    int it_row = 0, it_part = 0;
    // skip rows without tiles (they are written at the end)
    auto skip_empty = [&]() {
        while (it_row < nrw && lane_read(rp_hi, it_row) == lane_read(rp_lo, it_row)) it_row++;
    };
    skip_empty();
    auto issue_item = [&](int buf) __attribute__((always_inline)) {
        if (it_row >= nrw) {
            g_row[buf] = -1;
            return;
        }
        const int t0 = lane_read(rp_lo, it_row), t1 = lane_read(rp_hi, it_row);
        const int nsl_row = (t1 - t0 + 1) >> 1;
        const int first_slot = it_part * kSlots;
        const int nsl = min(kSlots, nsl_row - first_slot);
        const bool last = first_slot + nsl == nsl_row;
        const bool odd_tail = last && ((t1 - t0) & 1);  // the last slot holds one tile only
        g_row[buf] = it_row;
        g_nsl[buf] = nsl;
        g_last[buf] = last;
        const int tf = t0 + 2 * first_slot;  // first tile of the item
        // per-lane base pointer; slot p adds an immediate p*1024 B
        const _Float16 *wp = a.tiles + (size_t)(tf + sel) * 256 + r16 * 16 + koff;
#pragma unroll
        for (int p = 0; p < kSlots; p++) {
            if (p < nsl) {
                if (odd_tail && p == nsl - 1) {
                    // lanes of the missing second tile: zero weights
                    w[buf][p] = zero8;
                    if (sel == 0) w[buf][p] = *reinterpret_cast<const h8 *>(wp + p * 512);
                } else {
                    w[buf][p] = *reinterpret_cast<const h8 *>(wp + p * 512);
                }
            } else if (p & 1) {
                w[buf][p] = zero8;  // partner of the last slot inside a two-slot step
            }
        }
        // tiles past the row (zero weights) take the column of its last tile
        colv[buf] = a.col_idx[min(tf + r16, t1 - 1)];
        if (last) {  // the item that finishes the row carries its bias
            bias_v[buf] = h4{0, 0, 0, 0};
            if (a.bias)
                bias_v[buf] = *reinterpret_cast<const h4 *>(a.bias + (rb_begin + wave + nwave * it_row) * 16 + g * 4);
            if (RES32) load_resid(it_row, rsd[RES32 ? buf : 0], rgm[RES32 ? buf : 0], rbt[RES32 ? buf : 0]);
        }
        if (last) {
            it_row++;
            it_part = 0;
            skip_empty();
        } else {
            it_part++;
        }
    };
    // Row groups requested before the strip is written; the others follow when the registers of
    // the strip vectors are free again (only the 12-wave producer, at 170 registers per lane, has any)
    constexpr int kEarly = (MT == 1 && RES32) ? 2 : kNB;
#pragma unroll
    for (int buf = 0; buf < kEarly; buf++) issue_item(buf);

    // NORM: per-row (mean, rstd) and the affine vectors go to LDS behind the strip
    if constexpr (NORM) {
        if (wave == 0) {
            float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
            for (int k = 0; k < kMaxStatGroups / 2; k++) {
                const bool real = (lane >> 5) * (kMaxStatGroups / 2) + k < a.st_groups;
                s1 += real ? st_part[k].x : 0.0f;
                s2 += real ? st_part[k].y : 0.0f;
            }
            s1 += __shfl_xor(s1, 32, 64);
            s2 += __shfl_xor(s2, 32, 64);
            const float inv_h = 1.0f / (float)a.in;
            const float mean = s1 * inv_h;
            const float2 st = float2{mean, rsqrtf(fmaxf(__builtin_fmaf(-mean, mean, s2 * inv_h), 0.0f) + a.ln_eps)};
            if (lane < rows_here) {
                stat_lds[lane] = st;
                if (NORM32 && a.fin_out && group == 0)
                    *reinterpret_cast<float2 *>(a.fin_out + 2 * (size_t)(tok0 + lane)) = st;
            }
        }
#pragma unroll
        for (int k = 0; k < 2; k++) {
            const int c = threadIdx.x + k * nthr;
            if (c < vec_per_row) {
                *reinterpret_cast<h8 *>(gam_lds + c * 8) = aff[k][0];
                *reinterpret_cast<h8 *>(bet_lds + c * 8) = aff[k][1];
            }
        }
    }

    // ---- fused SkipLayerNorm: statistics in fp32 per row (wave64 butterflies), the
    // normalised row goes to LDS as fp16 — the value a separate LayerNorm kernel would
    // have stored — and, from block-row group 0, to ln_out
    if (LN) {
        auto unpack = [](uint2 raw, float (&f)[4]) {
            const h2 lo = __builtin_bit_cast(h2, raw.x), hi = __builtin_bit_cast(h2, raw.y);
            f[0] = (float)lo[0]; f[1] = (float)lo[1]; f[2] = (float)hi[0]; f[3] = (float)hi[1];
        };
        const float inv_h = 1.0f / (float)a.in;
#pragma unroll
        for (int rr = 0; rr < kLnRows; rr++) {
            const int r = wave + 8 * rr;  // 8 waves: always inside the strip
            const bool row_ok = r < rows_here;
            float x[kLnNit][4];
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < kLnNit; i++) {
                const bool ok = lane + 64 * i < ln_chunks;
                float y[4];
                unpack(ln_s[rr][i], x[i]);
                unpack(ln_k[rr][i], y);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    x[i][j] = ok ? x[i][j] + y[j] : 0.0f;
                    sum += x[i][j];
                }
            }
            const float mean = wave_sum(sum) * inv_h;
            float sq = 0.0f;
#pragma unroll
            for (int i = 0; i < kLnNit; i++) {
                const bool ok = lane + 64 * i < ln_chunks;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float d = ok ? x[i][j] - mean : 0.0f;
                    sq += d * d;
                }
            }
            const float rstd = rsqrtf(wave_sum(sq) * inv_h + a.ln_eps);
#pragma unroll
            for (int i = 0; i < kLnNit; i++) {
                const int c = lane + 64 * i;
                float gg[4], bb[4];
                unpack(ln_g[i], gg);
                unpack(ln_b[i], bb);
                h4 o;
#pragma unroll
                for (int j = 0; j < 4; j++)
                    o[j] = row_ok ? (_Float16)((x[i][j] - mean) * rstd * gg[j] + bb[j]) : (_Float16)0;
                if (c < ln_chunks) {
                    *reinterpret_cast<h4 *>(xs + r * lds_ld + c * 4) = o;  // rows past T stay zero
                    if (group == 0 && row_ok)
                        *reinterpret_cast<h4 *>(a.ln_out + (size_t)(tok0 + r) * a.in + c * 4) = o;
                }
            }
        }
        __syncthreads();
    }
    // ---- strip copy: write the first batch, then the rest
    if (NORM) __syncthreads();  // statistics and affine vectors are in LDS
    // value written for strip vector (r, c): the loaded one, or its normalisation
    auto strip_value = [&](h8 v, h8 skp, int r, int c) {
        if (!NORM) return v;
        const float2 st = stat_lds[r];
        const h8 gm = *reinterpret_cast<const h8 *>(gam_lds + c * 8);
        const h8 bt = *reinterpret_cast<const h8 *>(bet_lds + c * 8);
        h8 o;
#pragma unroll
        for (int e = 0; e < 8; e++)
            o[e] = (_Float16)norm_value((float)v[e] + (float)skp[e], st.x, st.y, (float)gm[e], (float)bt[e]);
        if (group == 0) *reinterpret_cast<h8 *>(a.ln_out + (size_t)(tok0 + r) * a.in + c * 8) = o;
        return o;
    };
    // the same from the binary32 strip; the block-row groups of a strip each write back an equal
    // run of its vectors (no run at all when neither output is asked for)
    const bool norm_wr = NORM32 && (a.ln_out32 || a.ln_out);
    const int own_per = (total_vec + ngroups - 1) / ngroups;
    const int own_lo = norm_wr ? group * own_per : 0;
    const int own_hi = norm_wr ? min(total_vec, own_lo + own_per) : 0;
    auto strip_value32 = [&](f4 lo, f4 hi, int r, int c, int idx) {
        const float2 st = stat_lds[r];
        const h8 gm = *reinterpret_cast<const h8 *>(gam_lds + c * 8);
        const h8 bt = *reinterpret_cast<const h8 *>(bet_lds + c * 8);
        f4 y0, y1;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            y0[e] = norm_value(lo[e], st.x, st.y, (float)gm[e], (float)bt[e]);
            y1[e] = norm_value(hi[e], st.x, st.y, (float)gm[4 + e], (float)bt[4 + e]);
        }
        const h8 o = {(_Float16)y0[0], (_Float16)y0[1], (_Float16)y0[2], (_Float16)y0[3],
                      (_Float16)y1[0], (_Float16)y1[1], (_Float16)y1[2], (_Float16)y1[3]};
        if (idx >= own_lo && idx < own_hi) {
            const size_t at = (size_t)(tok0 + r) * a.in + c * 8;
            if (a.ln_out32) {
                *reinterpret_cast<f4 *>(a.ln_out32 + at) = y0;
                *reinterpret_cast<f4 *>(a.ln_out32 + at + 4) = y1;
            }
            if (a.ln_out) *reinterpret_cast<h8 *>(a.ln_out + at) = o;
        }
        return o;
    };
    if (STAGE && !LN) {
        const int dr = nthr / vec_per_row, dc = nthr - dr * vec_per_row;  // (row, col) step of +nthr
        int r = threadIdx.x / vec_per_row, c = threadIdx.x - r * vec_per_row;
#pragma unroll
        for (int u = 0; u < kSU; u++) {
            const int idx = threadIdx.x + u * nthr;
            if (idx < total_vec)
                *reinterpret_cast<h8 *>(xs + r * lds_ld + c * 8) =
                    NORM32 ? strip_value32(s32[NORM32 ? u : 0][0], s32[NORM32 ? u : 0][1], r, c, idx)
                           : strip_value(sv[u], sk[SKIP16 ? u : 0], r, c);
            r += dr;
            c += dc;
            if (c >= vec_per_row) {
                c -= vec_per_row;
                r++;
            }
        }
        for (int base = threadIdx.x + kSU * nthr; base < total_vec; base += nthr * kSU) {
#pragma unroll
            for (int u = 0; u < kSU; u++) {
                const int v = min(base + u * nthr, total_vec - 1);
                if (NORM32) {
                    s32[NORM32 ? u : 0][0] = src32[2 * v];
                    s32[NORM32 ? u : 0][1] = src32[2 * v + 1];
                } else {
                    sv[u] = src[v];
                }
            }
            if (SKIP16) {
#pragma unroll
                for (int u = 0; u < kSU; u++) sk[u] = src_skip[min(base + u * nthr, total_vec - 1)];
            }
#pragma unroll
            for (int u = 0; u < kSU; u++) {
                const int idx = base + u * nthr;
                if (idx < total_vec)
                    *reinterpret_cast<h8 *>(xs + r * lds_ld + c * 8) =
                        NORM32 ? strip_value32(s32[NORM32 ? u : 0][0], s32[NORM32 ? u : 0][1], r, c, idx)
                               : strip_value(sv[u], sk[SKIP16 ? u : 0], r, c);
                r += dr;
                c += dc;
                if (c >= vec_per_row) {
                    c -= vec_per_row;
                    r++;
                }
            }
        }
        // rows beyond T (a partial last strip) read as zero
        for (int idx = total_vec + threadIdx.x; idx < MT * 16 * vec_per_row; idx += nthr) {
            const int rr = idx / vec_per_row, cc = idx - rr * vec_per_row;
            *reinterpret_cast<h8 *>(xs + rr * lds_ld + cc * 8) = zero8;
        }
#pragma unroll
        for (int buf = kEarly; buf < kNB; buf++) issue_item(buf);
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

    // ---- multiply
    f4 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = f4{0.f, 0.f, 0.f, 0.f};

    // bias + activation + store of one finished block-row, then clear
    float st1[MT], st2[MT];  // RES: this lane's sums over the values it wrote, per token block
#pragma unroll
    for (int m = 0; m < MT; m++) st1[m] = st2[m] = 0.0f;
    // RES32 with a residual that is formed here: mean and rstd of this lane's token of every block
    float2 tst[RES32 ? MT : 1];
    if (RES32 && a.rs_fin) {
#pragma unroll
        for (int m = 0; m < MT; m++)
            tst[RES32 ? m : 0] = *reinterpret_cast<const float2 *>(a.rs_fin + 2 * (size_t)min(tok0 + m * 16 + r16, a.T - 1));
    }
    auto flush = [&](int wave_row, h4 bv, const f4 (&rs)[MT], h4 gm, h4 bt) {
        const int f0 = (rb_begin + wave + nwave * wave_row) * 16 + g * 4;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            if (tok_ok[m]) {
                const int tok = tok0 + m * 16 + r16;
                h4 o;
                if (RES32) {  // the binary32 sum itself is the result
                    f4 v;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float rv = rs[m][j];
                        if (a.rs_fin)  // wave-uniform
                            rv = norm_value(rv, tst[RES32 ? m : 0].x, tst[RES32 ? m : 0].y, (float)gm[j], (float)bt[j]);
                        v[j] = acc[m][j] + (float)bv[j] + rv;
                        st1[m] += v[j];
                        st2[m] = __builtin_fmaf(v[j], v[j], st2[m]);
                    }
                    *reinterpret_cast<f4 *>(a.Y32 + (size_t)tok * a.out + f0) = v;
                    acc[m] = f4{0.f, 0.f, 0.f, 0.f};
                    continue;
                }
                if (RES) {
                    const h4 rv = *reinterpret_cast<const h4 *>(a.resid + (size_t)tok * a.out + f0);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        o[j] = (_Float16)(acc[m][j] + (float)bv[j]);
                        const float v = (float)o[j] + (float)rv[j];  // what the consumer will form
                        st1[m] += v;
                        st2[m] = __builtin_fmaf(v, v, st2[m]);
                    }
                } else if (a.Y32) {  // wave-uniform (a kernel argument)
                    f4 o32;
#pragma unroll
                    for (int j = 0; j < 4; j++) o32[j] = act_fixed<ACT>(acc[m][j] + (float)bv[j]);
                    *reinterpret_cast<f4 *>(a.Y32 + (size_t)tok * a.out + f0) = o32;
                    acc[m] = f4{0.f, 0.f, 0.f, 0.f};
                    continue;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) o[j] = (_Float16)act_fixed<ACT>(acc[m][j] + (float)bv[j]);
                }
                *reinterpret_cast<h4 *>(a.Y + (size_t)tok * a.out + f0) = o;
            }
            acc[m] = f4{0.f, 0.f, 0.f, 0.f};
        }
    };

    while (g_row[0] >= 0) {
#pragma unroll
        for (int buf = 0; buf < kNB; buf++) {
            if (g_row[buf] >= 0) {
                const int nsl = g_nsl[buf];
#pragma unroll
                for (int p0 = 0; p0 < kSlots; p0 += 2) {
                    if (p0 < nsl) {  // wave-uniform; slot p0+1 is real or zero-weighted
                        h8 x[2][MT];
                        int ca[2], cd[2];  // column of a slot's first tile; second minus first
#pragma unroll
                        for (int q = 0; q < 2; q++) {
                            ca[q] = lane_read(colv[buf], 2 * (p0 + q));
                            cd[q] = lane_read(colv[buf], 2 * (p0 + q) + 1) - ca[q];
                        }
#pragma unroll
                        for (int q = 0; q < 2; q++)
#pragma unroll
                            for (int m = 0; m < MT; m++) {
                                x[q][m] = *reinterpret_cast<const h8 *>(xrow[m] + (ca[q] + sel * cd[q]) * 16);
                                if (!STAGE && !tok_ok[m]) x[q][m] = zero8;
                            }
#pragma unroll
                        for (int q = 0; q < 2; q++)
#pragma unroll
                            for (int m = 0; m < MT; m++)
                                acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[buf][p0 + q], x[q][m], acc[m], 0, 0, 0);
                    }
                }
                if (g_last[buf]) flush(g_row[buf], bias_v[buf], rsd[RES32 ? buf : 0], rgm[RES32 ? buf : 0], rbt[RES32 ? buf : 0]);
                issue_item(buf);  // request the item after next into the buffer just drained
            }
        }
    }
    // block-rows without any tile still produce act(bias)
    for (int r = 0; r < nrw; r++) {
        if (lane_read(rp_hi, r) == lane_read(rp_lo, r)) {
            h4 bv = {0, 0, 0, 0};
            if (a.bias) bv = *reinterpret_cast<const h4 *>(a.bias + (rb_begin + wave + nwave * r) * 16 + g * 4);
            f4 rs[MT];
            h4 gm = {0, 0, 0, 0}, bt = {0, 0, 0, 0};
            if (RES32) load_resid(r, rs, gm, bt);
            flush(r, bv, rs, gm, bt);
        }
    }
    if (RES) {
        // per token: the four lanes that share it, then the waves (through LDS, in wave
        // order), then one float2 per token and block-row group — no atomics, so the sums
        // and everything normalised with them are reproducible
#pragma unroll
        for (int m = 0; m < MT; m++) {
            st1[m] += __shfl_xor(st1[m], 16, 64);
            st1[m] += __shfl_xor(st1[m], 32, 64);
            st2[m] += __shfl_xor(st2[m], 16, 64);
            st2[m] += __shfl_xor(st2[m], 32, 64);
        }
        __syncthreads();  // every wave is done reading the strip
        float2 *red = reinterpret_cast<float2 *>(smem_raw);
        if (g == 0) {
#pragma unroll
            for (int m = 0; m < MT; m++) red[wave * (MT * 16) + m * 16 + r16] = float2{st1[m], st2[m]};
        }
        __syncthreads();
        if ((int)threadIdx.x < rows_here) {
            float s1 = 0.0f, s2 = 0.0f;
            for (int wv = 0; wv < nwave; wv++) {
                const float2 pr = red[wv * (MT * 16) + threadIdx.x];
                s1 += pr.x;
                s2 += pr.y;
            }
            *reinterpret_cast<float2 *>(a.st_out + ((size_t)group * a.T + tok0 + threadIdx.x) * 2) = float2{s1, s2};
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

// LDS of one workgroup: the padded strip (when staged).
static size_t bsr_lds_bytes(int mt, bool stage, int in, int rows_per_wg) {
    (void)rows_per_wg;
    return stage ? (size_t)mt * 16 * (in + kLdsPad) * sizeof(_Float16) : 0;
}

// Launch geometry, from sweeps over 128..16384 token rows of the BERT-base and BERT-large
// matrices.  The kernel is bound by what one compute unit can fetch (its strip of X plus its
// share of W, about 35 GB/s per unit whatever is in flight), so the fastest geometry is almost
// always one workgroup per compute unit: strips of MT*16 rows, each split over
// floor(256 / strips) groups of block-rows.  Wider strips fetch W fewer times but leave each
// workgroup fewer block-rows; they pay once a workgroup still gets two per wave (64-row strips)
// or about one (32-row strips).  6 waves instead of 8 where that deals the block-rows evenly
// and as fast (6 or fewer, or 18, per workgroup).
static BsrPlan plan_bsr(int T, int in, int out) {
    const size_t lds_cap = 160 * 1024;
    const size_t row_bytes = (size_t)(in + kLdsPad) * sizeof(_Float16);
    const int nbr = out / 16;
    BsrPlan p{};
    if (16 * row_bytes > lds_cap) {
        // no strip fits the LDS: X fragments are read from global memory, 4 waves, two
        // block-rows per wave or an even split over 256 workgroups, whichever is more
        p.mt = 2;
        p.stage = false;
        p.threads = 256;
        const int strips = (T + 31) / 32;
        const int groups = strips >= 256 ? 1 : 256 / strips;
        int rpw = (nbr + groups - 1) / groups;
        if (rpw < 8) rpw = 8;
        if (rpw > nbr) rpw = nbr;
        // a wave keeps one block-row's [lo, hi) per lane: at most kMaxWaveRows block-rows per wave
        const int cap = kMaxWaveRows * (p.threads / 64);
        if (rpw > cap) rpw = cap;
        p.rows_per_wg = rpw;
        p.lds = 0;
        return p;
    }
    auto rows_per_wg_for = [&](int mt) {
        const int strips = (T + mt * 16 - 1) / (mt * 16);
        const int groups = strips >= 256 ? 1 : 256 / strips;
        return (nbr + groups - 1) / groups;
    };
    if (64 * row_bytes <= lds_cap && T >= 64 && rows_per_wg_for(4) >= 16) p.mt = 4;
    else if (32 * row_bytes <= lds_cap / 2 && T >= 32 && rows_per_wg_for(2) >= 5) p.mt = 2;
    else p.mt = 1;
    p.stage = true;
    int rpw = rows_per_wg_for(p.mt);
    p.threads = (rpw <= 6 || rpw == 18) ? 384 : 512;
    // 16-row strips (inputs too wide for 32 rows) with 24 to 48 block-rows per workgroup: 12 waves of
    // two to four rows instead of 8 waves of three to six, two row groups in flight per wave
    // (2048 x 3072 -> 768: 13.6 -> 11.6 us, 16384 rows: 103 -> 87 us).  With fewer rows per
    // workgroup the 8-wave form, which keeps four row groups in flight, is the faster one, and so it
    // is on 32-row strips.
    if (p.mt == 1 && rpw >= 24 && rpw <= 48) p.threads = 768;
    const int cap = kMaxWaveRows * (p.threads / 64);
    if (rpw > cap) rpw = cap;
    p.rows_per_wg = rpw;
    p.lds = bsr_lds_bytes(p.mt, p.stage, in, rpw);
    return p;
}

// Geometry of the kernels with the fused SkipLayerNorm prologue: 8 waves, staged strip.
static BsrPlan plan_bsr_ln(int T, int in, int out) {
    const size_t lds_cap = 160 * 1024;
    const size_t row_bytes = (size_t)(in + kLdsPad) * sizeof(_Float16);
    const int nbr = out / 16;
    BsrPlan p{};
    p.stage = 16 * row_bytes <= lds_cap;
    // 32-row strips once they give every compute unit work; 16-row strips below that (half
    // the rows to normalise per workgroup, twice the workgroups)
    p.mt = (T >= 512 && 32 * row_bytes <= lds_cap / 2) ? 2 : 1;
    p.threads = 512;
    // one workgroup per compute unit, as in plan_bsr
    const int strips = (T + p.mt * 16 - 1) / (p.mt * 16);
    const int groups = strips >= 256 ? 1 : 256 / strips;
    int rpw = (nbr + groups - 1) / groups;
    if (rpw > kMaxWaveRows * 8) rpw = kMaxWaveRows * 8;
    p.rows_per_wg = rpw;
    p.lds = bsr_lds_bytes(p.mt, p.stage, in, rpw);
    return p;
}

// Geometry of the kernels with the NORM prologue or the RES epilogue: staged strips of 16 or
// 32 rows; a RES producer splits a row over at most kMaxStatGroups block-row groups.
// stage == false in the result means the shape is not supported by these kernels.
static BsrPlan plan_bsr_fx(int T, int in, int out, int fx) {
    const size_t lds_cap = 160 * 1024;
    const size_t row_bytes = (size_t)(in + kLdsPad) * sizeof(_Float16);
    const size_t extra = (fx & kFxNorm) ? (size_t)4 * in : 0;  // gamma and beta
    const int nbr = out / 16;
    BsrPlan p{};
    auto fits = [&](int mt, size_t cap) { return mt * 16 * (row_bytes + sizeof(float2)) + extra <= cap; };
    p.stage = fits(1, lds_cap);
    p.mt = (T >= 32 && fits(2, lds_cap / 2)) ? 2 : 1;
    p.threads = 512;
    const int nwave = 8;
    const int strips = (T + p.mt * 16 - 1) / (p.mt * 16);
    int groups = strips >= 256 ? 1 : 256 / strips;
    if ((fx & kFxRes) && groups > kMaxStatGroups) groups = kMaxStatGroups;
    int rpw = (nbr + groups - 1) / groups;
    rpw = ((rpw + nwave - 1) / nwave) * nwave;
    if (rpw > nbr) rpw = nbr;
    if (rpw > kMaxWaveRows * nwave) {
        rpw = kMaxWaveRows * nwave;
        if ((fx & kFxRes) && (nbr + rpw - 1) / rpw > kMaxStatGroups) p.stage = false;  // out > 131072
    }
    p.rows_per_wg = rpw;
    p.lds = p.mt * 16 * (row_bytes + sizeof(float2)) + extra;
    const size_t red = (size_t)nwave * p.mt * 16 * sizeof(float2);
    if ((fx & kFxRes) && p.lds < red) p.lds = red;
    return p;
}

// Geometry of the binary32 split-normalisation kernels: that of plan_bsr (one workgroup per
// compute unit, 32-row strips where a workgroup still gets five block-rows), staged strips only,
// a RES producer split over at most kMaxStatGroups block-row groups.
static BsrPlan plan_bsr_fx32(int T, int in, int out, int fx) {
    const size_t lds_cap = 160 * 1024;
    const size_t row_bytes = (size_t)(in + kLdsPad) * sizeof(_Float16);
    const size_t extra = (fx & kFxNorm) ? (size_t)4 * in : 0;  // gamma and beta
    const int nbr = out / 16;
    BsrPlan p{};
    auto fits = [&](int mt, size_t cap) { return mt * 16 * (row_bytes + sizeof(float2)) + extra <= cap; };
    auto rows_per_wg_for = [&](int mt) {
        const int strips = (T + mt * 16 - 1) / (mt * 16);
        int groups = strips >= 256 ? 1 : 256 / strips;
        if ((fx & kFxRes) && groups > kMaxStatGroups) groups = kMaxStatGroups;
        return (nbr + groups - 1) / groups;
    };
    p.stage = fits(1, lds_cap);
    p.mt = (T >= 32 && fits(2, lds_cap / 2) && rows_per_wg_for(2) >= 5) ? 2 : 1;
    int rpw = rows_per_wg_for(p.mt);
    p.threads = (rpw <= 6 || rpw == 18) ? 384 : 512;
    // a producer on 16-row strips whose block-rows deal evenly to 12 waves runs 12: with a row or two
    // per wave, all its weights are requested before the strip has arrived
    if ((fx & kFxRes) && p.mt == 1 && rpw % 12 == 0 && rpw <= 24) p.threads = 768;
    // a consumer runs up to 12 waves of two block-rows: more instruction streams for the
    // normalisation and a shorter chain of rows per wave
    // (at least 6: the affine vectors of a row, in / 8 <= 640 16-byte pieces, are staged by two passes of the workgroup)
    if (fx & kFxNorm) p.threads = rpw > 12 ? 768 : 64 * std::max(6, (rpw + 1) / 2);
    const int cap = kMaxWaveRows * (p.threads / 64);
    if (rpw > cap) rpw = cap;
    if ((fx & kFxRes) && (nbr + rpw - 1) / rpw > kMaxStatGroups) p.stage = false;
    p.rows_per_wg = rpw;
    p.lds = p.mt * 16 * (row_bytes + sizeof(float2)) + extra;
    const size_t red = (size_t)(p.threads / 64) * p.mt * 16 * sizeof(float2);
    if ((fx & kFxRes) && p.lds < red) p.lds = red;
    return p;
}

template <int MT, bool STAGE, int ACT, int LN = 0, int FX = 0>
static int launch_bsr_act(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    auto kernel = bsr16_linear_kernel<MT, STAGE, ACT, LN, FX>;
    if (p.lds > 64 * 1024) {
        static bool raised = false;  // per instantiation
        if (!raised) {
            ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            raised = true;
        }
    }
    const int nbr = args.out / 16;
    const int ngroups = (nbr + p.rows_per_wg - 1) / p.rows_per_wg;
    const int nstrips = (args.T + MT * 16 - 1) / (MT * 16);
    const int strip_rounds = (nstrips + kXcds - 1) / kXcds;
    const dim3 grid((unsigned)(strip_rounds * kXcds * ngroups));
    kernel<<<grid, p.threads, p.lds, stream>>>(args);
    return check_launch("bsr16_linear_kernel");
}

template <int MT, bool STAGE>
static int launch_bsr(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    if constexpr (STAGE && MT <= 2) {
        if (p.threads > 512) {
            switch (args.act) {
                case ET_ACT_RELU: return launch_bsr_act<MT, STAGE, ET_ACT_RELU, 0, kFxWide>(args, p, stream);
                case ET_ACT_GELU: return launch_bsr_act<MT, STAGE, ET_ACT_GELU, 0, kFxWide>(args, p, stream);
                default: return launch_bsr_act<MT, STAGE, ET_ACT_NONE, 0, kFxWide>(args, p, stream);
            }
        }
    }
    ET_REQUIRE(p.threads <= 512, ET_ERR_INVALID_ARG, "tile-sparse Linear: %d threads need the 12-wave form", p.threads);
    switch (args.act) {
        case ET_ACT_RELU: return launch_bsr_act<MT, STAGE, ET_ACT_RELU>(args, p, stream);
        case ET_ACT_GELU: return launch_bsr_act<MT, STAGE, ET_ACT_GELU>(args, p, stream);
        default: return launch_bsr_act<MT, STAGE, ET_ACT_NONE>(args, p, stream);
    }
}

// fused SkipLayerNorm prologue: staged strips of 16 or 32 rows, 8 waves, in <= 1024
template <int MT, int NIT>
static int dispatch_bsr_ln_act(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    switch (args.act) {
        case ET_ACT_RELU: return launch_bsr_act<MT, true, ET_ACT_RELU, NIT>(args, p, stream);
        case ET_ACT_GELU: return launch_bsr_act<MT, true, ET_ACT_GELU, NIT>(args, p, stream);
        default: return launch_bsr_act<MT, true, ET_ACT_NONE, NIT>(args, p, stream);
    }
}
template <int MT>
static int dispatch_bsr_ln_mt(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    switch ((args.in + 255) / 256) {  // 4-element chunks per lane
        case 1: return dispatch_bsr_ln_act<MT, 1>(args, p, stream);
        case 2: return dispatch_bsr_ln_act<MT, 2>(args, p, stream);
        case 3: return dispatch_bsr_ln_act<MT, 3>(args, p, stream);
        default: return dispatch_bsr_ln_act<MT, 4>(args, p, stream);
    }
}
static int dispatch_bsr_ln(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    return p.mt == 2 ? dispatch_bsr_ln_mt<2>(args, p, stream) : dispatch_bsr_ln_mt<1>(args, p, stream);
}

template <int MT, int FX>
static int dispatch_bsr_fx_act(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    switch (args.act) {
        case ET_ACT_RELU: return launch_bsr_act<MT, true, ET_ACT_RELU, 0, FX>(args, p, stream);
        case ET_ACT_GELU: return launch_bsr_act<MT, true, ET_ACT_GELU, 0, FX>(args, p, stream);
        default: return launch_bsr_act<MT, true, ET_ACT_NONE, 0, FX>(args, p, stream);
    }
}
static int dispatch_bsr_norm(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    return p.mt == 2 ? dispatch_bsr_fx_act<2, kFxNorm>(args, p, stream) : dispatch_bsr_fx_act<1, kFxNorm>(args, p, stream);
}
static int dispatch_bsr_norm32(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    ET_REQUIRE(args.in / 8 <= 2 * p.threads, ET_ERR_UNSUPPORTED,
               "tile-sparse Linear: %d inputs need more than two passes of %d threads for the affine vectors", args.in,
               p.threads);
    return p.mt == 2 ? dispatch_bsr_fx_act<2, kFxNorm | kFxNorm32>(args, p, stream)
                     : dispatch_bsr_fx_act<1, kFxNorm | kFxNorm32>(args, p, stream);
}
static int dispatch_bsr_res32(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    if (args.resid16) {  // 8 waves at most: this kernel is not built for the 12-wave launch
        ET_REQUIRE(p.threads <= 512, ET_ERR_INVALID_ARG, "tile-sparse Linear: the binary16-residual producer runs at most 8 waves");
        return p.mt == 2 ? launch_bsr_act<2, true, ET_ACT_NONE, 0, kFxRes | kFxRes32 | kFxRes16>(args, p, stream)
                         : launch_bsr_act<1, true, ET_ACT_NONE, 0, kFxRes | kFxRes32 | kFxRes16>(args, p, stream);
    }
    return p.mt == 2 ? launch_bsr_act<2, true, ET_ACT_NONE, 0, kFxRes | kFxRes32>(args, p, stream)
                     : launch_bsr_act<1, true, ET_ACT_NONE, 0, kFxRes | kFxRes32>(args, p, stream);
}
static int dispatch_bsr_res(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    return p.mt == 2 ? launch_bsr_act<2, true, ET_ACT_NONE, 0, kFxRes>(args, p, stream)
                     : launch_bsr_act<1, true, ET_ACT_NONE, 0, kFxRes>(args, p, stream);
}

static int dispatch_bsr(const BsrArgs &args, const BsrPlan &p, hipStream_t stream) {
    ET_REQUIRE(p.rows_per_wg >= 1 && p.rows_per_wg <= kMaxWaveRows * (p.threads / 64), ET_ERR_UNSUPPORTED,
               "tile-sparse Linear: %d block-rows per workgroup of %d waves exceed %d per wave", p.rows_per_wg,
               p.threads / 64, kMaxWaveRows);
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
                 act,
                 nullptr, nullptr, nullptr, nullptr, nullptr, 0.0f, nullptr, 0, nullptr, nullptr};
    BsrPlan p = plan_bsr(T, in, out);
    args.rows_per_wg = p.rows_per_wg;
    return dispatch_bsr(args, p, as_stream(stream));
}

int et_linear_bsr16_f16_f32out(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles,
                               const et_f16 *bias, const et_f16 *X, float *Y, int T, int in, int out,
                               int act, et_stream stream) {
    int s = bsr_check(row_ptr, col_idx, tiles, X, reinterpret_cast<et_f16 *>(Y), T, in, out, act);
    if (s != ET_OK) return s;
    ET_REQUIRE((reinterpret_cast<uintptr_t>(Y) & 15) == 0, ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_f16_f32out: Y must be 16-byte aligned");
    if (T == 0) return ET_OK;
    BsrArgs args{};
    args.row_ptr = row_ptr;
    args.col_idx = col_idx;
    args.tiles = reinterpret_cast<const _Float16 *>(tiles);
    args.bias = reinterpret_cast<const _Float16 *>(bias);
    args.X = reinterpret_cast<const _Float16 *>(X);
    args.T = T;
    args.in = in;
    args.out = out;
    args.act = act;
    args.Y32 = Y;
    BsrPlan p = plan_bsr(T, in, out);
    args.rows_per_wg = p.rows_per_wg;
    return dispatch_bsr(args, p, as_stream(stream));
}

int et_skipln_linear_bsr16_f16(const et_f16 *src, const et_f16 *skip, const et_f16 *gamma,
                               const et_f16 *beta, float eps, et_f16 *ln_out, const int32_t *row_ptr,
                               const int32_t *col_idx, const et_f16 *tiles, const et_f16 *bias, et_f16 *Y,
                               int T, int in, int out, int act, et_stream stream) {
    ET_REQUIRE(src && skip && gamma && beta && ln_out, ET_ERR_INVALID_ARG,
               "et_skipln_linear_bsr16_f16: NULL pointer");
    int s = bsr_check(row_ptr, col_idx, tiles, ln_out, Y, T, in, out, act);
    if (s != ET_OK) return s;
    if (T == 0) return ET_OK;
    // the fused prologue keeps a row in registers as 4 chunks of 4 values per lane and needs a
    // staged strip; otherwise the two operators run back to back
    // (and must not normalise in place: every block-row group of a strip reads src and skip)
    BsrPlan p = plan_bsr_ln(T, in, out);
    if (in > 1024 || !p.stage || ln_out == src || ln_out == skip) {
        s = et_skip_layernorm_f16(ln_out, src, skip, gamma, beta, T, in, eps, stream);
        if (s != ET_OK) return s;
        return et_linear_bsr16_f16(row_ptr, col_idx, tiles, bias, ln_out, Y, T, in, out, act, stream);
    }
    BsrArgs args{row_ptr,
                 col_idx,
                 reinterpret_cast<const _Float16 *>(tiles),
                 reinterpret_cast<const _Float16 *>(bias),
                 nullptr,
                 reinterpret_cast<_Float16 *>(Y),
                 T,
                 in,
                 out,
                 p.rows_per_wg,
                 act,
                 reinterpret_cast<const _Float16 *>(src),
                 reinterpret_cast<const _Float16 *>(skip),
                 reinterpret_cast<const _Float16 *>(gamma),
                 reinterpret_cast<const _Float16 *>(beta),
                 reinterpret_cast<_Float16 *>(ln_out),
                 eps,
                 nullptr, 0, nullptr, nullptr};
    return dispatch_bsr_ln(args, p, as_stream(stream));
}

int et_linear_bsr16_fused_ln_supported(int T, int in, int out) {
    if (T <= 0 || in <= 0 || out <= 0 || T % 16 || in % 16 || out % 16) return 0;
    return plan_bsr_fx(T, in, out, kFxNorm).stage && plan_bsr_fx(T, in, out, kFxRes).stage ? 1 : 0;
}

int et_linear_bsr16_resid_stats_f16(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles,
                                    const et_f16 *bias, const et_f16 *X, const et_f16 *resid, et_f16 *V,
                                    float *stats, int *stat_groups, int T, int in, int out, et_stream stream) {
    ET_REQUIRE(resid && stats && stat_groups, ET_ERR_INVALID_ARG, "et_linear_bsr16_resid_stats_f16: NULL pointer");
    int s = bsr_check(row_ptr, col_idx, tiles, X, V, T, in, out, ET_ACT_NONE);
    if (s != ET_OK) return s;
    BsrPlan p = plan_bsr_fx(T, in, out, kFxRes);
    ET_REQUIRE(p.stage, ET_ERR_UNSUPPORTED, "et_linear_bsr16_resid_stats_f16: in=%d out=%d outside the staged range", in,
               out);
    *stat_groups = (out / 16 + p.rows_per_wg - 1) / p.rows_per_wg;
    if (T == 0) return ET_OK;
    BsrArgs args{row_ptr,
                 col_idx,
                 reinterpret_cast<const _Float16 *>(tiles),
                 reinterpret_cast<const _Float16 *>(bias),
                 reinterpret_cast<const _Float16 *>(X),
                 reinterpret_cast<_Float16 *>(V),
                 T,
                 in,
                 out,
                 p.rows_per_wg,
                 ET_ACT_NONE,
                 nullptr, nullptr, nullptr, nullptr, nullptr, 0.0f,
                 nullptr, 0,
                 reinterpret_cast<const _Float16 *>(resid),
                 stats};
    return dispatch_bsr_res(args, p, as_stream(stream));
}

int et_norm_linear_bsr16_f16(const et_f16 *V, const et_f16 *skip, const float *stats, int stat_groups,
                             const et_f16 *gamma, const et_f16 *beta, float eps, et_f16 *ln_out, const int32_t *row_ptr,
                             const int32_t *col_idx, const et_f16 *tiles, const et_f16 *bias, et_f16 *Y, int T,
                             int in, int out, int act, et_stream stream) {
    ET_REQUIRE(skip && stats && gamma && beta && ln_out, ET_ERR_INVALID_ARG, "et_norm_linear_bsr16_f16: NULL pointer");
    ET_REQUIRE(stat_groups >= 1 && stat_groups <= kMaxStatGroups, ET_ERR_INVALID_ARG,
               "et_norm_linear_bsr16_f16: stat_groups=%d must be in [1, %d]", stat_groups, kMaxStatGroups);
    ET_REQUIRE(ln_out != V && ln_out != skip, ET_ERR_INVALID_ARG,
               "et_norm_linear_bsr16_f16: ln_out must not alias V or skip");
    int s = bsr_check(row_ptr, col_idx, tiles, V, Y, T, in, out, act);
    if (s != ET_OK) return s;
    BsrPlan p = plan_bsr_fx(T, in, out, kFxNorm);
    ET_REQUIRE(p.stage, ET_ERR_UNSUPPORTED, "et_norm_linear_bsr16_f16: in=%d outside the staged range", in);
    if (T == 0) return ET_OK;
    BsrArgs args{row_ptr,
                 col_idx,
                 reinterpret_cast<const _Float16 *>(tiles),
                 reinterpret_cast<const _Float16 *>(bias),
                 reinterpret_cast<const _Float16 *>(V),
                 reinterpret_cast<_Float16 *>(Y),
                 T,
                 in,
                 out,
                 p.rows_per_wg,
                 act,
                 nullptr,
                 reinterpret_cast<const _Float16 *>(skip),
                 reinterpret_cast<const _Float16 *>(gamma),
                 reinterpret_cast<const _Float16 *>(beta),
                 reinterpret_cast<_Float16 *>(ln_out),
                 eps,
                 stats, stat_groups,
                 nullptr, nullptr};
    return dispatch_bsr_norm(args, p, as_stream(stream));
}

static bool fx32_shape_ok(int T, int in, int out) {
    return T > 0 && in > 0 && out > 0 && T % 16 == 0 && in % 16 == 0 && out % 16 == 0;
}
int et_linear_bsr16_resid_stats_f32_supported(int T, int in, int out) {
    return fx32_shape_ok(T, in, out) && plan_bsr_fx32(T, in, out, kFxRes).stage ? 1 : 0;
}
int et_norm_linear_bsr16_f32in_supported(int T, int in, int out) {
    return fx32_shape_ok(T, in, out) && plan_bsr_fx32(T, in, out, kFxNorm).stage ? 1 : 0;
}

static int resid_stats_f32(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, const et_f16 *bias,
                           const et_f16 *X, const float *resid, const et_f16 *resid16, const float *resid_fin,
                           const et_f16 *resid_gamma, const et_f16 *resid_beta, float *V, float *stats, int *stat_groups,
                           int T, int in, int out, et_stream stream);

int et_linear_bsr16_resid_stats_f32(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles,
                                    const et_f16 *bias, const et_f16 *X, const float *resid, const float *resid_fin,
                                    const et_f16 *resid_gamma, const et_f16 *resid_beta, float *V, float *stats,
                                    int *stat_groups, int T, int in, int out, et_stream stream) {
    ET_REQUIRE(resid, ET_ERR_INVALID_ARG, "et_linear_bsr16_resid_stats_f32: NULL pointer");
    return resid_stats_f32(row_ptr, col_idx, tiles, bias, X, resid, nullptr, resid_fin, resid_gamma, resid_beta, V, stats,
                           stat_groups, T, in, out, stream);
}

int et_linear_bsr16_resid16_stats_f32(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles,
                                      const et_f16 *bias, const et_f16 *X, const et_f16 *resid16, float *V, float *stats,
                                      int *stat_groups, int T, int in, int out, et_stream stream) {
    ET_REQUIRE(resid16, ET_ERR_INVALID_ARG, "et_linear_bsr16_resid16_stats_f32: NULL pointer");
    ET_REQUIRE((reinterpret_cast<uintptr_t>(resid16) & 7) == 0, ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_resid16_stats_f32: the residual must be 8-byte aligned");
    return resid_stats_f32(row_ptr, col_idx, tiles, bias, X, nullptr, resid16, nullptr, nullptr, nullptr, V, stats,
                           stat_groups, T, in, out, stream);
}

static int resid_stats_f32(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, const et_f16 *bias,
                           const et_f16 *X, const float *resid, const et_f16 *resid16, const float *resid_fin,
                           const et_f16 *resid_gamma, const et_f16 *resid_beta, float *V, float *stats, int *stat_groups,
                           int T, int in, int out, et_stream stream) {
    ET_REQUIRE(V && stats && stat_groups, ET_ERR_INVALID_ARG, "et_linear_bsr16_resid_stats_f32: NULL pointer");
    ET_REQUIRE(resid_fin == nullptr || (resid_gamma && resid_beta), ET_ERR_INVALID_ARG,
               "et_linear_bsr16_resid_stats_f32: a residual to normalise needs its affine vectors");
    ET_REQUIRE(V != resid, ET_ERR_INVALID_ARG, "et_linear_bsr16_resid_stats_f32: V must not alias the residual");
    ET_REQUIRE(((reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(resid)) & 15) == 0, ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_resid_stats_f32: V and resid must be 16-byte aligned");
    int s = bsr_check(row_ptr, col_idx, tiles, X, reinterpret_cast<et_f16 *>(V), T, in, out, ET_ACT_NONE);
    if (s != ET_OK) return s;
    BsrPlan p = plan_bsr_fx32(T, in, out, kFxRes);
    ET_REQUIRE(p.stage, ET_ERR_UNSUPPORTED, "et_linear_bsr16_resid_stats_f32: in=%d out=%d outside the staged range", in,
               out);
    if (resid16 && p.threads > 512) p.threads = 512;
    *stat_groups = (out / 16 + p.rows_per_wg - 1) / p.rows_per_wg;
    if (T == 0) return ET_OK;
    BsrArgs args{};
    args.row_ptr = row_ptr;
    args.col_idx = col_idx;
    args.tiles = reinterpret_cast<const _Float16 *>(tiles);
    args.bias = reinterpret_cast<const _Float16 *>(bias);
    args.X = reinterpret_cast<const _Float16 *>(X);
    args.T = T;
    args.in = in;
    args.out = out;
    args.rows_per_wg = p.rows_per_wg;
    args.act = ET_ACT_NONE;
    args.st_out = stats;
    args.Y32 = V;
    args.resid32 = resid;
    args.resid16 = reinterpret_cast<const _Float16 *>(resid16);
    args.rs_fin = resid_fin;
    args.rs_gamma = reinterpret_cast<const _Float16 *>(resid_gamma);
    args.rs_beta = reinterpret_cast<const _Float16 *>(resid_beta);
    return dispatch_bsr_res32(args, p, as_stream(stream));
}

int et_norm_linear_bsr16_f32in(const float *V, const float *stats, int stat_groups, const et_f16 *gamma,
                               const et_f16 *beta, float eps, float *fin_out, float *ln_out32, et_f16 *ln_out16,
                               const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, const et_f16 *bias,
                               et_f16 *Y, int T, int in, int out, int act, et_stream stream) {
    ET_REQUIRE(V && stats && gamma && beta, ET_ERR_INVALID_ARG, "et_norm_linear_bsr16_f32in: NULL pointer");
    ET_REQUIRE(stat_groups >= 1 && stat_groups <= kMaxStatGroups, ET_ERR_INVALID_ARG,
               "et_norm_linear_bsr16_f32in: stat_groups=%d must be in [1, %d]", stat_groups, kMaxStatGroups);
    ET_REQUIRE(ln_out32 == nullptr || ln_out32 != V, ET_ERR_INVALID_ARG,
               "et_norm_linear_bsr16_f32in: ln_out32 must not alias V");
    ET_REQUIRE(((reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(ln_out32) |
                 reinterpret_cast<uintptr_t>(ln_out16)) & 15) == 0,
               ET_ERR_UNSUPPORTED, "et_norm_linear_bsr16_f32in: V and the outputs must be 16-byte aligned");
    int s = bsr_check(row_ptr, col_idx, tiles, reinterpret_cast<const et_f16 *>(V), Y, T, in, out, act);
    if (s != ET_OK) return s;
    BsrPlan p = plan_bsr_fx32(T, in, out, kFxNorm);
    ET_REQUIRE(p.stage, ET_ERR_UNSUPPORTED, "et_norm_linear_bsr16_f32in: in=%d outside the staged range", in);
    if (T == 0) return ET_OK;
    BsrArgs args{};
    args.row_ptr = row_ptr;
    args.col_idx = col_idx;
    args.tiles = reinterpret_cast<const _Float16 *>(tiles);
    args.bias = reinterpret_cast<const _Float16 *>(bias);
    args.Y = reinterpret_cast<_Float16 *>(Y);
    args.T = T;
    args.in = in;
    args.out = out;
    args.rows_per_wg = p.rows_per_wg;
    args.act = act;
    args.ln_gamma = reinterpret_cast<const _Float16 *>(gamma);
    args.ln_beta = reinterpret_cast<const _Float16 *>(beta);
    args.ln_out = reinterpret_cast<_Float16 *>(ln_out16);
    args.ln_eps = eps;
    args.st_in = stats;
    args.st_groups = stat_groups;
    args.X32 = V;
    args.ln_out32 = ln_out32;
    args.fin_out = fin_out;
    return dispatch_bsr_norm32(args, p, as_stream(stream));
}

// Tuning hook: same computation with an explicit launch geometry.  mt in
// {1,2,4}; stage selects the LDS-staged strip; threads a multiple of 64 up to
// 768 (above 512: 16- and 32-row strips).  Not part of the drop-in surface.
int et_linear_bsr16_f16_geom(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles,
                             const et_f16 *bias, const et_f16 *X, et_f16 *Y, int T, int in,
                             int out, int act, int mt, int stage, int threads, int rows_per_wg,
                             et_stream stream) {
    int s = bsr_check(row_ptr, col_idx, tiles, X, Y, T, in, out, act);
    if (s != ET_OK) return s;
    ET_REQUIRE((mt == 1 || mt == 2 || mt == 4) && threads >= 64 && threads <= 768 &&
                   threads % 64 == 0 && rows_per_wg >= 1,
               ET_ERR_INVALID_ARG, "et_linear_bsr16_f16_geom: mt=%d threads=%d rows_per_wg=%d", mt,
               threads, rows_per_wg);
    if (T == 0) return ET_OK;
    BsrPlan p;
    p.mt = mt;
    p.stage = stage != 0;
    p.threads = threads;
    p.rows_per_wg = rows_per_wg;
    p.lds = bsr_lds_bytes(mt, p.stage, in, rows_per_wg);
    ET_REQUIRE(rows_per_wg <= kMaxWaveRows * (threads / 64), ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_f16_geom: at most %d block-rows per wave", kMaxWaveRows);
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
                 act,
                 nullptr, nullptr, nullptr, nullptr, nullptr, 0.0f, nullptr, 0, nullptr, nullptr};
    return dispatch_bsr(args, p, as_stream(stream));
}

}  // extern "C"
