// Dense GEMM for gfx950 on direct-to-LDS loads: C[M x N] = act(A[M x K] * B^T + bias), A and B
// both K-contiguous (B stored [N x K]), M and N multiples of the tile, K a multiple of 64.
//
// The 64x64-per-wave kernel in gemm.hip reads 1 byte of LDS per 32 flops, which at the
// MFMA peak is the whole bandwidth of the LDS port, and stages through registers; it tops
// out near a third of the matrix peak.  Here a workgroup of 4 waves (2 x 2) computes a tile of
// 64 TMW x 64 TNW and each wave a block of TMW x TNW v_mfma_f32_32x32x16_f16 tiles.  The
// largest tile, 256 x 256 (eight waves of 128 x 64, two per SIMD; the RAGGED form four waves of
// 128 x 128 with 256 accumulators in AGPRs), is for problems that fill the device with it; smaller problems
// take smaller tiles (more workgroups, several per compute unit) at the price of more operand
// traffic from the L2 per flop.  Latencies are covered inside the wave: K advances in stages
// of 64 through two LDS buffers (the 256 x 256 tile: stages of 32 through four, loads three
// stages ahead), a later stage is loaded straight from global memory into
// an idle buffer while the current one is multiplied (staging through registers and
// ds_write costs a third of the rate: the LDS port is then the bound), the fragment reads of
// the next K slice and the loads are issued between the MFMAs that hide them, in an order fixed in
// the source, and the one workgroup barrier of a stage sits before its last K slice.
//
// The MFMA A operand is the B matrix (output features) and vice versa, so a lane ends with
// 4 consecutive features of one row of C per 8-row group of a tile; the epilogue transposes
// through LDS to store whole row segments.
#include "gemm.hip.h"

namespace et {

constexpr int kDmaK = 64;                // K per stage: one 128-byte line of every row
constexpr int kDmaXcds = 8;
constexpr int kSbM = 4, kSbN = 8;        // tile block one XCD works on at a time
constexpr size_t dma_lds_bytes(int tmw, int tnw, int nbuf, int ks = kDmaK, int nwn = 2) {  // buffers of (BM + BN) rows of ks k-values
    return (size_t)nbuf * (64 * tmw + 32 * nwn * tnw) * ks * sizeof(_Float16);
}
// s_waitcnt immediate for vmcnt(n) alone on gfx9: vmcnt in bits 3:0 and 15:14, expcnt 6:4 and
// lgkmcnt 11:8 left at their maxima
constexpr int wait_vm(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }
#define ET_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define ET_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

typedef float f16v __attribute__((ext_vector_type(16)));

// TMW x TNW: 32 x 32 MFMA tiles per wave.  IDX: the result columns are scattered (c_scatter) or
// their bias is gathered (bias_idx).  RAGGED: M, N and K are multiples of 16 only; rows past the
// end of an operand are loaded from its last row and never stored, the chunks of the last K
// stage past the end of K are zeroed in LDS before they are read.
// BT: B is stored [K x N] (N contiguous) instead of [N x K]; its stage lies in LDS as loaded, k-major,
// and a lane gathers the 8 k-values of a fragment with 2-byte reads (64 x 64 tiles only).
// Problem z = blockIdx.y of a batch uses the operand offsets of GemmArgs.
// KS: k-values per stage, 64 or (whole tiles only) 32: half the stage, twice the buffers in the same LDS, so the
// loads of a stage are issued three stages ahead and spread over two K slices.
// NWN: waves along N, 2 (four waves, one per SIMD) or (whole tiles only) 4: eight waves, two per SIMD, so that a wave
// held up at a load or at the barrier leaves the matrix pipe to the other.
template <int TMW, int TNW, int NBUF, bool IDX, bool RAGGED = false, bool BT = false, int KS = kDmaK, int NWN = 2>
__global__ __launch_bounds__(128 * NWN) void gemm_f16_dma_kernel(const GemmArgs ga) {
    static_assert(NWN == 2 || (NWN == 4 && !RAGGED && !BT), "eight waves are written for whole tiles");
    constexpr int kWaves = 2 * NWN;
    static_assert(NBUF >= 2 && NBUF <= 4 && (NBUF - 1) * (2 * TMW + 2 * TNW) * KS / kDmaK <= 63, "vmcnt holds 63 loads");
    static_assert(KS == kDmaK || (KS == 32 && !RAGGED && !BT), "half stages are written for whole tiles");
    static_assert(!BT || (TMW == 1 && TNW == 1 && RAGGED), "the k-major B stage is written for the 64 x 64 tile");
    GemmArgs g = ga;
    {
        const long long zo = blockIdx.y / g.batch_inner, zi = blockIdx.y % g.batch_inner;
        g.A += zo * g.sAo + zi * g.sAi;
        g.B += zo * g.sBo + zi * g.sBi;
        g.C += zo * g.sCo + zi * g.sCi;
        if (g.bias) g.bias += zo * g.sBias_o + zi * g.sBias_i;
    }
    constexpr int BM = 64 * TMW, BN = 32 * NWN * TNW;  // workgroup tile: 2 x NWN waves
    constexpr int WM = 32 * TMW, WN = 32 * TNW;  // wave block
    extern __shared__ __align__(16) unsigned char dma_smem[];
    _Float16 *As = reinterpret_cast<_Float16 *>(dma_smem);  // [NBUF][BM][KS], chunks swizzled
    _Float16 *Bs = As + NBUF * BM * KS;                      // [NBUF][BN][KS]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: LDS targets of the loads stay scalar
    const int wm = wave / NWN, wn = wave % NWN;
    const int l32 = lane & 31, kg = lane >> 5;
    // Workgroup id -> tile, XCD-aware.  Workgroups go to the 8 XCDs round-robin by id and each XCD runs them in
    // order; consecutive workgroups of an XCD are given consecutive tiles of an order that walks the result in
    // blocks of group_rows x 8 tiles (4 x 8: 4 panels of A, 8 of B), so the XCD's L2 serves about 12 panels to 32
    // workgroups instead of up to 64.  The order counts existing tiles only (a block at the right or lower edge
    // is narrower or shorter) and the groups are dealt to the XCDs in turn, so every XCD gets the same number of
    // tiles to within one group; dealing whole 4 x 8 blocks instead gave the XCDs with odd numbers only the
    // half-empty blocks of a result 12 tiles wide.
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    const int sbm = g.group_rows, gsh = sbm == 4 ? 5 : sbm == 2 ? 4 : 3;  // a group: sbm x 8 = 1 << gsh tiles
    const int xcd = blockIdx.x % kDmaXcds, j = blockIdx.x / kDmaXcds;
    const int t = ((((j >> gsh) * kDmaXcds + xcd)) << gsh) + (j & ((1 << gsh) - 1));
    if (t >= tiles_m * tiles_n) return;  // padding of the grid (whole workgroup)
    int ty, tx;
    {
        const int per_br = sbm * tiles_n, full_br = tiles_m / sbm;  // tiles of a full block row; such rows
        const int br = min(t / per_br, full_br);
        const int rem = t - br * per_br;
        if (br < full_br && (tiles_n & (kSbN - 1)) == 0) {  // whole blocks only: shifts
            const int q = rem & ((1 << gsh) - 1);
            ty = br * sbm + (q >> 3);
            tx = (rem >> gsh) * kSbN + (q & 7);
        } else {
            const int rows = br < full_br ? sbm : tiles_m - full_br * sbm;  // tile rows of this block row
            const int per_bc = rows * kSbN, full_bc = tiles_n / kSbN;
            const int bc = min(rem / per_bc, full_bc);
            const int q = rem - bc * per_bc;
            const int w = bc < full_bc ? kSbN : tiles_n - full_bc * kSbN;  // tile columns of this block
            ty = br * sbm + q / w;
            tx = bc * kSbN + q % w;
        }
    }
    const int m0 = ty * BM, n0 = tx * BN;

    f16v acc[TMW][TNW];  // [token tile][feature tile]
#pragma unroll
    for (int i = 0; i < TMW; i++)
#pragma unroll
        for (int j = 0; j < TNW; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // Stage loads go straight from global memory to LDS (global_load_lds_dwordx4): a wave
    // instruction fills 1 KB of consecutive LDS, 16 bytes per lane, from addresses the lanes
    // choose.  Here that is 8 rows of 128 bytes, 8 lanes a row (whole lines of the operand);
    // within the row the lane at position p fetches chunk p ^ swz(row), so that the fragment
    // reads below, 16 rows apart by one chunk column, spread over all banks with no padding.
    const int lrow = lane >> 3, lpos = lane & 7;
    // K-contiguous operands (kWhole; all but BT): a lane's loads differ between stages only by the stage's k0, so a
    // load is a scalar base that advances by one line per stage plus a 32-bit lane offset computed once; every stage
    // issues its loads (past the last stage they fetch the last stage again, into a buffer nobody reads any more),
    // which keeps the loads in the block of the multiplications, where they can be placed between them, and the
    // number of outstanding loads the same in every stage.  RAGGED: rows past the end of an operand take the offset
    // of its last row, and the last stage, when K ends inside it, has offsets of its own: chunks past the end of K
    // fetch the last chunk of the row instead (and are zeroed in LDS once they have landed).
    constexpr bool kWhole = !BT;
    constexpr bool kImm = !RAGGED;  // (a clamped row may have a smaller offset than the immediate it would have to undo)
    // A stage row holds KS k-values = kLpr 16-byte chunks; one load instruction fills kRpi rows.  The chunk at
    // position p of row r is chunk p ^ swz(r) of the operand: rows that share their banks (2 rows of 128 bytes,
    // 4 rows of 64 bytes span all banks) get different chunks at one position.
    constexpr int kLpr = KS / 8, kRpi = 64 / kLpr;
    constexpr int kLA = BM / kWaves / kRpi, kLB = BN / kWaves / kRpi;  // loads per wave and stage
    auto swz_of = [](int r) { return KS == 64 ? (r >> 1) & 7 : (r >> 2) & 3; };
    // The instruction's immediate offset is added to the global address and to the LDS address alike: loads
    // 4j .. 4j + 3 of an operand share one LDS base (M0) and differ in the immediate, 1024 (v % 4), which the
    // lane's global offset has subtracted again.  One write of M0 per four loads instead of one per load.
    unsigned offA[kLA], offB[kLB];  // bytes from the tile's first row at k = 0, minus the immediate
    unsigned tailA[RAGGED ? kLA : 1], tailB[RAGGED ? kLB : 1];  // the same for a last stage that K ends in
    const int k_tail0 = (g.K - 1) / KS * KS;   // first k of the last stage
    const int k_tail = g.K - k_tail0;          // k-values of the last stage, 16 .. KS
    if (kWhole) {
        const int lr = lane / kLpr, lp = lane % kLpr;
#pragma unroll
        for (int v = 0; v < kLA; v++) {
            const int r = wave * (BM / kWaves) + v * kRpi + lr;
            const int row = RAGGED ? min(m0 + r, g.M - 1) - m0 : r;
            const int c8 = (lp ^ swz_of(r)) * 8;
            offA[v] = (unsigned)((row * g.lda + c8) * 2 - (kImm ? (v % 4) * 1024 : 0));
            if (RAGGED) tailA[v] = (unsigned)((row * g.lda + min(c8, k_tail - 8)) * 2);
        }
#pragma unroll
        for (int v = 0; v < kLB; v++) {
            const int r = wave * (BN / kWaves) + v * kRpi + lr;
            const int row = RAGGED ? min(n0 + r, g.N - 1) - n0 : r;
            const int c8 = (lp ^ swz_of(r)) * 8;
            offB[v] = (unsigned)((row * g.ldb + c8) * 2 - (kImm ? (v % 4) * 1024 : 0));
            if (RAGGED) tailB[v] = (unsigned)((row * g.ldb + min(c8, k_tail - 8)) * 2);
        }
    }
    const char *a_tile = reinterpret_cast<const char *>(g.A + (size_t)m0 * g.lda);
    const char *b_tile = reinterpret_cast<const char *>(g.B + (size_t)n0 * g.ldb);
    // loads [first, first + count) of a stage's kLA + kLB (whole tiles)
    auto load_part = [&](int buf, int k0, int first, int count) {
        const char *ak = a_tile + (size_t)k0 * 2, *bk = b_tile + (size_t)k0 * 2;  // uniform
        auto four = [&](const char *src, _Float16 *dst, int sub) {  // sub = v % 4 (a constant once unrolled)
            if (sub == 0) __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(src), ET_LDS_PTR(dst), 16, 0, 0);
            else if (sub == 1) __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(src), ET_LDS_PTR(dst), 16, 1024, 0);
            else if (sub == 2) __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(src), ET_LDS_PTR(dst), 16, 2048, 0);
            else __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(src), ET_LDS_PTR(dst), 16, 3072, 0);
        };
        const bool tail = RAGGED && k0 == k_tail0 && k_tail < KS;  // uniform
#pragma unroll
        for (int v = 0; v < kLA; v++)
            if (v >= first && v < first + count) {
                const unsigned off = RAGGED && tail ? tailA[RAGGED ? v : 0] : offA[v];
                four(ak + off, As + (buf * BM + wave * (BM / kWaves) + (kImm ? (v / 4) * 4 : v) * kRpi) * KS, kImm ? v % 4 : 0);
            }
#pragma unroll
        for (int v = 0; v < kLB; v++)
            if (kLA + v >= first && kLA + v < first + count) {
                const unsigned off = RAGGED && tail ? tailB[RAGGED ? v : 0] : offB[v];
                four(bk + off, Bs + (buf * BN + wave * (BN / kWaves) + (kImm ? (v / 4) * 4 : v) * kRpi) * KS, kImm ? v % 4 : 0);
            }
    };
    auto load_stage = [&](int buf, int k0) {
        if constexpr (kWhole) {
            load_part(buf, k0, 0, kLA + kLB);
            return;
        }
#pragma unroll
        for (int v = 0; v < 2 * TMW; v++) {  // a wave loads a quarter of the rows of each operand
            const int r0 = wave * (BM / 4) + v * 8, r = r0 + lrow;
            const int c = lpos ^ ((r >> 1) & 7);
            const int row = RAGGED ? min(m0 + r, g.M - 1) : m0 + r;
            const int k = RAGGED ? min(k0 + c * 8, g.K - 8) : k0 + c * 8;
            __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(g.A + (size_t)row * g.lda + k),
                                             ET_LDS_PTR(As + (buf * BM + r0) * kDmaK), 16, 0, 0);
        }
#pragma unroll
        for (int v = 0; v < 2 * TNW; v++) {
            const int r0 = wave * (BN / 4) + v * 8, r = r0 + lrow;
            if (BT) {  // LDS row r = k-value k0 + r of the stage, 64 columns of B from n0
                const int krow = min(k0 + r, g.K - 1), n = min(n0 + lpos * 8, g.N - 8);
                __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(g.B + (size_t)krow * g.ldb + n),
                                                 ET_LDS_PTR(Bs + (buf * kDmaK + r0) * BN), 16, 0, 0);
            } else {
                const int c = lpos ^ ((r >> 1) & 7);
                const int row = RAGGED ? min(n0 + r, g.N - 1) : n0 + r;
                const int k = RAGGED ? min(k0 + c * 8, g.K - 8) : k0 + c * 8;
                __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(g.B + (size_t)row * g.ldb + k),
                                                 ET_LDS_PTR(Bs + (buf * BN + r0) * kDmaK), 16, 0, 0);
            }
        }
    };
    // RAGGED: zeros over the chunks of the last stage that lie past the end of K, in the rows
    // this wave loaded (after its loads have landed, before the barrier that releases the buffer)
    const int ktail = g.K - (g.K - 1) / kDmaK * kDmaK;  // k-values of the last stage, 16..64
    auto zero_tail = [&](int buf) {
        const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int v = 0; v < 2 * TMW; v++) {
            const int r = wave * (BM / 4) + v * 8 + lrow;
            if ((lpos ^ ((r >> 1) & 7)) * 8 >= ktail)
                *reinterpret_cast<h8 *>(As + (buf * BM + r) * kDmaK + lpos * 8) = zero8;
        }
#pragma unroll
        for (int v = 0; v < 2 * TNW; v++) {
            const int r = wave * (BN / 4) + v * 8 + lrow;
            if (BT) {  // whole k-rows past the end of K
                if (r >= ktail) *reinterpret_cast<h8 *>(Bs + (buf * kDmaK + r) * BN + lpos * 8) = zero8;
            } else if ((lpos ^ ((r >> 1) & 7)) * 8 >= ktail) {
                *reinterpret_cast<h8 *>(Bs + (buf * BN + r) * kDmaK + lpos * 8) = zero8;
            }
        }
    };
    // fragments of one 16-wide K slice: the token tiles and feature tiles of the wave's block.
    // Rows WM wm + 32 i + l32: the swizzle term (row >> 1) & 7 depends on the lane only.
    struct Frag { h8 x[TMW], w[TNW]; };
    const int swz = swz_of(l32);
    const _Float16 *a_rows = As + (wm * WM + l32) * KS, *b_rows = Bs + (wn * WN + l32) * KS;
    auto read_frag = [&](Frag &f, int buf, int ks) {
        const int chunk = ((ks * 2 + kg) ^ swz) * 8;
#pragma unroll
        for (int i = 0; i < TMW; i++)
            f.x[i] = *reinterpret_cast<const h8 *>(a_rows + buf * BM * KS + chunk + i * 32 * KS);
#pragma unroll
        for (int j = 0; j < TNW; j++) {
            if (BT) {
                const _Float16 *col = Bs + (buf * kDmaK + ks * 16 + kg * 8) * BN + wn * WN + l32;
#pragma unroll
                for (int e = 0; e < 8; e++) f.w[j][e] = col[e * BN];
            } else {
                f.w[j] = *reinterpret_cast<const h8 *>(b_rows + buf * BN * KS + chunk + j * 32 * KS);
            }
        }
    };
    auto multiply = [&](const Frag &f) {
#pragma unroll
        for (int i = 0; i < TMW; i++)
#pragma unroll
            for (int j = 0; j < TNW; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.w[j], f.x[i], acc[i][j], 0, 0, 0);
    };

    const int nstage = RAGGED ? (g.K + kDmaK - 1) / kDmaK : g.K / KS;
    // Stage s is multiplied from LDS buffer s % NBUF; the loads of kAhead later stages are in
    // flight meanwhile.  A direct-to-LDS load has landed when vmcnt says so, and vmcnt counts
    // in issue order: "stage s + 1 has landed" is "at most the loads of the stages after it
    // are outstanding".
    constexpr int kAhead = NBUF - 1;
    constexpr int kStageLoads = kWhole ? kLA + kLB : 2 * TMW + 2 * TNW;  // per wave
    auto wait_stages = [&](int later) {  // wait until at most `later` whole stages are outstanding
        if (later <= 0) __builtin_amdgcn_s_waitcnt(wait_vm(0));
        else if (later == 1) __builtin_amdgcn_s_waitcnt(wait_vm(kStageLoads));
        else __builtin_amdgcn_s_waitcnt(wait_vm(2 * kStageLoads));
    };
    // Workgroup barrier that orders LDS accesses only.  __syncthreads() carries a fence that
    // waits for every outstanding global access, the direct-to-LDS loads of the later stages
    // included, which is exactly what a deeper pipeline must not do; here this wave's LDS reads
    // are waited for, the barrier is passed, and the compiler moves no memory access across.
    auto lds_barrier = [] { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    // Order of issue inside one K slice.  The wave's instruction stream is the only thing that feeds the matrix
    // pipe of its SIMD, so the LDS reads of the next slice go between the MFMAs of the current one instead of in a
    // run in front of the MFMAs that need them (left alone the scheduler puts every read directly in front of its
    // first use and the pipe drains while it returns: 2 x 4 of 16 MFMAs apart, then a wait).  Where the slice is not
    // written out by hand (below), the pattern is given to the scheduler: kNM / kND MFMAs, one LDS read, ...
    constexpr int kNM = TMW * TNW, kND = TMW + TNW;
    constexpr int kSlices = KS / 16;                  // K slices (steps) of a stage
    constexpr int kLoadSteps = KS == 32 ? 2 : 1;      // steps of a stage that issue a share of a later stage's loads
    constexpr int kStepLoads = (kStageLoads + kLoadSteps - 1) / kLoadSteps;  // in the first such step; the rest in the second
    constexpr int kStepLoads2 = kStageLoads - kStepLoads;
    auto interleave = [&] {
        if constexpr (kNM >= kND) {
            constexpr int per = kNM / kND;  // MFMAs per LDS read
#pragma unroll
            for (int i = 0; i < kND; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, per, 0);  // MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);    // LDS read
            }
            __builtin_amdgcn_sched_group_barrier(0x008, kNM - per * kND, 0);
        }
    };
    // Whole tiles with at least as many MFMAs as fragments in a K slice: the slice is written out in the order it is
    // to be issued in, one MFMA at a time with a fence for the scheduler behind it: after every kNM / kND MFMAs
    // one fragment of the next slice is read from LDS, and `nload` loads of a later stage (from number `first`)
    // are dealt evenly between the MFMAs (the four waves of a workgroup issue their loads in the same slices, and
    // a wave whose load waits for the compute unit's one address unit issues no MFMA behind it).
    constexpr bool kManual = kWhole && kNM >= kND;
    static_assert(!kManual || ((kStepLoads % kNM == 0 || kNM % kStepLoads == 0) && (kLoadSteps == 1 || kStepLoads2 == kStepLoads)),
                  "the loads of a slice are dealt evenly to its MFMAs");
    auto step = [&](const Frag &fm, Frag &fr, int rbuf, int rks, int nload, int lbuf, int k_later, int first) {
        const int chunk = ((rks * 2 + kg) ^ swz) * 8;
        // more loads than MFMAs: nload / kNM behind every MFMA; fewer: one behind every (kNM / nload)-th
        const int lpm = nload >= kNM ? nload / kNM : 0;
        const int every = (nload > 0 && nload < kNM) ? kNM / nload : 1;
#pragma unroll
        for (int m = 0; m < kNM; m++) {
            const int i = m / TNW, j = m % TNW;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fm.w[j], fm.x[i], acc[i][j], 0, 0, 0);
            // fragment idx of the next slice behind MFMA (idx kNM) / kND: evenly over the slice
            const int idx = (m * kND + kNM - 1) / kNM;
            if (idx < kND && (idx * kNM) / kND == m) {
                if (idx < TMW) fr.x[idx] = *reinterpret_cast<const h8 *>(a_rows + rbuf * BM * KS + chunk + idx * 32 * KS);
                else fr.w[idx - TMW] = *reinterpret_cast<const h8 *>(b_rows + rbuf * BN * KS + chunk + (idx - TMW) * 32 * KS);
            }
            if (lpm > 0) load_part(lbuf, k_later, first + m * lpm, lpm);
            else if (nload > 0 && m % every == every / 2) load_part(lbuf, k_later, first + m / every, 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    Frag f0, f1;
    if constexpr (kWhole) {
#pragma unroll
        for (int p = 0; p < kAhead; p++) load_stage(p, min(p, nstage - 1) * KS);
        __builtin_amdgcn_s_waitcnt(wait_vm((kAhead - 1) * kStageLoads));  // stage 0 has landed
    } else {
#pragma unroll
        for (int p = 0; p < kAhead; p++)
            if (p < nstage) load_stage(p, p * kDmaK);
        wait_stages(min(kAhead, nstage) - 1);
    }
    if (RAGGED && nstage == 1 && ktail < kDmaK) zero_tail(0);
    lds_barrier();
    read_frag(f0, 0, 0);
    // One stage, with the matrix pipe fed across the barrier: every K slice is read from LDS
    // while the one before it is multiplied, the first slice of the next stage included, so the
    // barrier of the stage sits before its last slice.  The loads of stage s + kAhead are issued
    // in stage s into the buffer stage s - 1 was read from (its last readers passed
    // the previous barrier); stage s + 1 is waited for just before the barrier.  The fragment
    // read after the barrier of the last stage touches valid LDS and is never used; the loop
    // has a single exit (a second one in the middle makes the register allocator copy the
    // accumulators).
    int cur = 0;
    for (int s = 0; s < nstage; s++) {
        const int nxt = cur + 1 == NBUF ? 0 : cur + 1;
        const int prev = cur == 0 ? NBUF - 1 : cur - 1;
        const int k_later = min(s + kAhead, nstage - 1) * KS;  // whole tiles: past the end, the last stage again
        if constexpr (kManual) {
            step(f0, f1, cur, 1, kStepLoads, prev, k_later, 0);
            if constexpr (kSlices == 4) {
                step(f1, f0, cur, 2, 0, prev, k_later, 0);
                step(f0, f1, cur, 3, 0, prev, k_later, 0);
            }
            // outstanding at most: the stages after s + 1 as far as they have been issued
            __builtin_amdgcn_s_waitcnt(wait_vm((kAhead - 2) * kStageLoads + kStepLoads));
            if (RAGGED && s + 2 == nstage && ktail < kDmaK) zero_tail(nxt);
            lds_barrier();
            step(f1, f0, nxt, 0, kLoadSteps == 2 ? kStepLoads : 0, prev, k_later, kStepLoads);
        } else {
            if constexpr (kWhole) {
                read_frag(f1, cur, 1);
                load_part(prev, k_later, 0, kStepLoads);
            } else {
                if (s + kAhead < nstage) load_stage(prev, (s + kAhead) * kDmaK);
                read_frag(f1, cur, 1);
            }
            multiply(f0);
            interleave();
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (kSlices == 4) {
                read_frag(f0, cur, 2);
                multiply(f1);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
                read_frag(f1, cur, 3);
                multiply(f0);
                interleave();
                __builtin_amdgcn_sched_barrier(0);
            }
            // outstanding at most: the stages after s + 1 as far as they have been issued
            if constexpr (kWhole) __builtin_amdgcn_s_waitcnt(wait_vm((kAhead - 2) * kStageLoads + kStepLoads));
            else wait_stages(min(kAhead - 1, nstage - 2 - s));
            if (RAGGED && s + 2 == nstage && ktail < kDmaK) zero_tail(nxt);
            lds_barrier();
            read_frag(f0, nxt, 0);
            if constexpr (kWhole && kLoadSteps == 2) load_part(prev, k_later, kStepLoads, kStepLoads2);
            multiply(f1);
            interleave();
            __builtin_amdgcn_sched_barrier(0);
        }
        cur = nxt;
    }
    // the loads issued past the last stage have landed before the staging LDS is written again
    if constexpr (kWhole) __builtin_amdgcn_s_waitcnt(wait_vm(0));
    __syncthreads();  // the staging LDS becomes the transposition buffer of the epilogue

    // Epilogue.  acc[i][j][e] is token WM wm + 32 i + l32, feature WN wn + 32 j + 8 (e / 4) +
    // 4 kg + e % 4 of the tile: a lane holds 4 consecutive features of one row, 32 rows per
    // instruction.  Each wave passes its 32 x WN strips through its own LDS region and stores
    // rows of 2 WN contiguous bytes.
    constexpr int kEpLd = WN + 8;
    constexpr int kRowChunks = WN / 8;  // 16-byte chunks of a stored row: 4, 8 or 16
    _Float16 *ep = reinterpret_cast<_Float16 *>(dma_smem) + wave * 32 * kEpLd;
    const int nbase = n0 + wn * WN;
    // unconditional loads (from B when there is no bias) and a select: a load under a branch
    // is waited for on the spot
    const bool has_bias = g.bias != nullptr;
    const int32_t *col_idx = g.c_scatter ? g.c_scatter : g.bias_idx;  // bias index of result column n
    h4 bias4[TNW][4];
#pragma unroll
    for (int j = 0; j < TNW; j++)
#pragma unroll
        for (int q = 0; q < 4; q++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                int n = nbase + j * 32 + q * 8 + kg * 4 + e;
                if (RAGGED) n = min(n, g.N - 1);
                _Float16 bv;
                if (IDX) {
                    const int bi = col_idx ? col_idx[n] : n;
                    bv = (has_bias ? g.bias : g.B)[has_bias ? bi : 0];
                } else {
                    bv = (has_bias ? g.bias : g.B)[has_bias ? n : 0];
                }
                bias4[j][q][e] = has_bias ? bv : (_Float16)0.0f;
            }
    // Scattered columns are stored one 2-byte element per lane, kScLanes consecutive result
    // columns of one row per group of lanes: ascending c_scatter keeps those stores within a
    // few neighbouring sectors of the row of C.
    constexpr int kScLanes = WN < 64 ? WN : 64;  // lanes per row
    constexpr int kScCols = WN / kScLanes;       // column groups
    constexpr int kScRows = 64 / kScLanes;       // rows per instruction
    const bool scatter = IDX && g.c_scatter != nullptr;  // a gathered bias alone keeps the vector stores
    int scat[kScCols];
    if (IDX) {
#pragma unroll
        for (int e = 0; e < kScCols; e++) {
            const int n = nbase + e * kScLanes + lane % kScLanes;
            scat[e] = scatter ? g.c_scatter[RAGGED ? min(n, g.N - 1) : n] : n;
        }
    }
    const int act = g.act;
#pragma unroll
    for (int i = 0; i < TMW; i++) {
#pragma unroll
        for (int j = 0; j < TNW; j++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                h4 o;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    o[e] = (_Float16)apply_act(acc[i][j][q * 4 + e] + (float)bias4[j][q][e], act);
                *reinterpret_cast<h4 *>(ep + l32 * kEpLd + j * 32 + q * 8 + kg * 4) = o;
            }
        __syncthreads();
        if (scatter) {
#pragma unroll
            for (int v = 0; v < 32 / kScRows; v++) {
                const int r = v * kScRows + lane / kScLanes;
                const int m = m0 + wm * WM + i * 32 + r;
                _Float16 *crow = g.C + (size_t)m * g.ldc;
#pragma unroll
                for (int e = 0; e < kScCols; e++) {
                    const bool inside = !RAGGED || (m < g.M && nbase + e * kScLanes + lane % kScLanes < g.N);
                    if (inside) crow[scat[e]] = ep[r * kEpLd + e * kScLanes + lane % kScLanes];
                }
            }
        } else {
#pragma unroll
            for (int v = 0; v < 32 * kRowChunks / 64; v++) {
                const int idx = lane + v * 64, r = idx / kRowChunks, c = idx % kRowChunks;
                const h8 val = *reinterpret_cast<const h8 *>(ep + r * kEpLd + c * 8);
                const int m = m0 + wm * WM + i * 32 + r;
                // N is a multiple of 16: a chunk of 8 columns is inside or outside as a whole
                if (!RAGGED || (m < g.M && nbase + c * 8 < g.N))
                    *reinterpret_cast<h8 *>(g.C + (size_t)m * g.ldc + nbase + c * 8) = val;
            }
        }
        __syncthreads();
    }
}

// Tile choice, from measurements on dense Linears of 1024..16384 rows: a larger tile halves the
// operand traffic from the L2 per flop but needs enough workgroups to keep every compute unit
// busy through whole rounds (a 256 x 256 workgroup owns its compute unit; two 128 x 128, three
// 128 x 64 or five 64 x 64 ones share it and cover each other's prologue and epilogue).
// 256 x 128 tiles were measured and never won.
struct DmaTile { int tmw, tnw, nbuf; bool ragged; };
static bool pick_dma_tile(const GemmArgs &g, int batch, bool trans_b, DmaTile *out) {
    const bool ragged = g.M % 64 || g.N % 64 || g.K % kDmaK || batch != 1 || !trans_b;
    if (ragged) {
        // 64 x 64 tiles with the edges clamped and masked; large ragged problems are left to the
        // 128 x 128 tiles of the register-staged kernel
        const long long w = (long long)((g.M + 63) / 64) * ((g.N + 63) / 64) * batch;
        if (g.M % 16 || g.N % 16 || g.K % 16) return false;
        if (batch == 1 && trans_b) {
            // enough workgroups for the larger tiles, as for whole tiles below (a row- or column-pruned
            // Linear keeps any multiple of 16 features: 2048 x 768 -> 2928 26.7 -> 21.4 us with 128 x 64 tiles)
            const long long m128 = (g.M + 127) / 128;
            if ((long long)((g.M + 255) / 256) * ((g.N + 255) / 256) >= 1024) { *out = {4, 4, 2, true}; return true; }
            if (m128 * ((g.N + 127) / 128) >= 512) { *out = {2, 2, 2, true}; return true; }
            if (m128 * ((g.N + 63) / 64) >= 512) { *out = {2, 1, 2, true}; return true; }
        }
        if (w > 1536) return false;
        // Batched problems and B stored k-major run on this instantiation too, where they are
        // bound by the latency of a long K loop in few workgroups (the stacked VO product of the
        // pre-computed-VO attention: 32 -> 22 us); gathering the k-major fragments with 2-byte LDS
        // reads costs more than it saves elsewhere (Linear_VO 28 -> 78 us), those stay on the
        // register-staged kernel.
        if ((batch != 1 || !trans_b) && (w > 256 || g.K / kDmaK < 16)) return false;
        *out = {1, 1, (w <= 512 && g.K / kDmaK >= 24) ? 3 : 2, true};  // third buffer: as below
        return true;
    }
    auto wgs = [&](int tmw, int tnw) -> long long {
        const int bm = 64 * tmw, bn = 64 * tnw;
        return (g.M % bm || g.N % bn) ? 0 : (long long)(g.M / bm) * (g.N / bn);
    };
    const long long w44 = wgs(4, 4), w11 = wgs(1, 1);
    // whole rounds of one workgroup per compute unit, or so many that the last one hardly counts
    if (w44 >= 256 && (w44 % 256 == 0 || w44 >= 1024)) { *out = {4, 4, 2, false}; return true; }
    if (wgs(2, 2) >= 512) { *out = {2, 2, 2, false}; return true; }
    if (wgs(2, 1) >= 512) { *out = {2, 1, 2, false}; return true; }
    // few workgroups with a long K loop are bound by the latency of a stage: a third buffer keeps
    // two stages in flight (2048 x 3072 -> 768: 29.5 -> 24.7 us; from 12 stages on it still gives
    // 3-5 %: 2048 x 768 -> 768 9.6 -> 9.1 us); elsewhere it only costs occupancy
    *out = {1, 1, (w11 <= 512 && g.K / kDmaK >= 12) ? 3 : 2, false};
    return true;
}

// The kernel moves 16 bytes at a time: operands and result 16-byte aligned, leading dimensions
// multiples of 8.
bool gemm_dma_applies(const GemmArgs &g, int batch, bool trans_b) {
    DmaTile t;
    const auto misaligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) != 0; };
    if (batch < 1 || batch > 65535 || g.a_gather || g.M <= 0) return false;
    if (g.lda % 8 || g.ldb % 8 || g.ldc % 8 || misaligned(g.A) || misaligned(g.B) || misaligned(g.C)) return false;
    if (g.lda > (1 << 21) || g.ldb > (1 << 21)) return false;  // a tile's rows are addressed with 32-bit byte offsets
    if (batch > 1 && ((g.sAo | g.sAi | g.sBo | g.sBi | g.sCo | g.sCi) & 7)) return false;  // every problem aligned
    return pick_dma_tile(g, batch, trans_b, &t);
}

template <int TMW, int TNW, int NBUF, bool IDX, bool RAGGED, bool BT = false, int KS = kDmaK, int NWN = 2>
static int launch_dma_variant(const GemmArgs &g, int batch, hipStream_t stream) {
    constexpr int BM = 64 * TMW, BN = 32 * NWN * TNW;
    constexpr size_t lds = dma_lds_bytes(TMW, TNW, NBUF, KS, NWN);
    const int tiles_m = (g.M + BM - 1) / BM, tiles_n = (g.N + BN - 1) / BN;
    // groups of group_rows x 8 tiles are dealt to the XCDs in turn: the size (32, 16 or 8 tiles) that leaves the
    // fullest XCD the fewest tiles, the larger on a tie
    const long long total = (long long)tiles_m * tiles_n;
    int sbm = kSbM;
    long long best = -1;
    for (int cand = kSbM; cand >= 1; cand /= 2) {
        const long long gsz = (long long)cand * kSbN, ngr = (total + gsz - 1) / gsz;
        const long long most = (ngr + kDmaXcds - 1) / kDmaXcds * gsz;
        if (best < 0 || most < best) { best = most; sbm = cand; }
    }
    const long long groups = (total + sbm * kSbN - 1) / (sbm * kSbN);
    const long long rounds = (groups + kDmaXcds - 1) / kDmaXcds;
    const dim3 grid((unsigned)(rounds * kDmaXcds * sbm * kSbN), (unsigned)batch);
    GemmArgs ga = g;
    ga.group_rows = sbm;
    auto kernel = gemm_f16_dma_kernel<TMW, TNW, NBUF, IDX, RAGGED, BT, KS, NWN>;
    static bool raised = false;  // more than 64 KB of dynamic LDS needs the attribute, once per kernel
    if (!raised) {
        ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    kernel<<<grid, 128 * NWN, lds, stream>>>(ga);
    return check_launch("gemm_f16_dma_kernel");
}

template <int TMW, int TNW, int NBUF, bool RAGGED = false, bool BT = false, int KS = kDmaK, int NWN = 2>
static int launch_dma_tile(const GemmArgs &g, int batch, hipStream_t stream) {
    return (g.c_scatter || g.bias_idx) ? launch_dma_variant<TMW, TNW, NBUF, true, RAGGED, BT, KS, NWN>(g, batch, stream)
                                       : launch_dma_variant<TMW, TNW, NBUF, false, RAGGED, BT, KS, NWN>(g, batch, stream);
}

int launch_gemm_dma(const GemmArgs &g, int batch, bool trans_b, hipStream_t stream) {
    DmaTile t{};
    if (!pick_dma_tile(g, batch, trans_b, &t)) return ET_ERR_UNSUPPORTED;
    if (t.ragged) {
        if (!trans_b)
            return t.nbuf == 3 ? launch_dma_tile<1, 1, 3, true, true>(g, batch, stream)
                               : launch_dma_tile<1, 1, 2, true, true>(g, batch, stream);
        if (t.tmw == 4) return launch_dma_tile<4, 4, 2, true>(g, batch, stream);
        if (t.tmw == 2) return t.tnw == 2 ? launch_dma_tile<2, 2, 2, true>(g, batch, stream)
                                          : launch_dma_tile<2, 1, 2, true>(g, batch, stream);
        return t.nbuf == 3 ? launch_dma_tile<1, 1, 3, true>(g, batch, stream)
                           : launch_dma_tile<1, 1, 2, true>(g, batch, stream);
    }
    switch (t.tmw * 100 + t.tnw * 10 + t.nbuf) {
        // 256 x 256: eight waves of 128 x 64, half stages through four buffers (four waves of 128 x 128 in the same
        // LDS: 0.5-2 % slower)
        case 442: return launch_dma_tile<4, 2, 4, false, false, 32, 4>(g, 1, stream);
        case 222: return launch_dma_tile<2, 2, 2>(g, 1, stream);
        case 212: return launch_dma_tile<2, 1, 2>(g, 1, stream);
        case 112: return launch_dma_tile<1, 1, 2>(g, 1, stream);
        case 113: return launch_dma_tile<1, 1, 3>(g, 1, stream);
        default: return ET_ERR_UNSUPPORTED;
    }
}

}  // namespace et
