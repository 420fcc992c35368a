// On-chip attention over a pre-computed VO projection (E.T.'s FusedAttention with the probabilities
// kept in registers): kernel, launch forms and the C entry point.  The fused Q.K^T / softmax / P.V
// kernel is in attention.hip, the forms that write the probabilities to memory in attention_vo.hip.
#include <math.h>

#include "common.hip.h"

namespace et {

constexpr int kXcds = 8;  // accelerator dies, each with a private L2
constexpr float kLog2e = 1.4426950408889634f;

// On-the-fly attention over a pre-computed VO projection (Fused_attention/Fused_attention.cu:10-116):
//     out[q][n] = sum_h softmax_h(q, :) . (VO_h[:, n] + b_VO,h[n]) + b_O[n]
// The probabilities never leave the chip, and no operand of the two products is staged for more
// than one wave: the projection is handed over key-contiguous, VOt[b][h][n][key], so that a lane's
// 8 values of a VO^T fragment are one 16-byte load, and a K fragment is a 16-byte load of one K row
// (the forms with a wave per head load whole rows instead and turn them into fragments through a
// wave-private piece of LDS, see kStaged).  The
// rows of a score tile are dealt to the keys so that the 8 probabilities a lane holds after the
// softmax (rows 4g..4g+3 of two tiles) are the keys 8g..8g+7 of a 32-key group, the order the
// VO^T fragment has in memory.
//
// A workgroup owns 16 or 32 queries of one sequence and 64 output columns; its waves take the
// heads h = wave, wave + NW, ... and never wait for one another while they work: the K fragments
// of the next (head, key block) are requested as soon as the scores of the current one are
// formed, the VO^T fragments before them.  At the end the waves add their fp32 sums through LDS
// and each output element is written once, by one lane (the reference adds fp16 atomics of all
// heads into an output it never clears).  The per-head bias of the projection is added here, in
// fp32, as the sum over heads: the probabilities of a row add up to one.  A query without any
// live key gets b_O alone.
struct MhaVoArgs {
    const _Float16 *Q, *K;      // [B*S x ld], head h in columns [h*hd, (h+1)*hd)
    const _Float16 *VOt;        // [B][nh][N][S]
    const _Float16 *bias_vo;    // [nh][N] or nullptr
    _Float16 *out;              // [B*S x out_width]
    const _Float16 *bias_o;     // [out_width] or nullptr
    const int32_t *col_scatter; // [N] output column of each VO column, or nullptr (identity)
    const _Float16 *mask;       // [S x S] additive or nullptr
    const int32_t *lens;        // [B] or nullptr
    int ldq, ldk, S, nh, hd, N, out_width, B;
    float scale_log2e;
    int causal;
};

constexpr int kVoCols = 64;  // output columns of a workgroup

// NW waves share the heads of a workgroup (wave w takes h = w, w + NW, ...), QT 16-query tiles per
// wave.  One head per wave and QT = 1 is the latency form (12 waves for BERT-base: every head's
// chain of load, scores, softmax and product runs at once); fewer waves with QT = 2 reuse each
// fragment for two query tiles and halve the operand traffic per query.
// VC: output columns of a workgroup, 64 or 32
template <int HD, int KBLK, bool MASKED, int NW, int QT, bool PF, int VC>
__global__ __launch_bounds__(64 * NW) void mha_vo_otf_kernel(const MhaVoArgs a) {
    constexpr int KS = HD / 32;        // K=32 MFMA steps over the head dimension
    constexpr int DB = VC / 16;   // 16-wide blocks of the output columns
    constexpr int NKB = KBLK / 16;     // score tiles of a key block
    constexpr int kStripQ = 16 * QT;
    constexpr int kTiles = QT * DB;
    __shared__ float red[NW][kTiles][4][64];
    __shared__ int alive[kStripQ];
    // Fragments through LDS (heads of 64 and 128).  A fragment load straight from memory touches 16
    // rows with 64 bytes each: half a cache line per row, and the memory pipeline of a CU passes such
    // an instruction at the cost of 16 whole lines (a wave per head, all heads at once, spent 6.5 us of
    // a 15 us launch waiting for K that way).  Instead a load instruction takes whole rows — 8 rows of
    // 128 bytes or 4 of 256 — and the wave turns 32 keys (K) or 16 columns (VO^T) at a time into
    // fragments through a piece of LDS of its own: written as loaded, read back in fragment order, the
    // 16-byte chunks of a row XOR-swizzled so that both directions spread over all banks.  One wave's
    // LDS instructions execute in order, so the piece is reused without a barrier.
    // (The large-grid forms, which prefetch the next block's fragments while they multiply, keep the
    // direct fragment loads: there the chip is full, the loads hide behind arithmetic and the LDS
    // round trip only costs — 40.3 against 37.9 us at eight sequences.)
    constexpr bool kStaged = HD >= 64 && !PF;
    constexpr int kCPR = HD / 8;                   // 16-byte chunks of a K row
    constexpr int kRPI = 64 / kCPR;                // K rows per load instruction
    constexpr int kNI = kStaged ? KBLK / kRPI : 1; // load instructions per key block
    constexpr int kPI = 32 / kRPI;                 // ... per 32-key piece
    constexpr int kCPV = KBLK / 8;                 // 16-byte chunks of a VO^T row inside a key block
    constexpr int kRPV = 64 / kCPV;                // VO^T rows per load instruction
    constexpr int kNIV = kStaged ? VC / kRPV : 1;
    constexpr int kPIV = 16 / kRPV;                // ... per 16-column piece
    constexpr int kPieceHalfs = kStaged ? (32 * HD > 16 * KBLK ? 32 * HD : 16 * KBLK) : 8;
    __shared__ __align__(16) _Float16 piece_lds[NW][kPieceHalfs];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int S = a.S;
    // workgroup id -> (sequence, column slice, query strip): the strips of one (sequence, slice)
    // read the same VO^T rows and get ids that land on one XCD
    const int qstrips = (S + kStripQ - 1) / kStripQ;
    const int nslices = (a.N + VC - 1) / VC;
    const int xcd = blockIdx.x % kXcds, k_in_xcd = blockIdx.x / kXcds;
    const int unit = xcd + kXcds * (k_in_xcd / qstrips);
    if (unit >= a.B * nslices) return;  // padding of the last round (whole workgroup)
    const int qstrip = k_in_xcd % qstrips;
    const int b = unit / nslices, slice = unit - b * nslices;
    const size_t row0 = (size_t)b * S;
    int q[QT];
    bool q_ok[QT];
#pragma unroll
    for (int t = 0; t < QT; t++) {
        q[t] = qstrip * kStripQ + t * 16 + r16;
        q_ok[t] = q[t] < S;
    }
    int klimit = S;
    if (a.lens) klimit = min(S, max(a.lens[b], 0));
    if (a.causal) klimit = min(klimit, (qstrip + 1) * kStripQ);
    const int hd = a.hd;
    const int n0 = slice * VC;
    const int nlive = min(VC, a.N - n0);  // live columns of the slice (a multiple of 16)
    const int nblocks = (klimit + KBLK - 1) / KBLK;

    // No load below is followed by a select in its own basic block: the compiler would wait for
    // the load there.  Addresses are clamped into the operand instead (32-bit element offsets
    // from a wave-uniform base); what a clamped load brings is finite and meets a zero (Q columns
    // past the head are zeroed when the fragments are taken into use), a probability of exactly
    // zero (keys past the limit), or is never stored (columns past the slice).
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const _Float16 *q_seq = a.Q + row0 * a.ldq;
    const _Float16 *k_seq = a.K + row0 * a.ldk;
    unsigned qoff[QT][KS], kcol[KS], vrow[DB];
    bool col_ok[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        col_ok[ks] = 32 * ks + 8 * g < hd;
        kcol[ks] = col_ok[ks] ? 32 * ks + 8 * g : 0;
#pragma unroll
        for (int t = 0; t < QT; t++) qoff[t][ks] = (unsigned)(q_ok[t] ? q[t] : 0) * (unsigned)a.ldq + kcol[ks];
    }
#pragma unroll
    for (int d = 0; d < DB; d++) vrow[d] = (unsigned)(16 * d < nlive ? 16 * d + r16 : 0) * (unsigned)S;

    h8 qf[QT][KS], qn[PF ? QT : 1][PF ? KS : 1];  // qn: the next head's Q, requested while this head is multiplied
    h8 kf[NKB][KS];
    // Q fragments: B operand, lane supplies Q[q][32ks + 8g .. +7]
    auto load_q = [&](int h) {
        const _Float16 *qh = q_seq + h * hd;
#pragma unroll
        for (int t = 0; t < QT; t++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                if constexpr (PF) qn[t][ks] = *reinterpret_cast<const h8 *>(qh + qoff[t][ks]);
                else qf[t][ks] = *reinterpret_cast<const h8 *>(qh + qoff[t][ks]);  // taken into use at once
            }
    };
    auto take_q = [&]() {
#pragma unroll
        for (int t = 0; t < QT; t++)
#pragma unroll
            for (int ks = 0; ks < KS; ks++) qf[t][ks] = (q_ok[t] && col_ok[ks]) ? (PF ? qn[PF ? t : 0][PF ? ks : 0] : qf[t][ks]) : zero8;
    };
    // K fragments: A operand of tile kb, row r16 of the tile is key 32(kb/2) + 8(r16/4) + 4(kb%2) + r16%4
    h8 kraw[kNI];
    _Float16 *piece = piece_lds[wave];
    const int k_row = lane / kCPR, k_chunk = lane % kCPR;       // staged form: this lane's place in a load instruction
    const unsigned k_col = k_chunk * 8 < hd ? k_chunk * 8 : 0;  // (columns past the head meet zeros of Q)
    // Places in the piece, in halfs.  A row's 16-byte chunks are XORed with three bits that differ
    // over the 16 rows of a score tile: key & 3, and bit 3 of the key (inside the piece).  For the
    // writer bit 3 depends on the instruction only, for the reader on nothing but the lane, so two
    // bases each and compile-time offsets address everything (registers are what this form lacks).
    int kw[2], kr[2];
#pragma unroll
    for (int p = 0; p < 2; p++) {
        kw[p] = (k_row * kCPR + (k_chunk ^ ((k_row & 3) | (p << 2)))) * 8;
        const int key = 8 * (r16 >> 2) + (r16 & 3);  // first tile of the piece; the second is 4 keys on
        kr[p] = (key * kCPR + ((4 * p + g) ^ ((r16 & 3) | (((r16 >> 2) & 1) << 2)))) * 8;
    }
    static_assert(!kStaged || kRPI == 4 || kRPI == 8, "rows per instruction");
    // VO^T: a row's chunks are XORed with row & 7 (the 16 rows of a piece are the 16 lanes of a fragment read)
    const int v_row = lane / kCPV, v_chunk = lane % kCPV;
    int vw[2], vr[2];
#pragma unroll
    for (int p = 0; p < 2; p++) {
        vw[p] = (v_row * kCPV + (v_chunk ^ ((v_row + 4 * p) & 7))) * 8;
        vr[p] = (r16 * kCPV + ((4 * p + g) ^ (r16 & 7))) * 8;
    }
    static_assert(!kStaged || kRPV == 4 || kRPV == 8, "rows per instruction");
    auto load_k = [&](int h, int k0) {
        const _Float16 *kh = k_seq + h * hd;
        if constexpr (kStaged) {
#pragma unroll
            for (int i = 0; i < kNI; i++) {
                const int key = min(k0 + i * kRPI + k_row, klimit - 1);
                kraw[i] = *reinterpret_cast<const h8 *>(kh + ((unsigned)key * (unsigned)a.ldk + k_col));
            }
            return;
        }
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) {
            const int key = min(k0 + 32 * (kb >> 1) + 8 * (r16 >> 2) + 4 * (kb & 1) + (r16 & 3), klimit - 1);
            const unsigned krow = (unsigned)key * (unsigned)a.ldk;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) kf[kb][ks] = *reinterpret_cast<const h8 *>(kh + (krow + kcol[ks]));
        }
    };

    int h = wave, blk = 0;
    bool have = h < a.nh && nblocks > 0;
    if (PF && have) {
        load_q(h);
        load_k(h, 0);
        take_q();
    }
    // The sum over this wave's heads of the normalised products: in registers, or (the forms with a wave
    // per head, which have none to spare) in the wave's rows of `red`, which the reduction at the end
    // reads anyway.
    constexpr bool kAccLds = !PF;
    f4 acc[kAccLds ? 1 : QT][kAccLds ? 1 : DB];
    if constexpr (!kAccLds) {
#pragma unroll
        for (int t = 0; t < QT; t++)
#pragma unroll
            for (int d = 0; d < DB; d++) acc[t][d] = f4{0.f, 0.f, 0.f, 0.f};
    }
    f4 o[QT][DB];
    float m_run[QT], l_part[QT];
#pragma unroll
    for (int t = 0; t < QT; t++) {
        m_run[t] = -INFINITY;
        l_part[t] = 0.0f;
#pragma unroll
        for (int d = 0; d < DB; d++) {
            o[t][d] = f4{0.f, 0.f, 0.f, 0.f};
        }
    }
    bool first_head = true;

    while (have) {  // wave-uniform
        const int k0 = blk * KBLK;
        if (!PF) {  // without the prefetch: this block's K (and the head's Q) now, VO^T once the scores stand
            load_k(h, k0);
            if (blk == 0) {
                load_q(h);
                take_q();
            }
        }
        // ---- VO^T fragments of this block: lane supplies VOt[n0 + 16d + r16][k0 + 32 s2 + 8g .. +7]
        h8 vf[NKB / 2][DB];
        h8 vraw[kNIV];
        auto load_v = [&]() {
            const _Float16 *vo_h = a.VOt + ((size_t)(b * a.nh + h) * a.N + n0) * S;
            if constexpr (kStaged) {
                const int key = k0 + (lane % kCPV) * 8;
                const unsigned kc = key < klimit ? key : 0;
#pragma unroll
                for (int i = 0; i < kNIV; i++) {
                    const int n = i * kRPV + lane / kCPV;  // column of the slice = row of VO^T
                    vraw[i] = *reinterpret_cast<const h8 *>(vo_h + ((unsigned)(n < nlive ? n : 0) * (unsigned)S + kc));
                }
                return;
            }
#pragma unroll
            for (int s2 = 0; s2 < NKB / 2; s2++) {
                const int key = k0 + 32 * s2 + 8 * g;
                const unsigned kc = key < klimit ? key : 0;
#pragma unroll
                for (int d = 0; d < DB; d++) vf[s2][d] = *reinterpret_cast<const h8 *>(vo_h + (vrow[d] + kc));
            }
        };
        if (PF) load_v();
        // additive mask of the block: lane holds keys key0..key0+3 of query q[t] per score tile
        h4 mraw[MASKED ? QT : 1][MASKED ? NKB : 1];
        if (MASKED) {
#pragma unroll
            for (int t = 0; t < QT; t++)
#pragma unroll
                for (int kb = 0; kb < NKB; kb++) {
                    const int key0 = k0 + 32 * (kb >> 1) + 8 * g + 4 * (kb & 1);
                    const bool live = q_ok[t] && key0 < S;
                    mraw[MASKED ? t : 0][MASKED ? kb : 0] =
                        *reinterpret_cast<const h4 *>(a.mask + (live ? (size_t)q[t] * S + key0 : 0));
                }
        }
        // ---- scores S^T = K Q^T
        f4 sc[QT][NKB];
        if constexpr (kStaged) {
            // the rows loaded by load_k become fragments 32 keys (two score tiles) at a time and are
            // multiplied at once, so that only two tiles' fragments are held in registers
#pragma unroll
            for (int s2 = 0; s2 < KBLK / 32; s2++) {
#pragma unroll
                for (int j = 0; j < kPI; j++)  // rows j * kRPI + k_row of the piece
                    *reinterpret_cast<h8 *>(piece + kw[((j * kRPI) >> 3) & 1] + j * kRPI * kCPR * 8) = kraw[s2 * kPI + j];
#pragma unroll
                for (int t2 = 0; t2 < 2; t2++) {
                    const int kb = 2 * s2 + t2;
                    h8 kfr[KS];
#pragma unroll
                    for (int ks = 0; ks < KS; ks++)  // row 8 (r16 / 4) + 4 t2 + r16 % 4, chunk 4 ks + g
                        kfr[ks] = *reinterpret_cast<const h8 *>(piece + kr[ks & 1] + (4 * t2 * kCPR + 8 * (ks >> 1)) * 8);
#pragma unroll
                    for (int t = 0; t < QT; t++) {
                        sc[t][kb] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int ks = 0; ks < KS; ks++)
                            sc[t][kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kfr[ks], qf[t][ks], sc[t][kb], 0, 0, 0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);  // pieces one after the other: fragments of one piece in registers at a time
            }
        } else {
#pragma unroll
            for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                for (int t = 0; t < QT; t++) {
                    sc[t][kb] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < KS; ks++)
                        sc[t][kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf[kb][ks], qf[t][ks], sc[t][kb], 0, 0, 0);
                }
        }
        // ---- request the next (head, block) of this wave
        int h_next = h, blk_next = blk + 1;
        if (blk_next == nblocks) {
            blk_next = 0;
            h_next = h + NW;
        }
        const bool more = h_next < a.nh;
        if (PF && more) {  // wave-uniform; nothing in this block uses what it loads
            load_k(h_next, blk_next * KBLK);
            if (blk_next == 0) load_q(h_next);
        }
        if (!PF) load_v();
        // ---- scale, mask, running max; probabilities
        h8 pf[QT][NKB / 2];
#pragma unroll
        for (int t = 0; t < QT; t++) {
            float m_blk = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < NKB; kb++) {
                const int key0 = k0 + 32 * (kb >> 1) + 8 * g + 4 * (kb & 1);
                float mk[4] = {0.f, 0.f, 0.f, 0.f};
                if (MASKED) {
                    const bool live = q_ok[t] && key0 < S;
#pragma unroll
                    for (int j = 0; j < 4; j++) mk[j] = live ? (float)mraw[MASKED ? t : 0][MASKED ? kb : 0][j] * kLog2e : 0.0f;
                }
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int key = key0 + j;
                    float sv = sc[t][kb][j] * a.scale_log2e + mk[j];
                    if (key >= klimit || (a.causal && key > q[t])) sv = -INFINITY;
                    sc[t][kb][j] = sv;
                    m_blk = fmaxf(m_blk, sv);
                }
            }
            m_blk = rows_max(m_blk);
            const float m_new = fmaxf(m_run[t], m_blk);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run[t] - m_use);
            m_run[t] = m_new;
            if (!__all(alpha == 1.0f)) {
                l_part[t] *= alpha;
#pragma unroll
                for (int d = 0; d < DB; d++) o[t][d] *= alpha;
            }
            const h2 ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
            for (int s2 = 0; s2 < NKB / 2; s2++)
#pragma unroll
                for (int pr = 0; pr < 4; pr++) {
                    const int kb = 2 * s2 + (pr >> 1), j = 2 * (pr & 1);
                    const h2 hp = {(_Float16)__builtin_amdgcn_exp2f(sc[t][kb][j] - m_use),
                                   (_Float16)__builtin_amdgcn_exp2f(sc[t][kb][j + 1] - m_use)};
                    l_part[t] = __builtin_amdgcn_fdot2(hp, ones, l_part[t], false);
                    pf[t][s2][2 * pr] = hp[0];
                    pf[t][s2][2 * pr + 1] = hp[1];
                }
        }
        // ---- O^T += VO^T P^T
        if constexpr (kStaged) {
            // the rows loaded by load_v become fragments 16 columns at a time and are multiplied at once
#pragma unroll
            for (int d = 0; d < DB; d++) {
#pragma unroll
                for (int j = 0; j < kPIV; j++)  // rows j * kRPV + v_row of the piece
                    *reinterpret_cast<h8 *>(piece + vw[(j * kRPV >> 2) & 1] + j * kRPV * kCPV * 8) = vraw[d * kPIV + j];
                h8 vfr[NKB / 2];
#pragma unroll
                for (int s2 = 0; s2 < NKB / 2; s2++)  // row r16, chunk 4 s2 + g
                    vfr[s2] = *reinterpret_cast<const h8 *>(piece + vr[s2 & 1] + 8 * (s2 >> 1) * 8);
#pragma unroll
                for (int s2 = 0; s2 < NKB / 2; s2++) {
                    if (k0 + 32 * s2 >= klimit) continue;  // wave-uniform
#pragma unroll
                    for (int t = 0; t < QT; t++)
                        o[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vfr[s2], pf[t][s2], o[t][d], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int s2 = 0; s2 < NKB / 2; s2++) {
                if (k0 + 32 * s2 >= klimit) continue;  // wave-uniform
#pragma unroll
                for (int d = 0; d < DB; d++)
#pragma unroll
                    for (int t = 0; t < QT; t++)
                        o[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[s2][d], pf[t][s2], o[t][d], 0, 0, 0);
            }
        }
        // ---- the head is done: add its normalised product, start the next head
        if (blk_next == 0) {
#pragma unroll
            for (int t = 0; t < QT; t++) {
                const float l = rows_sum(l_part[t]);
                const float inv = l > 0.0f ? 1.0f / l : 0.0f;
                if (first_head && wave == 0 && g == 0) {
                    int at = t * 16 + r16;
                    asm volatile("" : "+v"(at));  // formed here: hoisted out of the loop, the address is a register spilled
                    alive[at] = l > 0.0f;  // taken from one head: mask and lens are shared by all heads of a query
                }
#pragma unroll
                for (int d = 0; d < DB; d++) {
                    if constexpr (kAccLds) {
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            float v = o[t][d][j] * inv;
                            if (!first_head) v += red[wave][t * DB + d][j][lane];
                            red[wave][t * DB + d][j][lane] = v;
                        }
                    } else {
                        acc[kAccLds ? 0 : t][kAccLds ? 0 : d] += o[t][d] * inv;
                    }
                    o[t][d] = f4{0.f, 0.f, 0.f, 0.f};
                }
                m_run[t] = -INFINITY;
                l_part[t] = 0.0f;
            }
            if (PF && more) take_q();
            first_head = false;
        }
        h = h_next;
        blk = blk_next;
        have = more;
    }
    if (nblocks == 0 && threadIdx.x < kStripQ) alive[threadIdx.x] = 0;

    // ---- add the waves' sums; wave w finishes the tiles w, w + NW, ...
    if constexpr (kAccLds) {
        if (first_head) {  // a wave without a head of its own (wave-uniform)
#pragma unroll
            for (int tile = 0; tile < kTiles; tile++)
#pragma unroll
                for (int j = 0; j < 4; j++) red[wave][tile][j][lane] = 0.0f;
        }
    } else {
#pragma unroll
        for (int t = 0; t < QT; t++)
#pragma unroll
            for (int d = 0; d < DB; d++)
#pragma unroll
                for (int j = 0; j < 4; j++) red[wave][t * DB + d][j][lane] = acc[kAccLds ? 0 : t][kAccLds ? 0 : d][j];
    }
    __syncthreads();
    for (int tile = wave; tile < kTiles; tile += NW) {
        const int t = tile / DB, d = tile - t * DB;
        const int qq = qstrip * kStripQ + t * 16 + r16;
        if (16 * d >= nlive || qq >= S) continue;
        float y[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            y[j] = 0.0f;
#pragma unroll
            for (int w = 0; w < NW; w++) y[j] += red[w][tile][j][lane];
        }
        const int n = n0 + 16 * d + 4 * g;
        if (a.bias_vo && alive[t * 16 + r16]) {
            for (int hh = 0; hh < a.nh; hh++) {
                const h4 bv = *reinterpret_cast<const h4 *>(a.bias_vo + (size_t)hh * a.N + n);
#pragma unroll
                for (int j = 0; j < 4; j++) y[j] += (float)bv[j];
            }
        }
        _Float16 *orow = a.out + (row0 + qq) * a.out_width;
        if (a.col_scatter) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int c = a.col_scatter[n + j];
                orow[c] = (_Float16)(y[j] + (a.bias_o ? (float)a.bias_o[c] : 0.0f));
            }
        } else {
            h4 bo = {0, 0, 0, 0};
            if (a.bias_o) bo = *reinterpret_cast<const h4 *>(a.bias_o + n);
            h4 o4;
#pragma unroll
            for (int j = 0; j < 4; j++) o4[j] = (_Float16)(y[j] + (float)bo[j]);
            *reinterpret_cast<h4 *>(orow + n) = o4;
        }
    }
}

template <int HD, int KBLK, int NW, int QT, bool PF, int VC = kVoCols>
static int launch_mha_vo_otf_form(const MhaVoArgs &args, hipStream_t stream) {
    constexpr int kStripQ = 16 * QT;
    const int qstrips = (args.S + kStripQ - 1) / kStripQ, nslices = (args.N + VC - 1) / VC;
    const long long rounds = ((long long)args.B * nslices + kXcds - 1) / kXcds;
    const dim3 grid((unsigned)(rounds * kXcds * qstrips));
    if constexpr (NW <= 8) {  // the 12-wave forms have no masked variant (168 registers do not hold it)
        if (args.mask) {
            mha_vo_otf_kernel<HD, KBLK, true, NW, QT, PF, VC><<<grid, 64 * NW, 0, stream>>>(args);
            return check_launch("mha_vo_otf_kernel");
        }
    }
    mha_vo_otf_kernel<HD, KBLK, false, NW, QT, PF, VC><<<grid, 64 * NW, 0, stream>>>(args);
    return check_launch("mha_vo_otf_kernel");
}

// A workgroup reads the K of all heads and its VO^T slice of all heads (392 KB at 128 keys, 12 heads
// of 64, 64 columns), and a CU takes in 60 to 80 GB/s: that, not arithmetic, sets the time of a small
// grid, and a wave per head (no wave walks several heads) is the fastest form while the grid is a few
// hundred workgroups; a grid that leaves more than half of the CUs idle gives each workgroup 32
// columns instead of 64 (three quarters of the bytes per CU on twice the CUs).  Beyond that the chip
// is full either way and the form that reuses each fragment for two query tiles moves half the
// bytes per query.
template <int HD, int KBLK> static int launch_mha_vo_otf(const MhaVoArgs &args, hipStream_t stream) {
    const long long small_grid = (long long)args.B * ((args.N + kVoCols - 1) / kVoCols) * ((args.S + 15) / 16);
    if (small_grid > 512) return launch_mha_vo_otf_form<HD, KBLK, 4, 2, true>(args, stream);
    if (args.nh <= 4) return launch_mha_vo_otf_form<HD, KBLK, 4, 1, true>(args, stream);
    // (an additive mask costs registers: with it the 12-wave forms would spill, 8 waves walk the heads instead)
    if (args.nh <= 8 || args.mask) return launch_mha_vo_otf_form<HD, KBLK, 8, 1, false>(args, stream);
    if (small_grid <= 128) return launch_mha_vo_otf_form<HD, KBLK, 12, 1, false, 32>(args, stream);
    return launch_mha_vo_otf_form<HD, KBLK, 12, 1, false>(args, stream);
}

}  // namespace et

using namespace et;

extern "C" {

int et_mha_vo_otf_f16(const et_f16 *Q, const et_f16 *K, int ldq, int ldk, const et_f16 *VOt, const et_f16 *bias_vo,
                      et_f16 *out, const et_f16 *bias_o, const int32_t *col_scatter, const et_f16 *mask,
                      const int32_t *lens, int B, int S, int nh, int hd, int N, int out_width, float scale, int flags,
                      et_stream stream) {
    ET_REQUIRE(Q && K && VOt && out, ET_ERR_INVALID_ARG, "et_mha_vo_otf_f16: NULL pointer");
    ET_REQUIRE(B >= 0 && S > 0 && nh > 0 && hd > 0, ET_ERR_INVALID_ARG, "et_mha_vo_otf_f16: B=%d S=%d nh=%d hd=%d", B,
               S, nh, hd);
    ET_REQUIRE((flags & ~ET_MHA_CAUSAL) == 0, ET_ERR_INVALID_ARG, "et_mha_vo_otf_f16: flags=%d", flags);
    ET_REQUIRE(S % 16 == 0 && hd % 16 == 0 && hd <= 128, ET_ERR_UNSUPPORTED,
               "et_mha_vo_otf_f16: S=%d and head dim %d must be multiples of 16, the head dim at most 128", S, hd);
    ET_REQUIRE(N > 0 && N % 16 == 0 && out_width >= N && out_width % 4 == 0, ET_ERR_INVALID_ARG,
               "et_mha_vo_otf_f16: N=%d out_width=%d", N, out_width);
    ET_REQUIRE(col_scatter != nullptr || N == out_width, ET_ERR_INVALID_ARG,
               "et_mha_vo_otf_f16: N < out_width needs the column list");
    ET_REQUIRE(ldq >= nh * hd && ldk >= nh * hd && ldq % 8 == 0 && ldk % 8 == 0, ET_ERR_INVALID_ARG,
               "et_mha_vo_otf_f16: row strides %d %d", ldq, ldk);
    ET_REQUIRE((reinterpret_cast<uintptr_t>(VOt) & 15) == 0 && (reinterpret_cast<uintptr_t>(Q) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(K) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0 &&
                   (reinterpret_cast<uintptr_t>(bias_vo) & 7) == 0 && (reinterpret_cast<uintptr_t>(bias_o) & 7) == 0 &&
                   (reinterpret_cast<uintptr_t>(mask) & 7) == 0,
               ET_ERR_UNSUPPORTED, "et_mha_vo_otf_f16: operands must be 16-byte aligned (biases, mask, out: 8)");
    const long long strips = (S + 15) / 16, slices = (N + kVoCols - 1) / kVoCols;
    ET_REQUIRE(((long long)B * slices + kXcds) * strips < (1ll << 31), ET_ERR_UNSUPPORTED,
               "et_mha_vo_otf_f16: B=%d S=%d N=%d make too many workgroups", B, S, N);
    if (B == 0) return ET_OK;
    if (col_scatter && N < out_width) {
        // columns no surviving VO column maps to carry the output bias alone
        int s = et_fill_rows_bias_f16(out, bias_o, B * S, out_width, stream);
        if (s != ET_OK) return s;
    }
    MhaVoArgs a{};
    a.Q = reinterpret_cast<const _Float16 *>(Q);
    a.K = reinterpret_cast<const _Float16 *>(K);
    a.VOt = reinterpret_cast<const _Float16 *>(VOt);
    a.bias_vo = reinterpret_cast<const _Float16 *>(bias_vo);
    a.out = reinterpret_cast<_Float16 *>(out);
    a.bias_o = reinterpret_cast<const _Float16 *>(bias_o);
    a.col_scatter = col_scatter;
    a.mask = reinterpret_cast<const _Float16 *>(mask);
    a.lens = lens;
    a.ldq = ldq;
    a.ldk = ldk;
    a.S = S;
    a.nh = nh;
    a.hd = hd;
    a.N = N;
    a.out_width = out_width;
    a.B = B;
    a.scale_log2e = scale * kLog2e;
    a.causal = (flags & ET_MHA_CAUSAL) ? 1 : 0;
    if (hd <= 32) return launch_mha_vo_otf<32, 128>(a, as_stream(stream));
    if (hd <= 64) return launch_mha_vo_otf<64, 128>(a, as_stream(stream));
    return launch_mha_vo_otf<128, 64>(a, as_stream(stream));
}

}  // extern "C"
