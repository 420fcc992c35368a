// Fused multi-head self-attention for gfx950: scores, mask, softmax and P*V in
// one kernel; the score matrix lives in registers only.
//
// Grid (query strip, head, sequence).  A workgroup stages one block of up to
// 128 keys of its head in LDS — K as [key][hd] and V transposed as [hd][key]
// — and each wave owns 16 query rows.  Both contractions are computed
// transposed so that no register shuffle is needed between them:
//   S^T = K * Q^T : MFMA A = K rows (from LDS), B = Q rows (registers);
//                   lane (r = lane%16, g = lane/16) ends with the scores of
//                   query r against keys 16*kb + 4g..4g+3 of every key block.
//   O^T = V^T * P^T: the contraction index of v_mfma_f32_16x16x32_f16 is
//                   mapped so that the 8 values a lane must supply as the B
//                   operand are exactly the 2x4 probabilities it already holds
//                   (key blocks 2s and 2s+1); the A operand reads the same
//                   keys of V^T from LDS as two 8-byte loads.
// Softmax is the running-max form over key blocks (one block when S <= 128):
// fp32 scores, exp2 with log2(e) folded into the scale, row max/sum reduced
// in-lane and then across the four 16-lane groups with two wave64 butterflies.
// Probabilities are rounded to fp16 only as MFMA operands; the normalisation
// by the fp32 row sum happens once on the fp32 accumulators.
#include <math.h>

#include <type_traits>

#include "common.hip.h"

namespace et {

struct MhaArgs {
    const _Float16 *Q, *K, *V;
    _Float16 *Z;
    const _Float16 *mask;  // [S x S] additive or nullptr
    const int32_t *lens;   // [B] or nullptr
    int ldq, ldk, ldv, ldz;
    int S, nh;
    int hd;             // head size, a multiple of 8; the kernel template is the next of 32, 64, 128, 256
    int nbh;            // sequences * heads
    float scale_log2e;  // scale * log2(e)
    int causal;
    // compact-V form only: V is [rows x nnz] holding the surviving V columns;
    // head h owns compact columns [v_head_ptr[h], v_head_ptr[h+1]), which stand
    // for the full-width columns v_col_id[.] (all inside head h's slice of Z).
    const int32_t *v_col_id;
    const int32_t *v_head_ptr;
    int v_nnz = 0;  // entries of v_col_id (> 0 in the compact-V form)
};

constexpr int kXcds = 8;                // accelerator dies, each with a private L2
constexpr int kKeyBlock = 128;          // keys staged per iteration
constexpr int kNKB = kKeyBlock / 16;    // 16-key MFMA blocks per iteration
constexpr float kLog2e = 1.4426950408889634f;

template <int HD>
struct MhaLds {
    static constexpr int ldk = HD + 8;           // halfs per staged K row
    static constexpr int ldvt = kKeyBlock + 8;   // halfs per staged V^T row
    static constexpr int k_halfs = kKeyBlock * ldk;
    static constexpr int vt_halfs = HD * ldvt;
    static constexpr size_t bytes = (size_t)(k_halfs + vt_halfs) * sizeof(_Float16);
};

// Layout of a V^T row (one head dimension, kKeyBlock keys) in LDS.
//
// Order of the keys.  The P*V product contracts 32 keys per MFMA and lane (r16, g) supplies, as
// its 8 values, the scores it holds from two 16x16 score tiles: keys 4g..4g+3 of the first and
// of the second.  Key k = 32s + 16a + 4g + j is therefore stored at position 32s + 8g + 4a + j:
// the 8 values of a lane are consecutive and one 16-byte read fetches them (two 8-byte reads
// cost 1.55x as much LDS time).
//
// Swizzle.  The rows are written transposed, 8 bytes (4 keys of one dimension) per lane, and
// the lanes of one store instruction differ in the dimension group dg = row / 8: rows 16 apart
// fall in the same banks (4-way conflict, 3x the store time).  Bits of row / 16 are XORed into
// the position bits that the 32 lanes of a store pass do not vary themselves: bit 4 (16-key
// chunks, g ^ 2) and bit 5 (32-key groups); 128-wide heads have a third bit to place, which
// swaps the two 4-key halves of a lane's 8 values (bit 2).  For 64-wide heads the 4-key groups
// are dealt to the lanes of a wave with bits 1 and 2 of their index exchanged (vt_unit_keys), so
// that a pass varies g's low bit and a instead of both bits of g.  A reader applies the same XOR,
// which for it is uniform over the wave.  Stores and fragment reads are then conflict-free.
template <int HD> __device__ __forceinline__ constexpr int vt_swizzle(int row16) {
    if (HD <= 32) return (row16 & 1) << 5;
    if (HD <= 64) return ((row16 & 1) << 4) | (((row16 >> 1) & 1) << 5);
    return ((row16 & 1) << 4) | (((row16 >> 1) & 1) << 5) | (((row16 >> 2) & 1) << 2);
}
// 4-key group staged by unit number kg (units are dealt to consecutive threads)
template <int HD> __device__ __forceinline__ constexpr int vt_unit_keys(int kg) {
    if (HD > 32 && HD <= 64) return (kg & ~6) | ((kg & 2) << 1) | ((kg & 4) >> 1);
    return kg;
}

// QT = 16-query tiles per wave: with QT = 2 every K and V^T fragment read from LDS feeds
// two MFMAs and a workgroup covers 32*NW queries per staged key block.
//
// Some variants prefetch the next key block through registers (mha_prefetches).  The 4-wave one
// is held to the 168 registers of three resident waves per SIMD; left alone the allocator takes
// a few more and the third wave is lost, which costs more than the prefetch gains.
template <int HD, int NW, bool COMPACT, int QT> constexpr bool mha_prefetches() {
    if (HD == 128 && !COMPACT && NW == 8 && QT == 1) return true;  // 202 registers: two waves per SIMD either way
    return HD <= 64 && !COMPACT && ((NW == 4 && QT == 1) || (NW == 8 && QT == 2));
}
template <int HD, int NW, bool COMPACT, int QT> constexpr bool mha_three_waves() {
    return mha_prefetches<HD, NW, COMPACT, QT>() && NW == 4;
}

template <int HD, bool COMPACT, int NW, int QT>
__global__ __launch_bounds__(64 * NW)
    __attribute__((amdgpu_waves_per_eu(mha_three_waves<HD, NW, COMPACT, QT>() ? 3 : 1, mha_three_waves<HD, NW, COMPACT, QT>() ? 3 : 8))) void
    mha_fused_kernel(const MhaArgs a) {
    using L = MhaLds<HD>;
    constexpr int KS = HD / 32;  // K=32 MFMA steps over the head dimension
    constexpr int DB = HD / 16;  // 16-wide output blocks of the head dimension
    extern __shared__ __align__(16) unsigned char smem_raw[];
    _Float16 *Ks = reinterpret_cast<_Float16 *>(smem_raw);
    _Float16 *Vt = Ks + L::k_halfs;

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    constexpr int nwave = NW;
    constexpr int nthr = 64 * NW;
    constexpr int kStripQ = 16 * NW * QT;  // queries per workgroup
    const int r16 = lane & 15;
    const int g = lane >> 4;
    const int S = a.S;
    // Workgroup id -> (sequence*head, query strip), XCD-aware: workgroups go to the 8
    // XCDs round-robin by id, so the query strips of one (sequence, head) are given ids
    // that land on the same XCD and share its K and V in that L2.
    const int qstrips = (S + kStripQ - 1) / kStripQ;
    const int xcd = blockIdx.x % kXcds, k_in_xcd = blockIdx.x / kXcds;
    const int bh = xcd + kXcds * (k_in_xcd / qstrips);
    if (bh >= a.nbh) return;  // padding of the last round (whole workgroup)
    const int qstrip = k_in_xcd % qstrips;
    const int b = bh / a.nh, h = bh - b * a.nh;
    const size_t row0 = (size_t)b * S;  // first token row of this sequence
    int q[QT];       // this lane's queries
    bool q_ok[QT];
#pragma unroll
    for (int t = 0; t < QT; t++) {
        q[t] = qstrip * kStripQ + (wave * QT + t) * 16 + r16;
        q_ok[t] = q[t] < S;
    }
    int klimit = S;
    if (a.lens) klimit = min(S, max(a.lens[b], 0));
    // under a causal mask no query of this strip sees a key past the strip's last query
    if (a.causal) klimit = min(klimit, (qstrip + 1) * kStripQ);
    // compact-V: this head's surviving V columns
    // head sizes between the template sizes: columns [hd, HD) of Q, K and V read as zero
    // (no effect on scores or outputs) and are not written
    const int hd = a.hd;
    int vc0 = 0, vlive = hd;
    bool v_vec = false;  // this head's compact columns can be read as aligned 16-byte vectors
    if (COMPACT) {
        vc0 = a.v_head_ptr[h];
        vlive = min(a.v_head_ptr[h + 1] - vc0, hd);
        v_vec = ((vc0 | vlive | a.ldv) & 7) == 0 && vlive > 0 && (reinterpret_cast<uintptr_t>(a.V) & 15) == 0;
    }
    // compact-V: the full-width positions of this head's surviving columns are requested now
    // and used in the epilogue (kCid ids per thread cover the up to 128 columns of a head)
    constexpr int kCid = COMPACT ? (128 + nthr - 1) / nthr : 1;
    int my_cid[kCid];
    if (COMPACT) {
#pragma unroll
        for (int i = 0; i < kCid; i++)
            // clamped into the array also for a head without surviving columns that sits at its end
            my_cid[i] = a.v_col_id[min(vc0 + min((int)threadIdx.x + i * nthr, max(vlive - 1, 0)), a.v_nnz - 1)];
    }

    // Q fragments: B operand, lane supplies Q[q][32*ks + 8g .. +7]
    h8 qf[QT][KS];
#pragma unroll
    for (int t = 0; t < QT; t++) {
        const _Float16 *qp = a.Q + (row0 + (q_ok[t] ? q[t] : 0)) * a.ldq + h * hd + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const bool live = q_ok[t] && 32 * ks + 8 * g < hd;
            qf[t][ks] = *reinterpret_cast<const h8 *>(qp + (live ? 32 * ks : 0));
            if (!live) qf[t][ks] = h8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    f4 o[QT][DB];
    float m_run[QT];   // running max of this lane's query (log2 domain)
    float l_part[QT];  // this lane's share of the running row sum
#pragma unroll
    for (int t = 0; t < QT; t++) {
#pragma unroll
        for (int d = 0; d < DB; d++) o[t][d] = f4{0.f, 0.f, 0.f, 0.f};
        m_run[t] = -INFINITY;
        l_part[t] = 0.0f;
    }

    // ---- staging of one block of keys: K rows and V in units of 4 keys x 8 dims, which
    // go to LDS transposed.  load_block issues every global load of a block (one memory
    // round trip); store_block writes them to LDS.  The loads of block i+1 are issued
    // before block i is multiplied.
    constexpr int vec_per_row = HD / 8;
    constexpr int KV = kKeyBlock * vec_per_row / nthr;  // K vectors per thread
    constexpr int dgroups = HD / 8;
    constexpr int v_units = (kKeyBlock / 4) * dgroups;  // V units of 4 keys x 8 dims
    constexpr int VU = (v_units + nthr - 1) / nthr;       // ... per thread
    static_assert(KV >= 1 && kKeyBlock * vec_per_row % nthr == 0, "K block must split evenly");
    h8 kreg[KV];
    h8 vreg[VU][4];
    auto load_block = [&](int k0) {
#pragma unroll
        for (int i = 0; i < KV; i++) {
            const int v = threadIdx.x + i * nthr;
            const int r = v / vec_per_row, c = v - r * vec_per_row;
            kreg[i] = h8{0, 0, 0, 0, 0, 0, 0, 0};
            if (k0 + r < S && c * 8 < hd)
                kreg[i] = *reinterpret_cast<const h8 *>(a.K + (row0 + k0 + r) * a.ldk + h * hd + c * 8);
        }
#pragma unroll
        for (int j = 0; j < VU; j++) {
            const int u = threadIdx.x + j * nthr;
            const int dg = u % dgroups, kg = vt_unit_keys<HD>(u / dgroups);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = (u < v_units) ? k0 + kg * 4 + i : S;  // surplus threads load nothing
                vreg[j][i] = h8{0, 0, 0, 0, 0, 0, 0, 0};
                if (COMPACT) {
                    // Every load is unconditional, from a clamped address, and the value is
                    // selected afterwards: a load under a branch gets a basic block of its own and
                    // is waited for on the spot, one memory round trip per element.
                    const bool key_ok = key < S;
                    const _Float16 *vp = a.V + (row0 + (key_ok ? key : 0)) * a.ldv + (vlive > 0 ? vc0 : 0);
                    if (v_vec) {  // workgroup-uniform: 16-byte vectors of surviving columns
                        const bool live = key_ok && dg * 8 < vlive;
                        const h8 t = *reinterpret_cast<const h8 *>(vp + (live ? dg * 8 : 0));
                        vreg[j][i] = live ? t : h8{0, 0, 0, 0, 0, 0, 0, 0};
                    } else {  // compact columns that start at an arbitrary element
#pragma unroll
                        for (int d = 0; d < 8; d++) {
                            const bool live = key_ok && dg * 8 + d < vlive;
                            const _Float16 t = vp[live ? dg * 8 + d : 0];
                            vreg[j][i][d] = live ? t : (_Float16)0;
                        }
                    }
                } else if (key < S && dg * 8 < hd) {
                    vreg[j][i] = *reinterpret_cast<const h8 *>(a.V + (row0 + key) * a.ldv + h * hd + dg * 8);
                }
            }
        }
    };
    auto store_block = [&]() {
#pragma unroll
        for (int i = 0; i < KV; i++) {
            const int v = threadIdx.x + i * nthr;
            const int r = v / vec_per_row, c = v - r * vec_per_row;
            *reinterpret_cast<h8 *>(Ks + r * L::ldk + c * 8) = kreg[i];
        }
#pragma unroll
        for (int j = 0; j < VU; j++) {
            const int u = threadIdx.x + j * nthr;
            const int dg = u % dgroups, kg = vt_unit_keys<HD>(u / dgroups);
            if (u < v_units) {
                // keys 4kg..4kg+3 = (s, a, g) = (kg / 8, (kg / 4) % 2, kg % 4); rows 8dg..8dg+7 share row / 16
                const int pos = (32 * (kg >> 3) + 8 * (kg & 3) + 4 * ((kg >> 2) & 1)) ^ vt_swizzle<HD>(dg >> 1);
#pragma unroll
                for (int d = 0; d < 8; d++) {
                    h4 col = {vreg[j][0][d], vreg[j][1][d], vreg[j][2][d], vreg[j][3][d]};
                    *reinterpret_cast<h4 *>(Vt + (dg * 8 + d) * L::ldvt + pos) = col;
                }
            }
        }
    };

    // Holding the next block's loads in registers through the multiplication costs 32 VGPRs: it
    // is done where that still fits the resident waves the variant runs with anyway (3-4 % at
    // 512 and 2048 keys); elsewhere it spills or loses a wave, and is off.
    constexpr bool kPrefetch = mha_prefetches<HD, NW, COMPACT, QT>();
    const int nblocks = (klimit + kKeyBlock - 1) / kKeyBlock;
    if (kPrefetch && nblocks > 0) load_block(0);
    for (int blk = 0; blk < nblocks; blk++) {
        const int k0 = blk * kKeyBlock;
        if (blk > 0) __syncthreads();  // every wave is done with the previous block
        if (!kPrefetch) load_block(k0);
        store_block();
        __syncthreads();
        if (kPrefetch && blk + 1 < nblocks) load_block(k0 + kKeyBlock);

        // The multiplication of one staged block.  FAST (wave-uniform) = nothing is added to the
        // scores and every key of the block is live for every query of the workgroup, or dead
        // for every query (right padding):
        // no per-16-key branches (the LDS reads of the whole block can be issued ahead of
        // the MFMAs) and the softmax costs one max, one multiply-add, one exp2, half a
        // conversion and half a dot-accumulate per score.
        auto multiply = [&](auto fast_tag) {
            constexpr bool FAST = decltype(fast_tag)::value;
            // ---- scores of the wave's queries against the 128 staged keys
            f4 sc[QT][kNKB];
#pragma unroll
            for (int kb = 0; kb < kNKB; kb++) {
#pragma unroll
                for (int t = 0; t < QT; t++) sc[t][kb] = f4{0.f, 0.f, 0.f, 0.f};
                if (FAST || k0 + kb * 16 < klimit) {  // wave-uniform: skip fully padded key blocks
                    const _Float16 *kp = Ks + (kb * 16 + r16) * L::ldk + 8 * g;
#pragma unroll
                    for (int ks = 0; ks < KS; ks++) {
                        const h8 kf = *reinterpret_cast<const h8 *>(kp + 32 * ks);
#pragma unroll
                        for (int t = 0; t < QT; t++)
                            sc[t][kb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[t][ks], sc[t][kb], 0, 0, 0);
                    }
                }
            }

            if (FAST && k0 + kKeyBlock > klimit) {  // wave-uniform
                // The block ends in padded keys: their raw scores become -inf, in place.  Key
                // 16kb + 4g + j is padded when 16kb + j >= klimit - k0 - 4g (the left side a
                // constant once unrolled).  (A separate instantiation of this lambda for the
                // case made the allocator spill in the variants held to 168 registers.)
                const int lim = klimit - k0 - 4 * g;
#pragma unroll
                for (int t = 0; t < QT; t++)
#pragma unroll
                    for (int kb = 0; kb < kNKB; kb++)
#pragma unroll
                        for (int j = 0; j < 4; j++)
                            sc[t][kb][j] = (kb * 16 + j >= lim) ? -INFINITY : sc[t][kb][j];
            }
            // ---- scale, mask, block max, running max (FAST keeps the raw scores: the scale
            // is positive there, so the max commutes with it, and it is applied inside the
            // exponent's multiply-add)
            float m_use[QT];
#pragma unroll
            for (int t = 0; t < QT; t++) {
                float m_blk = -INFINITY;
                if (FAST) {
#pragma unroll
                    for (int kb = 0; kb < kNKB; kb++)
#pragma unroll
                        for (int j = 0; j < 4; j++) m_blk = fmaxf(m_blk, sc[t][kb][j]);
                    m_blk *= a.scale_log2e;
                } else {
#pragma unroll
                    for (int kb = 0; kb < kNKB; kb++) {
                        const int key0 = k0 + kb * 16 + 4 * g;
                        float mk[4] = {0.f, 0.f, 0.f, 0.f};
                        if (a.mask && q_ok[t] && key0 < S) {
                            const h4 mv = *reinterpret_cast<const h4 *>(a.mask + (size_t)q[t] * S + key0);
#pragma unroll
                            for (int j = 0; j < 4; j++) mk[j] = (float)mv[j] * kLog2e;
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
                }
                m_blk = rows_max(m_blk);

                const float m_new = fmaxf(m_run[t], m_blk);
                // all keys so far masked: keep everything at zero without inf - inf
                m_use[t] = (m_new == -INFINITY) ? 0.0f : m_new;
                const float alpha = __builtin_amdgcn_exp2f(m_run[t] - m_use[t]);  // m_run = -inf gives 0
                m_run[t] = m_new;
                // the running max seldom moves after the first blocks: skip the rescaling of
                // the accumulators when no lane of the wave needs it
                if (!__all(alpha == 1.0f)) {
                    l_part[t] *= alpha;
#pragma unroll
                    for (int d = 0; d < DB; d++) o[t][d] *= alpha;
                }
            }

            // ---- probabilities (fp32 sum, fp16 operands) and O^T += V^T P^T
            const h2 ones = {(_Float16)1.0f, (_Float16)1.0f};
            const int g8 = 8 * g, g8x = (8 * g) ^ 16;  // the lane's 8-key chunk of a 32-key group, plain and swizzled
#pragma unroll
            for (int s2 = 0; s2 < kNKB / 2; s2++) {
                if (!FAST && k0 + s2 * 32 >= klimit) continue;  // both key blocks fully padded
                h8 pf[QT];
#pragma unroll
                for (int t = 0; t < QT; t++) {
                    // the lane's 8 values: keys 4g..4g+3 of score tile 2*s2, then of tile 2*s2+1;
                    // each fp16 pair is formed once and feeds both the MFMA and the row sum
#pragma unroll
                    for (int pr = 0; pr < 4; pr++) {
                        const int kb = 2 * s2 + (pr >> 1), j = 2 * (pr & 1);
                        float e0, e1;
                        if (FAST) {
                            e0 = sc[t][kb][j] * a.scale_log2e - m_use[t];
                            e1 = sc[t][kb][j + 1] * a.scale_log2e - m_use[t];
                        } else {
                            e0 = sc[t][kb][j] - m_use[t];
                            e1 = sc[t][kb][j + 1] - m_use[t];
                        }
                        // raw v_exp_f32: results below the normal range flush to zero, which
                        // the conversion to fp16 would do anyway
                        const h2 hp = {(_Float16)__builtin_amdgcn_exp2f(e0), (_Float16)__builtin_amdgcn_exp2f(e1)};
                        // the row sum uses the values that enter the MFMA
                        l_part[t] = __builtin_amdgcn_fdot2(hp, ones, l_part[t], false);
                        pf[t][2 * pr] = hp[0];
                        pf[t][2 * pr + 1] = hp[1];
                    }
                }
                // The V^T fragments of the step are read unconditionally (dimension blocks past the
                // head size or the surviving columns hold zeros) so that the reads go out together;
                // a read under a branch is waited for on the spot.  Only compact V skips the
                // products of dead blocks (wave-uniform).
                // (at most 8 fragments, 32 registers, at a time: 256-wide heads take two rounds)
                constexpr int DC = DB < 8 ? DB : 8;
#pragma unroll
                for (int d0 = 0; d0 < DB; d0 += DC) {
                    h8 vf[DC];
#pragma unroll
                    for (int dd = 0; dd < DC; dd++) {
                        const int d = d0 + dd;
                        const int swz = vt_swizzle<HD>(d);  // a constant once d is unrolled
                        const h8 vr = *reinterpret_cast<const h8 *>(Vt + (d * 16 + r16) * L::ldvt +
                                                                     ((s2 * 32) ^ (swz & 32)) + ((swz & 16) ? g8x : g8));
                        vf[dd] = (swz & 4) ? h8{vr[4], vr[5], vr[6], vr[7], vr[0], vr[1], vr[2], vr[3]} : vr;
                    }
#pragma unroll
                    for (int dd = 0; dd < DC; dd++) {
                        const int d = d0 + dd;
                        if (COMPACT && d * 16 >= vlive) continue;
#pragma unroll
                        for (int t = 0; t < QT; t++)
                            o[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[dd], pf[t], o[t][d], 0, 0, 0);
                    }
                }
            }
        };
        const bool plain = a.mask == nullptr && a.scale_log2e > 0.0f &&
                          (!a.causal || k0 + kKeyBlock <= qstrip * kStripQ + 1);
        if (plain) multiply(std::true_type{});
        else multiply(std::false_type{});
    }

    // ---- normalise and store: lane holds dims 16d + 4g..4g+3 of query r16
    float inv[QT];
#pragma unroll
    for (int t = 0; t < QT; t++) {
        float l = l_part[t];
        l = rows_sum(l);
        inv[t] = l > 0.0f ? 1.0f / l : 0.0f;
    }
    if (!COMPACT) {
#pragma unroll
        for (int t = 0; t < QT; t++) {
            if (!q_ok[t]) continue;
            _Float16 *zp = a.Z + (row0 + q[t]) * a.ldz + h * hd + 4 * g;
#pragma unroll
            for (int d = 0; d < DB; d++) {
                if (16 * d >= hd) continue;  // wave-uniform
                h4 out;
#pragma unroll
                for (int j = 0; j < 4; j++) out[j] = (_Float16)(o[t][d][j] * inv[t]);
                // a head size that is a multiple of 8 only ends inside the last block: lanes past it store nothing
                if (16 * d + 4 * g < hd) *reinterpret_cast<h4 *>(zp + 16 * d) = out;
            }
        }
    }
    if (COMPACT) {
        // Full-width Z: surviving columns are scattered to v_col_id, the pruned columns of this
        // head's slice get zeros.  Every element of the slice is written exactly once (the
        // liveness mask tells the two sets apart), so no store has to be ordered against another.
        // The column ids were requested at the start of the kernel; mask and compact-to-full map
        // go through LDS here, where every wave of the workgroup arrives.
        __shared__ unsigned live_mask[4];  // bit c: column c of this head's slice of Z survives
        __shared__ int full_col[128];      // compact column -> column of Z
        __shared__ int n_outside;          // surviving columns that lie outside this head's slice
        if (threadIdx.x < 4) live_mask[threadIdx.x] = 0u;
        if (threadIdx.x == 4) n_outside = 0;
        __syncthreads();  // also: every wave is done with the staged K and V
#pragma unroll
        for (int i = 0; i < kCid; i++) {
            const int j = threadIdx.x + i * nthr;
            if (j < vlive) {
                full_col[j] = my_cid[i];
                const int c = my_cid[i] - h * hd;
                if (c >= 0 && c < HD) atomicOr(&live_mask[c >> 5], 1u << (c & 31));
                if (c < 0 || c >= hd) atomicAdd(&n_outside, 1);
            }
        }
        __syncthreads();
        if (n_outside == 0) {
            // The usual case, every surviving column inside the head's own slice: the wave
            // assembles its 16 queries x hd slice in LDS (zeros, then the surviving columns at
            // their places) and stores whole 8-byte pieces of rows, 4 per lane and tile, instead
            // of up to 32 two-byte stores.  One wave's LDS instructions complete in order, so
            // the three steps need no barrier.
            constexpr int ldt = HD + 8;
            _Float16 *zt = Ks + wave * 16 * ldt;  // the K stage is free: NW * 16 rows <= 128
            static_assert(NW * 16 <= kKeyBlock && HD + 8 <= MhaLds<HD>::ldk, "slice tiles fit the K stage");
            int zl[DB][4];
#pragma unroll
            for (int d = 0; d < DB; d++)
#pragma unroll
                for (int j = 0; j < 4; j++) zl[d][j] = full_col[min(d * 16 + 4 * g + j, 127)] - h * hd;
#pragma unroll
            for (int t = 0; t < QT; t++) {
                const h4 zero4 = {0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < HD / 16; i++) {
                    const int v = lane + 64 * i;  // 8-byte piece of the 16 x HD tile
                    *reinterpret_cast<h4 *>(zt + (v / (HD / 4)) * ldt + (v % (HD / 4)) * 4) = zero4;
                }
#pragma unroll
                for (int d = 0; d < DB; d++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (d * 16 + 4 * g + j < vlive) zt[r16 * ldt + zl[d][j]] = (_Float16)(o[t][d][j] * inv[t]);
                const int qbase = qstrip * kStripQ + (wave * QT + t) * 16;
#pragma unroll
                for (int i = 0; i < HD / 16; i++) {
                    const int v = lane + 64 * i;
                    const int rr = v / (HD / 4), cc = (v % (HD / 4)) * 4;
                    const h4 piece = *reinterpret_cast<const h4 *>(zt + rr * ldt + cc);
                    if (qbase + rr < S && cc < hd)
                        *reinterpret_cast<h4 *>(a.Z + (row0 + qbase + rr) * a.ldz + h * hd + cc) = piece;
                }
            }
            return;
        }
        int zc[DB][4];
#pragma unroll
        for (int d = 0; d < DB; d++)
#pragma unroll
            for (int j = 0; j < 4; j++) zc[d][j] = full_col[min(d * 16 + 4 * g + j, 127)];
        unsigned live_w[4];
#pragma unroll
        for (int w = 0; w < 4; w++) live_w[w] = live_mask[w];
#pragma unroll
        for (int t = 0; t < QT; t++) {
            if (q_ok[t]) {
                _Float16 *zrow = a.Z + (row0 + q[t]) * a.ldz;
#pragma unroll
                for (int d = 0; d < DB; d++) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int dc = d * 16 + 4 * g + j;  // as a compact index, and as a column of the slice
                        if (dc < vlive) zrow[zc[d][j]] = (_Float16)(o[t][d][j] * inv[t]);
                        if (dc < hd && !((live_w[dc >> 5] >> (dc & 31)) & 1u)) zrow[h * hd + dc] = (_Float16)0;
                    }
                }
            }
        }
    }
}

template <int HD, bool COMPACT, int NW, int QT>
static int launch_mha_nw(const MhaArgs &args, hipStream_t stream) {
    auto kernel = mha_fused_kernel<HD, COMPACT, NW, QT>;
    constexpr size_t lds = MhaLds<HD>::bytes;
    if (lds > 64 * 1024) {
        static bool raised = false;
        if (!raised) {
            ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            raised = true;
        }
    }
    const int qstrips = (args.S + 16 * NW * QT - 1) / (16 * NW * QT);
    const int rounds = (args.nbh + kXcds - 1) / kXcds;
    kernel<<<dim3((unsigned)(rounds * kXcds * qstrips)), 64 * NW, lds, stream>>>(args);
    return check_launch("mha_fused_kernel");
}

// 4 waves per workgroup and one 16-query tile per wave; 2 or 1 waves when 4 would leave a
// half-empty strip (S = 32, 96, 16, ...).  Larger workgroups stage each key block for more
// queries and pay once the grid still fills the chip: 8 waves (128 queries) from 256 such
// workgroups on (2048 keys, 16 x 16 heads: 546 -> 516 us; 128-wide heads 592 -> 570 us), and 8
// waves with two query tiles each (256 queries; every K and V^T fragment read from LDS feeds two
// MFMAs) from 512 on (-> 464 us; 214 registers, two waves per SIMD).  128-wide heads: the 8-wave
// form prefetches the next block through registers (565 -> 532 us at 2048 keys, 16 x 8 heads),
// the two-tile form takes all 256 registers and spills 45, and is still the faster one (503 us).
// Two tiles on 4 waves lose more to the missing third wave than they save (735 us).
template <int HD, bool COMPACT>
static int launch_mha(const MhaArgs &args, int B, hipStream_t stream) {
    (void)B;
    const int qblocks = args.S / 16;
    if constexpr (!COMPACT) {
        if (HD == 64 && qblocks % 16 == 0 && (long)args.nbh * (qblocks / 16) >= 512)
            return launch_mha_nw<(HD == 64 ? HD : 64), COMPACT, 8, 2>(args, stream);
        if (HD == 128 && qblocks % 16 == 0 && (long)args.nbh * (qblocks / 16) >= 512)
            return launch_mha_nw<(HD == 128 ? HD : 128), COMPACT, 8, 2>(args, stream);
        if (HD >= 64 && qblocks % 8 == 0 && (long)args.nbh * (qblocks / 8) >= 256)
            return launch_mha_nw<HD, COMPACT, 8, 1>(args, stream);
    }
    if (qblocks % 4 == 0) return launch_mha_nw<HD, COMPACT, 4, 1>(args, stream);
    if (qblocks % 2 == 0) return launch_mha_nw<HD, COMPACT, 2, 1>(args, stream);
    return launch_mha_nw<HD, COMPACT, 1, 1>(args, stream);
}

}  // namespace et

using namespace et;

extern "C" {

int et_mha_fused_f16(const et_f16 *Q, const et_f16 *K, const et_f16 *V, int ldq, int ldk, int ldv,
                     et_f16 *Z, int ldz, const et_f16 *mask, const int32_t *lens, int B, int S,
                     int nh, int hd, float scale, int flags, et_stream stream) {
    ET_REQUIRE(Q && K && V && Z, ET_ERR_INVALID_ARG, "et_mha_fused_f16: NULL pointer");
    ET_REQUIRE(B >= 0 && S > 0 && nh > 0 && hd > 0, ET_ERR_INVALID_ARG,
               "et_mha_fused_f16: B=%d S=%d nh=%d hd=%d", B, S, nh, hd);
    ET_REQUIRE((flags & ~ET_MHA_CAUSAL) == 0, ET_ERR_INVALID_ARG, "et_mha_fused_f16: flags=%d",
               flags);
    ET_REQUIRE(S % 16 == 0, ET_ERR_UNSUPPORTED, "et_mha_fused_f16: S=%d must be a multiple of 16",
               S);
    // the reference example's 800 / 4 = 200-wide heads (example/main.cu:24-31) are the reason for the 256 form
    ET_REQUIRE(hd % 8 == 0 && hd <= 256, ET_ERR_UNSUPPORTED,
               "et_mha_fused_f16: head dim %d must be a multiple of 8, at most 256", hd);
    const int width = nh * hd;
    ET_REQUIRE(ldq >= width && ldk >= width && ldv >= width && ldz >= width, ET_ERR_INVALID_ARG,
               "et_mha_fused_f16: row strides (%d %d %d %d) smaller than nh*hd=%d", ldq, ldk, ldv,
               ldz, width);
    ET_REQUIRE(ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0 && ldz % 4 == 0, ET_ERR_UNSUPPORTED,
               "et_mha_fused_f16: row strides must keep 16-byte alignment");
    ET_REQUIRE(((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) |
                 reinterpret_cast<uintptr_t>(V)) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(Z) & 7) == 0,
               ET_ERR_UNSUPPORTED, "et_mha_fused_f16: operands must be 16-byte aligned");
    ET_REQUIRE((long long)B * nh * (S / 16) < (1LL << 30), ET_ERR_UNSUPPORTED, "et_mha_fused_f16: grid too large");
    if (B == 0) return ET_OK;
    MhaArgs args;
    args.Q = reinterpret_cast<const _Float16 *>(Q);
    args.K = reinterpret_cast<const _Float16 *>(K);
    args.V = reinterpret_cast<const _Float16 *>(V);
    args.Z = reinterpret_cast<_Float16 *>(Z);
    args.mask = reinterpret_cast<const _Float16 *>(mask);
    args.lens = lens;
    args.ldq = ldq;
    args.ldk = ldk;
    args.ldv = ldv;
    args.ldz = ldz;
    args.S = S;
    args.nh = nh;
    args.hd = hd;
    args.nbh = B * nh;
    args.scale_log2e = scale * kLog2e;
    args.causal = (flags & ET_MHA_CAUSAL) ? 1 : 0;
    args.v_col_id = nullptr;
    args.v_head_ptr = nullptr;
    if (hd <= 32) return launch_mha<32, false>(args, B, as_stream(stream));
    if (hd <= 64) return launch_mha<64, false>(args, B, as_stream(stream));
    if (hd <= 128) return launch_mha<128, false>(args, B, as_stream(stream));
    // Heads up to 256 wide: 4 waves share the staging of a 128-key block (137 KB of LDS), each with one
    // 16-query tile.  One workgroup per compute unit and one wave per SIMD, so a wave has the whole
    // register file (8 waves at 256 registers spill 68 bytes per lane); a strip shorter than 64 queries
    // leaves waves without queries, which stage and otherwise idle.
    return launch_mha_nw<256, false, 4, 1>(args, as_stream(stream));
}

int et_mha_compactv_f16(const et_f16 *Q, const et_f16 *K, const et_f16 *Vc, int ldq, int ldk, int ldvc,
                        const int32_t *v_col_id, const int32_t *v_head_ptr, int nnz_col, et_f16 *Z,
                        int ldz, const et_f16 *mask, const int32_t *lens, int B, int S, int nh, int hd,
                        int vhd, float scale, int flags, et_stream stream) {
    ET_REQUIRE(Q && K && Vc && Z && v_col_id && v_head_ptr, ET_ERR_INVALID_ARG,
               "et_mha_compactv_f16: NULL pointer");
    ET_REQUIRE(B >= 0 && S > 0 && nh > 0 && hd > 0 && nnz_col >= 0, ET_ERR_INVALID_ARG,
               "et_mha_compactv_f16: B=%d S=%d nh=%d hd=%d nnz_col=%d", B, S, nh, hd, nnz_col);
    ET_REQUIRE((flags & ~ET_MHA_CAUSAL) == 0, ET_ERR_INVALID_ARG, "et_mha_compactv_f16: flags=%d", flags);
    ET_REQUIRE(S % 16 == 0, ET_ERR_UNSUPPORTED, "et_mha_compactv_f16: S=%d must be a multiple of 16", S);
    ET_REQUIRE(hd % 16 == 0 && hd <= 128, ET_ERR_UNSUPPORTED,
               "et_mha_compactv_f16: head dim %d must be a multiple of 16, at most 128", hd);
    ET_REQUIRE(vhd == hd, ET_ERR_UNSUPPORTED,
               "et_mha_compactv_f16: V head width %d must equal the Q/K head width %d", vhd, hd);
    ET_REQUIRE(ldq >= nh * hd && ldk >= nh * hd && ldz >= nh * vhd && ldvc >= nnz_col, ET_ERR_INVALID_ARG,
               "et_mha_compactv_f16: row strides too small");
    ET_REQUIRE(ldq % 8 == 0 && ldk % 8 == 0 && ldz % 4 == 0, ET_ERR_UNSUPPORTED,
               "et_mha_compactv_f16: row strides must keep 16-byte alignment");
    ET_REQUIRE((long long)B * nh * (S / 16) < (1LL << 30), ET_ERR_UNSUPPORTED, "et_mha_compactv_f16: grid too large");
    if (B == 0) return ET_OK;
    if (nnz_col == 0) {  // every V column pruned: Z is zero
        ET_REQUIRE(ldz == nh * vhd, ET_ERR_UNSUPPORTED, "et_mha_compactv_f16: nnz_col = 0 needs a contiguous Z");
        return et_fill_f16(Z, (size_t)B * S * ldz, 0, stream);
    }
    MhaArgs args;
    args.v_nnz = nnz_col;
    args.Q = reinterpret_cast<const _Float16 *>(Q);
    args.K = reinterpret_cast<const _Float16 *>(K);
    args.V = reinterpret_cast<const _Float16 *>(Vc);
    args.Z = reinterpret_cast<_Float16 *>(Z);
    args.mask = reinterpret_cast<const _Float16 *>(mask);
    args.lens = lens;
    args.ldq = ldq;
    args.ldk = ldk;
    args.ldv = ldvc;
    args.ldz = ldz;
    args.S = S;
    args.nh = nh;
    args.hd = hd;
    args.nbh = B * nh;
    args.scale_log2e = scale * kLog2e;
    args.causal = (flags & ET_MHA_CAUSAL) ? 1 : 0;
    args.v_col_id = v_col_id;
    args.v_head_ptr = v_head_ptr;
    if (hd <= 32) return launch_mha<32, true>(args, B, as_stream(stream));
    if (hd <= 64) return launch_mha<64, true>(args, B, as_stream(stream));
    return launch_mha<128, true>(args, B, as_stream(stream));
}

}  // extern "C"
