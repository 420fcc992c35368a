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

#include <algorithm>
#include <memory>
#include <new>
#include <vector>

#include <type_traits>

#include "common.hip.h"
#include "bsr_packed.hip.h"

namespace et {

#define ET_QM_CONST(T, p) ((const __attribute__((address_space(4))) T *)(p))

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
#include "attention_core.inc"
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


// ---- QKV projection inside the attention kernel --------------------------------------------------------
// One workgroup per (sequence, head), sequences of at most 128 tokens, heads of 64: the workgroup normalises
// its sequence's rows of the previous layer's binary32 sum while it stages them (the consumer half of the
// split SkipLayerNorm, 64 rows at a time), multiplies them with its head's 12 block-rows of the tile-sparse
// W_qkv (a pack: one block-row per wave, the wave's slots in registers), leaves Q, K and V^T of the head in
// LDS in the layouts the attention core reads, and runs that core on them.  Q, K and V never exist in memory
// and the layer has one launch fewer.  The heads of a sequence run on one XCD, so the sum comes from HBM once.
struct QkvMhaArgs {
    MhaArgs m;               // Z, ldz, mask, lens, S, nh, hd, nbh, scale_log2e, causal (Q, K, V unused)
    const _Float16 *pw;      // [nh][12][cap] slots of 1 KiB in lane order (two tiles each, zero slots as padding)
    const uint32_t *poff;    // [nh][12][cap] byte offsets (column * 32) of a slot's two tiles, 16 bits each
    const int32_t *pn;       // [nh][12] slots of every block-row
    const _Float16 *bias;    // [3 * nh * 64] (Q | K | V, as the rows of W_qkv) or nullptr
    int cap, in, T, B;
    const float *X32;        // [T][in] the binary32 sum
    const float *st_in;      // [st_groups][T][2] partial (sum, sum of squares) of every row
    int st_groups;
    const _Float16 *gamma, *beta;
    float eps;
    float *fin_out;          // [T][2] mean and rstd of every row, written by head 0 (may be null)
    const float *bias32;     // FOLDED: bias + W beta as binary32 (gamma is inside the slots; gamma, beta, bias unused)
};
constexpr int kQkvWaves = 12;   // Q, K, V x 4 block-rows of a 64-wide head
constexpr int kQkvRows = 64;    // token rows staged at a time
constexpr int kQkvIn = 768;     // input width the kernel is written for: 96 threads per row, 8 rows per pass of 768 threads

// PF of a thread's eight rows of the second 64 are requested before the products of the first 64 (they arrive while the
// matrix cores work).  NPASS = 1 keeps the wave's slots in registers across both halves; NPASS = 2 to 4 (block-rows of
// more than 12 slots) fetches them in parts of 8 or 4 for every 64 rows.
// FOLDED: the pack holds W diag(gamma) and bias + W beta, so that a row is normalised with one multiply-add per value,
// (x - mean) rstd, and the affine part of the normalisation costs nothing (the workgroups of the 12 heads of a sequence
// each normalise all of it).
template <int CAP, int PF, int NPASS, bool FOLDED>
__global__ __launch_bounds__(kQkvWaves * 64) void qkv_mha_kernel(const QkvMhaArgs qa) {
    constexpr int HD = 64, QT = 1;
    constexpr bool COMPACT = false;
    using L = MhaLds<HD>;
    constexpr int KS = HD / 32, DB = HD / 16;
    constexpr int SU = 8;  // 64 rows / (768 threads / 96 units): the host checks 64 == SU * dr
    const MhaArgs &a = qa.m;
    extern __shared__ __align__(256) unsigned char qm_smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, g = lane >> 4, sel = g >> 1, gbit = g & 1;
    constexpr int in = kQkvIn, stride = in * 2, upr = in >> 3;  // compile-time: the addresses below are adds of constants
    const int S = a.S;
    unsigned char *xs = qm_smem;                                                  // [64][in] binary16, swizzled
    _Float16 *Qs = reinterpret_cast<_Float16 *>(qm_smem + (size_t)kQkvRows * stride);  // [128][ldk]
    _Float16 *Ks = Qs + L::k_halfs;                                               // [128][ldk]
    _Float16 *Vt = Ks + L::k_halfs;                                               // [64][ldvt]
    float2 *stat = reinterpret_cast<float2 *>(Vt + L::vt_halfs);                 // [128] -mean * rstd and rstd of the sequence's rows
    _Float16 *gb = reinterpret_cast<_Float16 *>(stat + kKeyBlock);               // gamma | beta
    float2 *spart = reinterpret_cast<float2 *>(xs);                              // [16][128] partial sums, before xs is written

    const int xcd = blockIdx.x % kXcds, k_in_xcd = blockIdx.x / kXcds;
    const int b = xcd + kXcds * (k_in_xcd / a.nh), h = k_in_xcd % a.nh;
    if (b >= qa.B) return;  // padding of the last round (whole workgroup)
    const size_t row0 = (size_t)b * S;
    const int nhalf = (S + kQkvRows - 1) / kQkvRows;

    // ---- requests in the order their results are needed (they return in order): the partial row sums, gamma and
    // beta, the first 64 rows, then the wave's slots
    // partial sums: thread t takes row t % 128 of groups t / 128, + 6 and + 12
    const int st_row = threadIdx.x & (kKeyBlock - 1), st_g = threadIdx.x >> 7;
    float2 ps[3];
    {
        const int tok = min(st_row, S - 1);
#pragma unroll
        for (int k = 0; k < 3; k++)
            ps[k] = *reinterpret_cast<const float2 *>(qa.st_in + ((size_t)min(st_g + 6 * k, qa.st_groups - 1) * qa.T + row0 + tok) * 2);
    }
    // thread t owns columns 4c .. 4c + 3 and in / 2 + 4c .. + 3, c = t % upr, of staged rows t / upr + 8 u: the lanes of
    // a request read consecutive 16 bytes
    constexpr int n_dr = kQkvWaves * 64 / upr;
    static_assert(n_dr * upr == kQkvWaves * 64 && SU * n_dr == kQkvRows, "768 threads cover 8 rows of 96 units");
    const int n_r0 = (int)threadIdx.x / upr, n_c8 = (int)threadIdx.x - n_r0 * upr;
    h8 gam_in = {}, bet_in = {};
    if (!FOLDED && (int)threadIdx.x < upr) {
        gam_in = reinterpret_cast<const h8 *>(qa.gamma)[threadIdx.x];
        bet_in = reinterpret_cast<const h8 *>(qa.beta)[threadIdx.x];
    }
    f4 s32[SU][2];
    const char *xbase = reinterpret_cast<const char *>(qa.X32 + row0 * in);  // wave-uniform
    // rows [from, to) of the thread's eight in the given half (the thread's place passes through an empty asm: seen as
    // loop-invariant, the addresses of all sixteen rows are computed up front, 32 registers that spill)
    auto request_rows = [&](int half, auto from, auto to) {
        int r0_now = n_r0, c8_now = n_c8;
        asm volatile("" : "+v"(r0_now), "+v"(c8_now));
#pragma unroll
        for (int u = decltype(from)::value; u < decltype(to)::value; u++) {
            // (a wave-uniform base and a 32-bit offset per lane: the sequence's rows are less than 4 GB)
            const int tok = min(half * kQkvRows + r0_now + u * n_dr, S - 1);
            const unsigned off = (unsigned)tok * (unsigned)(in * 4) + 16u * (unsigned)c8_now;
            s32[u][0] = *reinterpret_cast<const f4 *>(xbase + off);
            s32[u][1] = *reinterpret_cast<const f4 *>(xbase + off + 2u * (unsigned)in);
        }
    };
    using i0 = std::integral_constant<int, 0>;
    using iPF = std::integral_constant<int, PF>;
    using iSU = std::integral_constant<int, SU>;
    // ---- mean and rstd of the sequence's rows: the partial sums are added per row in group order through LDS, by the
    // first two waves, while the others already request their rows.  (Results return in the order of the requests of
    // the whole compute unit: the few bytes the statistics wait for are requested, and awaited, ahead of all rows.)
#pragma unroll
    for (int k = 0; k < 3; k++)
        if (st_g + 6 * k < kMaxStatGroups) spart[(st_g + 6 * k) * kKeyBlock + st_row] = ps[k];
    if (!FOLDED && (int)threadIdx.x < upr) {
        reinterpret_cast<h8 *>(gb)[threadIdx.x] = gam_in;
        reinterpret_cast<h8 *>(gb + in)[threadIdx.x] = bet_in;
    }
    __syncthreads();
    if (threadIdx.x < kKeyBlock) {
        float s1 = 0.0f, s2 = 0.0f;
        for (int gi = 0; gi < qa.st_groups; gi++) {
            const float2 pr = spart[gi * kKeyBlock + threadIdx.x];
            s1 += pr.x;
            s2 += pr.y;
        }
        const float mean = s1 / (float)in;
        const float2 mine = {mean, rsqrtf(fmaxf(__builtin_fmaf(-mean, mean, s2 / (float)in), 0.0f) + qa.eps)};
        stat[threadIdx.x] = float2{-mean * mine.y, mine.y};
        if (qa.fin_out && h == 0 && (int)threadIdx.x < S)
            *reinterpret_cast<float2 *>(qa.fin_out + 2 * (row0 + threadIdx.x)) = mine;
    }
    request_rows(0, i0{}, iSU{});

    // ---- this wave's block-row of W_qkv: part 0 / 1 / 2 = Q / K / V, four block-rows of the head each
    const int part = wave >> 2, sub = wave & 3;
    const int rb = part * (a.nh * 4) + 4 * h + sub;  // block-row of W_qkv
    const size_t slab = (size_t)h * kQkvWaves + wave;
    const int nsl = ET_QM_CONST(int32_t, qa.pn)[slab];
    uint32_t offs[CAP];
    {
        const auto *op = ET_QM_CONST(uint32_t, qa.poff) + slab * CAP;
#pragma unroll
        for (int q4 = 0; q4 < CAP / 4; q4++) {
            if (4 * q4 < nsl) {
#pragma unroll
                for (int r = 0; r < 4; r++) offs[4 * q4 + r] = op[4 * q4 + r];
            }
        }
    }
    const size_t wp_off = slab * CAP * 512 + lane * 8;
    constexpr bool HOLD = NPASS == 1;
    constexpr int WN = CAP / NPASS;  // slots in registers at a time
    static_assert(WN % 4 == 0 && WN * NPASS == CAP, "slots are fetched in groups of four");
    h8 w[WN];
    // (the slab's offset and the swizzle term pass through an empty asm: seen as loop-invariant, the per-slot addresses
    // and LDS offsets are computed once in front of the loop, three registers per slot that then spill.  The offset
    // and not the pointer: a pointer out of an asm has no address space left, and its loads would count as LDS
    // accesses as well.)
    auto request_slots = [&](int first) {
        size_t off_now = wp_off + (size_t)first * 512;
        asm volatile("" : "+v"(off_now));
        const _Float16 *wp_now = qa.pw + off_now;
#pragma unroll
        for (int q4 = 0; q4 < WN / 4; q4++) {
            if (first + 4 * q4 < nsl) {
#pragma unroll
                for (int r = 0; r < 4; r++) w[4 * q4 + r] = *reinterpret_cast<const h8 *>(wp_now + (4 * q4 + r) * 512);
            }
        }
    };
    if constexpr (HOLD) request_slots(0);
    // bias: Q and K lanes end with features 4g .. 4g + 3 of a token, V lanes with feature r16 of four tokens.  Kept as
    // loaded and widened where it is added: a conversion here would wait for every request above.
    uint2 bias_bits = {0u, 0u};
    f4 bias_f = {0.f, 0.f, 0.f, 0.f};
    if constexpr (FOLDED) {
        if (part < 2) bias_f = *reinterpret_cast<const f4 *>(qa.bias32 + rb * 16 + g * 4);
        else bias_f[0] = qa.bias32[rb * 16 + r16];
    } else if (qa.bias) {
        if (part < 2) bias_bits = *reinterpret_cast<const uint2 *>(qa.bias + rb * 16 + g * 4);
        else bias_bits.x = *reinterpret_cast<const unsigned short *>(qa.bias + rb * 16 + r16);
    }
    const unsigned kx = (unsigned)((gbit ^ r16) & 15) << 4;

    if (nhalf * kQkvRows < kKeyBlock) {
        // keys that no round stages must hold finite values: their probabilities are exactly zero, and 0 x NaN is not
        uint4 *z = reinterpret_cast<uint4 *>(Ks);
        for (int i = threadIdx.x; i < (int)((L::k_halfs + L::vt_halfs) * sizeof(_Float16) / 16); i += blockDim.x)
            z[i] = uint4{0u, 0u, 0u, 0u};
    }
    __syncthreads();  // the statistics are complete and the partial sums read: xs may be written

    for (int half = 0; half < nhalf; half++) {
        const int tokbase = half * kQkvRows;
        if (half > 0) request_rows(half, iPF{}, iSU{});  // what was not requested ahead
        {
            // (the thread's place passes through an empty asm: the offsets made from it below are the same in both
            // halves, and held across the products they cost the registers that the variants with many slots lack)
            int r0_now = n_r0, c8_now = n_c8;
            asm volatile("" : "+v"(r0_now), "+v"(c8_now));
            h4 gam0 = {}, gam1 = {}, bet0 = {}, bet1 = {};
            if constexpr (!FOLDED) {
                gam0 = reinterpret_cast<const h4 *>(gb)[c8_now], gam1 = reinterpret_cast<const h4 *>(gb)[upr + c8_now];
                bet0 = reinterpret_cast<const h4 *>(gb + in)[c8_now], bet1 = reinterpret_cast<const h4 *>(gb + in)[upr + c8_now];
            }
            // Where the thread's two 8-byte pieces of row r0 + 8 u go: the row's swizzle term (row & 15) is r0 for even
            // u and r0 + 8 for odd u (r0 < 8), so four offsets and a multiple of a constant name all sixteen places.
            const unsigned unit0 = (unsigned)c8_now >> 1, unit1 = (unsigned)(upr + c8_now) >> 1;  // upr is even
            const unsigned at0 = (unsigned)r0_now * stride + (((unsigned)c8_now & 1u) << 3);
            const unsigned wr0[2] = {at0 + ((unit0 ^ (unsigned)r0_now) << 4), at0 + ((unit0 ^ (unsigned)(r0_now + 8)) << 4)};
            const unsigned wr1[2] = {at0 + ((unit1 ^ (unsigned)r0_now) << 4), at0 + ((unit1 ^ (unsigned)(r0_now + 8)) << 4)};
            // (the place of the next 64's rows passes through an empty asm: computed per row, two instructions, instead
            // of eight offsets held from the top of the loop)
            const int next_row = tokbase + kQkvRows + r0_now;
            const unsigned next_off = 16u * (unsigned)c8_now;
            const float2 *strow = stat + tokbase + r0_now;  // -mean * rstd and rstd of the thread's rows, 8 apart
            float2 st_next = strow[0];
#pragma unroll
            for (int u = 0; u < SU; u++) {
                const float2 st = st_next;
                if (u + 1 < SU) st_next = strow[(u + 1) * n_dr];  // one row ahead: its read is not waited for on the spot
                h4 lo, hi;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    if constexpr (FOLDED) {
                        lo[e] = (_Float16)__builtin_fmaf(s32[u][0][e], st.y, st.x);
                        hi[e] = (_Float16)__builtin_fmaf(s32[u][1][e], st.y, st.x);
                    } else {
                        lo[e] = (_Float16)__builtin_fmaf(__builtin_fmaf(s32[u][0][e], st.y, st.x), (float)gam0[e], (float)bet0[e]);
                        hi[e] = (_Float16)__builtin_fmaf(__builtin_fmaf(s32[u][1][e], st.y, st.x), (float)gam1[e], (float)bet1[e]);
                    }
                }
                *reinterpret_cast<h4 *>(xs + wr0[u & 1] + u * n_dr * stride) = lo;
                *reinterpret_cast<h4 *>(xs + wr1[u & 1] + u * n_dr * stride) = hi;
                if constexpr (HOLD) {
                    // the registers of a row go to the same row of the next 64 the moment they are free: the memory
                    // pipe stays busy through the normalisation and the products
                    if (u < PF && half + 1 < nhalf) {
                        const int tok = min(next_row + u * n_dr, S - 1);
                        const unsigned off = (unsigned)tok * (unsigned)(in * 4) + next_off;
                        s32[u][0] = *reinterpret_cast<const f4 *>(xbase + off);
                        s32[u][1] = *reinterpret_cast<const f4 *>(xbase + off + 2u * (unsigned)in);
                    }
                }
            }
        }
        if constexpr (!HOLD) {
            request_slots(0);  // (after the rows: they and a part of the slots do not fit in registers together)
            if (half + 1 < nhalf) request_rows(half + 1, i0{}, iPF{});  // in flight during the products
        }
        __syncthreads();
        // ---- the wave's block-row times the four 16-token tiles of the staged rows
        unsigned kx_now = kx, sel_now = (unsigned)sel << 4;
        asm volatile("" : "+v"(kx_now), "+v"(sel_now));
        f4 acc[4];
#pragma unroll
        for (int mt = 0; mt < 4; mt++) acc[mt] = f4{0.f, 0.f, 0.f, 0.f};
        // Q, K: features x tokens (a lane ends with four features of a token); V: tokens x features (a lane ends with
        // four consecutive tokens of a feature, a piece of a V^T row).  Two loops under one wave-uniform branch: as a
        // select per product the compiler computes both orientations.
        auto products = [&](auto swapped, auto first) {
            constexpr int P0 = decltype(first)::value;
#pragma unroll
            for (int p = 0; p < WN; p++) {
                if ((p & 3) == 0 && P0 + p >= nsl) break;  // wave-uniform: nothing was fetched beyond
                const unsigned o = ((offs[P0 + p] >> sel_now) & 0xffffu) ^ kx_now;
#pragma unroll
                for (int mt = 0; mt < 4; mt++) {
                    const h8 x = *reinterpret_cast<const h8 *>(xs + (unsigned)((mt * 16 + r16) * stride) + o);
                    if constexpr (decltype(swapped)::value) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x, w[p], acc[mt], 0, 0, 0);
                    else acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[p], x, acc[mt], 0, 0, 0);
                }
            }
        };
        if (part < 2) products(std::false_type{}, i0{});
        else products(std::true_type{}, i0{});
        auto next_part = [&](auto first) {
            __builtin_amdgcn_sched_barrier(0);  // not above the products that still read the registers' last contents
            request_slots(decltype(first)::value);
            if (part < 2) products(std::false_type{}, first);
            else products(std::true_type{}, first);
        };
        if constexpr (NPASS >= 2) next_part(std::integral_constant<int, WN>{});
        if constexpr (NPASS >= 3) next_part(std::integral_constant<int, 2 * WN>{});
        if constexpr (NPASS >= 4) next_part(std::integral_constant<int, 3 * WN>{});
        static_assert(NPASS <= 4, "parts of the slots");
        float bq[4];
        if constexpr (FOLDED) {
#pragma unroll
            for (int e = 0; e < 4; e++) bq[e] = part < 2 ? bias_f[e] : bias_f[0];
        } else if (part < 2) {
            const h4 t = __builtin_bit_cast(h4, bias_bits);
#pragma unroll
            for (int e = 0; e < 4; e++) bq[e] = (float)t[e];
        } else {
            const float t = (float)__builtin_bit_cast(_Float16, (unsigned short)bias_bits.x);
#pragma unroll
            for (int e = 0; e < 4; e++) bq[e] = t;
        }
#pragma unroll
        for (int mt = 0; mt < 4; mt++) {
            const h4 v = {(_Float16)(acc[mt][0] + bq[0]), (_Float16)(acc[mt][1] + bq[1]), (_Float16)(acc[mt][2] + bq[2]),
                          (_Float16)(acc[mt][3] + bq[3])};
            if (part < 2) {
                _Float16 *dst = (part == 0 ? Qs : Ks) + (tokbase + mt * 16 + r16) * L::ldk + sub * 16 + 4 * g;
                *reinterpret_cast<h4 *>(dst) = v;
            } else {
                // keys 4kg .. 4kg + 3, kg = 16 half + 4 mt + g, at their place in the V^T row of feature 16 sub + r16
                const int pos = (32 * (2 * half + (mt >> 1)) + 8 * g + 4 * (mt & 1)) ^ vt_swizzle<HD>(sub);
                *reinterpret_cast<h4 *>(Vt + (sub * 16 + r16) * L::ldvt + pos) = v;
            }
        }
        if (half + 1 < nhalf) __syncthreads();  // every wave is done with the staged rows
    }
    __syncthreads();  // Q, K and V^T of the head are complete
    if (wave * 16 >= S) return;  // 16 queries per wave: the waves beyond the sequence are done

    // ---- the attention core on the staged head (one key block: S <= 128)
    int q[QT] = {wave * 16 + r16};
    bool q_ok[QT] = {q[0] < S};
    int klimit = S;
    if (a.lens) klimit = min(S, max(a.lens[b], 0));
    if (a.causal) klimit = min(klimit, (wave + 1) * 16);
    const int vlive = HD;
    h8 qf[QT][KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[0][ks] = *reinterpret_cast<const h8 *>(Qs + (wave * 16 + r16) * L::ldk + 32 * ks + 8 * g);
    f4 o[QT][DB];
    float m_run[QT] = {-INFINITY}, l_part[QT] = {0.0f};
#pragma unroll
    for (int d = 0; d < DB; d++) o[0][d] = f4{0.f, 0.f, 0.f, 0.f};
    const int k0 = 0;
    if (klimit > 0) {
#include "attention_core.inc"
        const bool plain = a.mask == nullptr && a.scale_log2e > 0.0f && !a.causal;
        if (plain) multiply(std::true_type{});
        else multiply(std::false_type{});
    }
    float l = rows_sum(l_part[0]);
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    if (q_ok[0]) {
        _Float16 *zp = a.Z + (row0 + q[0]) * a.ldz + h * HD + 4 * g;
#pragma unroll
        for (int d = 0; d < DB; d++) {
            h4 out;
#pragma unroll
            for (int j = 0; j < 4; j++) out[j] = (_Float16)(o[0][d][j] * inv);
            *reinterpret_cast<h4 *>(zp + 16 * d) = out;
        }
    }
}

template <int CAP, int PF, int NPASS, bool FOLDED> static int launch_qkv_mha_f(const QkvMhaArgs &qa, size_t lds, hipStream_t stream) {
    auto kernel = qkv_mha_kernel<CAP, PF, NPASS, FOLDED>;
    static bool raised = false;  // per instantiation
    if (!raised) {
        ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised = true;
    }
    const int rounds = (qa.B + kXcds - 1) / kXcds;
    kernel<<<dim3((unsigned)(rounds * kXcds * qa.m.nh)), kQkvWaves * 64, lds, stream>>>(qa);
    return check_launch("qkv_mha_kernel");
}
// PFF, NPF: rows requested ahead and parts of the slots in the folded form, whose register needs differ
template <int CAP, int PF, int NPASS, int PFF = PF, int NPF = NPASS>
static int launch_qkv_mha(const QkvMhaArgs &qa, size_t lds, hipStream_t stream) {
    return qa.bias32 ? launch_qkv_mha_f<CAP, PFF, NPF, true>(qa, lds, stream) : launch_qkv_mha_f<CAP, PF, NPASS, false>(qa, lds, stream);
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


int et_norm_qkv_mha_f32in_supported(int B, int S, int in, int nhead, int hd) {
    return B > 0 && S > 0 && S % 16 == 0 && S <= kKeyBlock && in == 768 && nhead > 0 && hd == 64 ? 1 : 0;
}

// gamma != nullptr: the pack holds W diag(gamma) and, as binary32, bias + W beta
static int qkv_heads_pack_build(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, const et_f16 *bias,
                                const et_f16 *gamma, const et_f16 *beta, int in, int nhead, et_bsr_pack *pack) {
    ET_REQUIRE(pack != nullptr, ET_ERR_INVALID_ARG, "et_qkv_heads_pack_create: pack is NULL");
    *pack = nullptr;
    ET_REQUIRE(row_ptr && col_idx && tiles, ET_ERR_INVALID_ARG, "et_qkv_heads_pack_create: NULL pointer");
    ET_REQUIRE(et_norm_qkv_mha_f32in_supported(1, 16, in, nhead, 64) == 1, ET_ERR_UNSUPPORTED,
               "et_qkv_heads_pack_create: in=%d nhead=%d outside the fused form (768-wide input, heads of 64)", in, nhead);
    const int nbr = 3 * nhead * 4, bc = in / 16;  // block-rows of W_qkv: Q | K | V, four per head each
    std::vector<int32_t> rp((size_t)nbr + 1);
    ET_HIP(hipMemcpy(rp.data(), row_ptr, rp.size() * 4, hipMemcpyDeviceToHost));
    ET_REQUIRE(rp[0] == 0, ET_ERR_INVALID_ARG, "et_qkv_heads_pack_create: row_ptr must start at 0");
    for (int r = 0; r < nbr; r++)
        ET_REQUIRE(rp[(size_t)r + 1] >= rp[(size_t)r], ET_ERR_INVALID_ARG, "et_qkv_heads_pack_create: row_ptr decreases");
    const int ntile = rp[(size_t)nbr];
    std::vector<int32_t> ci((size_t)std::max(ntile, 1));
    if (ntile) ET_HIP(hipMemcpy(ci.data(), col_idx, (size_t)ntile * 4, hipMemcpyDeviceToHost));
    for (int t = 0; t < ntile; t++)
        ET_REQUIRE(ci[(size_t)t] >= 0 && ci[(size_t)t] < bc, ET_ERR_INVALID_ARG,
                   "et_qkv_heads_pack_create: column-tile index %d of tile %d outside [0, %d)", ci[(size_t)t], t, bc);
    int most = 1;
    for (int r = 0; r < nbr; r++) most = std::max(most, (rp[(size_t)r + 1] - rp[(size_t)r] + 1) / 2);
    const int cap = most <= 8 ? 8 : most <= 12 ? 12 : most <= 16 ? 16 : 24;  // the kernel's instantiations
    ET_REQUIRE(cap <= 24, ET_ERR_UNSUPPORTED, "et_qkv_heads_pack_create: a block-row of %d slots exceeds a wave's 24", most);
    const size_t nslab = (size_t)nhead * kQkvWaves;
    std::vector<int32_t> order(nslab * cap * 2, -1), tab(nslab, 0);
    std::vector<uint32_t> off(nslab * cap, 0);
    for (int h = 0; h < nhead; h++) {
        for (int wv = 0; wv < kQkvWaves; wv++) {
            const int rb = (wv >> 2) * (nhead * 4) + 4 * h + (wv & 3);
            const size_t slab = (size_t)h * kQkvWaves + wv;
            int p = 0;
            for (int t = rp[(size_t)rb]; t < rp[(size_t)rb + 1]; t += 2, p++) {
                const bool two = t + 1 < rp[(size_t)rb + 1];
                order[(slab * cap + p) * 2] = t;
                order[(slab * cap + p) * 2 + 1] = two ? t + 1 : -1;
                off[slab * cap + p] = (uint32_t)(ci[(size_t)t] * 32) | ((uint32_t)(ci[(size_t)(two ? t + 1 : t)] * 32) << 16);
            }
            tab[slab] = p;
        }
    }
    std::unique_ptr<et_bsr_pack_s> p(new (std::nothrow) et_bsr_pack_s);  // freed on every early return
    ET_REQUIRE(p != nullptr, ET_ERR_ALLOC, "et_qkv_heads_pack_create: out of host memory");
    p->in = in;
    p->out = nbr * 16;
    p->mt = 4;
    p->ngroups = nhead;
    p->nwave = kQkvWaves;
    p->cap = cap;
    p->flags = ET_PACK_QKV_HEADS;
    p->lds = (size_t)kQkvRows * in * 2 + (size_t)(2 * MhaLds<64>::k_halfs + MhaLds<64>::vt_halfs) * sizeof(_Float16) +
             kKeyBlock * sizeof(float2) + (size_t)in * 4;
    int s = ET_OK;
    if (gamma) {
        // W diag(gamma) as binary16 tiles and bias + W beta as binary32, made here from host copies
        const size_t nvals = (size_t)ntile * 256, nout = (size_t)nbr * 16;
        std::vector<_Float16> ht(std::max<size_t>(nvals, 1)), hg((size_t)in), hb((size_t)in), hbias(nout);
        std::vector<float> b32(nout, 0.0f);
        if (nvals) ET_HIP(hipMemcpy(ht.data(), tiles, nvals * 2, hipMemcpyDeviceToHost));
        ET_HIP(hipMemcpy(hg.data(), gamma, (size_t)in * 2, hipMemcpyDeviceToHost));
        ET_HIP(hipMemcpy(hb.data(), beta, (size_t)in * 2, hipMemcpyDeviceToHost));
        if (bias) {
            ET_HIP(hipMemcpy(hbias.data(), bias, nout * 2, hipMemcpyDeviceToHost));
            for (size_t o = 0; o < nout; o++) b32[o] = (float)hbias[o];
        }
        for (int rb = 0; rb < nbr; rb++) {
            for (int t = rp[(size_t)rb]; t < rp[(size_t)rb + 1]; t++) {
                const size_t c0 = (size_t)ci[(size_t)t] * 16;
                for (int r = 0; r < 16; r++) {
                    float dot = 0.0f;
                    for (int c = 0; c < 16; c++) {
                        _Float16 &w = ht[(size_t)t * 256 + (size_t)r * 16 + c];  // tile row r = output feature, column c = input
                        dot += (float)w * (float)hb[c0 + c];
                        w = (_Float16)((float)w * (float)hg[c0 + c]);
                    }
                    b32[(size_t)rb * 16 + r] += dot;
                }
            }
        }
        void *d_scaled = nullptr;
        s = check_hip(hipMalloc(&d_scaled, std::max<size_t>(nvals * 2, 16)), "hipMalloc");
        if (s == ET_OK && nvals) s = check_hip(hipMemcpy(d_scaled, ht.data(), nvals * 2, hipMemcpyHostToDevice), "hipMemcpy");
        if (s == ET_OK) s = pack_upload(*p, off, tab, order, static_cast<const et_f16 *>(d_scaled));
        (void)hipFree(d_scaled);
        if (s == ET_OK) s = et_malloc(&p->bias32, nout * 4);
        if (s == ET_OK) s = check_hip(hipMemcpy(p->bias32, b32.data(), nout * 4, hipMemcpyHostToDevice), "hipMemcpy");
    } else {
        s = pack_upload(*p, off, tab, order, tiles);
    }
    if (s != ET_OK) return s;
    *pack = p.release();
    return ET_OK;
}

int et_qkv_heads_pack_create(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, int in, int nhead,
                             et_bsr_pack *pack) {
    return qkv_heads_pack_build(row_ptr, col_idx, tiles, nullptr, nullptr, nullptr, in, nhead, pack);
}

int et_qkv_heads_pack_create_folded(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, const et_f16 *bias,
                                    const et_f16 *gamma, const et_f16 *beta, int in, int nhead, et_bsr_pack *pack) {
    ET_REQUIRE(gamma && beta, ET_ERR_INVALID_ARG, "et_qkv_heads_pack_create_folded: gamma and beta must be set");
    return qkv_heads_pack_build(row_ptr, col_idx, tiles, bias, gamma, beta, in, nhead, pack);
}

int et_norm_qkv_mha_f32in(et_bsr_pack pack, const float *V, const float *stats, int stat_groups, const et_f16 *gamma,
                          const et_f16 *beta, float eps, float *fin_out, const et_f16 *bias_qkv, et_f16 *Z, int ldz,
                          const et_f16 *mask, const int32_t *lens, int B, int S, float scale, int flags, et_stream stream) {
    ET_REQUIRE(pack != nullptr && (pack->flags & ET_PACK_QKV_HEADS), ET_ERR_INVALID_ARG,
               "et_norm_qkv_mha_f32in: needs a pack from et_qkv_heads_pack_create");
    const bool folded = pack->bias32 != nullptr;
    ET_REQUIRE(V && stats && Z && (folded || (gamma && beta)), ET_ERR_INVALID_ARG, "et_norm_qkv_mha_f32in: NULL pointer");
    const int nh = pack->ngroups, in = pack->in;
    ET_REQUIRE(B >= 0 && et_norm_qkv_mha_f32in_supported(std::max(B, 1), S, in, nh, 64) == 1, ET_ERR_UNSUPPORTED,
               "et_norm_qkv_mha_f32in: B=%d S=%d: sequences of a multiple of 16 up to %d tokens", B, S, kKeyBlock);
    ET_REQUIRE(stat_groups >= 1 && stat_groups <= kMaxStatGroups, ET_ERR_INVALID_ARG, "et_norm_qkv_mha_f32in: stat_groups=%d",
               stat_groups);
    ET_REQUIRE((flags & ~ET_MHA_CAUSAL) == 0, ET_ERR_INVALID_ARG, "et_norm_qkv_mha_f32in: flags=%d", flags);
    ET_REQUIRE(ldz >= nh * 64 && ldz % 4 == 0 && (reinterpret_cast<uintptr_t>(Z) & 7) == 0 &&
                   (reinterpret_cast<uintptr_t>(V) & 15) == 0,
               ET_ERR_UNSUPPORTED, "et_norm_qkv_mha_f32in: Z must be 8-byte and V 16-byte aligned, ldz >= nhead * 64");
    if (B == 0) return ET_OK;
    QkvMhaArgs qa{};
    qa.m.Z = reinterpret_cast<_Float16 *>(Z);
    qa.m.mask = reinterpret_cast<const _Float16 *>(mask);
    qa.m.lens = lens;
    qa.m.ldz = ldz;
    qa.m.S = S;
    qa.m.nh = nh;
    qa.m.hd = 64;
    qa.m.nbh = B * nh;
    qa.m.scale_log2e = scale * kLog2e;
    qa.m.causal = (flags & ET_MHA_CAUSAL) ? 1 : 0;
    qa.pw = static_cast<const _Float16 *>(pack->pw);
    qa.poff = static_cast<const uint32_t *>(pack->poff);
    qa.pn = static_cast<const int32_t *>(pack->ptab);
    qa.bias = reinterpret_cast<const _Float16 *>(bias_qkv);
    qa.cap = pack->cap;
    qa.in = in;
    qa.T = B * S;
    qa.B = B;
    qa.X32 = V;
    qa.st_in = stats;
    qa.st_groups = stat_groups;
    qa.gamma = reinterpret_cast<const _Float16 *>(gamma);
    qa.beta = reinterpret_cast<const _Float16 *>(beta);
    qa.eps = eps;
    qa.fin_out = fin_out;
    qa.bias32 = static_cast<const float *>(pack->bias32);
    switch (pack->cap) {
        case 8: return launch_qkv_mha<8, 8, 1>(qa, pack->lds, as_stream(stream));
        case 12: return launch_qkv_mha<12, 4, 1, 8>(qa, pack->lds, as_stream(stream));
        case 16: return launch_qkv_mha<16, 4, 2, 4, 4>(qa, pack->lds, as_stream(stream));
        case 24: return launch_qkv_mha<24, 4, 3>(qa, pack->lds, as_stream(stream));
        default: return fail(ET_ERR_INVALID_ARG, "et_norm_qkv_mha_f32in: no kernel for %d slots per wave", pack->cap);
    }
}

}  // extern "C"
