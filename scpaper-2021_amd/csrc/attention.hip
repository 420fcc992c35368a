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
#include <atomic>
#include <memory>
#include <mutex>
#include <new>
#include <vector>

#include <type_traits>

#include "common.hip.h"
#include "bsr_packed.hip.h"
#include "../../include/et_tuning.h"

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
// Eight bytes stored and sixteen bytes loaded at device scope: the access goes past the L2 of the issuing
// accelerator die (each die has its own, and they are not kept coherent with one another inside a launch), so
// a workgroup on another die reads what was written without either side writing back or invalidating a
// whole cache.
__device__ __forceinline__ void store_device_scope(_Float16 *p, h4 v) {
    __hip_atomic_store(reinterpret_cast<unsigned long long *>(p), __builtin_bit_cast(unsigned long long, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ h8 load_device_scope(const _Float16 *p) {
    typedef unsigned long long u2 __attribute__((ext_vector_type(2)));
    const unsigned long long *q = reinterpret_cast<const unsigned long long *>(p);
    u2 r;
    r[0] = __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    r[1] = __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_bit_cast(h8, r);
}

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
    constexpr bool kCoherentZ = false;
#include "attention_body.inc"
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


// ---- attention and the tile-sparse output projection in one launch ------------------------------------
// E.T.'s O-fused attention (Attention/kernel_fuseO.cu:138-243) runs the attention of every (head, query
// strip), waits at a grid-wide barrier of a cooperative launch and then multiplies Z with the tile-sparse
// W_O.  Here nothing waits: a workgroup runs the fused attention of its (sequence, head, query strip),
// stores its slice of Z, and adds one to the arrival count of its (sequence, query strip).  The workgroup
// whose addition completes the count — all heads of those tokens are in memory — stages the finished rows of
// Z (and the weight's row pointers and column indices) in LDS and multiplies them with W_O: a wave per block-row
// of the weight, two tiles per MFMA, the tile
// fragments of the next three groups of six tile pairs on their way while a group is multiplied.  Every other
// workgroup has left by then, so the launch needs no co-residency and no spinning, and the projection of
// the first finished strips overlaps the attention of the rest.  The last arriver puts the count back to
// zero: the counts are zero before and after every launch.
// What it costs: the projecting workgroup takes in the whole weight by itself (236 KB for 768 x 768 at 80 %
// sparsity; a compute unit takes in 20 GB/s of lines its L2 does not hold, 90 GB/s of lines it does), and the
// loop measures 1.1 us per group of six tile pairs whatever the number of live tiles in it, 13 groups per wave
// (as compiled it still waits for all of its requests once per turn of the four register sets): 14 us for the
// projection of a strip, against 4 us for a launch of its own that spreads the weight over a few hundred
// workgroups.  25 against 8 us for one sequence of 128 tokens, 28 against 9 us for eight.  The class layer
// therefore keeps the two launches; this entry point is for callers that need one.
struct FuseOArgs {
    const int32_t *row_ptr, *col_idx;  // W_O [emdim x nh*hd] as 16x16 tiles (tile rows = output features)
    const _Float16 *tiles;
    const _Float16 *bias;              // [emdim] or nullptr
    _Float16 *out;                     // [B*S x emdim]
    int emdim;
    unsigned *arrived;                 // [B * query strips]
};

constexpr int kFuseOPairs = 6;            // tile pairs of a block-row requested together
constexpr int kFuseOCounters = 16384;     // arrival counts built into the library (per device)
static __device__ __align__(256) unsigned fuseo_arrived[kFuseOCounters];

template <int HD, int NW, int QT>
__global__ __launch_bounds__(64 * NW) void mha_fuseo_kernel(const MhaArgs a, const FuseOArgs f) {
    constexpr bool COMPACT = false;
    constexpr bool kCoherentZ = true;
#include "attention_body.inc"
    // ---- arrival.  Z was stored at device scope, and such a store counts as complete only once it has
    // reached the memory side: when every wave's stores are complete the count moves.  A device-wide fence
    // would order the same, but it writes back the whole L2 of the die and invalidates it, 2.4 us for every
    // workgroup of the launch, one after the other on a die.
    __shared__ unsigned is_last;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // also: every wave is done with the staged K and V
    if (threadIdx.x == 0) {
        unsigned *cnt = f.arrived + (size_t)b * qstrips + qstrip;
        const unsigned before = __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = before + 1u == (unsigned)a.nh;
        if (last) __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = last ? 1u : 0u;
    }
    __syncthreads();
    if (!is_last) return;

    // ---- the projection of the strip.  Order of the requests: the row pointers, the rows of Z, then the first
    // tile fragments.
    constexpr int TT = NW * QT;  // 16-token tiles of the strip
    constexpr int P = kFuseOPairs;
    constexpr int ZU = 24;       // 16-byte vectors of Z a thread requests together (768-wide rows on 4 waves: all of them)
    const int nbr = f.emdim / 16;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    // the wave owns block-rows wave, wave + NW, ...: its k-th row is wave + NW k.  The row pointers go to LDS
    // behind the rows of Z: a load of them between the tile requests would have to be waited for, and the
    // requests made before it with it (loads return in order).
    const int nrows = nbr > wave_u ? (nbr - wave_u + NW - 1) / NW : 0;

    const int width = a.nh * hd;       // a multiple of 16
    const int ldzs = width + 8;        // halfs; rows 16 bytes apart in the banks
    _Float16 *Zs = reinterpret_cast<_Float16 *>(smem_raw);
    const int vpr = width / 8;
    const int nvec = kStripQ * vpr;
    h8 zt[ZU];
    auto z_request = [&](int v0) {
#pragma unroll
        for (int i = 0; i < ZU; i++) {
            const int v = min(v0 + i * nthr + (int)threadIdx.x, nvec - 1);
            const int r = v / vpr, c = v - r * vpr;
            const int row = min(qstrip * kStripQ + r, S - 1);
            zt[i] = load_device_scope(a.Z + (row0 + row) * a.ldz + c * 8);
        }
    };
    // rows past the sequence as zeros.  Every store is unconditional (surplus threads repeat the last vector):
    // a store under a branch leaves its load unwaited on the other path as far as the compiler can tell, and
    // the first write to that register in the projection loop then waits for every outstanding request.
    auto z_place = [&](int v0) {
#pragma unroll
        for (int i = 0; i < ZU; i++) {
            const int v = min(v0 + i * nthr + (int)threadIdx.x, nvec - 1);
            const int r = v / vpr, c = v - r * vpr;
            *reinterpret_cast<h8 *>(Zs + r * ldzs + c * 8) =
                (qstrip * kStripQ + r < S) ? zt[i] : h8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    };
    int *rps = reinterpret_cast<int *>(Zs + kStripQ * ldzs);
    for (int i0 = 0; i0 <= nbr; i0 += nthr) {  // one pass up to 64 NW - 1 block-rows
        const int i = min(i0 + (int)threadIdx.x, nbr);
        const int v = f.row_ptr[i];
        if (i0 == 0) {
            z_request(0);
            __builtin_amdgcn_sched_barrier(0);
        }
        rps[i] = v;
    }
    __syncthreads();
    // ... and the column indices behind them (room for every tile of a full weight): read from LDS where they
    // are used, they do not take part in the count of outstanding memory requests
    int *cols = rps + nbr + 1;
    const int ntile = min(rps[nbr], nbr * (width / 16));
    for (int i = threadIdx.x; i < ntile; i += nthr) cols[i] = f.col_idx[i];
    if (ntile == 0 && threadIdx.x == 0) cols[0] = 0;

    // a weight without tiles: the loads below go to valid dummy addresses and meet the zero operand
    const _Float16 *tbase = ntile > 0 ? f.tiles : a.Z + row0 * a.ldz;
    const int jmax = max(ntile - 1, 0);
    const int half_k = 8 * (g & 1), second = g >> 1;
    const h8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    // chunk = up to P tile pairs of one block-row: (row of the wave, first tile, end of the row's tiles);
    // three chunks are on their way while one is multiplied
    struct Chunk {
        int k, j, j1;
    };
    // (the row's bias comes with every chunk: requested where the row ends, it would be waited for on the
    // spot, and with it every request made before it)
    const _Float16 *bbase = f.bias ? f.bias + 4 * g : tbase;
    const int bstep = f.bias ? 16 : 0;
    auto request = [&](const Chunk &ch, h8 (&w)[P], h4 &bq) {
        bq = *reinterpret_cast<const h4 *>(bbase + (size_t)min(wave_u + NW * ch.k, nbr - 1) * bstep);
#pragma unroll
        for (int p = 0; p < P; p++) {
            const int jt = ch.j + 2 * p + second;
            const int jc = min(jt, jmax);
            w[p] = *reinterpret_cast<const h8 *>(tbase + (size_t)jc * 256 + r16 * 16 + half_k);
        }
    };
    auto after = [&](const Chunk &ch) {  // the rest of the row, or the start of the wave's next row
        Chunk nx = {ch.k, ch.j + 2 * P, ch.j1};
        if (nx.j >= ch.j1 && ch.k < nrows) {  // wave-uniform
            nx.k = ch.k + 1;
            if (nx.k < nrows) {
                nx.j = __builtin_amdgcn_readfirstlane(rps[wave_u + NW * nx.k]);
                nx.j1 = __builtin_amdgcn_readfirstlane(rps[wave_u + NW * nx.k + 1]);
            } else {
                nx.j = nx.j1 = ch.j1;  // past the end: requests that meet nothing
            }
        }
        return nx;
    };
    h8 w0[P], w1[P], w2[P], w3[P];
    h4 b0, b1, b2, b3;
    Chunk ch0 = {0, 0, 0};
    if (nrows > 0) {
        ch0.j = __builtin_amdgcn_readfirstlane(rps[wave_u]);
        ch0.j1 = __builtin_amdgcn_readfirstlane(rps[wave_u + 1]);
    }
    // (the first tile requests wait until the rows of Z are placed: with both in registers at once the
    // kernel is out of registers, and the compiler then reuses a register a request is still due to fill,
    // which it can only do after waiting for every request)
    z_place(0);
    for (int v0 = ZU * nthr; v0 < nvec; v0 += ZU * nthr) {
        z_request(v0);
        z_place(v0);
    }
    __builtin_amdgcn_sched_barrier(0);
    request(ch0, w0, b0);
    Chunk ch1 = after(ch0);
    request(ch1, w1, b1);
    Chunk ch2 = after(ch1);
    request(ch2, w2, b2);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();

    // ---- out[token][16n + ..] = bias + sum over the tiles of block-row n
    f4 acc[TT];
#pragma unroll
    for (int tt = 0; tt < TT; tt++) acc[tt] = f4{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const Chunk &cur, const Chunk &nxt, const h8 (&w)[P], const h4 &bq) {
        // the Z fragments of two tile pairs are read together and multiplied then: one wave per SIMD has
        // nothing else to cover the LDS latency with, and read by read it adds up to most of the projection
        constexpr int PH = 2;
#pragma unroll
        for (int p0 = 0; p0 < P; p0 += PH) {
            h8 zf[PH][TT];
#pragma unroll
            for (int pp = 0; pp < PH; pp++) {
                const bool live = cur.j + 2 * (p0 + pp) + second < cur.j1;
                const int col = cols[min(cur.j + 2 * (p0 + pp) + second, jmax)];
                const _Float16 *zp = Zs + r16 * ldzs + col * 16 + half_k;
#pragma unroll
                for (int tt = 0; tt < TT; tt++) zf[pp][tt] = *reinterpret_cast<const h8 *>(zp + tt * 16 * ldzs);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int pp = 0; pp < PH; pp++) {
                const bool live = cur.j + 2 * (p0 + pp) + second < cur.j1;
                const h8 wf = live ? w[p0 + pp] : zero8;
#pragma unroll
                for (int tt = 0; tt < TT; tt++)
                    acc[tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, zf[pp][tt], acc[tt], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (nxt.k != cur.k) {  // the row is complete: lane holds features 16n + 4g .. +3 of token r16 of every tile
            const int n = wave_u + NW * cur.k;
            float bv[4];
#pragma unroll
            for (int j = 0; j < 4; j++) bv[j] = f.bias ? (float)bq[j] : 0.0f;
#pragma unroll
            for (int tt = 0; tt < TT; tt++) {
                const int row = qstrip * kStripQ + tt * 16 + r16;
                h4 o4;
#pragma unroll
                for (int j = 0; j < 4; j++) o4[j] = (_Float16)(acc[tt][j] + bv[j]);
                if (row < S) *reinterpret_cast<h4 *>(f.out + (row0 + row) * f.emdim + n * 16 + 4 * g) = o4;
                acc[tt] = f4{0.f, 0.f, 0.f, 0.f};
            }
        }
    };
    // The four register sets take turns (a set is requested again right after it was multiplied); moving
    // the fragments from set to set instead would make every turn wait for all of them.
    Chunk ch3 = ch2;
    // (scheduling barriers: left alone, the compiler moves requests down to where their values are used and
    // then has to wait for all of them)
    while (true) {  // every exit is wave-uniform
        if (ch0.k >= nrows) break;
        ch3 = after(ch2);
        request(ch3, w3, b3);
        __builtin_amdgcn_sched_barrier(0);
        multiply(ch0, ch1, w0, b0);
        __builtin_amdgcn_sched_barrier(0);
        if (ch1.k >= nrows) break;
        ch0 = after(ch3);
        request(ch0, w0, b0);
        __builtin_amdgcn_sched_barrier(0);
        multiply(ch1, ch2, w1, b1);
        __builtin_amdgcn_sched_barrier(0);
        if (ch2.k >= nrows) break;
        ch1 = after(ch0);
        request(ch1, w1, b1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(ch2, ch3, w2, b2);
        __builtin_amdgcn_sched_barrier(0);
        if (ch3.k >= nrows) break;
        ch2 = after(ch1);
        request(ch2, w2, b2);
        __builtin_amdgcn_sched_barrier(0);
        multiply(ch3, ch0, w3, b3);
        __builtin_amdgcn_sched_barrier(0);
    }
}

static std::mutex g_fuseo_mutex;
static std::atomic<unsigned *> g_fuseo_counts[64];

// Device address of the arrival counts on the current device (looked up on first use; the array is
// zero when the library is loaded and every launch leaves it zero).
static int fuseo_counts(unsigned **out) {
    int dev = -1;
    ET_HIP(hipGetDevice(&dev));
    ET_REQUIRE(dev >= 0 && dev < 64, ET_ERR_UNSUPPORTED, "et_mha_fuseo_f16: device ordinal %d", dev);
    unsigned *p = g_fuseo_counts[dev].load(std::memory_order_acquire);
    if (!p) {
        std::lock_guard<std::mutex> lock(g_fuseo_mutex);
        p = g_fuseo_counts[dev].load(std::memory_order_relaxed);
        if (!p) {
            void *sym = nullptr;
            ET_HIP(hipGetSymbolAddress(&sym, HIP_SYMBOL(fuseo_arrived)));
            ET_REQUIRE(sym != nullptr, ET_ERR_LAUNCH, "et_mha_fuseo_f16: hipGetSymbolAddress returned NULL");
            p = static_cast<unsigned *>(sym);
            g_fuseo_counts[dev].store(p, std::memory_order_release);
        }
    }
    *out = p;
    return ET_OK;
}

// row pointers and (room for) the column index of every tile of a full weight, kept in LDS behind the rows of Z
static size_t fuseo_index_bytes(int width, int emdim) {
    return ((size_t)(emdim / 16) + 1 + (size_t)(emdim / 16) * (width / 16)) * sizeof(int);
}
constexpr size_t kLdsPerWorkgroup = 160 * 1024 - 256;  // the arrival flag is a static allocation of its own

template <int HD, int NW>
static int launch_fuseo_nw(const MhaArgs &args, const FuseOArgs &fo, hipStream_t stream) {
    auto kernel = mha_fuseo_kernel<HD, NW, 1>;
    const size_t strip = (size_t)16 * NW * (args.nh * args.hd + 8) * sizeof(_Float16) + fuseo_index_bytes(args.nh * args.hd, fo.emdim);
    const size_t lds = std::max(MhaLds<HD>::bytes, strip);
    ET_REQUIRE(lds <= kLdsPerWorkgroup, ET_ERR_UNSUPPORTED, "et_mha_fuseo_f16: a strip of %d rows of Z (%zu B) exceeds LDS",
               16 * NW, strip);
    static std::atomic<size_t> raised{64 * 1024};
    if (lds > raised.load(std::memory_order_acquire)) {
        ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)kLdsPerWorkgroup));
        raised.store(kLdsPerWorkgroup, std::memory_order_release);
    }
    const int qstrips = (args.S + 16 * NW - 1) / (16 * NW);
    const int rounds = (args.nbh + kXcds - 1) / kXcds;
    kernel<<<dim3((unsigned)(rounds * kXcds * qstrips)), 64 * NW, lds, stream>>>(args, fo);
    return check_launch("mha_fuseo_kernel");
}

// waves: 0 picks; 1, 2 or 4 waves (16, 32 or 64 tokens per workgroup and projection strip)
template <int HD>
static int launch_fuseo(const MhaArgs &args, const FuseOArgs &fo, int waves, hipStream_t stream) {
    const int qblocks = args.S / 16;
    const size_t row_bytes = (size_t)(args.nh * args.hd + 8) * sizeof(_Float16);
    if (waves == 0) {
        waves = qblocks % 4 == 0 ? 4 : qblocks % 2 == 0 ? 2 : 1;
        while (waves > 1 && 16 * waves * row_bytes + fuseo_index_bytes(args.nh * args.hd, fo.emdim) > kLdsPerWorkgroup) waves >>= 1;
    }
    if (waves == 4) return launch_fuseo_nw<HD, 4>(args, fo, stream);
    if (waves == 2) return launch_fuseo_nw<HD, 2>(args, fo, stream);
    return launch_fuseo_nw<HD, 1>(args, fo, stream);
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

int et_mha_fuseo_f16_geom(const et_f16 *Q, const et_f16 *K, const et_f16 *V, int ldq, int ldk, int ldv, et_f16 *Z,
                          int ldz, const et_f16 *mask, const int32_t *lens, int B, int S, int nh, int hd,
                          float scale, int flags, const int32_t *o_row_ptr, const int32_t *o_col_idx,
                          const et_f16 *o_tiles, const et_f16 *o_bias, et_f16 *out, int emdim, int waves,
                          et_stream stream) {
    ET_REQUIRE(Q && K && V && Z && o_row_ptr && out, ET_ERR_INVALID_ARG, "et_mha_fuseo_f16: NULL pointer");
    ET_REQUIRE(B >= 0 && S > 0 && nh > 0 && hd > 0 && emdim > 0, ET_ERR_INVALID_ARG,
               "et_mha_fuseo_f16: B=%d S=%d nh=%d hd=%d emdim=%d", B, S, nh, hd, emdim);
    ET_REQUIRE((flags & ~ET_MHA_CAUSAL) == 0, ET_ERR_INVALID_ARG, "et_mha_fuseo_f16: flags=%d", flags);
    ET_REQUIRE(waves == 0 || waves == 1 || waves == 2 || waves == 4, ET_ERR_INVALID_ARG,
               "et_mha_fuseo_f16: waves=%d", waves);
    ET_REQUIRE(S % 16 == 0, ET_ERR_UNSUPPORTED, "et_mha_fuseo_f16: S=%d must be a multiple of 16", S);
    ET_REQUIRE(hd % 8 == 0 && hd <= 128, ET_ERR_UNSUPPORTED,
               "et_mha_fuseo_f16: head dim %d must be a multiple of 8, at most 128", hd);
    const int width = nh * hd;
    ET_REQUIRE(width % 16 == 0 && emdim % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_mha_fuseo_f16: nh*hd=%d and emdim=%d must be multiples of 16", width, emdim);
    ET_REQUIRE(ldq >= width && ldk >= width && ldv >= width && ldz >= width, ET_ERR_INVALID_ARG,
               "et_mha_fuseo_f16: row strides (%d %d %d %d) smaller than nh*hd=%d", ldq, ldk, ldv, ldz, width);
    ET_REQUIRE(ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0 && ldz % 8 == 0, ET_ERR_UNSUPPORTED,
               "et_mha_fuseo_f16: row strides must keep 16-byte alignment");
    ET_REQUIRE(((reinterpret_cast<uintptr_t>(Q) | reinterpret_cast<uintptr_t>(K) | reinterpret_cast<uintptr_t>(V) |
                 reinterpret_cast<uintptr_t>(Z) | reinterpret_cast<uintptr_t>(o_tiles)) & 15) == 0 &&
                   ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(o_bias)) & 7) == 0,
               ET_ERR_UNSUPPORTED, "et_mha_fuseo_f16: operands must be 16-byte aligned (out, bias: 8)");
    // one arrival count per (sequence, 16-query block) at most
    ET_REQUIRE((long long)B * (S / 16) <= kFuseOCounters, ET_ERR_UNSUPPORTED,
               "et_mha_fuseo_f16: B*S/16=%lld exceeds the %d arrival counts built into the library; run "
               "et_mha_fused_f16 and et_linear_bsr16_f16 instead",
               (long long)B * (S / 16), kFuseOCounters);
    ET_REQUIRE((size_t)16 * (width + 8) * sizeof(_Float16) + fuseo_index_bytes(width, emdim) <= kLdsPerWorkgroup, ET_ERR_UNSUPPORTED,
               "et_mha_fuseo_f16: 16 rows of Z and the index arrays of a %d x %d weight exceed LDS", emdim, width);
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
    FuseOArgs fo;
    fo.row_ptr = o_row_ptr;
    fo.col_idx = o_col_idx;
    fo.tiles = reinterpret_cast<const _Float16 *>(o_tiles);
    fo.bias = reinterpret_cast<const _Float16 *>(o_bias);
    fo.out = reinterpret_cast<_Float16 *>(out);
    fo.emdim = emdim;
    int st = fuseo_counts(&fo.arrived);
    if (st != ET_OK) return st;
    if (hd <= 32) return launch_fuseo<32>(args, fo, waves, as_stream(stream));
    if (hd <= 64) return launch_fuseo<64>(args, fo, waves, as_stream(stream));
    return launch_fuseo<128>(args, fo, waves, as_stream(stream));
}

int et_mha_fuseo_f16(const et_f16 *Q, const et_f16 *K, const et_f16 *V, int ldq, int ldk, int ldv, et_f16 *Z,
                     int ldz, const et_f16 *mask, const int32_t *lens, int B, int S, int nh, int hd, float scale,
                     int flags, const int32_t *o_row_ptr, const int32_t *o_col_idx, const et_f16 *o_tiles,
                     const et_f16 *o_bias, et_f16 *out, int emdim, et_stream stream) {
    return et_mha_fuseo_f16_geom(Q, K, V, ldq, ldk, ldv, Z, ldz, mask, lens, B, S, nh, hd, scale, flags, o_row_ptr,
                                 o_col_idx, o_tiles, o_bias, out, emdim, 0, stream);
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
