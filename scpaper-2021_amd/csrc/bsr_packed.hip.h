// Tile-sparse Linear, packed form (device side, shared by the kernels that run packs):  Y[T x out] = act(X[T x in] * W^T + bias), W in 16x16 tiles
// (the mathematics of Linear/SPMM_tile.cu:249-324; tile order inside a block-row is free).
//
// At a few hundred to a few thousand token rows a launch of this product is a chain of memory
// round trips, not arithmetic: row pointers, then the tiles and columns they name, then the
// product, then the store.  This form removes every dependent load.  A "pack" is a copy of the
// weight laid out for one launch geometry (et_bsr16_pack_create, built once per weight):
//
//   * the block-rows of W are cut into groups (one workgroup each, per token strip), the tiles of
//     a block-row are paired into "slots" (two tiles = one v_mfma_f32_16x16x32_f16), and the
//     slots of a group, in row order, are dealt evenly to the waves of the workgroup — a block-row
//     may be split between consecutive waves;
//   * every wave's run of slots is padded with zero slots to the same capacity CAP, so the
//     address of slot p of wave w of group g is arithmetic: all weight loads of a wave are
//     issued as the kernel starts, with immediate offsets from one base, together with the
//     token strip, the bias and the residual;
//   * per wave a bit mask says after which slots a block-row (or the wave's part of it) ends; the
//     wave then parks its accumulator as a "part" in LDS.  After one barrier every block-row is
//     finished by one wave, which adds its parts in slot order (so the result does not depend on
//     how the slots were dealt), applies bias / activation / residual and stores.
//
// The strip of X lies in LDS unpadded with its 16-byte units XOR-swizzled by the row (rows are
// whole multiples of 256 bytes): the 16 rows a fragment read touches fall into 16 distinct
// 16-byte bank groups for any grouping of the lanes into quads.  Plain strips are fetched with
// direct-to-LDS loads; a binary32 strip that is normalised on the way (the consumer half of the
// split SkipLayerNorm) passes through registers.
#pragma once
#include <vector>

#include "common.hip.h"

namespace et {

#define ET_PK_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define ET_PK_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

constexpr int kPkXcds = 8;
constexpr int kPkMaxWaves = 16;
constexpr int kPkTabSlots = 2 * kPkMaxWaves;     // slots of every wave, rounded up to whole fours
constexpr int kPkTabRows = 3 * kPkMaxWaves;      // first block-row and number of block-rows of the group
constexpr int kPkTabHead = 3 * kPkMaxWaves + 4;  // ints ahead of the per-row part table of a group

// Operands that no kernel ever writes (tables, column offsets, bias, affine vectors), read through the
// constant address space: with a wave-uniform address such a load goes through the scalar cache and
// costs the vector memory pipeline, which is what bounds these kernels, nothing.
#define ET_PK_CONST(T, p) ((const __attribute__((address_space(4))) T *)(p))

struct PackArgs {
    const _Float16 *pw;      // [ngroups][nwave][CAP] slots of 1 KiB in lane order (two tiles each), zero slots as padding
    const uint32_t *poff;    // [ngroups][nwave][cap]: byte offsets (column * 32) of a slot's two tiles, 16 bits each
    const int32_t *ptab;     // [ngroups][tab_stride]: masks[16], first part[16], slots[16], first block-row,
                             // block-rows, 0, 0, part_start[rows_per_wg + 1]
    const _Float16 *bias;
    const _Float16 *X;       // binary16 strip source (plain prologue)
    _Float16 *Y;             // binary16 result, or
    float *Y32;              // binary32 result
    int T, in, out;
    int rows_per_wg, ngroups, tab_stride;  // rows_per_wg: the most block-rows any group holds
    int cap;                               // slots per wave of the pack (a multiple of 4)
    int act;
    // binary32 strip that is normalised while staged (NORM32)
    const float *X32;
    const float *st_in;      // [st_groups][T][2] partial (sum, sum of squares) of every row of X32
    int st_groups;
    const _Float16 *gamma, *beta;
    float eps;
    float *fin_out;          // [T][2] mean and rstd of every row, written by block-row group 0 (may be null)
    // residual epilogue with row sums (RES32): Y32 = acc + bias + residual, st_out[group][T][2]
    const float *resid32;
    const _Float16 *resid16;  // when set, the residual in binary16 (resid32 unused)
    const float *rs_fin;      // when set, the residual is the normalisation of resid32 by these [T][2] (mean, rstd)
    const _Float16 *rs_gamma, *rs_beta;
    float *st_out;
};

__device__ __forceinline__ float pk_act(float x, int act) {
    if (act == ET_ACT_RELU) return x > 0.0f ? x : 0.0f;
    if (act == ET_ACT_GELU) return gelu_tanh(x);
    return x;
}

// most waves a workgroup of the CAP-slot kernel may have (registers: a slot is four per lane, and
// the normalising prologue holds its share of the binary32 strip)
constexpr int pk_max_waves(int cap, bool norm, int su = 1) {
    return norm ? (su >= 8 ? 8 : cap <= 12 ? 16 : cap <= 16 ? 12 : 8) : (cap <= 16 ? 16 : 12);
}

// Which part of a launch a workgroup works on: workgroup id -> (token strip, block-row group).
// Workgroups are handed to the XCDs round-robin by id, so the groups of one strip share an XCD (one
// L2).  With unit32 set, a 16-row strip goes to the XCD its 32-row neighbourhood would go to as a
// 32-row strip: launches with different strip heights then keep a token on one XCD.
struct PkItem {
    int strip, group, tok0, rb_begin, rows_here;
    bool live;  // false: padding of the last round of strips (the whole workgroup has nothing to do)
};
template <int MT> __device__ __forceinline__ PkItem pk_item(const PackArgs &a, int wg, bool unit32) {
    PkItem it;
    const int nstrips = (a.T + MT * 16 - 1) / (MT * 16);
    const int xcd = wg % kPkXcds, k = wg / kPkXcds;
    const int j = k / a.ngroups;
    it.group = k % a.ngroups;
    it.strip = (unit32 && MT == 1) ? 2 * (xcd + kPkXcds * (j >> 1)) + (j & 1) : xcd + kPkXcds * j;
    it.live = it.strip < nstrips;
    it.tok0 = it.strip * (MT * 16);
    // the groups hold about equally many slots, not equally many block-rows: their bounds are in the table
    const auto *tab = ET_PK_CONST(int32_t, a.ptab) + (size_t)it.group * a.tab_stride;
    it.rb_begin = tab[kPkTabRows];
    it.rows_here = tab[kPkTabRows + 1];
    return it;
}

// One launch's work of a workgroup, in the steps a kernel strings together.  Everything a step
// requests from memory is held in members (registers) until a later step uses it, so a kernel that
// runs several packs one after the other can request the weights of the next while it finishes
// the current one.
// DYN: CAP is the most slots a wave may have; the pack's own count (PackArgs::cap, a multiple of 4) is
// read at run time and slots beyond it are neither fetched nor multiplied.
template <int MT, int CAP, bool NORM32, bool RES32, int SU, bool DYN = false> struct PkPhase {
    static_assert(!(NORM32 && RES32), "a consumer of a normalised strip stores plain results");
    static_assert(CAP % 4 == 0, "slots are handled four at a time");
    static constexpr int EPF = RES32 ? 1 : 2;  // block-rows per wave whose epilogue operands are requested ahead
    static constexpr int kStatPass = NORM32 ? (2 * SU + 7) / 8 : 1;

    int lane, wave, nwave, r16, g, sel, gbit;
    PkItem it;
    int stride, upr;  // bytes, and 16-byte units, of a strip row in LDS
    unsigned char *xs, *parts;
    const __attribute__((address_space(4))) int32_t *tab;
    // requested by request_weights
    uint32_t mask;
    int seg, nsl;  // first part of this wave; its slots, rounded up to whole fours
    int ps0[EPF], ps1[EPF];
    h8 w[CAP];
    uint32_t offs[CAP];  // wave-uniform: both tiles' byte offsets of every slot
    h4 bias_pf[EPF];
    h4 gm_pf[RES32 ? EPF : 1], bt_pf[RES32 ? EPF : 1];
    h8 gam, bet;
    // requested by request_inputs
    float2 st_a[kStatPass], st_b[kStatPass];
    f4 s32[NORM32 ? SU : 1][2];
    f4 rs_pf[RES32 ? EPF : 1][MT];
    float2 tst[RES32 ? MT : 1];
    int n_dr, n_r0, n_c8, n_ra;

    __device__ __forceinline__ void setup(const PackArgs &a, unsigned char *smem, int wg, bool unit32) {
        lane = threadIdx.x & 63;
        wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        nwave = blockDim.x >> 6;
        r16 = lane & 15;
        g = lane >> 4;
        sel = g >> 1;
        gbit = g & 1;
        it = pk_item<MT>(a, wg, unit32);
        stride = a.in * 2;
        upr = a.in >> 3;
        xs = smem;
        parts = smem + MT * 16 * stride;
        tab = ET_PK_CONST(int32_t, a.ptab) + (size_t)it.group * a.tab_stride;
        n_dr = 1;
        n_r0 = n_c8 = n_ra = 0;
        if constexpr (NORM32) {
            // thread t owns unit c8 = t % upr of strip rows t / upr + u * dr
            n_dr = (int)blockDim.x / upr;  // the host picks the wave count so that this is exact and 16 * MT = SU * dr
            n_r0 = (int)threadIdx.x / upr;
            n_c8 = (int)threadIdx.x - n_r0 * upr;
            n_ra = (wave * 64) / upr;  // a wave's threads lie in base rows n_ra and n_ra + 1 (upr >= 64)
        }
    }

    // the four values 4g .. 4g + 3 of the 16 that belong to block-row `row` of a per-feature vector:
    // the 32 bytes are read with a wave-uniform address, a lane picks its 8
    __device__ __forceinline__ h4 row_quad(const _Float16 *vec, int row) const {
        const auto *p = ET_PK_CONST(uint32_t, vec) + row * 8;
        uint32_t d[8];
#pragma unroll
        for (int k = 0; k < 8; k++) d[k] = p[k];
        const uint32_t lo = g == 0 ? d[0] : g == 1 ? d[2] : g == 2 ? d[4] : d[6];
        const uint32_t hi = g == 0 ? d[1] : g == 1 ? d[3] : g == 2 ? d[5] : d[7];
        const h2 a2 = __builtin_bit_cast(h2, lo), b2 = __builtin_bit_cast(h2, hi);
        return h4{a2[0], a2[1], b2[0], b2[1]};
    }
    __device__ __forceinline__ h4 load_bias(const PackArgs &a, int i) const {
        h4 b = {0, 0, 0, 0};
        if (a.bias) b = row_quad(a.bias, it.rb_begin + i);
        return b;
    }
    __device__ __forceinline__ void load_affine(const PackArgs &a, int i, h4 &gm, h4 &bt) const {
        gm = bt = h4{0, 0, 0, 0};
        if (a.rs_fin) {  // wave-uniform
            gm = row_quad(a.rs_gamma, it.rb_begin + i);
            bt = row_quad(a.rs_beta, it.rb_begin + i);
        }
    }
    __device__ __forceinline__ void load_resid(const PackArgs &a, int i, f4 (&rs)[MT]) const {
        const int f0 = (it.rb_begin + i) * 16 + g * 4;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const int tok = min(it.tok0 + m * 16 + r16, a.T - 1);
            if (a.resid16) {  // wave-uniform
                const h4 r = *reinterpret_cast<const h4 *>(a.resid16 + (size_t)tok * a.out + f0);
                rs[m] = f4{(float)r[0], (float)r[1], (float)r[2], (float)r[3]};
            } else {
                rs[m] = *reinterpret_cast<const f4 *>(a.resid32 + (size_t)tok * a.out + f0);
            }
        }
    }

    // Everything that is a property of the weight: tables (wave-uniform addresses: scalar loads),
    // the wave's CAP slots at immediate offsets from one base, the byte offsets of their columns for
    // this half of the wave, bias and affine vectors.  In NPART parts (a chain requests them between
    // the units of the previous step's epilogue): part 0 carries the small operands; the groups of four
    // slots are dealt to the parts round-robin.
    template <int NPART = 1> __device__ __forceinline__ void request_weights(const PackArgs &a, int part = 0) {
        const size_t wslab = (size_t)(it.group * nwave + wave);
        const int cap = DYN ? a.cap : CAP;  // wave-uniform
        if (part == 0) {
            mask = (uint32_t)tab[wave];
            seg = tab[kPkMaxWaves + wave];
            nsl = tab[kPkTabSlots + wave];
#pragma unroll
            for (int e = 0; e < EPF; e++) {
                const int i = min(wave + nwave * e, it.rows_here - 1);
                ps0[e] = tab[kPkTabHead + i];
                ps1[e] = tab[kPkTabHead + i + 1];
            }
            if constexpr (NORM32) {
                gam = reinterpret_cast<const h8 *>(a.gamma)[n_c8];
                bet = reinterpret_cast<const h8 *>(a.beta)[n_c8];
            }
            const auto *op = ET_PK_CONST(uint32_t, a.poff) + wslab * cap;
#pragma unroll
            for (int q = 0; q < CAP / 4; q++) {
                if (4 * q < nsl) {
#pragma unroll
                    for (int r = 0; r < 4; r++) offs[4 * q + r] = op[4 * q + r];
                }
            }
#pragma unroll
            for (int e = 0; e < EPF; e++) {
                if (wave + nwave * e < it.rows_here) {  // wave-uniform: a wave without that block-row asks for nothing
                    bias_pf[e] = load_bias(a, wave + nwave * e);
                    if constexpr (RES32) load_affine(a, wave + nwave * e, gm_pf[e], bt_pf[e]);
                }
            }
        }
        const _Float16 *wp = a.pw + wslab * cap * 512 + lane * 8;
#pragma unroll
        for (int q = 0; q < CAP / 4; q++) {  // groups of four slots, dealt to the parts round-robin
            if ((NPART == 1 || q % NPART == part) && 4 * q < nsl) {
#pragma unroll
                for (int r = 0; r < 4; r++) w[4 * q + r] = *reinterpret_cast<const h8 *>(wp + (4 * q + r) * 512);
            }
        }
    }

    // Everything that an earlier launch (or an earlier step of a chain) produced: the binary32 strip
    // with its row sums (NORM32), the residual and its row statistics (RES32).  A plain strip is
    // fetched by stage(), straight into LDS.
    __device__ __forceinline__ void request_inputs(const PackArgs &a) {
        if constexpr (NORM32) {
            // lane L: partial sums of block-row group L % 8 (and L % 8 + 8) of row slot L / 8;
            // slot s = strip row n_ra + (s & 1) + (s >> 1) * dr
#pragma unroll
            for (int ps = 0; ps < kStatPass; ps++) {
                const int slot = ps * 8 + (lane >> 3);
                const int row = min(n_ra + (slot & 1) + (slot >> 1) * n_dr, MT * 16 - 1);
                const int tok = min(it.tok0 + row, a.T - 1);
                const int gi = lane & 7;
                st_a[ps] = *reinterpret_cast<const float2 *>(a.st_in + ((size_t)min(gi, a.st_groups - 1) * a.T + tok) * 2);
                st_b[ps] = float2{0.0f, 0.0f};
                if (a.st_groups > 8)  // wave-uniform
                    st_b[ps] = *reinterpret_cast<const float2 *>(a.st_in + ((size_t)min(gi + 8, a.st_groups - 1) * a.T + tok) * 2);
            }
#pragma unroll
            for (int u = 0; u < SU; u++) {
                const int tok = min(it.tok0 + n_r0 + u * n_dr, a.T - 1);
                const f4 *p = reinterpret_cast<const f4 *>(a.X32 + (size_t)tok * a.in) + 2 * n_c8;
                s32[u][0] = p[0];
                s32[u][1] = p[1];
            }
        }
        if constexpr (RES32) {
            if (wave < it.rows_here) {  // wave-uniform: this wave finishes at least one block-row
#pragma unroll
                for (int e = 0; e < EPF; e++)
                    if (wave + nwave * e < it.rows_here) load_resid(a, wave + nwave * e, rs_pf[e]);
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    tst[m] = float2{0.0f, 1.0f};
                    if (a.rs_fin)
                        tst[m] = *reinterpret_cast<const float2 *>(a.rs_fin + 2 * (size_t)min(it.tok0 + m * 16 + r16, a.T - 1));
                }
            }
        }
    }

    // The strip into LDS: normalised on the way (NORM32), or by direct-to-LDS loads.  Ends with every
    // load of this wave complete; the caller's barrier then makes the strip visible to all waves.
    __device__ __forceinline__ void stage(const PackArgs &a) {
        if constexpr (NORM32) {
            // statistics of the wave's row slots: eight lanes per slot, added by a butterfly
            float mean_l[kStatPass], rstd_l[kStatPass];
            const float inv_h = 1.0f / (float)a.in;
#pragma unroll
            for (int ps = 0; ps < kStatPass; ps++) {
                const int gi = lane & 7;
                float s1 = (gi < a.st_groups ? st_a[ps].x : 0.0f) + (gi + 8 < a.st_groups ? st_b[ps].x : 0.0f);
                float s2 = (gi < a.st_groups ? st_a[ps].y : 0.0f) + (gi + 8 < a.st_groups ? st_b[ps].y : 0.0f);
#pragma unroll
                for (int d = 1; d < 8; d <<= 1) {
                    s1 += __shfl_xor(s1, d, 64);
                    s2 += __shfl_xor(s2, d, 64);
                }
                const float mean = s1 * inv_h;
                mean_l[ps] = mean;
                rstd_l[ps] = rsqrtf(fmaxf(__builtin_fmaf(-mean, mean, s2 * inv_h), 0.0f) + a.eps);
                // block-row group 0 leaves (mean, rstd) of the strip's rows for the next producer: each row
                // by the wave in which the row's first thread lies
                if (a.fin_out && it.group == 0 && gi == 0) {
                    const int slot = ps * 8 + (lane >> 3);
                    const int base = n_ra + (slot & 1);
                    const int row = base + (slot >> 1) * n_dr;
                    if ((slot >> 1) < SU && base < n_dr && base * upr >= wave * 64 && base * upr < wave * 64 + 64 &&
                        it.tok0 + row < a.T)
                        *reinterpret_cast<float2 *>(a.fin_out + 2 * (size_t)(it.tok0 + row)) = float2{mean_l[ps], rstd_l[ps]};
                }
            }
#pragma unroll
            for (int u = 0; u < SU; u++) {
                const int slot = 2 * u + (n_r0 - n_ra);
                float mean = 0.0f, rstd = 0.0f;
#pragma unroll
                for (int ps = 0; ps < kStatPass; ps++) {
                    const float mv = __shfl(mean_l[ps], (slot & 7) << 3, 64), rv = __shfl(rstd_l[ps], (slot & 7) << 3, 64);
                    if (kStatPass == 1 || (slot >> 3) == ps) {
                        mean = mv;
                        rstd = rv;
                    }
                }
                const int row = n_r0 + u * n_dr;
                h8 o;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    o[e] = (_Float16)norm_value(s32[u][0][e], mean, rstd, (float)gam[e], (float)bet[e]);
                    o[4 + e] = (_Float16)norm_value(s32[u][1][e], mean, rstd, (float)gam[4 + e], (float)bet[4 + e]);
                }
                *reinterpret_cast<h8 *>(xs + row * stride + ((n_c8 ^ (row & 15)) << 4)) = o;
            }
        } else {
            // direct-to-LDS: instruction j fills LDS bytes [1024 j, 1024 j + 1024) of the strip; the lane
            // that fills unit pu of a row fetches the row's unit pu ^ (row & 15)
            const int n_inst = MT * 16 * upr / 64;
            int row = (wave * 64 + lane) / upr;
            int pu = (wave * 64 + lane) - row * upr;
            const int d_u = nwave * 64;
            const int d_row = d_u / upr, d_pu = d_u - d_row * upr;
            for (int j = wave; j < n_inst; j += nwave) {
                const int lu = pu ^ (row & 15);
                const int tok = min(it.tok0 + row, a.T - 1);
                __builtin_amdgcn_global_load_lds(ET_PK_GLOBAL_PTR(a.X + (size_t)tok * a.in + lu * 8),
                                                 ET_PK_LDS_PTR(xs + j * 1024), 16, 0, 0);
                row += d_row;
                pu += d_pu;
                if (pu >= upr) {
                    pu -= upr;
                    row++;
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    }

    // byte offset of slot p's tile for this half of the wave (a wave-uniform word, a per-lane field)
    __device__ __forceinline__ unsigned slot_off(int p) const { return (offs[p] >> (sel << 4)) & 0xffffu; }

    // Slot p of the wave: B operand = 16 tokens x (8 values of each of the slot's two column tiles)
    // read from the swizzled strip.  Where the mask says that a block-row (or this wave's part of it)
    // ends, the accumulator is parked in LDS.
    __device__ __forceinline__ void multiply() {
        const unsigned kx = (unsigned)((gbit ^ r16) & 15) << 4;
        unsigned rowbase[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) rowbase[m] = (unsigned)((m * 16 + r16) * stride);
        f4 acc[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) acc[m] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < CAP; p++) {
            if ((p & 3) == 0 && p >= nsl) break;  // wave-uniform: nothing was fetched beyond
            const unsigned o = slot_off(p) ^ kx;
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const h8 x = *reinterpret_cast<const h8 *>(xs + rowbase[m] + o);
                acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[p], x, acc[m], 0, 0, 0);
            }
            if ((mask >> p) & 1u) {  // wave-uniform
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    *reinterpret_cast<f4 *>(parts + (seg * MT + m) * 1024 + lane * 16) = acc[m];
                    acc[m] = f4{0.f, 0.f, 0.f, 0.f};
                }
                seg++;
            }
        }
    }

    // Local block-row i is finished by wave i % nwave: its parts added in slot order, bias,
    // activation or residual, store; RES32 also leaves the row sums of what the workgroup stored.
    // Contains one workgroup barrier when RES32.
    // hook(u) is called before unit u of the work (a unit = one of the first EPF block-rows of the
    // wave; kUnits of them): a chain puts the next step's weight requests there.
    static constexpr int kUnits = EPF;
    struct NoHook {
        __device__ __forceinline__ void operator()(int) const {}
    };
    __device__ __forceinline__ void epilogue(const PackArgs &a) { epilogue(a, NoHook()); }
    template <typename Hook> __device__ __forceinline__ void epilogue(const PackArgs &a, Hook hook) {
        bool tok_ok[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) tok_ok[m] = it.tok0 + m * 16 + r16 < a.T;
        float st1[MT], st2[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) st1[m] = st2[m] = 0.0f;
        // binary16 results of a whole 32-row strip leave in 16-byte pieces
        const bool wide16 = MT == 2 && !RES32 && a.Y32 == nullptr && it.tok0 + 32 <= a.T;  // wave-uniform
        auto finish = [&](int i, int s0, int s1, h4 bv, const f4 (&rs)[MT], h4 gm, h4 bt) {
            f4 sum[MT];
            uint2 out16[MT];
#pragma unroll
            for (int m = 0; m < MT; m++) sum[m] = f4{0.f, 0.f, 0.f, 0.f};
            for (int s = s0; s < s1; s++) {
#pragma unroll
                for (int m = 0; m < MT; m++) sum[m] += *reinterpret_cast<const f4 *>(parts + (s * MT + m) * 1024 + lane * 16);
            }
            const int f0 = (it.rb_begin + i) * 16 + g * 4;
#pragma unroll
            for (int m = 0; m < MT; m++) {
                if (!tok_ok[m]) continue;
                const size_t at = (size_t)(it.tok0 + m * 16 + r16) * a.out + f0;
                if constexpr (RES32) {
                    f4 v;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float rv = rs[m][j];
                        if (a.rs_fin) rv = norm_value(rv, tst[m].x, tst[m].y, (float)gm[j], (float)bt[j]);  // wave-uniform
                        v[j] = sum[m][j] + (float)bv[j] + rv;
                        st1[m] += v[j];
                        st2[m] = __builtin_fmaf(v[j], v[j], st2[m]);
                    }
                    *reinterpret_cast<f4 *>(a.Y32 + at) = v;
                } else if (a.Y32) {  // wave-uniform
                    f4 v;
#pragma unroll
                    for (int j = 0; j < 4; j++) v[j] = pk_act(sum[m][j] + (float)bv[j], a.act);
                    *reinterpret_cast<f4 *>(a.Y32 + at) = v;
                } else {
                    h4 v;
#pragma unroll
                    for (int j = 0; j < 4; j++) v[j] = (_Float16)pk_act(sum[m][j] + (float)bv[j], a.act);
                    if (!wide16) *reinterpret_cast<h4 *>(a.Y + at) = v;
                    out16[m] = __builtin_bit_cast(uint2, v);
                }
            }
            if constexpr (MT == 2 && !RES32) {
                if (wide16) {
                    // 16-byte stores: the lanes of an even and the next odd 16-lane row hold features 4g .. 4g + 7
                    // of the same two tokens; the even row takes both quads of the first token, the odd row
                    // those of the second (one row swap per register), and every lane stores 8 features
                    const auto lo = __builtin_amdgcn_permlane16_swap(out16[0].x, out16[1].x, false, false);
                    const auto hi = __builtin_amdgcn_permlane16_swap(out16[0].y, out16[1].y, false, false);
                    const uint4 q = {(unsigned)lo[0], (unsigned)hi[0], (unsigned)lo[1], (unsigned)hi[1]};
                    const size_t at = (size_t)(it.tok0 + gbit * 16 + r16) * a.out + f0 - gbit * 4;
                    *reinterpret_cast<uint4 *>(a.Y + at) = q;
                }
            }
        };
#pragma unroll
        for (int e = 0; e < EPF; e++) {
            const int i = wave + nwave * e;
            hook(e);
            if (i < it.rows_here)
                finish(i, ps0[e], ps1[e], bias_pf[e], rs_pf[RES32 ? e : 0], gm_pf[RES32 ? e : 0], bt_pf[RES32 ? e : 0]);
        }
        for (int i = wave + nwave * EPF; i < it.rows_here; i += nwave) {
            const h4 bv = load_bias(a, i);
            f4 rs[MT];
            h4 gm = {0, 0, 0, 0}, bt = {0, 0, 0, 0};
            if constexpr (RES32) {
                load_resid(a, i, rs);
                load_affine(a, i, gm, bt);
            }
            finish(i, tab[kPkTabHead + i], tab[kPkTabHead + i + 1], bv, rs, gm, bt);
        }
        if constexpr (RES32) {
            // row sums of what this workgroup stored: the four lanes of a token, then the waves through
            // LDS in wave order, one float2 per token and block-row group — no atomics
#pragma unroll
            for (int m = 0; m < MT; m++) {
                st1[m] += __shfl_xor(st1[m], 16, 64);
                st1[m] += __shfl_xor(st1[m], 32, 64);
                st2[m] += __shfl_xor(st2[m], 16, 64);
                st2[m] += __shfl_xor(st2[m], 32, 64);
            }
            float2 *red = reinterpret_cast<float2 *>(xs);  // the strip is no longer read
            if (g == 0) {
#pragma unroll
                for (int m = 0; m < MT; m++) red[wave * (MT * 16) + m * 16 + r16] = float2{st1[m], st2[m]};
            }
            __syncthreads();
            const int rows_tok = min(MT * 16, a.T - it.tok0);
            if ((int)threadIdx.x < rows_tok) {
                float s1 = 0.0f, s2 = 0.0f;
                for (int wv = 0; wv < nwave; wv++) {
                    const float2 pr = red[wv * (MT * 16) + threadIdx.x];
                    s1 += pr.x;
                    s2 += pr.y;
                }
                *reinterpret_cast<float2 *>(a.st_out + ((size_t)it.group * a.T + it.tok0 + threadIdx.x) * 2) = float2{s1, s2};
            }
        }
    }
};

}  // namespace et

// A pack: device copies of the re-ordered weight and its tables, and the geometry they were built for.
struct et_bsr_pack_s {
    int in = 0, out = 0, T = 0;
    int mt = 0, ngroups = 0, rows_per_wg = 0, nwave = 0, cap = 0, su = 0, tab_stride = 0;
    int flags = 0;
    size_t lds = 0;
    void *pw = nullptr, *poff = nullptr, *ptab = nullptr;
    void *bias32 = nullptr;  // packs with a normalisation's affine part folded in: bias + W beta, binary32
    ~et_bsr_pack_s() {
        (void)et_free(pw);
        (void)et_free(poff);
        (void)et_free(ptab);
        (void)et_free(bias32);
    }
};

namespace et {
// device copies of a pack's tables and of its weight slabs (slot s = tiles order[2s], order[2s + 1]; negative: zeros)
int pack_upload(et_bsr_pack_s &p, const std::vector<uint32_t> &off, const std::vector<int32_t> &tab,
                const std::vector<int32_t> &order, const et_f16 *tiles);
// the row-loop form (bsr_rowloop.hip): its pack builder, from host copies of the structure, and its launch
int rowloop_pack_create(const std::vector<int32_t> &row_ptr, const std::vector<int32_t> &col_idx, const et_f16 *tiles, int T, int in,
                        int out, int flags, et_bsr_pack_s **pack);
int rowloop_launch(const PackArgs &a, const et_bsr_pack_s &p, hipStream_t stream);
// kernel arguments of a launch of `p` over T token rows (the operands are filled in by the caller)
inline PackArgs pk_base_args(const et_bsr_pack_s &p, const et_f16 *bias, int T) {
    PackArgs a{};
    a.pw = static_cast<const _Float16 *>(p.pw);
    a.poff = static_cast<const uint32_t *>(p.poff);
    a.ptab = static_cast<const int32_t *>(p.ptab);
    a.bias = reinterpret_cast<const _Float16 *>(bias);
    a.T = T;
    a.in = p.in;
    a.out = p.out;
    a.rows_per_wg = p.rows_per_wg;
    a.ngroups = p.ngroups;
    a.tab_stride = p.tab_stride;
    a.cap = p.cap;
    return a;
}
}  // namespace et
