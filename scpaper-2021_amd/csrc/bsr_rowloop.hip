// Tile-sparse Linear through a pack, many token rows:  Y[T x out] = act(X[T x in] * W^T + bias), W in 16x16 tiles
// (the mathematics of Linear/SPMM_tile.cu:249-324).
//
// From a few thousand token rows on a launch of this product is arithmetic and LDS traffic, and what
// the one-strip-per-workgroup forms pay per strip — fetching their share of the weight, a barrier
// between multiplying and storing, partial sums through LDS — is paid thousands of times.  Here a
// workgroup keeps its share of the weight in registers for the whole launch and walks over token
// strips:
//
//   * a pack built with ET_PACK_ROW_LOOP deals whole block-rows to the waves (a wave never shares a
//     block-row with another), so a wave finishes every block-row it multiplies by itself: bias,
//     activation and store come straight from the accumulator, nothing is parked in LDS and the
//     only barrier of a strip is the one that hands over the staged strip;
//   * three strip buffers: the direct-to-LDS loads of strip i + 2 are issued before strip i is
//     multiplied and have two multiplications to arrive;
//   * the block-row groups of a strip run on the same XCD, so the strip comes from HBM once.
//
// What is left per 16x16x32 product is the 1 KiB operand fragment a wave reads from the strip in
// LDS, and per strip the store of its results.
#include <algorithm>
#include <new>
#include <vector>

#include "bsr_packed.hip.h"
#include "../../include/et_tuning.h"

namespace et {

constexpr int kRlTabFirstRow = kPkMaxWaves;  // table slots shared with the other packs: masks, first row, slots, bounds

// Loads and stores of a wave share one memory counter, which counts down in issue order.  A wave
// that waited for "everything" before each strip would wait for the stores of the strip before, and each
// strip would pay the latency of its stores.  Here a wave waits for "everything but the last n", n
// being what it has issued since the loads it needs: the stores of the last two strips and its share of
// the loads of the strip after next.  The direct-to-LDS loads are issued from inline assembly: known to
// the compiler, every LDS read behind one would be made to wait for all of them (it cannot tell the
// buffers apart), which is the very stall this form exists to avoid.
__device__ __forceinline__ void rl_wait_vmcnt(int n) {  // wave-uniform n; the instruction takes an immediate
#define ET_RL_CASE(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    switch (n) {
        ET_RL_CASE(1) ET_RL_CASE(2) ET_RL_CASE(3) ET_RL_CASE(4) ET_RL_CASE(5) ET_RL_CASE(6) ET_RL_CASE(7) ET_RL_CASE(8)
        ET_RL_CASE(9) ET_RL_CASE(10) ET_RL_CASE(11) ET_RL_CASE(12) ET_RL_CASE(13) ET_RL_CASE(14) ET_RL_CASE(15) ET_RL_CASE(16)
        ET_RL_CASE(17) ET_RL_CASE(18) ET_RL_CASE(19) ET_RL_CASE(20) ET_RL_CASE(21) ET_RL_CASE(22) ET_RL_CASE(23) ET_RL_CASE(24)
        ET_RL_CASE(25) ET_RL_CASE(26) ET_RL_CASE(27) ET_RL_CASE(28) ET_RL_CASE(29) ET_RL_CASE(30) ET_RL_CASE(31) ET_RL_CASE(32)
        ET_RL_CASE(33) ET_RL_CASE(34) ET_RL_CASE(35) ET_RL_CASE(36) ET_RL_CASE(37) ET_RL_CASE(38) ET_RL_CASE(39) ET_RL_CASE(40)
        ET_RL_CASE(41) ET_RL_CASE(42) ET_RL_CASE(43) ET_RL_CASE(44) ET_RL_CASE(45) ET_RL_CASE(46) ET_RL_CASE(47) ET_RL_CASE(48)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;  // 0, and anything the immediate cannot say: wait for all
    }
#undef ET_RL_CASE
}
__device__ __forceinline__ void rl_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
// 16 bytes per lane from global memory (base + byte offset of the lane) to LDS bytes [lds_base + 16 lane, + 16);
// base and lds_base are wave-uniform
__device__ __forceinline__ void rl_load_to_lds(const void *base, unsigned lane_off, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(lds_base)
                 : "memory", "m0");
}

constexpr int kRlBuf = 3;  // strip buffers: the strip being multiplied and the two after it

// OUT32: the results are stored as binary32 (Y32; the unrounded accumulator plus bias, activated), one 16-byte store
// per lane and 16-row block instead of packed binary16.
template <int MT, int CAP, bool OUT32>
__global__ __launch_bounds__(pk_max_waves(CAP, false) * 64) void bsr16_rowloop_kernel(const PackArgs a) {
    extern __shared__ __align__(256) unsigned char rl_smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwave = blockDim.x >> 6;
    const int r16 = lane & 15, g = lane >> 4, sel = g >> 1, gbit = g & 1;
    // workgroup -> (XCD, block-row group, lane of strips): strips xcd + 8 (j + nj i), i = 0, 1, ...
    const int xcd = blockIdx.x % kPkXcds, k = blockIdx.x / kPkXcds;
    const int group = k % a.ngroups, j = k / a.ngroups, nj = (int)gridDim.x / kPkXcds / a.ngroups;
    const int nstrips = (a.T + MT * 16 - 1) / (MT * 16);
    const int step = kPkXcds * nj;
    const int stride = a.in * 2, upr = a.in >> 3;
    const unsigned strip_bytes = (unsigned)(MT * 16 * stride);
    const int s0 = xcd + kPkXcds * j;
    if (s0 >= nstrips) return;  // the whole workgroup: nothing to do
    const int rounds = (nstrips - s0 + step - 1) / step;
    const unsigned lds0 = (unsigned)(size_t)ET_PK_LDS_PTR(rl_smem);
    uint32_t *bias_l = reinterpret_cast<uint32_t *>(rl_smem + (size_t)kRlBuf * strip_bytes);  // [rows of the group][8]

    // This wave's share of a strip's direct-to-LDS loads: instruction i (i = wave, wave + nwave, ...) fills LDS
    // bytes [1024 i, 1024 i + 1024) of the strip; the lane that fills unit pu of a row fetches the row's unit
    // pu ^ (row & 15).  Rows past T repeat the last row.
    const int n_inst = MT * 16 * upr / 64;
    const int n_mine = wave < n_inst ? (n_inst - wave + nwave - 1) / nwave : 0;
    auto stage_issue = [&](int round) {
        const int tok0 = (s0 + round * step) * (MT * 16);
        const int last_row = min(MT * 16, a.T - tok0) - 1;
        const _Float16 *base = a.X + (size_t)tok0 * a.in;  // wave-uniform
        const unsigned lbase = lds0 + (unsigned)(round % kRlBuf) * strip_bytes;
        int row = (wave * 64 + lane) / upr;
        int pu = (wave * 64 + lane) - row * upr;
        const int d_u = nwave * 64;
        const int d_row = d_u / upr, d_pu = d_u - d_row * upr;
        for (int i = wave; i < n_inst; i += nwave) {
            const unsigned off = (unsigned)(min(row, last_row) * stride + ((pu ^ (row & 15)) << 4));
            rl_load_to_lds(base, off, lbase + (unsigned)i * 1024u);
            row += d_row;
            pu += d_pu;
            if (pu >= upr) {
                pu -= upr;
                row++;
            }
        }
    };
    stage_issue(0);
    if (rounds > 1) stage_issue(1);

    const auto *tab = ET_PK_CONST(int32_t, a.ptab) + (size_t)group * a.tab_stride;
    const uint32_t mask = (uint32_t)tab[wave];
    const int row_first = tab[kRlTabFirstRow + wave];
    const int nsl = tab[kPkTabSlots + wave];
    const int rb_begin = tab[kPkTabRows], rows_here = tab[kPkTabRows + 1];
    const int my_rows = __builtin_popcount(mask);  // one store instruction each, per whole strip
    // this wave's share of the weight: held for the whole launch
    h8 w[CAP];
    uint32_t offs[CAP];
    {
        const size_t wslab = (size_t)(group * nwave + wave);
        const auto *op = ET_PK_CONST(uint32_t, a.poff) + wslab * CAP;
        const _Float16 *wp = a.pw + wslab * CAP * 512 + lane * 8;
#pragma unroll
        for (int q = 0; q < CAP / 4; q++) {
            if (4 * q < nsl) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    offs[4 * q + r] = op[4 * q + r];
                    w[4 * q + r] = *reinterpret_cast<const h8 *>(wp + (4 * q + r) * 512);
                }
            }
        }
    }
    // the group's bias values into LDS (zeros without a bias): a row's quad is then an LDS read like the fragments
    for (int i = threadIdx.x; i < rows_here * 8; i += blockDim.x)
        bias_l[i] = a.bias ? reinterpret_cast<const uint32_t *>(a.bias)[(size_t)rb_begin * 8 + i] : 0u;
    // everything requested so far — the first two strips, the weights, the bias — is in place before the loop
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)

    const unsigned kx = (unsigned)((gbit ^ r16) & 15) << 4;
    unsigned rowbase[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) rowbase[m] = (unsigned)((m * 16 + r16) * stride);
    const int act = a.act;
    const int spr = OUT32 ? MT : MT == 2 ? 1 : MT;  // store instructions per block-row of a whole strip

    int slot = 0, s = s0;
    for (int r = 0; r < rounds; r++, s += step) {
        const bool whole = s * (MT * 16) + MT * 16 <= a.T;  // wave-uniform: no token row of the strip lies past T
        if (r >= 2) {
            // issued since the loads of strip r: the stores of rounds r - 2 and r - 1 (both whole strips: only the
            // last strip of all may be ragged, and it is the last of its workgroup) and the loads of strip r + 1
            rl_wait_vmcnt(2 * my_rows * spr + (r + 1 < rounds ? n_mine : 0));
        }
        rl_barrier();  // every wave's share of strip r has landed, and every wave is done with strip r - 1
        if (r + 2 < rounds) stage_issue(r + 2);  // into the buffer of strip r - 1
        const unsigned char *xs = rl_smem + (size_t)slot * strip_bytes;
        slot = slot + 1 == kRlBuf ? 0 : slot + 1;
        const int tok0 = s * (MT * 16);
        int row = row_first;
        f4 acc[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) acc[m] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < CAP; p++) {
            if ((p & 3) == 0 && p >= nsl) break;  // wave-uniform: nothing was fetched beyond
            const unsigned o = ((offs[p] >> (sel << 4)) & 0xffffu) ^ kx;
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const h8 x = *reinterpret_cast<const h8 *>(xs + rowbase[m] + o);
                acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w[p], x, acc[m], 0, 0, 0);
            }
            if ((mask >> p) & 1u) {  // wave-uniform: block-row `row` of the group is complete
                const uint2 bq = *reinterpret_cast<const uint2 *>(bias_l + row * 8 + g * 2);
                const h2 b01 = __builtin_bit_cast(h2, bq.x), b23 = __builtin_bit_cast(h2, bq.y);
                const float bv[4] = {(float)b01[0], (float)b01[1], (float)b23[0], (float)b23[1]};
                const int f0 = (rb_begin + row) * 16 + g * 4;
                float v[MT][4];
#pragma unroll
                for (int m = 0; m < MT; m++) {
#pragma unroll
                    for (int e = 0; e < 4; e++) v[m][e] = acc[m][e] + bv[e];
                    acc[m] = f4{0.f, 0.f, 0.f, 0.f};
                }
                if (act == ET_ACT_GELU) {  // wave-uniform
#pragma unroll
                    for (int m = 0; m < MT; m++)
#pragma unroll
                        for (int e = 0; e < 4; e++) v[m][e] = gelu_tanh(v[m][e]);
                } else if (act == ET_ACT_RELU) {
#pragma unroll
                    for (int m = 0; m < MT; m++)
#pragma unroll
                        for (int e = 0; e < 4; e++) v[m][e] = fmaxf(v[m][e], 0.0f);
                }
                uint2 out16[MT];
#pragma unroll
                for (int m = 0; m < MT; m++)
                    out16[m] = __builtin_bit_cast(uint2, h4{(_Float16)v[m][0], (_Float16)v[m][1], (_Float16)v[m][2], (_Float16)v[m][3]});
                if constexpr (OUT32) {
                    // whole strips: exactly MT store instructions (rows past T exist only in the last strip of all)
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        const int tok = tok0 + m * 16 + r16;
                        if (whole || tok < a.T) *reinterpret_cast<f4 *>(a.Y32 + (size_t)tok * a.out + f0) = f4{v[m][0], v[m][1], v[m][2], v[m][3]};
                    }
                } else if (whole) {  // exactly `spr` store instructions, whatever the lanes hold: the waits above count on it
                    if constexpr (MT == 2) {
                        // 16-byte stores: an even and the next odd 16-lane row hold features 4g .. 4g + 7 of the same
                        // two tokens; the even row takes both quads of the first token, the odd row those of the second
                        const auto lo = __builtin_amdgcn_permlane16_swap(out16[0].x, out16[MT - 1].x, false, false);
                        const auto hi = __builtin_amdgcn_permlane16_swap(out16[0].y, out16[MT - 1].y, false, false);
                        const uint4 q = {(unsigned)lo[0], (unsigned)hi[0], (unsigned)lo[1], (unsigned)hi[1]};
                        *reinterpret_cast<uint4 *>(a.Y + (size_t)(tok0 + gbit * 16 + r16) * a.out + f0 - gbit * 4) = q;
                    } else {
                        *reinterpret_cast<uint2 *>(a.Y + (size_t)(tok0 + r16) * a.out + f0) = out16[0];
                    }
                } else {
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        const int tok = tok0 + m * 16 + r16;
                        if (tok < a.T) *reinterpret_cast<uint2 *>(a.Y + (size_t)tok * a.out + f0) = out16[m];
                    }
                }
                row++;
            }
        }
    }
}

constexpr size_t kRlLdsBudget = 160 * 1024;

template <int MT, int CAP, bool OUT32> static int rl_launch(const PackArgs &a, const et_bsr_pack_s &p, hipStream_t stream) {
    auto kernel = bsr16_rowloop_kernel<MT, CAP, OUT32>;
    if (p.lds > 64 * 1024) {
        static bool raised = false;  // per instantiation
        if (!raised) {
            ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)kRlLdsBudget));
            raised = true;
        }
    }
    // one workgroup per compute unit, fewer when there are not that many (strip, group) pairs: lanes of strips per XCD
    const int nstrips = (a.T + MT * 16 - 1) / (MT * 16);
    const int per_xcd = (nstrips + kPkXcds - 1) / kPkXcds;
    const int nj = std::max(1, std::min(per_xcd, 32 / a.ngroups));
    kernel<<<dim3((unsigned)(kPkXcds * a.ngroups * nj)), p.nwave * 64, p.lds, stream>>>(a);
    return check_launch("bsr16_rowloop_kernel");
}

template <int MT, bool OUT32> static int rl_dispatch_cap(const PackArgs &a, const et_bsr_pack_s &p, hipStream_t stream) {
    switch (p.cap) {
        case 8: return rl_launch<MT, 8, OUT32>(a, p, stream);
        case 12: return rl_launch<MT, 12, OUT32>(a, p, stream);
        case 16: return rl_launch<MT, 16, OUT32>(a, p, stream);
        case 20: return rl_launch<MT, 20, OUT32>(a, p, stream);
        case 24: return rl_launch<MT, 24, OUT32>(a, p, stream);
        default: return fail(ET_ERR_INVALID_ARG, "tile-sparse Linear (row loop): no kernel for %d slots per wave", p.cap);
    }
}

int rowloop_launch(const PackArgs &a, const et_bsr_pack_s &p, hipStream_t stream) {
    if (a.Y32) return p.mt == 2 ? rl_dispatch_cap<2, true>(a, p, stream) : rl_dispatch_cap<1, true>(a, p, stream);
    return p.mt == 2 ? rl_dispatch_cap<2, false>(a, p, stream) : rl_dispatch_cap<1, false>(a, p, stream);
}

// The pack of the row-loop kernel: block-rows cut into `ngroups` contiguous groups of about equally
// many slots, the block-rows of a group into contiguous runs, one per wave, none fuller than `cap`
// slots.  A block-row without tiles gets one zero slot, so that its bias is still stored.
int rowloop_pack_create(const std::vector<int32_t> &rp, const std::vector<int32_t> &ci, const et_f16 *tiles, int T, int in, int out,
                        int flags, et_bsr_pack *pack) {
    const int nbr = out / 16;
    ET_REQUIRE(in % 128 == 0 && in <= 1536, ET_ERR_UNSUPPORTED,
               "et_bsr16_pack_create: in=%d outside the row-loop kernel's range (multiples of 128 up to 1536)", in);
    // 32-row strips where three of them fit the LDS, else 16-row strips
    const size_t lds_room = kRlLdsBudget - 8192;  // less the bias values of a group (up to 256 block-rows)
    const int mt = (size_t)kRlBuf * 32 * in * 2 <= lds_room ? 2 : 1;
    ET_REQUIRE((size_t)kRlBuf * mt * 16 * in * 2 <= lds_room, ET_ERR_UNSUPPORTED,
               "et_bsr16_pack_create: in=%d: three 16-row strips do not fit the LDS", in);
    struct Slot {
        int t0, t1, c0, c1;
        bool row_end;
    };
    std::vector<int> row_slots((size_t)nbr);
    long total = 0;
    for (int rb = 0; rb < nbr; rb++) {
        row_slots[(size_t)rb] = std::max(1, (rp[(size_t)rb + 1] - rp[(size_t)rb] + 1) / 2);
        total += row_slots[(size_t)rb];
    }
    // contiguous cut of rows [b, e) into at most `parts` runs none above `bound` slots; fills `ends` with the run ends
    auto cut = [&](int b, int e, int parts, long bound, std::vector<int> *ends) -> bool {
        int used = 0, rb = b;
        if (ends) ends->clear();
        while (rb < e) {
            if (++used > parts) return false;
            long sum = 0;
            while (rb < e && sum + row_slots[(size_t)rb] <= bound) sum += row_slots[(size_t)rb++];
            if (sum == 0) return false;  // a single row above the bound
            if (ends) ends->push_back(rb);
        }
        return true;
    };
    auto least_bound = [&](int b, int e, int parts) -> long {
        long lo = 1, hi = 1;
        for (int rb = b; rb < e; rb++) {
            lo = std::max<long>(lo, row_slots[(size_t)rb]);
            hi += row_slots[(size_t)rb];
        }
        while (lo < hi) {
            const long mid = (lo + hi) / 2;
            if (cut(b, e, parts, mid, nullptr)) hi = mid;
            else lo = mid + 1;
        }
        return lo;
    };
    // the fewest groups (each re-reads the strip) whose fullest wave fits the registers: 16 waves up to 16 slots
    // each, or 12 up to 24
    int ngroups = 0, nwave = 0, cap = 0;
    std::vector<int> gends;
    for (int ng = 1; ng <= 32 && !ngroups; ng *= 2) {
        if (ng > nbr) break;
        const long gb = least_bound(0, nbr, ng);
        std::vector<int> ge;
        cut(0, nbr, ng, gb, &ge);
        while ((int)ge.size() < ng) ge.push_back(nbr);  // trailing groups may be empty
        int widest = 0;
        for (int gi = 0, b = 0; gi < ng; b = ge[(size_t)gi++]) widest = std::max(widest, ge[(size_t)gi] - b);
        if (widest > 256) continue;  // the bias values of a group have 8 KB of LDS
        for (int wv : {16, 12}) {
            long fullest = 0;
            int b = 0;
            for (int gi = 0; gi < ng; gi++) {
                if (ge[(size_t)gi] > b) fullest = std::max(fullest, least_bound(b, ge[(size_t)gi], wv));
                b = ge[(size_t)gi];
            }
            const int c = std::max(8, (int)((fullest + 3) / 4 * 4));
            if (c <= (wv == 16 ? 16 : 24)) {
                ngroups = ng, nwave = wv, cap = c, gends = ge;
                break;
            }
        }
    }
    ET_REQUIRE(ngroups > 0, ET_ERR_UNSUPPORTED,
               "et_bsr16_pack_create: in=%d out=%d with %ld slots does not fit the row-loop kernel's 32 block-row groups", in, out,
               total);
    int rows_per_wg = 0;
    {
        int b = 0;
        for (int gi = 0; gi < ngroups; gi++) {
            rows_per_wg = std::max(rows_per_wg, gends[(size_t)gi] - b);
            b = gends[(size_t)gi];
        }
    }
    const size_t lds = (size_t)kRlBuf * mt * 16 * in * 2 + (size_t)rows_per_wg * 32;
    ET_REQUIRE(lds <= kRlLdsBudget, ET_ERR_UNSUPPORTED, "et_bsr16_pack_create: in=%d needs %zu bytes of LDS", in, lds);

    const int tab_stride = (kPkTabHead + 3) / 4 * 4;
    const size_t nslab = (size_t)ngroups * nwave;
    std::vector<int32_t> order(nslab * cap * 2, -1), tab((size_t)ngroups * tab_stride, 0);
    std::vector<uint32_t> off(nslab * cap, 0);
    int gb = 0;
    for (int gi = 0; gi < ngroups; gi++) {
        const int ge = gends[(size_t)gi];
        int32_t *tb = &tab[(size_t)gi * tab_stride];
        tb[kPkTabRows] = gb;
        tb[kPkTabRows + 1] = ge - gb;
        std::vector<int> wends;
        if (ge > gb) cut(gb, ge, nwave, least_bound(gb, ge, nwave), &wends);
        int rb = gb;
        for (int wv = 0; wv < nwave; wv++) {
            const int we = wv < (int)wends.size() ? wends[(size_t)wv] : rb;
            const size_t slab = (size_t)gi * nwave + wv;
            uint32_t m = 0;
            int p = 0;
            tb[kRlTabFirstRow + wv] = rb - gb;
            for (; rb < we; rb++) {
                const int t_begin = rp[(size_t)rb], t_end = rp[(size_t)rb + 1];
                if (t_begin == t_end) {  // no tiles: one zero slot
                    ET_REQUIRE(p < cap, ET_ERR_INVALID_ARG, "et_bsr16_pack_create: internal: wave over capacity");
                    p++;
                } else {
                    for (int t = t_begin; t < t_end; t += 2, p++) {
                        ET_REQUIRE(p < cap, ET_ERR_INVALID_ARG, "et_bsr16_pack_create: internal: wave over capacity");
                        const bool two = t + 1 < t_end;
                        order[(slab * cap + p) * 2] = t;
                        order[(slab * cap + p) * 2 + 1] = two ? t + 1 : -1;
                        off[slab * cap + p] = (uint32_t)(ci[(size_t)t] * 32) | ((uint32_t)(ci[(size_t)(two ? t + 1 : t)] * 32) << 16);
                    }
                }
                m |= 1u << (p - 1);
            }
            tb[wv] = (int32_t)m;
            tb[kPkTabSlots + wv] = (p + 3) / 4 * 4;
        }
        ET_REQUIRE(rb == ge, ET_ERR_INVALID_ARG, "et_bsr16_pack_create: internal: rows left over");
        gb = ge;
    }

    et_bsr_pack_s *p = new (std::nothrow) et_bsr_pack_s;
    ET_REQUIRE(p != nullptr, ET_ERR_ALLOC, "et_bsr16_pack_create: out of host memory");
    p->in = in;
    p->out = out;
    p->T = T;
    p->mt = mt;
    p->ngroups = ngroups;
    p->rows_per_wg = rows_per_wg;
    p->nwave = nwave;
    p->cap = cap;
    p->su = 0;
    p->tab_stride = tab_stride;
    p->flags = flags;
    p->lds = lds;
    const int s = pack_upload(*p, off, tab, order, tiles);
    if (s != ET_OK) {
        delete p;
        return s;
    }
    *pack = p;
    return ET_OK;
}

}  // namespace et
