// Tile-sparse Linear, packed form: the stand-alone kernels, the pack builder and the entry points
// (device code and the description of the form: bsr_packed.hip.h).
#include <algorithm>
#include <new>
#include <vector>

#include "bsr_packed.hip.h"
#include "../../include/et_tuning.h"

namespace et {

template <int MT, int CAP, bool NORM32, bool RES32, int SU>
__global__ __launch_bounds__(pk_max_waves(CAP, NORM32, SU) * 64) void bsr16_packed_kernel(const PackArgs a) {
    extern __shared__ __align__(256) unsigned char pk_smem[];
    PkPhase<MT, CAP, NORM32, RES32, SU> ph;
    ph.setup(a, pk_smem, blockIdx.x, false);
    if (!ph.it.live) return;
    // a strip that needs arithmetic before the barrier goes first in the load queue, then the weights;
    // a strip that goes straight into LDS is requested last (its arrival is what stage() waits for)
    if constexpr (NORM32) ph.request_inputs(a);
    ph.request_weights(a);
    if constexpr (!NORM32) ph.request_inputs(a);
    ph.stage(a);
    __syncthreads();
    ph.multiply();
    __syncthreads();
    ph.epilogue(a);
}

// Slot s of the pack = tiles order[2s] and order[2s + 1] (a zero tile where negative), stored in the
// order the lanes of a wave read it: the 16-byte piece of lane (r, g) — row r, values 8 (g & 1) .. + 7
// of tile g >> 1 — lies at byte 16 * lane, so a slot is one contiguous 1 KiB wave load.
__global__ void bsr_pack_gather_kernel(_Float16 *__restrict__ pw, const _Float16 *__restrict__ tiles,
                                       const int32_t *__restrict__ order, int nslots) {
    const int s = blockIdx.x, lane = threadIdx.x;
    if (s >= nslots || lane >= 64) return;
    const int src = order[2 * s + (lane >> 5)];
    const int piece = (lane & 15) * 2 + ((lane >> 4) & 1);
    const h8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const h8 *t = reinterpret_cast<const h8 *>(tiles + (size_t)(src < 0 ? 0 : src) * 256);
    reinterpret_cast<h8 *>(pw + (size_t)s * 512)[lane] = src < 0 ? zero : t[piece];
}

}  // namespace et

using namespace et;

namespace et {

constexpr size_t kPkLdsBudget = 160 * 1024;
static const int kPkCaps[] = {4, 8, 12, 16, 20, 24};

static size_t pk_lds_bytes(int mt, int in, int rows_per_wg, int nwave) {
    const size_t strip = (size_t)mt * 16 * in * 2;
    const size_t parts = (size_t)(rows_per_wg + nwave) * mt * 1024;
    const size_t red = (size_t)nwave * mt * 16 * sizeof(float2);
    return std::max(strip, red) + parts;
}

// strip vectors per thread of the normalising prologue for this wave count, or 0 when the
// threads do not deal evenly to the rows
static int pk_norm_su(int mt, int in, int nwave) {
    const int upr = in / 8;
    if (upr < 64 || (nwave * 64) % upr) return 0;
    const int dr = nwave * 64 / upr;
    if (dr < 1 || (16 * mt) % dr) return 0;
    const int su = 16 * mt / dr;
    if (mt == 2) return (su == 4 || su == 8) ? su : 0;
    return (su == 2 || su == 4 || su == 8) ? su : 0;
}

template <int MT, int CAP, bool NORM32, bool RES32, int SU>
static int pk_launch(const PackArgs &a, const et_bsr_pack_s &p, hipStream_t stream) {
    auto kernel = bsr16_packed_kernel<MT, CAP, NORM32, RES32, SU>;
    if (p.lds > 64 * 1024) {
        static bool raised = false;  // per instantiation
        if (!raised) {
            ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       160 * 1024));
            raised = true;
        }
    }
    const int nstrips = (a.T + MT * 16 - 1) / (MT * 16);
    const int rounds = (nstrips + kPkXcds - 1) / kPkXcds;
    kernel<<<dim3((unsigned)(rounds * kPkXcds * a.ngroups)), p.nwave * 64, p.lds, stream>>>(a);
    return check_launch("bsr16_packed_kernel");
}

template <int MT, bool NORM32, bool RES32, int SU>
static int pk_dispatch_cap(const PackArgs &a, const et_bsr_pack_s &p, hipStream_t stream) {
    switch (p.cap) {
        case 4: return pk_launch<MT, 4, NORM32, RES32, SU>(a, p, stream);
        case 8: return pk_launch<MT, 8, NORM32, RES32, SU>(a, p, stream);
        case 12: return pk_launch<MT, 12, NORM32, RES32, SU>(a, p, stream);
        case 16: return pk_launch<MT, 16, NORM32, RES32, SU>(a, p, stream);
        case 20: return pk_launch<MT, 20, NORM32, RES32, SU>(a, p, stream);
        case 24: return pk_launch<MT, 24, NORM32, RES32, SU>(a, p, stream);
        default: return fail(ET_ERR_INVALID_ARG, "tile-sparse Linear (packed): no kernel for %d slots per wave", p.cap);
    }
}

template <bool RES32> static int pk_dispatch_plain(const PackArgs &a, const et_bsr_pack_s &p, hipStream_t stream) {
    return p.mt == 2 ? pk_dispatch_cap<2, false, RES32, 1>(a, p, stream) : pk_dispatch_cap<1, false, RES32, 1>(a, p, stream);
}

static int pk_dispatch_norm(const PackArgs &a, const et_bsr_pack_s &p, hipStream_t stream) {
    if (p.mt == 2) {
        if (p.su == 4) return pk_dispatch_cap<2, true, false, 4>(a, p, stream);
        if (p.su == 8) return pk_dispatch_cap<2, true, false, 8>(a, p, stream);
    } else {
        if (p.su == 2) return pk_dispatch_cap<1, true, false, 2>(a, p, stream);
        if (p.su == 4) return pk_dispatch_cap<1, true, false, 4>(a, p, stream);
        if (p.su == 8) return pk_dispatch_cap<1, true, false, 8>(a, p, stream);
    }
    return fail(ET_ERR_INVALID_ARG, "tile-sparse Linear (packed): the pack was not built for a normalising consumer");
}

}  // namespace et

namespace et {
int pack_upload(et_bsr_pack_s &p, const std::vector<uint32_t> &off, const std::vector<int32_t> &tab,
                const std::vector<int32_t> &order, const et_f16 *tiles) {
    auto upload = [&](void **dst, const void *src, size_t bytes) -> int {
        int s = et_malloc(dst, std::max<size_t>(bytes, 16));
        if (s != ET_OK) return s;
        if (bytes) ET_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return ET_OK;
    };
    void *d_order = nullptr;
    int s = upload(&p.poff, off.data(), off.size() * 4);
    if (s == ET_OK) s = upload(&p.ptab, tab.data(), tab.size() * 4);
    if (s == ET_OK) s = check_hip(hipMalloc(&d_order, std::max<size_t>(order.size() * 4, 16)), "hipMalloc");
    if (s == ET_OK) s = check_hip(hipMemcpy(d_order, order.data(), order.size() * 4, hipMemcpyHostToDevice), "hipMemcpy");
    const size_t nslots = order.size() / 2;
    if (s == ET_OK) s = et_malloc(&p.pw, std::max<size_t>(nslots * 1024, 16));
    if (s == ET_OK && nslots) {
        bsr_pack_gather_kernel<<<(unsigned)nslots, 64>>>(static_cast<_Float16 *>(p.pw), reinterpret_cast<const _Float16 *>(tiles),
                                                         static_cast<const int32_t *>(d_order), (int)nslots);
        s = check_launch("bsr_pack_gather_kernel");
        if (s == ET_OK) s = check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize");
    }
    (void)hipFree(d_order);
    return s;
}
}  // namespace et

extern "C" {

int et_bsr16_pack_create_geom(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, int T, int in, int out,
                              int flags, int mt, int ngroups, int nwave, int cap, et_bsr_pack *pack) {
    ET_REQUIRE(pack != nullptr, ET_ERR_INVALID_ARG, "et_bsr16_pack_create: pack is NULL");
    *pack = nullptr;
    ET_REQUIRE(row_ptr && col_idx && tiles, ET_ERR_INVALID_ARG, "et_bsr16_pack_create: NULL pointer");
    ET_REQUIRE((flags & ~(ET_PACK_NORM_CONSUMER | ET_PACK_STATS_PRODUCER | ET_PACK_ROW_LOOP)) == 0 &&
                   (!(flags & ET_PACK_ROW_LOOP) || flags == ET_PACK_ROW_LOOP),
               ET_ERR_INVALID_ARG, "et_bsr16_pack_create: flags=%d", flags);
    ET_REQUIRE(T > 0 && in > 0 && out > 0 && T % 16 == 0 && out % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_bsr16_pack_create: T=%d in=%d out=%d must be positive multiples of 16", T, in, out);
    const bool consumer = (flags & ET_PACK_NORM_CONSUMER) != 0, producer = (flags & ET_PACK_STATS_PRODUCER) != 0;
    // strip rows are whole multiples of 256 bytes (the swizzle), a 16-row strip and its parts fit the LDS
    ET_REQUIRE(in % 128 == 0 && in <= 4096 && (!consumer || in >= 512), ET_ERR_UNSUPPORTED,
               "et_bsr16_pack_create: in=%d outside the packed kernel's range (multiples of 128 up to 4096%s)", in,
               consumer ? ", at least 512 for a normalising consumer" : "");
    ET_REQUIRE((mt == 0 || mt == 1 || mt == 2) && ngroups >= 0 && nwave >= 0 && nwave <= kPkMaxWaves && cap >= 0,
               ET_ERR_INVALID_ARG, "et_bsr16_pack_create: mt=%d ngroups=%d nwave=%d cap=%d", mt, ngroups, nwave, cap);
    const int nbr = out / 16, bc = in / 16;
    std::vector<int32_t> rp((size_t)nbr + 1);
    ET_HIP(hipMemcpy(rp.data(), row_ptr, rp.size() * 4, hipMemcpyDeviceToHost));
    ET_REQUIRE(rp[0] == 0, ET_ERR_INVALID_ARG, "et_bsr16_pack_create: row_ptr must start at 0");
    for (int r = 0; r < nbr; r++)
        ET_REQUIRE(rp[(size_t)r + 1] >= rp[(size_t)r], ET_ERR_INVALID_ARG, "et_bsr16_pack_create: row_ptr decreases");
    const int ntile = rp[(size_t)nbr];
    std::vector<int32_t> ci((size_t)std::max(ntile, 1));
    if (ntile) ET_HIP(hipMemcpy(ci.data(), col_idx, (size_t)ntile * 4, hipMemcpyDeviceToHost));
    for (int t = 0; t < ntile; t++)
        ET_REQUIRE(ci[(size_t)t] >= 0 && ci[(size_t)t] < bc, ET_ERR_INVALID_ARG,
                   "et_bsr16_pack_create: column-tile index %d of tile %d outside [0, %d)", ci[(size_t)t], t, bc);

    if (flags & ET_PACK_ROW_LOOP) {  // the form for many token rows has a geometry and a builder of its own
        ET_REQUIRE(mt == 0 && ngroups == 0 && nwave == 0 && cap == 0, ET_ERR_INVALID_ARG,
                   "et_bsr16_pack_create: a row-loop pack chooses its own geometry");
        return rowloop_pack_create(rp, ci, tiles, T, in, out, flags, pack);
    }
    // ---- strips and block-row groups: one workgroup per compute unit where the shape allows it
    if (mt == 0) mt = (T >= 32 && (size_t)32 * in * 2 <= 64 * 1024) ? 2 : 1;
    const int strips = (T + mt * 16 - 1) / (mt * 16);
    ET_REQUIRE(strips <= 1024, ET_ERR_UNSUPPORTED, "et_bsr16_pack_create: %d token rows are beyond the packed kernel's range", T);
    const bool auto_groups = ngroups == 0;
    if (auto_groups) ngroups = strips >= 256 ? 1 : 256 / strips;
    ngroups = std::min(ngroups, nbr);
    if (producer) ngroups = std::min(ngroups, kMaxStatGroups);

    struct Slot {
        int t0, t1, c0, c1, row;
        bool row_end;
    };
    // slots of every block-row (two tiles each, a zero tile where the count is odd)
    std::vector<int> row_slots((size_t)nbr);
    long total_slots = 0;
    for (int rb = 0; rb < nbr; rb++) {
        row_slots[(size_t)rb] = (rp[(size_t)rb + 1] - rp[(size_t)rb] + 1) / 2;
        total_slots += row_slots[(size_t)rb];
    }
    int rows_per_wg = 0, S = 0;
    std::vector<int> gbegin;  // first block-row of every group, and nbr at the end
    std::vector<std::vector<Slot>> gslots;
    auto build = [&]() {
        // contiguous groups with the smallest possible fullest group (no group empty): the least bound
        // a left-to-right cut can keep, found by bisection
        ngroups = std::max(1, std::min(ngroups, nbr));
        auto cut = [&](long bound, std::vector<int> *out) -> bool {
            int groups = 0, rb = 0;
            if (out) out->assign(1, 0);
            while (rb < nbr) {
                if (++groups > ngroups) return false;
                long sum = 0;
                const int left_after = ngroups - groups;  // groups still to be filled behind this one
                int n = 0;
                while (rb < nbr && nbr - rb > left_after && (n == 0 || sum + row_slots[(size_t)rb] <= bound)) {
                    sum += row_slots[(size_t)rb++];
                    n++;
                }
                if (sum > bound) return false;
                if (out) out->push_back(rb);
            }
            return groups == ngroups;
        };
        long lo = 0, hi = std::max<long>(total_slots, 1);
        for (int rb = 0; rb < nbr; rb++) lo = std::max<long>(lo, row_slots[(size_t)rb]);
        while (lo < hi) {
            const long mid = (lo + hi) / 2;
            if (cut(mid, nullptr)) hi = mid;
            else lo = mid + 1;
        }
        cut(lo, &gbegin);
        rows_per_wg = 0;
        gslots.assign((size_t)ngroups, {});
        S = 0;
        for (int gi = 0; gi < ngroups; gi++) {
            const int rb0 = gbegin[(size_t)gi], rb1 = gbegin[(size_t)gi + 1];
            rows_per_wg = std::max(rows_per_wg, rb1 - rb0);
            auto &v = gslots[(size_t)gi];
            for (int rb = rb0; rb < rb1; rb++) {
                for (int t = rp[(size_t)rb]; t < rp[(size_t)rb + 1]; t += 2) {
                    const bool two = t + 1 < rp[(size_t)rb + 1];
                    v.push_back(Slot{t, two ? t + 1 : -1, ci[(size_t)t], two ? ci[(size_t)t + 1] : ci[(size_t)t], rb - rb0,
                                     t + 2 >= rp[(size_t)rb + 1]});
                }
            }
            S = std::max(S, (int)v.size());
        }
    };
    // (waves, slots per wave) for the fullest group: the fewest slots fetched, then the most waves
    int su = 0;
    auto choose = [&]() -> bool {
        long best = -1;
        int best_w = 0, best_c = 0, best_su = 0;
        for (int c : kPkCaps) {
            if (cap && c != cap) continue;
            for (int wv = 1; wv <= pk_max_waves(c, consumer); wv++) {
                if (nwave && wv != nwave) continue;
                if ((long)wv * c < std::max(S, 1)) continue;
                int s = 1;
                if (consumer) {
                    s = pk_norm_su(mt, in, wv);
                    if (!s || wv > pk_max_waves(c, true, s)) continue;
                }
                if (pk_lds_bytes(mt, in, rows_per_wg, wv) > kPkLdsBudget) continue;
                const long cost = (long)wv * c * 64 - wv;  // slots fetched; ties go to more waves
                if (best < 0 || cost < best) {
                    best = cost;
                    best_w = wv;
                    best_c = c;
                    best_su = s;
                }
            }
        }
        if (best < 0) return false;
        nwave = best_w;
        cap = best_c;
        su = best_su;
        return true;
    };
    build();
    const int nwave_req = nwave, cap_req = cap;
    while (!choose()) {
        // too many slots for one workgroup: more, smaller groups (several workgroups per compute unit)
        nwave = nwave_req;
        cap = cap_req;
        const bool can_split = auto_groups && ngroups < nbr && (!producer || ngroups < kMaxStatGroups);
        ET_REQUIRE(can_split, ET_ERR_UNSUPPORTED,
                   "et_bsr16_pack_create: T=%d in=%d out=%d (%d slots in the fullest of %d block-row groups) does not fit "
                   "the packed kernel",
                   T, in, out, S, ngroups);
        ngroups = std::min(producer ? std::min(nbr, kMaxStatGroups) : nbr, ngroups * 2);
        build();
    }

    // ---- flatten
    const int tab_stride = (kPkTabHead + rows_per_wg + 1 + 3) / 4 * 4;
    const size_t nslab = (size_t)ngroups * nwave;
    std::vector<int32_t> order(nslab * cap * 2, -1), tab((size_t)ngroups * tab_stride, 0);
    std::vector<uint32_t> off(nslab * cap, 0);
    for (int gi = 0; gi < ngroups; gi++) {
        const auto &v = gslots[(size_t)gi];
        int32_t *tb = &tab[(size_t)gi * tab_stride];
        const int n = (int)v.size(), per = n / nwave, rem = n % nwave;
        tb[kPkTabRows] = gbegin[(size_t)gi];
        tb[kPkTabRows + 1] = gbegin[(size_t)gi + 1] - gbegin[(size_t)gi];
        std::vector<int> first_part((size_t)rows_per_wg + 1, -1);
        int pos = 0, nparts = 0;
        for (int wv = 0; wv < nwave; wv++) {
            const int cnt = per + (wv < rem ? 1 : 0);
            uint32_t m = 0;
            tb[kPkMaxWaves + wv] = nparts;
            const size_t slab = (size_t)gi * nwave + wv;
            for (int p = 0; p < cnt; p++, pos++) {
                const Slot &s = v[(size_t)pos];
                order[(slab * cap + p) * 2] = s.t0;
                order[(slab * cap + p) * 2 + 1] = s.t1;
                off[slab * cap + p] = (uint32_t)(s.c0 * 32) | ((uint32_t)(s.c1 * 32) << 16);
                const bool starts = p == 0 || v[(size_t)pos - 1].row_end;  // a part starts at the wave's first slot or after a row
                if (starts && first_part[(size_t)s.row] < 0) first_part[(size_t)s.row] = nparts;
                if (s.row_end || p == cnt - 1) {
                    m |= 1u << p;
                    nparts++;
                }
            }
            tb[wv] = (int32_t)m;
            tb[kPkTabSlots + wv] = (cnt + 3) / 4 * 4;
        }
        // part_start[i]: first part of local row i; rows without tiles take the next row's
        int next = nparts;
        first_part[(size_t)rows_per_wg] = nparts;
        for (int i = rows_per_wg - 1; i >= 0; i--) {
            if (first_part[(size_t)i] < 0) first_part[(size_t)i] = next;
            next = first_part[(size_t)i];
        }
        for (int i = 0; i <= rows_per_wg; i++) tb[kPkTabHead + i] = first_part[(size_t)i];
        ET_REQUIRE(nparts <= rows_per_wg + nwave, ET_ERR_INVALID_ARG, "et_bsr16_pack_create: internal: %d parts", nparts);
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
    p->su = consumer ? su : 0;
    p->tab_stride = tab_stride;
    p->flags = flags;
    p->lds = pk_lds_bytes(mt, in, rows_per_wg, nwave);
    const int s = pack_upload(*p, off, tab, order, tiles);
    if (s != ET_OK) {
        delete p;
        return s;
    }
    *pack = p;
    return ET_OK;
}

int et_bsr16_pack_create(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, int T, int in, int out,
                         int flags, int nwave, et_bsr_pack *pack) {
    return et_bsr16_pack_create_geom(row_ptr, col_idx, tiles, T, in, out, flags, 0, 0, nwave, 0, pack);
}

int et_bsr16_pack_destroy(et_bsr_pack pack) {
    delete pack;
    return ET_OK;
}

int et_bsr16_pack_info(et_bsr_pack pack, int *mt, int *ngroups, int *nwave, int *cap, int *lds_bytes) {
    ET_REQUIRE(pack != nullptr, ET_ERR_INVALID_ARG, "et_bsr16_pack_info: pack is NULL");
    if (mt) *mt = pack->mt;
    if (ngroups) *ngroups = pack->ngroups;
    if (nwave) *nwave = pack->nwave;
    if (cap) *cap = pack->cap;
    if (lds_bytes) *lds_bytes = (int)pack->lds;
    return ET_OK;
}

static int pk_check_T(const et_bsr_pack_s *pack, int T, const char *who) {
    ET_REQUIRE(pack != nullptr, ET_ERR_INVALID_ARG, "%s: pack is NULL", who);
    ET_REQUIRE(T >= 0 && T % 16 == 0, ET_ERR_UNSUPPORTED, "%s: T=%d must be a multiple of 16", who, T);
    return ET_OK;
}

int et_linear_bsr16_packed_f16(et_bsr_pack pack, const et_f16 *bias, const et_f16 *X, et_f16 *Y, float *Y32, int T,
                               int act, et_stream stream) {
    int s = pk_check_T(pack, T, "et_linear_bsr16_packed_f16");
    if (s != ET_OK) return s;
    ET_REQUIRE(X && ((Y != nullptr) != (Y32 != nullptr)), ET_ERR_INVALID_ARG,
               "et_linear_bsr16_packed_f16: X must be set, and exactly one of Y and Y32");
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_bsr16_packed_f16: act=%d", act);
    ET_REQUIRE((reinterpret_cast<uintptr_t>(X) & 15) == 0 && (reinterpret_cast<uintptr_t>(Y) & 7) == 0 &&
                   (reinterpret_cast<uintptr_t>(Y32) & 15) == 0,
               ET_ERR_UNSUPPORTED, "et_linear_bsr16_packed_f16: X and Y must be 16-byte aligned");
    if (T == 0) return ET_OK;
    PackArgs a = pk_base_args(*pack, bias, T);
    a.X = reinterpret_cast<const _Float16 *>(X);
    a.Y = reinterpret_cast<_Float16 *>(Y);
    a.Y32 = Y32;
    a.act = act;
    if (pack->flags & ET_PACK_ROW_LOOP) {
        ET_REQUIRE((reinterpret_cast<uintptr_t>(Y) & 15) == 0, ET_ERR_UNSUPPORTED,
                   "et_linear_bsr16_packed_f16: a row-loop pack stores its results 16-byte aligned");
        return rowloop_launch(a, *pack, as_stream(stream));
    }
    return pk_dispatch_plain<false>(a, *pack, as_stream(stream));
}

int et_linear_bsr16_packed_resid_stats_f32(et_bsr_pack pack, const et_f16 *bias, const et_f16 *X, const float *resid,
                                           const et_f16 *resid16, const float *resid_fin, const et_f16 *resid_gamma,
                                           const et_f16 *resid_beta, float *V, float *stats, int *stat_groups, int T,
                                           et_stream stream) {
    int s = pk_check_T(pack, T, "et_linear_bsr16_packed_resid_stats_f32");
    if (s != ET_OK) return s;
    ET_REQUIRE(X && V && stats && stat_groups && ((resid != nullptr) != (resid16 != nullptr)), ET_ERR_INVALID_ARG,
               "et_linear_bsr16_packed_resid_stats_f32: NULL pointer, or not exactly one of resid and resid16");
    ET_REQUIRE(resid_fin == nullptr || (resid && resid_gamma && resid_beta), ET_ERR_INVALID_ARG,
               "et_linear_bsr16_packed_resid_stats_f32: a residual to normalise needs its affine vectors");
    ET_REQUIRE(V != resid, ET_ERR_INVALID_ARG, "et_linear_bsr16_packed_resid_stats_f32: V must not alias the residual");
    ET_REQUIRE(((reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(resid) | reinterpret_cast<uintptr_t>(X)) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(resid16) & 7) == 0,
               ET_ERR_UNSUPPORTED, "et_linear_bsr16_packed_resid_stats_f32: X, V and resid must be 16-byte aligned");
    ET_REQUIRE(pack->ngroups <= kMaxStatGroups, ET_ERR_UNSUPPORTED,
               "et_linear_bsr16_packed_resid_stats_f32: the pack splits a row over %d block-row groups (build it with "
               "ET_PACK_STATS_PRODUCER)",
               pack->ngroups);
    *stat_groups = pack->ngroups;
    if (T == 0) return ET_OK;
    PackArgs a = pk_base_args(*pack, bias, T);
    a.X = reinterpret_cast<const _Float16 *>(X);
    a.Y32 = V;
    a.act = ET_ACT_NONE;
    a.resid32 = resid;
    a.resid16 = reinterpret_cast<const _Float16 *>(resid16);
    a.rs_fin = resid_fin;
    a.rs_gamma = reinterpret_cast<const _Float16 *>(resid_gamma);
    a.rs_beta = reinterpret_cast<const _Float16 *>(resid_beta);
    a.st_out = stats;
    return pk_dispatch_plain<true>(a, *pack, as_stream(stream));
}

int et_norm_linear_bsr16_packed_f32in(et_bsr_pack pack, const float *V, const float *stats, int stat_groups,
                                      const et_f16 *gamma, const et_f16 *beta, float eps, float *fin_out,
                                      const et_f16 *bias, et_f16 *Y, int T, int act, et_stream stream) {
    int s = pk_check_T(pack, T, "et_norm_linear_bsr16_packed_f32in");
    if (s != ET_OK) return s;
    ET_REQUIRE(V && stats && gamma && beta && Y, ET_ERR_INVALID_ARG, "et_norm_linear_bsr16_packed_f32in: NULL pointer");
    ET_REQUIRE(stat_groups >= 1 && stat_groups <= kMaxStatGroups, ET_ERR_INVALID_ARG,
               "et_norm_linear_bsr16_packed_f32in: stat_groups=%d must be in [1, %d]", stat_groups, kMaxStatGroups);
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_norm_linear_bsr16_packed_f32in: act=%d", act);
    ET_REQUIRE((pack->flags & ET_PACK_NORM_CONSUMER) && pack->su > 0, ET_ERR_INVALID_ARG,
               "et_norm_linear_bsr16_packed_f32in: the pack was not built with ET_PACK_NORM_CONSUMER");
    ET_REQUIRE(((reinterpret_cast<uintptr_t>(V) | reinterpret_cast<uintptr_t>(gamma) | reinterpret_cast<uintptr_t>(beta)) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(Y) & 7) == 0 && (reinterpret_cast<uintptr_t>(fin_out) & 7) == 0,
               ET_ERR_UNSUPPORTED, "et_norm_linear_bsr16_packed_f32in: V, gamma and beta must be 16-byte aligned");
    if (T == 0) return ET_OK;
    PackArgs a = pk_base_args(*pack, bias, T);
    a.Y = reinterpret_cast<_Float16 *>(Y);
    a.act = act;
    a.X32 = V;
    a.st_in = stats;
    a.st_groups = stat_groups;
    a.gamma = reinterpret_cast<const _Float16 *>(gamma);
    a.beta = reinterpret_cast<const _Float16 *>(beta);
    a.eps = eps;
    a.fin_out = fin_out;
    return pk_dispatch_norm(a, *pack, as_stream(stream));
}

}  // extern "C"
