// The token-local part of an encoder layer in ONE launch: output projection (+ residual, row sums)
// -> FFN up-projection (normalising that sum, + activation) -> FFN down-projection (+ residual, row
// sums) -> the next layer's QKV projection (normalising that sum).  Each of the four is the packed
// tile-sparse Linear of bsr_packed.hip.h; what the reference runs as separate kernels with
// SkipLayerNorm launches between them (Encoder/Encoder.h:81-96, Attention/Attention.h:246-265).
//
// Why one launch can do it.  Every one of these products maps token rows to token rows, and a
// workgroup with id i runs on XCD i % 8: a token strip is given to the same XCD in all four steps,
// so whatever a step reads was written by workgroups of the same XCD, into the L2 that XCD's
// compute units share.  Between two steps the 32 workgroups of an XCD meet at a counter in that L2
// (an atomic add and a bounded poll, about 0.9 us) instead of at a kernel boundary (about 2.3 us:
// drain, write-back and invalidation of every L2, dispatch).  No cache maintenance is needed in
// between: stores are complete at the L2 when their wave's memory counter reads zero, a compute
// unit's L1 is write-through and holds nothing of a buffer that is written in this launch before
// that buffer's writers have met its readers at the barrier (every buffer is read only after its
// last write).  The weights of a step depend on no other step: a workgroup requests the next step's
// slots when it has multiplied the current one, so they travel while it runs its epilogue and waits
// at the barrier.
//
// What is checked rather than assumed: the workgroups that share a counter (equal id % 8) compare
// the hardware's XCD ids they run on, and a poll gives up after a bounded number of rounds; either event is recorded in the
// status words behind the counters (et_encoder_chain_status), the launch still ends, and the
// caller goes back to separate launches.  All workgroups of the launch must be resident at once:
// one per compute unit, at most as many as the device has.
#include <algorithm>

#include "bsr_packed.hip.h"

namespace et {

constexpr int kChainWaves = 12;
// most slots per wave of the four steps (registers: a slot is four per lane, and the next step's
// slots are requested while the current step runs its epilogue)
constexpr int kChainCaps[4] = {8, 12, 24, 8};

struct ChainArgs {
    PackArgs ph[4];  // output projection, FFN up, FFN down, next QKV
    int nphase;      // 3: no QKV projection follows (last layer)
    unsigned *sync;  // counters: one 128-byte line per XCD; then status words
    int spin_limit;
    int wg_per_xcd;
};

// All workgroups of this XCD have passed `target / wg_per_xcd` barriers.  The wave's own stores are
// complete (at the L2) before it arrives.
__device__ __forceinline__ void chain_barrier(unsigned *counter, unsigned target, unsigned *status, int spin_limit) {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {  // nobody has given up yet
            int n = 0;
            while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                __builtin_amdgcn_s_sleep(1);
                if (++n > spin_limit) {
                    __hip_atomic_fetch_add(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    break;
                }
            }
        }
    }
    __syncthreads();
    asm volatile("" ::: "memory");
}

__global__ __launch_bounds__(kChainWaves * 64) void bsr16_chain_kernel(const ChainArgs c) {
    extern __shared__ __align__(256) unsigned char chain_smem[];
    const int xcd = blockIdx.x % kPkXcds;
    unsigned *counter = c.sync + xcd * 32;
    unsigned *status = c.sync + kPkXcds * 32;
    if (threadIdx.x == 0) {
        // the workgroups that share a counter must share an XCD: the first of them to come by leaves
        // the hardware's XCD id, the others compare
        const unsigned xcc = (__builtin_amdgcn_s_getreg((3 << 11) | 20) & 15u) + 1u;  // XCC_ID
        unsigned seen = 0;
        __hip_atomic_compare_exchange_strong(status + 2 + xcd, &seen, xcc, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
        if (seen != 0 && seen != xcc) __hip_atomic_fetch_add(status + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const unsigned per = (unsigned)c.wg_per_xcd;
    PkPhase<2, kChainCaps[0], false, true, 1, true> p0;
    PkPhase<2, kChainCaps[1], true, false, 4, true> p1;
    PkPhase<1, kChainCaps[2], false, true, 1, true> p2;
    PkPhase<2, kChainCaps[3], true, false, 4, true> p3;
    p0.setup(c.ph[0], chain_smem, blockIdx.x, true);
    p1.setup(c.ph[1], chain_smem, blockIdx.x, true);
    p2.setup(c.ph[2], chain_smem, blockIdx.x, true);
    p3.setup(c.ph[3], chain_smem, blockIdx.x, true);

    // ---- output projection
    if (p0.it.live) {
        p0.request_weights(c.ph[0]);
        p0.request_inputs(c.ph[0]);
        p0.stage(c.ph[0]);
        __syncthreads();
        p0.multiply();
    }
    // the next step's weights are requested between the units of this step's epilogue: a wave that
    // waits for the memory pipeline to take its request leaves the vector unit to the others
    if (p0.it.live) {
        __syncthreads();
        p0.epilogue(c.ph[0], [&](int u) {
            __builtin_amdgcn_sched_barrier(0);
            if (p1.it.live) p1.template request_weights<p0.kUnits>(c.ph[1], u);
            __builtin_amdgcn_sched_barrier(0);
        });
    } else if (p1.it.live) {
        p1.request_weights(c.ph[1]);
    }
    chain_barrier(counter, per, status, c.spin_limit);

    // ---- FFN up-projection
    if (p1.it.live) {
        p1.request_inputs(c.ph[1]);
        p1.stage(c.ph[1]);
        __syncthreads();
        p1.multiply();
    }
    if (p1.it.live) {
        __syncthreads();
        p1.epilogue(c.ph[1], [&](int u) {
            __builtin_amdgcn_sched_barrier(0);
            if (p2.it.live) p2.template request_weights<2 * p1.kUnits>(c.ph[2], u);  // half of them: registers
            __builtin_amdgcn_sched_barrier(0);
        });
    } else if (p2.it.live) {
#pragma unroll
        for (int u = 0; u < p1.kUnits; u++) p2.template request_weights<2 * p1.kUnits>(c.ph[2], u);
    }
    chain_barrier(counter, 2 * per, status, c.spin_limit);

    // ---- FFN down-projection
    if (p2.it.live) {
#pragma unroll
        for (int u = p1.kUnits; u < 2 * p1.kUnits; u++) p2.template request_weights<2 * p1.kUnits>(c.ph[2], u);
        p2.request_inputs(c.ph[2]);
        p2.stage(c.ph[2]);
        __syncthreads();
        p2.multiply();
    }
    if (p2.it.live) {
        __syncthreads();
        p2.epilogue(c.ph[2], [&](int u) {
            __builtin_amdgcn_sched_barrier(0);
            if (c.nphase > 3 && p3.it.live) p3.template request_weights<p2.kUnits>(c.ph[3], u);
            __builtin_amdgcn_sched_barrier(0);
        });
    } else if (c.nphase > 3 && p3.it.live) {
        p3.request_weights(c.ph[3]);
    }
    if (c.nphase <= 3) return;
    chain_barrier(counter, 3 * per, status, c.spin_limit);

    // ---- the next layer's QKV projection
    if (p3.it.live) {
        p3.request_inputs(c.ph[3]);
        p3.stage(c.ph[3]);
        __syncthreads();
        p3.multiply();
        __syncthreads();
        p3.epilogue(c.ph[3]);
    }
}

// workgroups per XCD that a step needs when a token stays on the XCD of its 32-row neighbourhood
static int chain_items_per_xcd(const et_bsr_pack_s &p, int T) {
    const int units = (T + 31) / 32;  // 32-row neighbourhoods
    const int rounds = (units + kPkXcds - 1) / kPkXcds;
    return rounds * (p.mt == 1 ? 2 : 1) * p.ngroups;
}

static int chain_check(const et_chain_desc *d, bool report) {
    auto no = [&](const char *why) {
        if (report) return fail(ET_ERR_UNSUPPORTED, "et_encoder_chain_f32: %s", why);
        return (int)ET_ERR_UNSUPPORTED;
    };
    if (!d || !d->o || !d->up || !d->down) return no("the three packs of the layer must be set");
    const et_bsr_pack_s *ps[4] = {d->o, d->up, d->down, d->qkv};
    const int n = d->qkv ? 4 : 3;
    for (int i = 0; i < n; i++) {
        if (ps[i]->nwave != kChainWaves) return no("every pack must be built for 12 waves");
        if (ps[i]->cap > kChainCaps[i] || ps[i]->cap % 4) return no("a pack has more slots per wave than its step of the chain holds (8 / 12 / 24 / 8)");
        if (d->T > ps[i]->T || d->T <= 0 || d->T % 16) return no("T must be a multiple of 16 within what the packs were built for");
    }
    if (d->o->mt != 2 || d->up->mt != 2 || d->down->mt != 1 || (d->qkv && d->qkv->mt != 2))
        return no("strip heights must be 32 / 32 / 16 / 32 rows");
    if (d->up->su != 4 || (d->qkv && d->qkv->su != 4)) return no("the normalising packs must deal four strip vectors per thread");
    if (d->o->ngroups > kMaxStatGroups || d->down->ngroups > kMaxStatGroups) return no("too many block-row groups for the row sums");
    if (d->o->out != d->up->in || d->up->out != d->down->in || d->down->out != d->o->out || (d->qkv && d->qkv->in != d->down->out))
        return no("the widths of the four projections do not chain");
    int per = 0;
    size_t lds = 0;
    for (int i = 0; i < n; i++) {
        per = std::max(per, chain_items_per_xcd(*ps[i], d->T));
        lds = std::max(lds, ps[i]->lds);
    }
    if (lds > 160 * 1024) return no("a step needs more than 160 KB of LDS");
    static int num_cu = 0;
    if (!num_cu) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return no("no device");
        num_cu = prop.multiProcessorCount;
    }
    if (per * kPkXcds > num_cu) return no("more workgroups than compute units: they could not all be resident");
    return ET_OK;
}

}  // namespace et

using namespace et;

extern "C" {

int et_encoder_chain_supported(const et_chain_desc *d) { return chain_check(d, true) == ET_OK ? 1 : 0; }

int et_encoder_chain_f32(const et_chain_desc *d, int *stat_groups2, et_stream stream) {
    int s = chain_check(d, true);
    if (s != ET_OK) return s;
    ET_REQUIRE(d->Z && d->V1 && d->stats1 && d->fin1 && d->H && d->V2 && d->stats2 && d->gamma1 && d->beta1 && d->sync &&
                   ((d->resid != nullptr) != (d->resid16 != nullptr)),
               ET_ERR_INVALID_ARG, "et_encoder_chain_f32: NULL pointer, or not exactly one of resid and resid16");
    ET_REQUIRE(d->resid_fin == nullptr || (d->resid && d->resid_gamma && d->resid_beta), ET_ERR_INVALID_ARG,
               "et_encoder_chain_f32: a residual to normalise needs its affine vectors");
    ET_REQUIRE(!d->qkv || (d->gamma2 && d->beta2 && d->QKV), ET_ERR_INVALID_ARG, "et_encoder_chain_f32: the QKV step needs gamma2, beta2 and QKV");
    ET_REQUIRE(d->act >= ET_ACT_NONE && d->act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_encoder_chain_f32: act=%d", d->act);
    auto al = [](const void *p, uintptr_t m) { return (reinterpret_cast<uintptr_t>(p) & m) == 0; };
    ET_REQUIRE(al(d->Z, 15) && al(d->V1, 15) && al(d->V2, 15) && al(d->H, 15) && al(d->resid, 15) && al(d->resid16, 7) &&
                   al(d->QKV, 7) && al(d->gamma1, 15) && al(d->beta1, 15) && al(d->gamma2, 15) && al(d->beta2, 15) &&
                   al(d->fin1, 7) && al(d->fin2, 7) && al(d->sync, 127),
               ET_ERR_UNSUPPORTED, "et_encoder_chain_f32: operands must be 16-byte aligned (sync: 128)");
    if (stat_groups2) *stat_groups2 = d->down->ngroups;

    ChainArgs c{};
    // output projection
    c.ph[0] = pk_base_args(*d->o, d->bias_o, d->T);
    c.ph[0].X = reinterpret_cast<const _Float16 *>(d->Z);
    c.ph[0].Y32 = d->V1;
    c.ph[0].resid32 = d->resid;
    c.ph[0].resid16 = reinterpret_cast<const _Float16 *>(d->resid16);
    c.ph[0].rs_fin = d->resid_fin;
    c.ph[0].rs_gamma = reinterpret_cast<const _Float16 *>(d->resid_gamma);
    c.ph[0].rs_beta = reinterpret_cast<const _Float16 *>(d->resid_beta);
    c.ph[0].st_out = d->stats1;
    // FFN up
    c.ph[1] = pk_base_args(*d->up, d->bias_up, d->T);
    c.ph[1].Y = reinterpret_cast<_Float16 *>(d->H);
    c.ph[1].act = d->act;
    c.ph[1].X32 = d->V1;
    c.ph[1].st_in = d->stats1;
    c.ph[1].st_groups = d->o->ngroups;
    c.ph[1].gamma = reinterpret_cast<const _Float16 *>(d->gamma1);
    c.ph[1].beta = reinterpret_cast<const _Float16 *>(d->beta1);
    c.ph[1].eps = d->eps1;
    c.ph[1].fin_out = d->fin1;
    // FFN down: the residual is LayerNorm1(V1), formed from V1 and the statistics the up-projection left
    c.ph[2] = pk_base_args(*d->down, d->bias_down, d->T);
    c.ph[2].X = reinterpret_cast<const _Float16 *>(d->H);
    c.ph[2].Y32 = d->V2;
    c.ph[2].resid32 = d->V1;
    c.ph[2].rs_fin = d->fin1;
    c.ph[2].rs_gamma = reinterpret_cast<const _Float16 *>(d->gamma1);
    c.ph[2].rs_beta = reinterpret_cast<const _Float16 *>(d->beta1);
    c.ph[2].st_out = d->stats2;
    c.nphase = 3;
    if (d->qkv) {
        c.ph[3] = pk_base_args(*d->qkv, d->bias_qkv, d->T);
        c.ph[3].Y = reinterpret_cast<_Float16 *>(d->QKV);
        c.ph[3].act = ET_ACT_NONE;
        c.ph[3].X32 = d->V2;
        c.ph[3].st_in = d->stats2;
        c.ph[3].st_groups = d->down->ngroups;
        c.ph[3].gamma = reinterpret_cast<const _Float16 *>(d->gamma2);
        c.ph[3].beta = reinterpret_cast<const _Float16 *>(d->beta2);
        c.ph[3].eps = d->eps2;
        c.ph[3].fin_out = d->fin2;
        c.nphase = 4;
    } else {
        c.ph[3] = c.ph[1];  // a valid description; never run
    }
    c.sync = d->sync;
    c.spin_limit = 100000;  // about 20 ms of polling before a workgroup gives up
    const et_bsr_pack_s *ps[4] = {d->o, d->up, d->down, d->qkv};
    size_t lds = 0;
    int per = 0;
    for (int i = 0; i < c.nphase; i++) {
        lds = std::max(lds, ps[i]->lds);
        per = std::max(per, chain_items_per_xcd(*ps[i], d->T));
    }
    c.wg_per_xcd = per;
    static bool raised = false;
    if (!raised) {
        ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(bsr16_chain_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   160 * 1024));
        raised = true;
    }
    bsr16_chain_kernel<<<dim3((unsigned)(per * kPkXcds)), kChainWaves * 64, lds, as_stream(stream)>>>(c);
    return check_launch("bsr16_chain_kernel");
}

int et_encoder_chain_status(const uint32_t *sync, int *gave_up, int *misplaced) {
    ET_REQUIRE(sync != nullptr, ET_ERR_INVALID_ARG, "et_encoder_chain_status: NULL pointer");
    uint32_t st[2] = {0, 0};
    ET_HIP(hipMemcpy(st, sync + kPkXcds * 32, sizeof st, hipMemcpyDeviceToHost));
    if (gave_up) *gave_up = (int)st[0];
    if (misplaced) *misplaced = (int)st[1];
    return ET_OK;
}

}  // extern "C"
