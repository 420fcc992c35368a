// Tile-sparse Linear, streaming form:  Y[T x out] = act(X[T x in] * W^T + bias), W in 16x16 tiles.
//
// The input width is walked in chunks of KC columns.  For every chunk a workgroup brings in, with
// direct-to-LDS loads (global_load_lds_dwordx4: no register passes through, so a whole chunk is in
// flight at once), the [16*MT x KC] piece of its token strip AND the weight tiles of its block-rows
// that fall into the chunk, one chunk ahead of the one it multiplies (two LDS buffers).  The
// matrix cores are fed from LDS only: per "slot" (two tiles of one block-row = one
// v_mfma_f32_16x16x32_f16) one 16-byte read of the weights, one 4-byte read of the column, MT
// 16-byte reads of X.  Accumulators stay in registers across chunks, so the width of the input
// is not limited by LDS and a weight tile read from L2 serves 16*MT token rows.
//
// This needs the tiles of a block-row grouped by chunk, and the tiles one workgroup needs for one
// chunk contiguous in memory.  A "plan" holds that re-ordered copy of the weight (tiles padded
// with zero tiles to whole slots) together with the tables that describe it; it is built once per
// weight and launch geometry (et_bsr16_plan_create) from the reference layout, which stays the
// interchange format (mat_type/tile_mat/tile_mat.h:3-58).  Same mathematics as the reference
// kernel (Linear/SPMM_tile.cu:249-324): tile order inside a block-row is free.
#include <algorithm>
#include <new>
#include <vector>

#include "common.hip.h"

namespace et {

#define ET_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define ET_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

constexpr int kSNW = 8;        // waves per workgroup
constexpr int kSMaxRpw = 4;    // block-rows per wave (accumulator sets held in registers)
constexpr int kSXcds = 8;

struct BsrStreamArgs {
    const _Float16 *stiles;   // [ngroups][nchunk][max_slots][2][16][16] re-ordered tiles, zero tiles as padding
    const int32_t *sq;        // [ngroups][nchunk][q_ints] per slot and tile: 16-byte-chunk index of the tile's
                              // columns inside its K chunk
    const int32_t *wseg;      // [ngroups][nchunk][kSNW][8]  slot offset inside the chunk, slots per owned row
    const _Float16 *bias;
    const _Float16 *X;
    _Float16 *Y;              // binary16 result, or
    float *Y32;               // binary32 result (exactly one of the two is set)
    int T, in, out;
    int rows_per_wg, ngroups, nchunk, rpw;
    int max_slots;            // slots of every (group, chunk) region, a multiple of kSNW
    int q_ints;               // ints of the column list of one (group, chunk), a multiple of 256
    int nbuf;                 // LDS buffers (chunks in flight + 1), 2..4
    int act;
};

__device__ __forceinline__ float stream_act(float x, int act) {
    if (act == ET_ACT_RELU) return x > 0.0f ? x : 0.0f;
    if (act == ET_ACT_GELU) return gelu_tanh(x);
    return x;
}

// s_waitcnt vmcnt(n) for a wave-uniform run-time n (the instruction takes an immediate)
__device__ __forceinline__ void wait_vmcnt(int n) {
#define ET_VM_CASE(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
    switch (n) {
        ET_VM_CASE(0) ET_VM_CASE(1) ET_VM_CASE(2) ET_VM_CASE(3) ET_VM_CASE(4) ET_VM_CASE(5) ET_VM_CASE(6) ET_VM_CASE(7)
        ET_VM_CASE(8) ET_VM_CASE(9) ET_VM_CASE(10) ET_VM_CASE(11) ET_VM_CASE(12) ET_VM_CASE(13) ET_VM_CASE(14)
        ET_VM_CASE(15) ET_VM_CASE(16) ET_VM_CASE(17) ET_VM_CASE(18) ET_VM_CASE(19) ET_VM_CASE(20) ET_VM_CASE(21)
        ET_VM_CASE(22) ET_VM_CASE(23) ET_VM_CASE(24) ET_VM_CASE(25) ET_VM_CASE(26) ET_VM_CASE(27) ET_VM_CASE(28)
        ET_VM_CASE(29) ET_VM_CASE(30) ET_VM_CASE(31) ET_VM_CASE(32) ET_VM_CASE(33) ET_VM_CASE(34) ET_VM_CASE(35)
        ET_VM_CASE(36) ET_VM_CASE(37) ET_VM_CASE(38) ET_VM_CASE(39) ET_VM_CASE(40) ET_VM_CASE(41) ET_VM_CASE(42)
        ET_VM_CASE(43) ET_VM_CASE(44) ET_VM_CASE(45) ET_VM_CASE(46) ET_VM_CASE(47) ET_VM_CASE(48)
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#undef ET_VM_CASE
}

template <int MT, int KC>
__global__ __launch_bounds__(kSNW * 64) void bsr16_stream_kernel(const BsrStreamArgs a) {
    constexpr int R = MT * 16;                  // token rows of the strip
    constexpr int kRowBytes = KC * 2;
    constexpr int kRowsPerInst = 1024 / kRowBytes;        // rows one direct-to-LDS instruction fills
    constexpr int kLanesPerRow = 64 / kRowsPerInst;       // 16-byte chunks of a chunk row
    constexpr int kXInst = R / kRowsPerInst;              // instructions per X chunk
    constexpr int kXPerWave = (kXInst + kSNW - 1) / kSNW;
    static_assert(KC == 128 || KC == 256 || KC == 512, "chunk width");
    extern __shared__ __align__(16) unsigned char stream_smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r16 = lane & 15, g = lane >> 4;
    const int sel = g >> 1;
    // workgroup id -> (token strip, block-row group): the groups of one strip share an XCD (one L2)
    const int nstrips = (a.T + R - 1) / R;
    const int xcd = blockIdx.x % kSXcds, k_in_xcd = blockIdx.x / kSXcds;
    const int strip = xcd + kSXcds * (k_in_xcd / a.ngroups);
    const int group = k_in_xcd % a.ngroups;
    if (strip >= nstrips) return;  // padding of the last round of strips (whole workgroup)
    const int tok0 = strip * R;
    const int nbr = a.out >> 4;
    const int rb_begin = group * a.rows_per_wg;
    const int rb_end = min(rb_begin + a.rows_per_wg, nbr);

    // one LDS buffer: X chunk | weight slots (+1 slot of slack) | column list (+ slack)
    const int x_bytes = R * KC * 2;
    const int w_bytes = (a.max_slots + 1) * 1024;
    const int buf_bytes = x_bytes + w_bytes + a.q_ints * 4 + 1024;
    auto xbuf = [&](int b) { return reinterpret_cast<_Float16 *>(stream_smem + b * buf_bytes); };
    auto wbuf = [&](int b) { return reinterpret_cast<_Float16 *>(stream_smem + b * buf_bytes + x_bytes); };
    auto qbuf = [&](int b) { return reinterpret_cast<int32_t *>(stream_smem + b * buf_bytes + x_bytes + w_bytes); };

    // ---- direct-to-LDS loads of chunk c into buffer b.  Every region has a fixed size, so nothing
    // here waits for a table and every wave issues the same number of loads for every chunk (which
    // is what lets "chunk c has landed" be expressed as a count of outstanding loads).
    const int lrow = lane / kLanesPerRow, lpos = lane % kLanesPerRow;
    const int w_per_wave = a.max_slots / kSNW;
    const int q_inst = a.q_ints / 256;  // 1 KiB each, issued by the first waves
    const int loads_per_chunk = max(0, min(kXPerWave, (kXInst - wave + kSNW - 1) / kSNW)) + w_per_wave +
                                (wave < q_inst ? 1 : 0);
    auto issue = [&](int c, int b) {
        _Float16 *xb = xbuf(b);
#pragma unroll
        for (int v = 0; v < kXPerWave; v++) {
            const int j = wave + kSNW * v;
            if (j < kXInst) {
                const int row = j * kRowsPerInst + lrow;
                // the lane at position p of a row fetches chunk p ^ (row & 15): the fragment reads below,
                // 16 rows apart by one chunk column, then spread over all banks without padding
                const int qsrc = lpos ^ (row & 15);
                const int tok = min(tok0 + row, a.T - 1);
                const int col = min(c * KC + qsrc * 8, a.in - 8);
                __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(a.X + (size_t)tok * a.in + col),
                                                 ET_LDS_PTR(xb + j * kRowsPerInst * KC), 16, 0, 0);
            }
        }
        const size_t region = (size_t)group * a.nchunk + c;
        const _Float16 *wsrc = a.stiles + region * a.max_slots * 512 + lane * 8;
        _Float16 *wb = wbuf(b);
        for (int v = 0; v < w_per_wave; v++) {
            const int s = wave + kSNW * v;
            __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(wsrc + (size_t)s * 512), ET_LDS_PTR(wb + s * 512), 16, 0, 0);
        }
        if (wave < q_inst)
            __builtin_amdgcn_global_load_lds(ET_GLOBAL_PTR(a.sq + region * a.q_ints + wave * 256 + lane * 4),
                                             ET_LDS_PTR(qbuf(b) + wave * 256), 16, 0, 0);
    };

    const int ahead = a.nbuf - 1;  // chunks in flight beyond the one being multiplied
    for (int c = 0; c < ahead && c < a.nchunk; c++) issue(c, c);

    // tables of this wave (lane L holds those of chunk 64 * block + L; reloaded every 64 chunks) and the
    // bias of its rows: requested behind the first chunks
    const int32_t *ws = a.wseg + ((size_t)group * a.nchunk * kSNW + wave) * 8;
    auto load_seg = [&](int block, int4 &lo, int &n3) {
        const int lc = min(block * 64 + lane, a.nchunk - 1);
        lo = *reinterpret_cast<const int4 *>(ws + (size_t)lc * kSNW * 8);
        n3 = ws[(size_t)lc * kSNW * 8 + 4];
    };
    int4 seg_lo;
    int seg_n3;
    load_seg(0, seg_lo, seg_n3);
    h4 bias_v[kSMaxRpw];
#pragma unroll
    for (int i = 0; i < kSMaxRpw; i++) {
        const int rb = min(rb_begin + wave + kSNW * i, nbr - 1);
        bias_v[i] = h4{0, 0, 0, 0};
        if (a.bias) bias_v[i] = *reinterpret_cast<const h4 *>(a.bias + rb * 16 + g * 4);
    }
    // the compiler waits for these ordinary loads with vmcnt(0) before their first use, which would
    // also wait for every chunk in flight: take them now, behind the chunks issued so far, so that
    // the waits below see direct-to-LDS loads only
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    int seg_base_l = seg_lo.x, seg_n0_l = seg_lo.y, seg_n1_l = seg_lo.z, seg_n2_l = seg_lo.w;

    f4 acc[kSMaxRpw][MT];
#pragma unroll
    for (int i = 0; i < kSMaxRpw; i++)
#pragma unroll
        for (int m = 0; m < MT; m++) acc[i][m] = f4{0.f, 0.f, 0.f, 0.f};

    // A operand: lane (r16, g) reads 8 halfs of row r16 of tile (g >> 1) at offset 8 * (g & 1)
    const int a_off = sel * 256 + r16 * 16 + (g & 1) * 8;  // halfs inside the slot

    int b = 0;
    for (int c = 0; c < a.nchunk; c++) {
        // chunk c has landed when at most the loads of the chunks issued after it are outstanding
        const int later = min(ahead - 1, a.nchunk - 1 - c);
        wait_vmcnt(max(later, 0) * loads_per_chunk);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");  // ... for every wave; buffer b-1 is free
        if (c + ahead < a.nchunk) issue(c + ahead, b == 0 ? a.nbuf - 1 : b - 1);
        if (c && (c & 63) == 0) {
            // the next 64 chunks' tables (an ordinary load: it waits for everything in flight, once per 64 chunks)
            load_seg(c >> 6, seg_lo, seg_n3);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            seg_base_l = seg_lo.x, seg_n0_l = seg_lo.y, seg_n1_l = seg_lo.z, seg_n2_l = seg_lo.w;
        }
        const _Float16 *xb = xbuf(b) + r16 * KC;
        const _Float16 *wb = wbuf(b) + a_off;
        const int32_t *qb = qbuf(b) + sel;
        const int cl = c & 63;  // lane that holds this chunk's tables
        int slot = __builtin_amdgcn_readlane(seg_base_l, cl);
        const int seg_n[4] = {__builtin_amdgcn_readlane(seg_n0_l, cl), __builtin_amdgcn_readlane(seg_n1_l, cl),
                              __builtin_amdgcn_readlane(seg_n2_l, cl), __builtin_amdgcn_readlane(seg_n3, cl)};
        // the wave's slots of this chunk are consecutive; the weights and the column of the next slot
        // are read while the current one is multiplied (one slot past the end is read and dropped)
        h8 w_next = *reinterpret_cast<const h8 *>(wb + slot * 512);
        int q_next = qb[slot * 2];
#pragma unroll
        for (int i = 0; i < kSMaxRpw; i++) {
            const int n = i < a.rpw ? seg_n[i] : 0;
            for (int s = 0; s < n; s++) {
                const h8 w = w_next;
                const int pos = (((q_next + (g & 1)) ^ r16) & (kLanesPerRow - 1)) * 8;  // halfs
                h8 x[MT];
#pragma unroll
                for (int m = 0; m < MT; m++) x[m] = *reinterpret_cast<const h8 *>(xb + m * 16 * KC + pos);
                slot++;
                w_next = *reinterpret_cast<const h8 *>(wb + slot * 512);
                q_next = qb[slot * 2];
#pragma unroll
                for (int m = 0; m < MT; m++) acc[i][m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w, x[m], acc[i][m], 0, 0, 0);
            }
        }
        b = b + 1 == a.nbuf ? 0 : b + 1;
    }

    // ---- bias, activation, store: lane (r16, g) holds C[feature 4g .. 4g+3][token r16] of every block
#pragma unroll
    for (int i = 0; i < kSMaxRpw; i++) {
        const int rb = rb_begin + wave + kSNW * i;
        if (i < a.rpw && rb < rb_end) {
            const int f0 = rb * 16 + g * 4;
            const h4 bv = bias_v[i];
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const int tok = tok0 + m * 16 + r16;
                if (tok < a.T) {
                    if (a.Y32) {
                        f4 o;
#pragma unroll
                        for (int j = 0; j < 4; j++) o[j] = stream_act(acc[i][m][j] + (float)bv[j], a.act);
                        *reinterpret_cast<f4 *>(a.Y32 + (size_t)tok * a.out + f0) = o;
                    } else {
                        h4 o;
#pragma unroll
                        for (int j = 0; j < 4; j++) o[j] = (_Float16)stream_act(acc[i][m][j] + (float)bv[j], a.act);
                        *reinterpret_cast<h4 *>(a.Y + (size_t)tok * a.out + f0) = o;
                    }
                }
            }
        }
    }
}

// stiles[s][t] = tiles[order[2s + t]], or a zero tile where order is negative
__global__ void bsr_stream_reorder_kernel(_Float16 *__restrict__ stiles, const _Float16 *__restrict__ tiles,
                                          const int32_t *__restrict__ order, int nhalf_tiles) {
    const int t = blockIdx.x;
    if (t >= nhalf_tiles) return;
    const int src = order[t];
    const h8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const h8 *s = reinterpret_cast<const h8 *>(tiles + (size_t)(src < 0 ? 0 : src) * 256);
    h8 *d = reinterpret_cast<h8 *>(stiles + (size_t)t * 256);
    if (threadIdx.x < 32) d[threadIdx.x] = src < 0 ? zero : s[threadIdx.x];
}

}  // namespace et

using namespace et;

// The plan: device copies of the re-ordered weight and its tables, and the geometry they were built for.
struct et_bsr_plan_s {
    int in = 0, out = 0;
    int mt = 0, kc = 0, rpw = 0, rows_per_wg = 0, ngroups = 0, nchunk = 0, nbuf = 0;
    int max_slots = 0;  // slots of every (group, chunk) region
    int q_ints = 0;
    void *stiles = nullptr, *sq = nullptr, *wseg = nullptr;
    ~et_bsr_plan_s() {
        (void)hipFree(stiles);
        (void)hipFree(sq);
        (void)hipFree(wseg);
    }
};

namespace et {

constexpr size_t kStreamLdsBudget = 160 * 1024;

static size_t stream_buf_bytes(int mt, int kc, int max_slots) {
    const size_t q_ints = ((size_t)max_slots * 2 + 255) / 256 * 256;
    return (size_t)mt * 16 * kc * 2 + ((size_t)max_slots + 1) * 1024 + q_ints * 4 + 1024;
}

// Geometry for T token rows: one workgroup per compute unit where the shape allows it.
static void stream_geometry(int T, int in, int out, int &mt, int &kc, int &rows_per_wg) {
    const int nbr = out / 16;
    if (mt == 0) {
        // wide strips re-use a weight tile for more token rows; narrow ones give more workgroups
        if (T >= 8192) mt = 8;
        else if (T >= 2048) mt = 4;
        else if (T >= 512) mt = 2;
        else mt = 1;
    }
    if (kc == 0) {
        kc = in >= 512 ? 512 : (in >= 256 ? 256 : 128);
        while (kc > 128 && (size_t)mt * 16 * kc * 2 > 32 * 1024) kc /= 2;  // three buffers and the weights must fit
    }
    if (rows_per_wg == 0) {
        const int strips = (T + mt * 16 - 1) / (mt * 16);
        const int groups = strips >= 256 ? 1 : 256 / strips;
        rows_per_wg = (nbr + groups - 1) / groups;
    }
    rows_per_wg = std::max(1, std::min(rows_per_wg, kSNW * kSMaxRpw));
    rows_per_wg = std::min(rows_per_wg, nbr);
}

template <int MT, int KC>
static int launch_stream(const BsrStreamArgs &a, size_t lds, hipStream_t stream) {
    auto kernel = bsr16_stream_kernel<MT, KC>;
    static bool raised = false;  // per instantiation
    if (lds > 64 * 1024 && !raised) {
        ET_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   160 * 1024));
        raised = true;
    }
    const int nstrips = (a.T + MT * 16 - 1) / (MT * 16);
    const int rounds = (nstrips + kSXcds - 1) / kSXcds;
    kernel<<<dim3((unsigned)(rounds * kSXcds * a.ngroups)), kSNW * 64, lds, stream>>>(a);
    return check_launch("bsr16_stream_kernel");
}

template <int MT>
static int dispatch_stream_kc(const BsrStreamArgs &a, int kc, size_t lds, hipStream_t stream) {
    switch (kc) {
        case 128: return launch_stream<MT, 128>(a, lds, stream);
        case 256: return launch_stream<MT, 256>(a, lds, stream);
        default: return launch_stream<MT, 512>(a, lds, stream);
    }
}

}  // namespace et

extern "C" {

int et_bsr16_plan_create(const int32_t *row_ptr, const int32_t *col_idx, const et_f16 *tiles, int T, int in,
                         int out, int mt, int kc, int rows_per_wg, et_bsr_plan *plan) {
    ET_REQUIRE(plan != nullptr, ET_ERR_INVALID_ARG, "et_bsr16_plan_create: plan is NULL");
    *plan = nullptr;
    ET_REQUIRE(row_ptr && col_idx && tiles, ET_ERR_INVALID_ARG, "et_bsr16_plan_create: NULL pointer");
    ET_REQUIRE(T > 0 && in > 0 && out > 0 && in % 16 == 0 && out % 16 == 0 && T % 16 == 0, ET_ERR_UNSUPPORTED,
               "et_bsr16_plan_create: T=%d in=%d out=%d must be positive multiples of 16", T, in, out);
    ET_REQUIRE(in >= 128, ET_ERR_UNSUPPORTED, "et_bsr16_plan_create: the streaming kernel needs in >= 128 (in=%d)", in);
    int nbuf_req = 0;
    if (mt >= 100) {  // tuning: mt = 100 * buffers + blocks per strip
        nbuf_req = mt / 100;
        mt %= 100;
    }
    ET_REQUIRE((mt == 0 || mt == 1 || mt == 2 || mt == 4 || mt == 8) && (kc == 0 || kc == 128 || kc == 256 || kc == 512) &&
                   rows_per_wg >= 0 && (nbuf_req == 0 || (nbuf_req >= 2 && nbuf_req <= 4)),
               ET_ERR_INVALID_ARG, "et_bsr16_plan_create: mt=%d kc=%d rows_per_wg=%d", mt, kc, rows_per_wg);
    const int nbr = out / 16, bc = in / 16;
    std::vector<int32_t> rp((size_t)nbr + 1);
    ET_HIP(hipMemcpy(rp.data(), row_ptr, rp.size() * 4, hipMemcpyDeviceToHost));
    ET_REQUIRE(rp[0] == 0, ET_ERR_INVALID_ARG, "et_bsr16_plan_create: row_ptr must start at 0");
    for (int r = 0; r < nbr; r++)
        ET_REQUIRE(rp[(size_t)r + 1] >= rp[(size_t)r], ET_ERR_INVALID_ARG, "et_bsr16_plan_create: row_ptr decreases");
    const int ntile = rp[(size_t)nbr];
    std::vector<int32_t> ci((size_t)std::max(ntile, 1));
    if (ntile) ET_HIP(hipMemcpy(ci.data(), col_idx, (size_t)ntile * 4, hipMemcpyDeviceToHost));
    for (int t = 0; t < ntile; t++)
        ET_REQUIRE(ci[(size_t)t] >= 0 && ci[(size_t)t] < bc, ET_ERR_INVALID_ARG,
                   "et_bsr16_plan_create: column-tile index %d of tile %d outside [0, %d)", ci[(size_t)t], t, bc);

    const bool auto_kc = kc == 0, auto_rows = rows_per_wg == 0;
    stream_geometry(T, in, out, mt, kc, rows_per_wg);
    int nchunk = 0, ngroups = 0, rpw = 0, max_slots = 0;
    // per (group, chunk): the tiles in stream order — wave, owned row (rb_begin + wave + 8 i), tiles of
    // the row inside the chunk, a zero tile where a row segment is odd — and the slots per (wave, row)
    struct Region {
        std::vector<int32_t> order, q;
    };
    std::vector<Region> regions;
    std::vector<int32_t> wseg;
    auto build = [&]() {
        nchunk = (in + kc - 1) / kc;
        const int kct = kc / 16;
        ngroups = (nbr + rows_per_wg - 1) / rows_per_wg;
        rpw = (rows_per_wg + kSNW - 1) / kSNW;
        regions.assign((size_t)ngroups * nchunk, Region());
        wseg.assign((size_t)ngroups * nchunk * kSNW * 8, 0);
        max_slots = 0;
        for (int g = 0; g < ngroups; g++) {
            const int rb_begin = g * rows_per_wg, rb_end = std::min(rb_begin + rows_per_wg, nbr);
            for (int c = 0; c < nchunk; c++) {
                Region &reg = regions[(size_t)g * nchunk + c];
                for (int w = 0; w < kSNW; w++) {
                    int32_t *seg = &wseg[(((size_t)g * nchunk + c) * kSNW + w) * 8];
                    seg[0] = (int32_t)(reg.order.size() / 2);
                    for (int i = 0; i < rpw; i++) {
                        const int rb = rb_begin + w + kSNW * i;
                        int n = 0;
                        if (rb < rb_end) {
                            for (int t = rp[(size_t)rb]; t < rp[(size_t)rb + 1]; t++) {
                                if (ci[(size_t)t] / kct == c) {
                                    reg.order.push_back(t);
                                    reg.q.push_back((ci[(size_t)t] - c * kct) * 2);
                                    n++;
                                }
                            }
                            if (n & 1) {
                                reg.order.push_back(-1);
                                reg.q.push_back(0);
                                n++;
                            }
                        }
                        seg[1 + i] = n / 2;
                    }
                }
                max_slots = std::max(max_slots, (int)(reg.order.size() / 2));
            }
        }
        max_slots = std::max(kSNW, (max_slots + kSNW - 1) / kSNW * kSNW);  // every wave copies max_slots / 8 slots
    };
    build();
    // an automatic geometry gives way until two buffers fit: narrower chunks first (they halve the
    // strip piece and the tiles of a chunk alike), then fewer block-rows per workgroup
    while (2 * stream_buf_bytes(mt, kc, max_slots) > kStreamLdsBudget) {
        if (auto_kc && kc > 128) kc /= 2;
        else if (auto_rows && rows_per_wg > 1) rows_per_wg = (rows_per_wg + 1) / 2;
        else break;
        build();
    }
    const size_t buf = stream_buf_bytes(mt, kc, max_slots);
    ET_REQUIRE(2 * buf <= kStreamLdsBudget, ET_ERR_UNSUPPORTED,
               "et_bsr16_plan_create: mt=%d kc=%d rows_per_wg=%d needs 2 x %zu bytes of LDS (%d slots in the fullest "
               "chunk), more than 160 KB",
               mt, kc, rows_per_wg, buf, max_slots);
    int nbuf = (int)std::min<size_t>(4, kStreamLdsBudget / buf);
    if (nbuf_req) nbuf = std::min(nbuf, nbuf_req);
    nbuf = std::max(2, std::min(nbuf, nchunk + 1));
    const int q_ints = (max_slots * 2 + 255) / 256 * 256;
    ET_REQUIRE(q_ints / 256 <= kSNW, ET_ERR_UNSUPPORTED, "et_bsr16_plan_create: %d slots per chunk are too many",
               max_slots);
    // "chunk c has landed" is a count of outstanding loads, and the counter tops out: fewer buffers
    // where a chunk takes many loads per wave
    const int loads_per_wave = (mt * 16 * kc * 2 / 1024 + kSNW - 1) / kSNW + max_slots / kSNW + 1;
    while (nbuf > 2 && (nbuf - 2) * loads_per_wave > 48) nbuf--;

    // flatten: fixed-size regions
    const size_t nreg = regions.size();
    std::vector<int32_t> order(nreg * (size_t)max_slots * 2, -1), sq(nreg * (size_t)q_ints, 0);
    for (size_t r = 0; r < nreg; r++) {
        std::copy(regions[r].order.begin(), regions[r].order.end(), order.begin() + (std::ptrdiff_t)(r * (size_t)max_slots * 2));
        std::copy(regions[r].q.begin(), regions[r].q.end(), sq.begin() + (std::ptrdiff_t)(r * (size_t)q_ints));
    }

    et_bsr_plan_s *p = new (std::nothrow) et_bsr_plan_s;
    ET_REQUIRE(p != nullptr, ET_ERR_ALLOC, "et_bsr16_plan_create: out of host memory");
    p->in = in;
    p->out = out;
    p->mt = mt;
    p->kc = kc;
    p->rpw = rpw;
    p->rows_per_wg = rows_per_wg;
    p->ngroups = ngroups;
    p->nchunk = nchunk;
    p->nbuf = nbuf;
    p->max_slots = max_slots;
    p->q_ints = q_ints;
    auto upload = [&](void **dst, const void *src, size_t bytes) -> int {
        ET_HIP(hipMalloc(dst, std::max<size_t>(bytes, 16)));
        if (bytes) ET_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return ET_OK;
    };
    void *d_order = nullptr;
    int s = upload(&p->sq, sq.data(), sq.size() * 4);
    if (s == ET_OK) s = upload(&p->wseg, wseg.data(), wseg.size() * 4);
    if (s == ET_OK) s = upload(&d_order, order.data(), order.size() * 4);
    const size_t nhalf = order.size();
    if (s == ET_OK) s = check_hip(hipMalloc(&p->stiles, std::max<size_t>(nhalf * 512, 16)), "hipMalloc");
    if (s == ET_OK && nhalf) {
        bsr_stream_reorder_kernel<<<(unsigned)nhalf, 64>>>(static_cast<_Float16 *>(p->stiles),
                                                           reinterpret_cast<const _Float16 *>(tiles),
                                                           static_cast<const int32_t *>(d_order), (int)nhalf);
        s = check_launch("bsr_stream_reorder_kernel");
        if (s == ET_OK) s = check_hip(hipDeviceSynchronize(), "hipDeviceSynchronize");
    }
    (void)hipFree(d_order);
    if (s != ET_OK) {
        delete p;
        return s;
    }
    *plan = p;
    return ET_OK;
}

int et_bsr16_plan_destroy(et_bsr_plan plan) {
    delete plan;
    return ET_OK;
}

int et_bsr16_plan_info(et_bsr_plan plan, int *mt, int *kc, int *rows_per_wg, int *lds_bytes) {
    ET_REQUIRE(plan != nullptr, ET_ERR_INVALID_ARG, "et_bsr16_plan_info: plan is NULL");
    if (mt) *mt = plan->mt;
    if (kc) *kc = plan->kc;
    if (rows_per_wg) *rows_per_wg = plan->rows_per_wg;
    if (lds_bytes) *lds_bytes = (int)(plan->nbuf * stream_buf_bytes(plan->mt, plan->kc, plan->max_slots));
    return ET_OK;
}

int et_linear_bsr16_planned_f16(et_bsr_plan plan, const et_f16 *bias, const et_f16 *X, et_f16 *Y, float *Y32,
                                int T, int act, et_stream stream) {
    ET_REQUIRE(plan && X && ((Y != nullptr) != (Y32 != nullptr)), ET_ERR_INVALID_ARG,
               "et_linear_bsr16_planned_f16: plan and X must be set, and exactly one of Y and Y32");
    ET_REQUIRE(act >= ET_ACT_NONE && act <= ET_ACT_GELU, ET_ERR_INVALID_ARG, "et_linear_bsr16_planned_f16: act=%d", act);
    ET_REQUIRE(T >= 0 && T % 16 == 0, ET_ERR_UNSUPPORTED, "et_linear_bsr16_planned_f16: T=%d must be a multiple of 16", T);
    ET_REQUIRE((reinterpret_cast<uintptr_t>(X) & 15) == 0 && (reinterpret_cast<uintptr_t>(Y) & 7) == 0 &&
                   (reinterpret_cast<uintptr_t>(Y32) & 15) == 0,
               ET_ERR_UNSUPPORTED, "et_linear_bsr16_planned_f16: X and Y must be 16-byte aligned");
    if (T == 0) return ET_OK;
    BsrStreamArgs a{};
    a.stiles = static_cast<const _Float16 *>(plan->stiles);
    a.sq = static_cast<const int32_t *>(plan->sq);
    a.wseg = static_cast<const int32_t *>(plan->wseg);
    a.bias = reinterpret_cast<const _Float16 *>(bias);
    a.X = reinterpret_cast<const _Float16 *>(X);
    a.Y = reinterpret_cast<_Float16 *>(Y);
    a.Y32 = Y32;
    a.T = T;
    a.in = plan->in;
    a.out = plan->out;
    a.rows_per_wg = plan->rows_per_wg;
    a.ngroups = plan->ngroups;
    a.nchunk = plan->nchunk;
    a.rpw = plan->rpw;
    a.max_slots = plan->max_slots;
    a.q_ints = plan->q_ints;
    a.nbuf = plan->nbuf;
    a.act = act;
    const size_t lds = (size_t)plan->nbuf * stream_buf_bytes(plan->mt, plan->kc, plan->max_slots);
    hipStream_t st = as_stream(stream);
    switch (plan->mt) {
        case 1: return dispatch_stream_kc<1>(a, plan->kc, lds, st);
        case 2: return dispatch_stream_kc<2>(a, plan->kc, lds, st);
        case 4: return dispatch_stream_kc<4>(a, plan->kc, lds, st);
        default: return dispatch_stream_kc<8>(a, plan->kc, lds, st);
    }
}

}  // extern "C"
