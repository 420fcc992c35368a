/*
 * et_abi.h — C ABI of the MI355X (gfx950) E.T. encoder engine.
 *
 * Everything the C++ class layer (the headers under include/et) and any foreign-language
 * binding needs goes through these entry points: plain pointers and sizes, no
 * C++ or framework types.  Unless a parameter is documented as "host", every
 * pointer is a device pointer.  Every function returns an int status
 * (ET_OK == 0, negative on failure) and never aborts; et_last_error() gives a
 * thread-local message for the most recent failure.
 *
 * Activations are row-major [tokens x features] IEEE binary16.  A Linear
 * weight is the PyTorch [out x in] matrix and y = x * W^T + b.  All
 * contractions accumulate in fp32 and round once when the result is stored.
 *
 * Each declaration cites the interface of the reference implementation
 * (paths relative to the reference repository root) that it replaces.
 */
#ifndef ET_ABI_H
#define ET_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint16_t et_f16;  /* IEEE binary16 bit pattern */
typedef void *et_stream;  /* hipStream_t; NULL = the null stream */
typedef void *et_event;   /* hipEvent_t */
typedef void *et_graph;   /* a captured HIP graph with its executable instance (opaque) */

enum et_status {
    ET_OK = 0,
    ET_ERR_INVALID_ARG = -1,  /* null pointer, negative size, bad enum        */
    ET_ERR_UNSUPPORTED = -2,  /* shape the kernels do not handle (e.g. % 16)  */
    ET_ERR_ALLOC = -3,        /* device or host allocation failed             */
    ET_ERR_LAUNCH = -4,       /* HIP reported an error for a launch or copy   */
    ET_ERR_IO = -5,           /* file missing / malformed                     */
    ET_ERR_NO_DEVICE = -6     /* no usable gfx950 device                      */
};

enum et_act { ET_ACT_NONE = 0, ET_ACT_RELU = 1, ET_ACT_GELU = 2 /* tanh form */ };

/* bit flags of et_mha_* */
enum et_mha_flags {
    ET_MHA_CAUSAL = 1  /* key j visible to query i iff j <= i */
};

const char *et_status_string(int status);
const char *et_last_error(void);
void et_set_last_error(const char *message); /* for layers built on this ABI */
/* library / device identification: fills name (<= cap bytes, NUL terminated),
 * compute-unit count and LDS bytes per workgroup of the current device. */
int et_device_info(char *name, int cap, int *num_cu, int *lds_bytes);

/* ------------------------------------------------------------------------
 * Device buffers, streams, timers.
 * Replaces culib::CUDA_ptr<T> (lib/CUDA_ptr.hpp:10-69), sync_streams
 * (lib/utils.cu:49-53), to_half_devptr (lib/utils.cu:36-47), __kernel_setVal
 * (lib/CUDA_ptr.cu:5-11) and the host timers (lib/wtime.h:5-35).
 * ------------------------------------------------------------------------ */
int et_malloc(void **ptr, size_t bytes);              /* zero-filled, like CUDA_ptr(size) */
int et_free(void *ptr);                               /* NULL is accepted */
/* Placement.  et_malloc cuts buffers from 64 MiB slabs (4 KiB granules), so that
 * buffers allocated one after the other lie next to one another whatever the
 * driver's allocator holds at the time; a request above 16 MiB gets an
 * allocation of its own.  Between et_pool_private_begin and
 * et_pool_private_end the calling thread's et_malloc calls are served from
 * slabs of their own, the first buffer lead_bytes (a multiple of 4096, at most
 * 32 MiB) into the first slab: a model built inside such a scope has the same
 * layout in every process, and its speed does not depend on what was allocated
 * before it (et_model_finalize opens one).  Scopes do not nest.  No reference
 * counterpart (lib/CUDA_ptr.hpp:18-31 calls cudaMalloc per buffer). */
int et_pool_private_begin(size_t lead_bytes);
int et_pool_private_end(void);
int et_memset(void *ptr, int byte, size_t bytes, et_stream stream);
int et_memcpy_h2d(void *dst, const void *src_host, size_t bytes);
int et_memcpy_d2h(void *dst_host, const void *src, size_t bytes);
int et_memcpy_d2d(void *dst, const void *src, size_t bytes, et_stream stream);
/* dst device; src host OR device memory, told apart by the address, like the
 * cudaMemcpyDefault copy of CUDA_ptr(ptr, n) (lib/CUDA_ptr.hpp:18-31).  Blocking. */
int et_memcpy_auto(void *dst, const void *src, size_t bytes);
int et_fill_f16(et_f16 *dst, size_t n, et_f16 value, et_stream stream);
int et_fill_i32(int32_t *dst, size_t n, int32_t value, et_stream stream);
int et_f32_to_f16(et_f16 *dst, const float *src, size_t n, et_stream stream); /* RN-even */
int et_f16_to_f32(float *dst, const et_f16 *src, size_t n, et_stream stream);
int et_stream_create(et_stream *stream);
int et_stream_destroy(et_stream stream);
int et_stream_sync(et_stream stream);
int et_device_sync(void);
int et_event_create(et_event *ev);
int et_event_destroy(et_event ev);
int et_event_record(et_event ev, et_stream stream);
int et_event_sync(et_event ev);
int et_event_elapsed_ms(float *ms, et_event start, et_event stop);

/* HIP-graph capture of a launch sequence: everything issued on `stream` between
 * begin and end is recorded instead of executed; et_graph_launch replays it with
 * one submission.  This is how the N-layer caller loop of the reference drivers
 * (test/Table2/template.hpp:46-48, example/main.cu:175-177) is issued without
 * per-kernel launch latency.  `stream` must come from et_stream_create.  The
 * entry points of this library allocate nothing and never synchronise, so any
 * sequence of them may be captured (run it once eagerly first). */
int et_graph_begin_capture(et_stream stream);
int et_graph_end_capture(et_stream stream, et_graph *graph);
int et_graph_launch(et_graph graph, et_stream stream);
int et_graph_destroy(et_graph graph);

/* ------------------------------------------------------------------------
 * Linear layers: Y[T x out] = act(X[T x in] * W^T + bias).
 * bias may be NULL (treated as zero).  T, in and out must be multiples of 16.
 * ------------------------------------------------------------------------ */

/* 16x16 block-sparse weight (tile_mat): row_ptr[out/16 + 1], col_idx[ntile]
 * (column-tile index of each tile, any order inside a block-row), tiles
 * [ntile][16][16] with tile rows = output features.
 * Replaces Linear<tile_mat>::forward (Linear/SPMM_tile.cu:312-324) and its
 * kernel (Linear/SPMM_tile.cu:249-310); act fuses Encoder's act<>
 * (Encoder/Encoder.h:27-37) into the epilogue. */
int et_linear_bsr16_f16(const int32_t *row_ptr, const int32_t *col_idx,
                        const et_f16 *tiles, const et_f16 *bias,
                        const et_f16 *X, et_f16 *Y, int T, int in, int out,
                        int act, et_stream stream);

/* et_linear_bsr16_f16 with the result stored as binary32 [T x out]: the fp32
 * accumulator after bias and activation, unrounded (Y 16-byte aligned).  The
 * projections that feed a SkipLayerNorm use it in the mixed-precision layer
 * (fp16 matrix-core operands, fp32 residual stream); the reference's mixed
 * kernels (Attention/mixed-precision/mixed_attn.cu:10-124) widen only the
 * score accumulation. */
int et_linear_bsr16_f16_f32out(const int32_t *row_ptr, const int32_t *col_idx,
                               const et_f16 *tiles, const et_f16 *bias,
                               const et_f16 *X, float *Y, int T, int in, int out,
                               int act, et_stream stream);

/* Tile-sparse Linear through a plan.  et_bsr16_plan_create re-orders the weight
 * once (device pointers in the reference layout in, a device-side copy grouped by
 * K chunk and workgroup out; blocking) for T token rows; the planned call then
 * streams token strips and weight tiles through LDS chunk by chunk, which lifts
 * the limit the plain call has on the input width and lets one weight tile serve
 * 16*mt token rows.  mt (1, 2, 4, 8 sixteen-row blocks per strip), kc (128, 256,
 * 512 columns per chunk) and rows_per_wg (block-rows per workgroup, at most 32)
 * select the launch geometry; 0 picks it from T.  A plan may be used with any T
 * that is a multiple of 16.  Exactly one of Y (binary16) and Y32 (binary32, the
 * accumulator unrounded) is non-NULL.  Same results as et_linear_bsr16_f16 up to
 * the order of the fp32 accumulation.  Replaces Linear<tile_mat>::forward
 * (Linear/SPMM_tile.cu:312-324) for callers that keep a Linear object. */
typedef struct et_bsr_plan_s *et_bsr_plan;
int et_bsr16_plan_create(const int32_t *row_ptr, const int32_t *col_idx,
                         const et_f16 *tiles, int T, int in, int out, int mt,
                         int kc, int rows_per_wg, et_bsr_plan *plan);
int et_bsr16_plan_destroy(et_bsr_plan plan);
/* the geometry a plan was built with, and the LDS bytes of a workgroup */
int et_bsr16_plan_info(et_bsr_plan plan, int *mt, int *kc, int *rows_per_wg,
                       int *lds_bytes);
int et_linear_bsr16_planned_f16(et_bsr_plan plan, const et_f16 *bias,
                                const et_f16 *X, et_f16 *Y, float *Y32, int T,
                                int act, et_stream stream);

/* Tile-sparse Linear through a pack: the launch form for a few hundred to a few
 * thousand token rows, where a launch is a chain of memory round trips rather
 * than arithmetic.  et_bsr16_pack_create copies the weight once (device
 * pointers in the reference layout in; blocking) into the order one launch
 * geometry for T token rows reads it: per workgroup and wave a fixed number of
 * two-tile slots, zero-padded, so that every load of a launch is issued when it
 * starts and none depends on another.  ET_UNSUPPORTED when the shape is outside
 * that form (in not a multiple of 128 or above 4096, more than 16384 rows, ...):
 * the caller then uses et_linear_bsr16_f16.  flags: ET_PACK_STATS_PRODUCER keeps
 * the block-row groups of a strip to the 16 that the row sums of
 * et_linear_bsr16_packed_resid_stats_f32 allow; ET_PACK_NORM_CONSUMER picks a
 * workgroup size that deals the binary32 strip of
 * et_norm_linear_bsr16_packed_f32in evenly (in >= 512).  nwave asks for that
 * many waves per workgroup (0: chosen with the rest of the geometry; the chain
 * call below takes packs of 12).  A pack is used with
 * the T it was built for, or any smaller multiple of 16.  The three calls
 * compute what et_linear_bsr16_f16 / et_linear_bsr16_f16_f32out,
 * et_linear_bsr16_resid_stats_f32 / et_linear_bsr16_resid16_stats_f32 (exactly
 * one of resid and resid16 set) and et_norm_linear_bsr16_f32in (without the
 * optional normalised outputs) compute, up to the order of the fp32
 * accumulation.  ET_PACK_ROW_LOOP (alone) builds the pack of the form for many
 * token rows instead — any number of them, in a multiple of 128 up to 1536:
 * a workgroup keeps its share of the weight in registers and walks over
 * token strips staged two ahead, whole block-rows per wave, results stored
 * straight from the accumulators; such a pack serves
 * et_linear_bsr16_packed_f16 (binary16 or binary32 result) only.  Replaces
 * Linear<tile_mat>::forward (Linear/SPMM_tile.cu:312-324) for callers that keep
 * a Linear object. */
typedef struct et_bsr_pack_s *et_bsr_pack;
enum et_pack_flags { ET_PACK_NORM_CONSUMER = 1, ET_PACK_STATS_PRODUCER = 2, ET_PACK_ROW_LOOP = 4, ET_PACK_QKV_HEADS = 8 };
int et_bsr16_pack_create(const int32_t *row_ptr, const int32_t *col_idx,
                         const et_f16 *tiles, int T, int in, int out, int flags,
                         int nwave, et_bsr_pack *pack);
int et_bsr16_pack_destroy(et_bsr_pack pack);
/* the geometry a pack was built with: 16-row blocks per token strip, block-row
 * groups, waves per workgroup, slots per wave, LDS bytes of a workgroup */
int et_bsr16_pack_info(et_bsr_pack pack, int *mt, int *ngroups, int *nwave,
                       int *cap, int *lds_bytes);
int et_linear_bsr16_packed_f16(et_bsr_pack pack, const et_f16 *bias,
                               const et_f16 *X, et_f16 *Y, float *Y32, int T,
                               int act, et_stream stream);
int et_linear_bsr16_packed_resid_stats_f32(et_bsr_pack pack, const et_f16 *bias,
                                           const et_f16 *X, const float *resid,
                                           const et_f16 *resid16,
                                           const float *resid_fin,
                                           const et_f16 *resid_gamma,
                                           const et_f16 *resid_beta, float *V,
                                           float *stats, int *stat_groups, int T,
                                           et_stream stream);
int et_norm_linear_bsr16_packed_f32in(et_bsr_pack pack, const float *V,
                                      const float *stats, int stat_groups,
                                      const et_f16 *gamma, const et_f16 *beta,
                                      float eps, float *fin_out,
                                      const et_f16 *bias, et_f16 *Y, int T,
                                      int act, et_stream stream);

/* The token-local part of an encoder layer in one launch (mixed-precision layer
 * with the split SkipLayerNorm, tile-sparse projections through packs of 12 waves):
 *   V1  = Z W_O^T + b_O + residual                      (binary32, row sums stats1)
 *   H   = act(LayerNorm1(V1) W_1^T + b_1)               (binary16; fin1 = mean, rstd of V1's rows)
 *   V2  = H W_2^T + b_2 + LayerNorm1(V1)                (binary32, row sums stats2)
 *   QKV = LayerNorm2(V2) W_qkv^T + b_qkv                (the NEXT layer's projection; fin2; skipped
 *                                                        when qkv is NULL)
 * i.e. et_linear_bsr16_packed_resid_stats_f32, et_norm_linear_bsr16_packed_f32in,
 * et_linear_bsr16_packed_resid_stats_f32 and et_norm_linear_bsr16_packed_f32in
 * with the same operands, bit for bit, but with the workgroups of each XCD
 * meeting at a counter in their L2 between the steps instead of at three kernel
 * boundaries.  The residual of the first step is resid (binary32; normalised by
 * resid_fin / resid_gamma / resid_beta when resid_fin is set) or resid16.
 * sync: ET_CHAIN_SYNC_WORDS words of device memory, 128-byte aligned, ALL ZERO when
 * the launch starts (et_fill_i32) and used by one launch at a time;
 * et_encoder_chain_status (blocking) reads back how many workgroups gave up
 * waiting at a barrier and how many ran on another XCD than the workgroups they
 * share a counter with —
 * both 0 in a valid run; otherwise the results are not to be used and the caller
 * returns to the separate calls.  All workgroups must be resident at once: no
 * other kernel that itself waits for this one may run beside it.
 * et_encoder_chain_supported: 1 when the packs form a chain this launch runs
 * (0: et_last_error says what does not fit).
 * Replaces the launches between the attention kernels of
 * Encoder<cfg>::forward (Encoder/Encoder.h:81-96) and the QKV Linear of
 * Attention<cfg, true>::forward (Attention/Attention.h:246-253). */
#define ET_CHAIN_SYNC_WORDS 288
typedef struct et_chain_desc {
    et_bsr_pack o;
    const et_f16 *bias_o, *Z;
    const float *resid;
    const et_f16 *resid16;
    const float *resid_fin;
    const et_f16 *resid_gamma, *resid_beta;
    float *V1, *stats1;
    et_bsr_pack up;
    const et_f16 *bias_up, *gamma1, *beta1;
    float eps1;
    float *fin1;
    et_f16 *H;
    int act;
    et_bsr_pack down;
    const et_f16 *bias_down;
    float *V2, *stats2;
    et_bsr_pack qkv;
    const et_f16 *bias_qkv, *gamma2, *beta2;
    float eps2;
    float *fin2;
    et_f16 *QKV;
    int T;
    uint32_t *sync;
} et_chain_desc;
int et_encoder_chain_supported(const et_chain_desc *desc);
int et_encoder_chain_f32(const et_chain_desc *desc, int *stat_groups2, et_stream stream);
int et_encoder_chain_status(const uint32_t *sync, int *gave_up, int *misplaced);

/* SkipLayerNorm fused into the tile-sparse Linear that consumes it:
 *   ln_out = LayerNorm(src + skip) * gamma + beta      (written, [T x in])
 *   Y      = act(ln_out * W^T + bias)
 * in one kernel: the normalisation happens while the token strip is staged on
 * chip, so the Linear does not wait for a LayerNorm kernel to drain.  Same values
 * as et_skip_layernorm_f16 followed by et_linear_bsr16_f16 (which is what runs
 * when in > 1024).  It saves a launch and repeats the normalisation in every
 * block-row group of a strip: the faster form up to about 256 token rows, the
 * two separate calls above that.  Replaces LN1->forward + linear1->forward +
 * act<>() of Encoder<cfg>::forward (Encoder/Encoder.h:85-89). */
int et_skipln_linear_bsr16_f16(const et_f16 *src, const et_f16 *skip,
                               const et_f16 *gamma, const et_f16 *beta, float eps,
                               et_f16 *ln_out, const int32_t *row_ptr,
                               const int32_t *col_idx, const et_f16 *tiles,
                               const et_f16 *bias, et_f16 *Y, int T, int in,
                               int out, int act, et_stream stream);

/* SkipLayerNorm split between the Linear that produces its first input and the
 * Linear that consumes its output, so that no normalisation kernel runs between
 * them:
 *
 *   et_linear_bsr16_resid_stats_f16   V = X W^T + bias as usual, plus, per token,
 *       the sum and the sum of squares of (V as stored + resid), split over
 *       *stat_groups block-row groups: stats[stat_groups][T][2] floats (the
 *       caller provides room for 16 groups).  No atomics: the sums are reproducible.
 *   et_norm_linear_bsr16_f16          ln_out = (V + skip - mean) * rstd * gamma + beta
 *       with mean / rstd from those sums (variance E[v^2] - mean^2, fp32; skip is
 *       the resid of the producer; the sum is formed in fp32 and never stored),
 *       written [T x in], and Y = act(ln_out W^T + bias) — one launch.
 *   et_norm_from_stats_f16            the normalisation alone (last layer of a stack);
 *       bit-identical to the ln_out of the fused form.
 *
 * Together they are SkipLayerNorm::forward (SkipLayerNorm/SkipLayerNorm.cu:73-82)
 * between two Linear<tile_mat>::forward calls, i.e. the LN1/LN2 steps of
 * Encoder<cfg>::forward (Encoder/Encoder.h:85-92), with the reference's rounding
 * points (Linear output and LayerNorm output in fp16).
 * et_linear_bsr16_fused_ln_supported returns 1 when both kernels take the shape
 * (the token strip, its statistics and the affine vectors must fit in LDS).
 * Measured on MI355X at 1024 x 768 the pair costs as much as the LayerNorm
 * kernel it removes (the producer gains 0.6-1.3 us, the consumer 2.2 us), so the
 * class layer keeps et_skipln_linear_bsr16_f16 + et_skip_layernorm_f16; these
 * entry points serve callers whose shapes make a separate pass over the
 * activations the larger cost. */
int et_linear_bsr16_fused_ln_supported(int T, int in, int out);
int et_linear_bsr16_resid_stats_f16(const int32_t *row_ptr, const int32_t *col_idx,
                                    const et_f16 *tiles, const et_f16 *bias,
                                    const et_f16 *X, const et_f16 *resid, et_f16 *V,
                                    float *stats, int *stat_groups, int T, int in,
                                    int out, et_stream stream);
int et_norm_linear_bsr16_f16(const et_f16 *V, const et_f16 *skip, const float *stats,
                             int stat_groups, const et_f16 *gamma, const et_f16 *beta,
                             float eps, et_f16 *ln_out, const int32_t *row_ptr,
                             const int32_t *col_idx, const et_f16 *tiles,
                             const et_f16 *bias, et_f16 *Y, int T, int in, int out,
                             int act, et_stream stream);
int et_norm_from_stats_f16(et_f16 *out, const et_f16 *V, const et_f16 *skip,
                           const float *stats, int stat_groups, const et_f16 *gamma,
                           const et_f16 *beta, int rows, int H, float eps,
                           et_stream stream);

/* The same split in the mixed-precision layer, where the residual stream is binary32:
 *
 *   et_linear_bsr16_resid_stats_f32   V = X W^T + bias + resid, binary32, unrounded (X
 *       binary16 [T x in], resid and V binary32 [T x out]), and per token the sum and the
 *       sum of squares of V over each of *stat_groups block-row groups:
 *       stats[stat_groups][T][2] (room for 16 groups).  With resid_fin != NULL the residual
 *       is not read but formed: the normalisation of `resid` (then the V of an earlier
 *       producer) with the row statistics resid_fin[T][2] (mean, rstd — what the consumer of
 *       that V left in fin_out) and resid_gamma / resid_beta: the rows the consumer formed
 *       from the same data, which therefore never have to be stored.
 *   et_norm_linear_bsr16_f32in        ln = (V - mean) * rstd * gamma + beta from those sums,
 *       formed while the token strip is staged; Y = act(ln W^T + bias) with ln rounded to
 *       binary16 as the matrix-core operand.
 *       Optional results (NULL = not wanted): fin_out
 *       [T][2] = mean and rstd of every row; ln_out32 / ln_out16 = the normalised rows as
 *       binary32 / binary16 (each row written by one workgroup).
 *   et_norm_from_stats_f32in          the normalisation alone (after the last layer).
 *
 * A layer then runs QKV (normalising the previous layer's sum), attention, O projection
 * (+ residual, sums), FFN-up (normalising) and FFN-down (+ residual, sums): five launches,
 * no SkipLayerNorm launch, and no normalised activation is ever written to memory.  The
 * *_supported functions return 1 when the shape is taken (the token strip must fit in
 * LDS).  Encoder/Encoder.h:85-92 with SkipLayerNorm (SkipLayerNorm/SkipLayerNorm.cu:73-82)
 * folded into its neighbours. */
int et_linear_bsr16_resid_stats_f32_supported(int T, int in, int out);
int et_norm_linear_bsr16_f32in_supported(int T, int in, int out);
int et_linear_bsr16_resid_stats_f32(const int32_t *row_ptr, const int32_t *col_idx,
                                    const et_f16 *tiles, const et_f16 *bias,
                                    const et_f16 *X, const float *resid,
                                    const float *resid_fin, const et_f16 *resid_gamma,
                                    const et_f16 *resid_beta, float *V, float *stats,
                                    int *stat_groups, int T, int in, int out,
                                    et_stream stream);
/* The producer with its residual in binary16 (the first layer of a stack adds the model's
 * binary16 input: no widened copy of it is needed); otherwise et_linear_bsr16_resid_stats_f32
 * with resid_fin NULL. */
int et_linear_bsr16_resid16_stats_f32(const int32_t *row_ptr, const int32_t *col_idx,
                                      const et_f16 *tiles, const et_f16 *bias, const et_f16 *X,
                                      const et_f16 *resid16, float *V, float *stats,
                                      int *stat_groups, int T, int in, int out, et_stream stream);
int et_norm_linear_bsr16_f32in(const float *V, const float *stats, int stat_groups,
                               const et_f16 *gamma, const et_f16 *beta, float eps,
                               float *fin_out, float *ln_out32, et_f16 *ln_out16,
                               const int32_t *row_ptr,
                               const int32_t *col_idx, const et_f16 *tiles,
                               const et_f16 *bias, et_f16 *Y, int T, int in, int out,
                               int act, et_stream stream);
int et_norm_from_stats_f32in(float *out32, et_f16 *out16, const float *V,
                             const float *stats, int stat_groups, const et_f16 *gamma,
                             const et_f16 *beta, int rows, int H, float eps,
                             et_stream stream);

/* Dense weight W[out x in] row-major.  Replaces Linear<base_mat>::forward
 * (Linear/Linear.h:53-64) = cuBLAS_mmul (mycublas/cublas.cu:4-22) + bias map. */
int et_linear_dense_f16(const et_f16 *W, const et_f16 *bias, const et_f16 *X,
                        et_f16 *Y, int T, int in, int out, int act,
                        et_stream stream);

/* General row-major GEMM  C[M x N] = A[M x K] * op(B), fp32 accumulation.
 * trans_b != 0: B is [N x K] (C = A * B^T); trans_b == 0: B is [K x N].
 * lda/ldb/ldc are row strides in elements.  batch > 1 applies element strides
 * strideA/strideB/strideC between problems (a stride of 0 shares the operand).
 * Replaces cuBLAS_mmul / cuBLAS_bmmul (mycublas/cublas.cu:4-55) and the
 * cublasHgemmStridedBatched call of Linear_VO (Fused_attention/Linear_VO.h:45-47). */
int et_gemm_f16(const et_f16 *A, const et_f16 *B, et_f16 *C, int M, int N,
                int K, int lda, int ldb, int ldc, int trans_b, int batch,
                long long strideA, long long strideB, long long strideC,
                et_stream stream);

/* Row-pruned weight (row_mat): rows[nnz_row x in] are the surviving output
 * features, row_id[nnz_row] (ascending) their positions in [0, out).
 * Surviving columns of Y get x*w + bias, pruned columns get bias alone.
 * Replaces Linear<row_mat>::forward (Linear/SPMM_row.cu:62-75). */
int et_linear_rowpruned_f16(const et_f16 *rows, const int32_t *row_id,
                            int nnz_row, const et_f16 *bias, const et_f16 *X,
                            et_f16 *Y, int T, int in, int out, int act,
                            et_stream stream);

/* Row-pruned weight, compact output Yc[T x nnz_row] = X * rows^T (+ bias[row_id[j]]
 * when bias != NULL): the compact-V producer of the attention-aware path.
 * Replaces Linear<row_mat>::forward(col_mat*, ...) (Linear/SPMM_row.cu:78-95). */
int et_linear_rowpruned_compact_f16(const et_f16 *rows, const int32_t *row_id,
                                    int nnz_row, const et_f16 *bias,
                                    const et_f16 *X, et_f16 *Yc, int T, int in,
                                    et_stream stream);

/* Column-pruned weight (col_mat): cols[out x nnz_col] row-major are the
 * surviving input features, col_id[nnz_col] (any order) their positions in
 * [0, in).  Y = X[:, col_id] * cols^T + bias.
 * Replaces Linear<col_mat>::forward (Linear/SPMM_col.cu:57-69). */
int et_linear_colpruned_f16(const et_f16 *cols, const int32_t *col_id,
                            int nnz_col, const et_f16 *bias, const et_f16 *X,
                            et_f16 *Y, int T, int in, int out, int act,
                            et_stream stream);

/* dst[T x nnz_col] = X[:, col_id]: the gather pass of the column-pruned Linear
 * (Linear/SPMM_col.cu:25-39).  nnz_col % 8 == 0; dst and col_id 16-byte aligned. */
int et_gather_cols_f16(et_f16 *dst, const et_f16 *X, const int32_t *col_id, int T,
                       int in, int nnz_col, et_stream stream);

/* et_linear_colpruned_f16 through a caller-owned workspace [T x nnz_col]: gather
 * once, then a dense GEMM over the compact activations — the reference's own
 * sequence (Linear/SPMM_col.cu:57-69).  The workspace-free call gathers inside
 * the GEMM, once per output-column block, and is the slower of the two whenever
 * out spans more than one block. */
int et_linear_colpruned_ws_f16(const et_f16 *cols, const int32_t *col_id,
                               int nnz_col, const et_f16 *bias, const et_f16 *X,
                               et_f16 *Y, et_f16 *workspace, int T, int in,
                               int out, int act, et_stream stream);

/* et_linear_colpruned_ws_f16 without a workspace argument and without any
 * allocation: the gathered activations [T x nnz_col] go to a buffer built into
 * the library (a file-scope device array of 8 MiB per GPU, held until the
 * process ends).  No counterpart in the reference; it is for callers that
 * cannot allocate device memory or pass a workspace: code under HIP-graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  Same result,
 * bit for bit, as the _ws form.  T * nnz_col * 2 bytes must fit 8 MiB
 * (ET_ERR_UNSUPPORTED otherwise).  All calls on one GPU share the buffer: calls
 * that may overlap on one GPU (different streams, or one graph replayed while
 * another call runs) race on it and must be ordered by the caller. */
int et_linear_colpruned_static_f16(const et_f16 *cols, const int32_t *col_id,
                                   int nnz_col, const et_f16 *bias, const et_f16 *X,
                                   et_f16 *Y, int T, int in, int out, int act,
                                   et_stream stream);

/* 1x16 vector-sparse weight (mat1x16): for row-set r (16 output features) and
 * part p (16 input features) the surviving 1x16 vectors are idx in
 * [tile_idx[r*(in/16+1)+p], tile_idx[r*(in/16+1)+p+1]); row_idx[idx] % 16 is
 * the row inside the set and data[16*idx .. 16*idx+15] the weights.
 * Completes Linear<mat1x16> (Linear/Linear.h:153-167), whose reference kernel
 * (Linear/SPMM1x16.cu:35-124) is never launched and stores nothing. */
int et_linear_vec1x16_f16(const int32_t *tile_idx, const int32_t *row_idx,
                          const et_f16 *data, const et_f16 *bias,
                          const et_f16 *X, et_f16 *Y, int T, int in, int out,
                          int act, et_stream stream);

/* Dense image W[out x in] of a 1x16 weight, written on the device.  A matrix
 * core multiplies whole 16x16 cells, and below about 95 % vector sparsity nearly
 * every cell holds a vector, so the products cannot be skipped: Linear<mat1x16>
 * expands its weight once at construction and runs et_linear_dense_f16 on the
 * image (3-5 times faster than et_linear_vec1x16_f16 at 80 %).  No counterpart
 * in the reference. */
int et_vec1x16_to_dense_f16(const int32_t *tile_idx, const int32_t *row_idx,
                            const et_f16 *data, et_f16 *W, int in, int out,
                            et_stream stream);

/* Dense image W[out x in] of a 16x16 BSR weight (device pointers; row_ptr[out/16+1],
 * col_idx and tiles as for et_linear_bsr16_f16; column-tile indices must be in
 * range; a position named twice keeps the later tile, so callers with such
 * weights stay on the tile kernel).  A tile-pruned matrix that keeps most of its
 * tiles is a dense matrix with holes: Linear<tile_mat> runs the dense GEMM on this
 * image below 50 % sparsity (55 % for inputs of 3072 and wider), where that is
 * the faster kernel.  No counterpart in the reference. */
int et_bsr16_to_dense_f16(const int32_t *row_ptr, const int32_t *col_idx,
                          const et_f16 *tiles, et_f16 *W, int in, int out,
                          et_stream stream);

/* Unstructured CSR weight over [out x in] (indices need not be sorted inside a
 * row).  T may be any size; out % 4 == 0.  Replaces Linear<csr_mat>::forward
 * (Linear/cusp.cu:23-82, cusparseSpMM + bias map); no workspace is allocated. */
int et_linear_csr_f16(const int32_t *indptr, const int32_t *indices,
                      const et_f16 *data, const et_f16 *bias, const et_f16 *X,
                      et_f16 *Y, int T, int in, int out, int act,
                      et_stream stream);

/* C[r][c] = bias[c] (0 when bias is NULL) for a dense [rows x cols] matrix. */
int et_fill_rows_bias_f16(et_f16 *C, const et_f16 *bias, int rows, int cols,
                          et_stream stream);

/* ------------------------------------------------------------------------
 * Fused multi-head self-attention (scores never leave the chip).
 *
 * Token rows [b*S, (b+1)*S) belong to sequence b.  Head h is the column slice
 * [h*hd, (h+1)*hd) of Q, K, V and Z; ldq/ldk/ldv/ldz are row strides in
 * elements, so Q, K, V may be slices of one [T x 3H] buffer.
 *   P = softmax(scale * Q_h K_h^T + mask),  Z_h = P V_h
 * mask: optional additive [S x S] binary16 matrix shared by all sequences and
 * heads (-inf removes a key).  lens: optional int32[B]; keys >= lens[b] of
 * sequence b get probability exactly 0 (right padding).  Scores, softmax and
 * both contractions are fp32-accumulated.  S % 16 == 0; hd a multiple of 8, at
 * most 256 (the reference's kernels ask for multiples of 16,
 * Fused_attention/test/testfused.cu:22, while its example model has 800 / 4 =
 * 200-wide heads, example/main.cu:24-31: both are taken).
 *
 * Replaces Multihead_atttion<OTF_attn_full> (Attention/Attention.cu:80-95,
 * Attention/OTFkernel_full.h:15-125), the single-buffer form
 * (Attention/Attention_single.cu:10-108, Attention/Attention.h:246-265) and
 * the mixed-precision form (Attention/mixed-precision/mixed_attn.cu:10-124).
 * ------------------------------------------------------------------------ */
int et_mha_fused_f16(const et_f16 *Q, const et_f16 *K, const et_f16 *V,
                     int ldq, int ldk, int ldv, et_f16 *Z, int ldz,
                     const et_f16 *mask, const int32_t *lens, int B, int S,
                     int nh, int hd, float scale, int flags, et_stream stream);

/* Fused attention and the tile-sparse output projection in ONE launch:
 *   Z = attention as et_mha_fused_f16 (Z is written, [B*S x ldz]),
 *   out[B*S x emdim] = Z[:, :nh*hd] * W_O^T + o_bias,
 * W_O [emdim x nh*hd] as 16x16 tiles (o_row_ptr[emdim/16 + 1], o_col_idx,
 * o_tiles as in et_linear_bsr16_f16; o_bias may be NULL).  Same values as
 * et_mha_fused_f16 followed by et_linear_bsr16_f16 up to the order of the fp32
 * accumulation.  The workgroup that completes the heads of a strip of tokens
 * projects that strip; no workgroup waits for another.  hd a multiple of 8, at
 * most 128; nh*hd and emdim multiples of 16; ldz % 8 == 0; Z and o_tiles
 * 16-byte aligned.  Arrival counts live in a device array built into the
 * library (allocates nothing): B*S/16 <= 16384, else ET_ERR_UNSUPPORTED, and
 * two of these calls that overlap in time on one GPU (different streams) race
 * on the counts — issue them on one stream.  For callers that need the pair
 * as one launch: the two separate launches are the faster form on this device
 * at every size measured (8 against 25 us for one sequence of 128 tokens, the
 * reference kernel's case; 26 against 129 us for 64 sequences).
 * Replaces Multihead_atttion_fuseO (Attention/kernel_fuseO.h:6-9, kernel
 * Attention/kernel_fuseO.cu:138-243, host :254-290), which joins the two parts
 * with a grid-wide barrier inside a cooperative launch. */
int et_mha_fuseo_f16(const et_f16 *Q, const et_f16 *K, const et_f16 *V,
                     int ldq, int ldk, int ldv, et_f16 *Z, int ldz,
                     const et_f16 *mask, const int32_t *lens, int B, int S,
                     int nh, int hd, float scale, int flags,
                     const int32_t *o_row_ptr, const int32_t *o_col_idx,
                     const et_f16 *o_tiles, const et_f16 *o_bias, et_f16 *out,
                     int emdim, et_stream stream);

/* Attention-aware pruning: W_V is row-pruned, so V arrives compact,
 * Vc[T x nnz_col] (row stride ldvc), holding only the surviving V columns.
 * v_col_id[nnz_col] (ascending) are their full-width positions and
 * v_head_ptr[nh+1] splits them by head (the columns of head h lie in its own
 * slice [h*vhd, (h+1)*vhd), as col_mat::set_metadata produces them,
 * mat_type/col_mat/col_mat.cu:34-58).  P*V runs over the surviving columns
 * only; Z is written full width [T x nh*vhd] with zeros in pruned columns.
 * Completes Multihead_atttion<Prune_attn> (Attention/Attention.cu:54-78), whose
 * reference kernel never stores Z (Attention/kernels.cu:453-458). */
int et_mha_compactv_f16(const et_f16 *Q, const et_f16 *K, const et_f16 *Vc,
                        int ldq, int ldk, int ldvc, const int32_t *v_col_id,
                        const int32_t *v_head_ptr, int nnz_col, et_f16 *Z,
                        int ldz, const et_f16 *mask, const int32_t *lens, int B,
                        int S, int nh, int hd, int vhd, float scale, int flags,
                        et_stream stream);

/* ---------------------------------------------------------------------------
 * The QKV projection inside the attention kernel (four launches per layer in
 * the split-normalisation stack instead of five): one workgroup per (sequence,
 * head) normalises its sequence's rows of the previous layer's binary32 sum V
 * with that sum's row statistics (what et_norm_linear_bsr16_f32in does for the
 * QKV projection), multiplies them with its head's block-rows of the
 * tile-sparse W_qkv, keeps Q, K and V of the head in LDS and runs the fused
 * attention of et_mha_fused_f16 on them; fin_out[T][2] receives mean and rstd
 * of every row (may be NULL).  W_qkv = [Q | K | V] rows as Attention's single
 * projection holds them (Attention/Attention.h:246-265); et_qkv_heads_pack_create
 * copies it once into the order the kernel reads (destroy with
 * et_bsr16_pack_destroy).  Limits, told by et_norm_qkv_mha_f32in_supported:
 * sequences of a multiple of 16 up to 128 tokens, 768-wide input, heads of 64.
 * Rows of V past a sequence's length are projected like the others and their
 * keys weighted with exactly zero: they must hold finite values.
 * Replaces Attention<cfg, isSingleKernel>::forward up to the O projection
 * (Attention/Attention_single.cu:10-108).
 * ------------------------------------------------------------------------ */
int et_norm_qkv_mha_f32in_supported(int B, int S, int in, int nhead, int hd);
int et_qkv_heads_pack_create(const int32_t *row_ptr, const int32_t *col_idx,
                             const et_f16 *tiles, int in, int nhead,
                             et_bsr_pack *pack);
/* The same pack with the affine part of the normalisation folded into the
 * weight: it holds W_qkv diag(gamma) (binary16) and bias_qkv + W_qkv beta
 * (binary32), so that the launch normalises a value with one multiply-add,
 * (v - mean) rstd — the twelve workgroups of a sequence each normalise all of it.
 * et_norm_qkv_mha_f32in then ignores its gamma, beta and bias_qkv arguments
 * (they may be NULL); a caller that changes gamma, beta, the bias or the weight
 * builds the pack again.  bias may be NULL (zeros). */
int et_qkv_heads_pack_create_folded(const int32_t *row_ptr, const int32_t *col_idx,
                                    const et_f16 *tiles, const et_f16 *bias,
                                    const et_f16 *gamma, const et_f16 *beta,
                                    int in, int nhead, et_bsr_pack *pack);
int et_norm_qkv_mha_f32in(et_bsr_pack pack, const float *V, const float *stats,
                          int stat_groups, const et_f16 *gamma,
                          const et_f16 *beta, float eps, float *fin_out,
                          const et_f16 *bias_qkv, et_f16 *Z, int ldz,
                          const et_f16 *mask, const int32_t *lens, int B, int S,
                          float scale, int flags, et_stream stream);

/* Softmax probabilities written to memory: P[b*S + q][h*S + key] (row stride
 * nh*S), the layout of the reference's __kernel_fused_attention_NOTF
 * (Fused_attention/Fused_attention.cu:118-206).  S <= 512. */
int et_mha_probs_f16(const et_f16 *Q, const et_f16 *K, int ldq, int ldk,
                     et_f16 *P, const et_f16 *mask, const int32_t *lens, int B,
                     int S, int nh, int hd, float scale, int flags,
                     et_stream stream);

/* Unfused baseline: probabilities through the workspace P[T x nh*S], then a
 * batched P*V GEMM per (sequence, head).  Replaces Multihead_atttion<Norm_attn>
 * (Attention/Attention.cu:8-36: batched GEMM, mask map, softmax kernel, GEMM). */
int et_mha_unfused_f16(const et_f16 *Q, const et_f16 *K, const et_f16 *V,
                       int ldq, int ldk, int ldv, et_f16 *Z, int ldz, et_f16 *P,
                       const et_f16 *mask, const int32_t *lens, int B, int S,
                       int nh, int hd, float scale, int flags,
                       et_stream stream);

/* Pre-multiplied value/output projection: VO[b][h] (S x N) = X[b] (S x H) *
 * W[h] (H x N) + bias[h]; W is [nh][H][N] row-major, bias [nh][N] (may be
 * NULL), VO is [B][nh][S][N].  Replaces Linear_VO::forward and
 * Linear_VO_prune::forward (Fused_attention/Linear_VO.h:39-58,79-95:
 * cublasHgemmStridedBatched + add_bias_VO). */
int et_linear_vo_f16(const et_f16 *W, const et_f16 *bias, const et_f16 *X,
                     et_f16 *VO, int B, int S, int H, int N, int nh,
                     et_stream stream);

/* The same projection from weights stored k-contiguous per head, Wt[nh][N][H]
 * (Wt[h][n][k] = W[h][k][n]): the layout the GEMM kernels read fastest
 * (one sequence of BERT-base: 12 us against 21 us).  et_transpose_heads_f16
 * makes Wt from W once, at construction; the Linear_VO classes do so. */
int et_transpose_heads_f16(et_f16 *dst, const et_f16 *src, int nh, int H, int N,
                           et_stream stream);
int et_linear_vo_t_f16(const et_f16 *Wt, const et_f16 *bias, const et_f16 *X,
                       et_f16 *VO, int B, int S, int H, int N, int nh,
                       et_stream stream);

/* E.T. attention over the pre-multiplied VO: out[b] = sum_h P_h[b] VO[b][h] +
 * bias_o, with P = softmax(scale * Q_h K_h^T + mask) written to the workspace
 * P[T x nh*S] on the way.  N is the width of VO; when col_scatter != NULL the N
 * result columns go to columns col_scatter[n] of out (row stride out_width) and
 * the other columns of out receive bias_o alone.  Replaces
 * Fused_Multihead_attention<NOTF_fused_attn> / <OTF_fused_attn> and
 * Fused_prune_Multihead_attention (Fused_attention/Fused_attention.cu:207-308)
 * plus the bias map of FusedAttention::forward (Fused_attention.h:109-115). */
int et_mha_vo_f16(const et_f16 *Q, const et_f16 *K, int ldq, int ldk,
                  const et_f16 *VO, et_f16 *P, et_f16 *out,
                  const et_f16 *bias_o, const int32_t *col_scatter,
                  const et_f16 *mask, const int32_t *lens, int B, int S, int nh,
                  int hd, int N, int out_width, float scale, int flags,
                  et_stream stream);

/* The same attention with the probabilities kept on chip (the reference's
 * OTF_fused_attn, Fused_attention/Fused_attention.cu:10-116), in two calls.
 * et_linear_vo_keys_f16 writes the projection key-contiguous and without its
 * bias, VOt[b][h][n][s] = sum_k Wt[h][n][k] X[b*S+s][k] (Wt as for
 * et_linear_vo_t_f16): both matrix-core operands of the attention kernel are
 * then 16-byte loads and nothing is staged through LDS.  et_mha_vo_otf_f16
 * gives the waves of a workgroup (32 queries x 64 output columns) a head each,
 * sums softmax_h * VO_h in fp32, adds sum_h bias_vo[h][n] (the probabilities of
 * a row add up to one; bias_vo [nh][N] or NULL) and bias_o, and writes every
 * element of out once: no P buffer, no atomics, out need not be cleared.  The
 * other arguments as et_mha_vo_f16.  With lens (or a causal strip) the keys
 * past a sequence's length, up to the next multiple of 8, are still read and
 * weighted with probabilities that are exactly zero: the rows of X behind them
 * (and so of VOt) must hold finite values. */
int et_linear_vo_keys_f16(const et_f16 *Wt, const et_f16 *X, et_f16 *VOt, int B,
                          int S, int H, int N, int nh, et_stream stream);
int et_mha_vo_otf_f16(const et_f16 *Q, const et_f16 *K, int ldq, int ldk,
                      const et_f16 *VOt, const et_f16 *bias_vo, et_f16 *out,
                      const et_f16 *bias_o, const int32_t *col_scatter,
                      const et_f16 *mask, const int32_t *lens, int B, int S,
                      int nh, int hd, int N, int out_width, float scale,
                      int flags, et_stream stream);

/* ------------------------------------------------------------------------
 * Normalisation and element-wise operators.
 * ------------------------------------------------------------------------ */

/* out[r] = LayerNorm(src[r] + skip[r]) * gamma + beta over H features,
 * statistics in fp32, one pass over HBM.  H % 4 == 0, H <= 8192.
 * Replaces SkipLayerNorm::forward (SkipLayerNorm/SkipLayerNorm.cu:73-82). */
int et_skip_layernorm_f16(et_f16 *out, const et_f16 *src, const et_f16 *skip,
                          const et_f16 *gamma, const et_f16 *beta, int rows,
                          int H, float eps, et_stream stream);

/* Mixed-precision SkipLayerNorm: src and skip are binary32 [rows x H] (a
 * projection's unrounded output and the residual stream), gamma and beta the
 * model's binary16 parameters; the result is written as binary32 to out32 (the
 * next residual) and, rounded once, as binary16 to out16 (the next
 * projection's operand).  Either output may be NULL.  Same statistics as
 * et_skip_layernorm_f16 (SkipLayerNorm/SkipLayerNorm.cu:22-63). */
int et_skip_layernorm_mixed(float *out32, et_f16 *out16, const float *src,
                            const float *skip, const et_f16 *gamma,
                            const et_f16 *beta, int rows, int H, float eps,
                            et_stream stream);

/* out[r] = LayerNorm(src[r]) * gamma + beta.
 * Replaces LayerNorm::forward (LayerNorm/LayerNorm.cu:51-57). */
int et_layernorm_f16(et_f16 *out, const et_f16 *src, const et_f16 *gamma,
                     const et_f16 *beta, int rows, int H, float eps,
                     et_stream stream);

/* In-place capable activations over n elements.  Replace act<GELU_OP> /
 * act<RELU_OP> (Encoder/Encoder.h:27-37, Encoder/Encoder.cu:25-68). */
int et_gelu_f16(et_f16 *out, const et_f16 *in, size_t n, et_stream stream);
int et_relu_f16(et_f16 *out, const et_f16 *in, size_t n, et_stream stream);

/* data[r][c] += bias[c] for a [rows x cols] matrix.  Replaces the cuda_map
 * bias lambdas (Linear/Linear.h:57-63, Fused_attention/Fused_attention.h:109-115). */
int et_bias_add_f16(et_f16 *data, const et_f16 *bias, int rows, int cols,
                    et_stream stream);

/* ------------------------------------------------------------------------
 * binary32 twins.  Same contracts as the _f16 functions of the same name with
 * every pointer a float pointer; values are stored, multiplied and accumulated
 * in binary32 (MFMA 16x16x4 f32 in the Linear).  They are the verification
 * path for dense fp32 models — an encoder layer built from them agrees with a
 * CPU fp32 forward to max-abs 1e-4 — and have no counterpart in the reference,
 * whose kernels are binary16 only (Linear/Linear.h:9, lib/mma.hpp:6-13).
 * et_linear_dense_f32: in % 16 == 0, out % 4 == 0, any T.
 * et_mha_fused_f32: S % 16 == 0, hd a multiple of 16 up to 128, 16*S floats of scores
 * must fit on chip (S <= 2048); mask is a float [S x S] matrix.
 * ------------------------------------------------------------------------ */
int et_linear_dense_f32(const float *W, const float *bias, const float *X, float *Y,
                        int T, int in, int out, int act, et_stream stream);
/* binary32 twins of the Linear layers over the sparse weight containers: the
 * structure arrays (row_ptr / col_idx, row_id, col_id, tile_idx / row_idx,
 * indptr / indices) mean what they mean in the _f16 function of the same name;
 * weights, bias, X and Y are float.  T may be any size.
 *   et_linear_bsr16_f32             Linear<tile_mat> (Linear/SPMM_tile.cu:312-324); in, out % 16 == 0
 *   et_linear_rowpruned_f32         Linear<row_mat>  (Linear/SPMM_row.cu:62-75): pruned columns of Y
 *                                   get act(bias); in % 16 == 0, nnz_row % 4 == 0
 *   et_linear_rowpruned_compact_f32 its compact-output form (Linear/SPMM_row.cu:78-95)
 *   et_linear_colpruned_f32         Linear<col_mat>  (Linear/SPMM_col.cu:57-69); the gather happens
 *                                   while X is staged, no workspace; nnz_col % 16 == 0, out % 4 == 0,
 *                                   col_id 16-byte aligned
 *   et_linear_vec1x16_f32           Linear<mat1x16>  (Linear/Linear.h:153-167); in, out % 16 == 0,
 *                                   at most 16 vectors per (row-set, part) cell
 *   et_linear_csr_f32               Linear<csr_mat>  (Linear/cusp.cu:23-82); out % 4 == 0 */
int et_linear_bsr16_f32(const int32_t *row_ptr, const int32_t *col_idx, const float *tiles,
                        const float *bias, const float *X, float *Y, int T, int in, int out,
                        int act, et_stream stream);
int et_linear_rowpruned_f32(const float *rows, const int32_t *row_id, int nnz_row,
                            const float *bias, const float *X, float *Y, int T, int in,
                            int out, int act, et_stream stream);
int et_linear_rowpruned_compact_f32(const float *rows, const int32_t *row_id, int nnz_row,
                                    const float *bias, const float *X, float *Yc, int T,
                                    int in, et_stream stream);
int et_linear_colpruned_f32(const float *cols, const int32_t *col_id, int nnz_col,
                            const float *bias, const float *X, float *Y, int T, int in,
                            int out, int act, et_stream stream);
int et_linear_vec1x16_f32(const int32_t *tile_idx, const int32_t *row_idx, const float *data,
                          const float *bias, const float *X, float *Y, int T, int in, int out,
                          int act, et_stream stream);
int et_linear_csr_f32(const int32_t *indptr, const int32_t *indices, const float *data,
                      const float *bias, const float *X, float *Y, int T, int in, int out,
                      int act, et_stream stream);
int et_mha_fused_f32(const float *Q, const float *K, const float *V, int ldq, int ldk,
                     int ldv, float *Z, int ldz, const float *mask,
                     const int32_t *lens, int B, int S, int nh, int hd, float scale,
                     int flags, et_stream stream);
int et_skip_layernorm_f32(float *out, const float *src, const float *skip,
                          const float *gamma, const float *beta, int rows, int H,
                          float eps, et_stream stream);
int et_layernorm_f32(float *out, const float *src, const float *gamma,
                     const float *beta, int rows, int H, float eps, et_stream stream);
int et_gelu_f32(float *out, const float *in, size_t n, et_stream stream);
int et_relu_f32(float *out, const float *in, size_t n, et_stream stream);

/* ------------------------------------------------------------------------
 * Encoder stack: nlayer post-LN encoder layers, layer i feeding layer i+1,
 *   a = Attn(x); y1 = SkipLN1(a, x); f = L2(act(L1(y1))); out = SkipLN2(f, y1)
 * assembled from host weights and run as ONE HIP-graph replay per forward.
 * This is the C form of the reference's model assembly and inference loop
 * (example/main.cu:24-182: Weights -> tile_mat -> Linear -> Attention ->
 * SkipLayerNorm -> Encoder, then model[i]->forward chained) over
 * Encoder<cfg>::forward (Encoder/Encoder.h:81-96) with the single-projection
 * attention (Attention/Attention.h:246-265).  The handle owns its weights and
 * scratch; forward takes caller-owned device buffers of batch*seq_len rows.
 * One handle serves one host thread at a time.
 * ------------------------------------------------------------------------ */
typedef struct et_model_s *et_model;

typedef struct et_model_desc {
    int kdim, vdim, seq_len, nhead, dimFF, emdim, nlayer; /* Model_t (Model.h:2-10) */
    int batch;     /* sequences per forward; activations have batch*seq_len rows */
    int act;       /* ET_ACT_RELU or ET_ACT_GELU (Encoder_config::act_t)          */
    float eps;     /* LayerNorm epsilon; <= 0 selects 1e-5                        */
    int causal;    /* != 0: causal mask (the reference's hard-wired one)          */
    int use_graph; /* != 0: replay a captured HIP graph; 0: launch kernel by kernel */
    int mixed;     /* 1 to 5: mixed precision — the residual stream (layer inputs, the two
                    * projections that feed a SkipLayerNorm, both SkipLayerNorm results)
                    * is kept in binary32 inside the stack, binary16 only as matrix-core
                    * operands; input and output of et_model_forward stay binary16.
                    * 1: SkipLayerNorm is folded into the neighbouring tile-sparse projections
                    *    where the shapes allow (five launches per layer; four, as under 4, for
                    *    the batch sizes where that measured faster: 96 to 400 (sequence, head)
                    *    pairs); 2: it keeps its own
                    *    launches (seven); 3: as 1, with everything between two attention
                    *    kernels in one launch (et_encoder_chain_f32: two launches per layer)
                    *    where the shapes allow and the device runs it as it must, else as 1;
                    *    4: as 1, with the QKV projection of every layer after the first inside
                    *    its attention kernel (et_norm_qkv_mha_f32in: four launches per layer)
                    *    where the shapes allow, else as 1; 5: as 1, always with five launches.
                    * 0: every activation is stored as binary16 (the reference's storage) */
} et_model_desc;

/* which matrix of a layer */
enum et_weight { ET_W_QKV = 0, ET_W_O = 1, ET_W_FF1 = 2, ET_W_FF2 = 3 };

int et_model_create(const et_model_desc *desc, et_model *out);
/* 16x16 BSR weight in the exporter's layout (example/npy2pt.py:75-119): host
 * row_ptr[out/16+1], column[ntile], data[ntile][256], bias[out] (NULL = 0).
 * fp32 values are rounded to fp16 (nearest-even); the _f16 form takes fp16 bits. */
int et_model_set_bsr16(et_model m, int layer, int which, const int32_t *row_ptr,
                       const int32_t *column, const float *data, int ntile,
                       const float *bias);
int et_model_set_bsr16_f16(et_model m, int layer, int which, const int32_t *row_ptr,
                           const int32_t *column, const et_f16 *data, int ntile,
                           const et_f16 *bias);
/* dense [out x in] weight (Linear<base_mat>); a layer is all-BSR or all-dense */
int et_model_set_dense(et_model m, int layer, int which, const float *W,
                       const float *bias);
int et_model_set_dense_f16(et_model m, int layer, int which, const et_f16 *W,
                           const et_f16 *bias);
/* SkipLayerNorm which = 0 (after attention) or 1 (after the FFN): host gamma, beta[emdim] */
int et_model_set_norm(et_model m, int layer, int which, const float *gamma,
                      const float *beta);
int et_model_set_norm_f16(et_model m, int layer, int which, const et_f16 *gamma,
                          const et_f16 *beta);
/* right padding: host lens[batch], keys >= lens[b] are ignored; NULL removes it */
int et_model_set_lens(et_model m, const int32_t *lens_host);
/* additive [seq_len x seq_len] mask from host memory; NULL removes it */
int et_model_set_mask(et_model m, const et_f16 *mask_host);
/* uploads the weights and builds the layer objects; weights are fixed afterwards */
int et_model_finalize(et_model m);
/* builds a finalized model from weights.txt + .npz archives (example/weights.hpp:32-47) */
int et_model_load(const char *weights_txt, const char *dir,
                  const et_model_desc *desc, et_model *out);
/* out, in: device [batch*seq_len x emdim].  Asynchronous; stream NULL = the
 * model's own stream (wait with et_model_sync).  in and out may not alias. */
int et_model_forward(et_model m, et_f16 *out, const et_f16 *in, et_stream stream);
/* one layer, launched kernel by kernel (Encoder<cfg>::forward) */
int et_model_forward_layer(et_model m, int layer, et_f16 *out, const et_f16 *in,
                           et_stream stream);
int et_model_sync(et_model m);
/* kernel launches per encoder layer of a finalized model in the mode it actually runs
 * (2: chain launches, 5: SkipLayerNorm folded into the projections, 7: SkipLayerNorm on its own;
 * 0 before et_model_finalize).  A model asked for mixed = 3 reports 5 once it has gone back to
 * separate launches. */
int et_model_launches_per_layer(et_model m, int *launches);
int et_model_destroy(et_model m);

/* The same stack in binary32 from end to end: weights, activations, input and
 * output are float; every layer is seven launches of the *_f32 entry points
 * above (QKV, attention, O, SkipLayerNorm, linear1 + activation, linear2,
 * SkipLayerNorm: Encoder/Encoder.h:81-96), replayed as one HIP graph when
 * desc.use_graph != 0.  desc.mixed is ignored; kdim == vdim == emdim.  A
 * layer's four matrices may each be dense or 16x16 tile-sparse.  No reference
 * counterpart (the reference computes in binary16 only): the binary32 twin of
 * et_model_*, for checking a pruned model's values without binary16 rounding.
 * Argument meaning as in the et_model_* function of the same name. */
typedef struct et_model_f32_s *et_model_f32;
int et_model_f32_create(const et_model_desc *desc, et_model_f32 *out);
int et_model_f32_set_bsr16(et_model_f32 m, int layer, int which, const int32_t *row_ptr,
                           const int32_t *column, const float *data, int ntile,
                           const float *bias);
int et_model_f32_set_dense(et_model_f32 m, int layer, int which, const float *W,
                           const float *bias);
int et_model_f32_set_norm(et_model_f32 m, int layer, int which, const float *gamma,
                          const float *beta);
int et_model_f32_set_lens(et_model_f32 m, const int32_t *lens_host);
int et_model_f32_finalize(et_model_f32 m);
int et_model_f32_forward(et_model_f32 m, float *out, const float *in, et_stream stream);
int et_model_f32_sync(et_model_f32 m);
int et_model_f32_destroy(et_model_f32 m);

/* ------------------------------------------------------------------------
 * Host-side construction of the sparse weight structures (integer work on
 * host pointers, usable without a GPU).  Outputs are caller-allocated; a
 * function that produces a data-dependent number of entries reports it through
 * its last argument and accepts NULL for the variable-length outputs on a
 * sizing call.  Random structure is seeded: ids are taken in ascending order
 * of their SplitMix64 key, which stands in for the reference's
 * std::random_shuffle.
 * ------------------------------------------------------------------------ */

/* out[0..n) = the seeded permutation of 0..n-1. */
int et_fmt_permutation(int64_t n, uint64_t seed, int64_t *out);
/* int(total * (1.0 - (double)sparsity)) — mat_type/tile_mat/tile_mat.cu:12.
 * Returns the count itself (not a status). */
int et_fmt_kept_count(int64_t total, float sparsity);
/* tile_mat::gen_sparse_mat structure (mat_type/tile_mat/tile_mat.cu:7-40):
 * row_ptr[nrow/16+1], row_offset[kept_count(total tiles)] in permuted order. */
int et_fmt_tile_pattern(int nrow, int ncol, float sparsity, uint64_t seed,
                        int32_t *row_ptr, int32_t *row_offset, int *ntile);
/* Exporter gen_csr (example/npy2pt.py:75-109): tiles of W[nrow x ncol] with a
 * non-zero element, block-rows in order, columns ascending; data[ntile][256]. */
int et_fmt_dense_to_bsr16(const float *W, int nrow, int ncol, int32_t *row_ptr,
                          int32_t *column, float *data, int *ntile);
/* row_mat::gen_sparse_mat ids (mat_type/row_mat/row_mat.cu:14-25), ascending. */
int et_fmt_row_ids(int nrow, float sparsity, uint64_t seed, int32_t *ids, int *count);
/* col_mat::gen_sparse_mat ids (mat_type/col_mat/col_mat.cu:22-32), permuted order. */
int et_fmt_col_ids(int ncol, float sparsity, uint64_t seed, int32_t *ids, int *count);
/* col_mat::set_metadata (mat_type/col_mat/col_mat.cu:34-58): out[nhead+1]. */
int et_fmt_head_ptr(const int32_t *col_id, int nnz_col, int nhead, int full_dim,
                    int32_t *out);
/* mat1x16 (mat_type/mat1x16/mat1x16.h:5-22) in the layout its kernel reads
 * (Linear/SPMM1x16.cu:52-74): tile_idx[(nrow/16)*(ncol/16+1)] global offsets,
 * row_idx[ntile], data[pad16(ntile)][16]. */
int et_fmt_dense_to_1x16(const float *W, int nrow, int ncol, int32_t *tile_idx,
                         int32_t *row_idx, float *data, int *ntile);
int et_fmt_1x16_pattern(int nrow, int ncol, float sparsity, uint64_t seed,
                        int32_t *tile_idx, int32_t *row_idx, int *ntile);
/* csr_mat (mat_type/csr_mat/csr_mat.h:11-42, generator csr_mat.cpp:25-67). */
int et_fmt_dense_to_csr(const float *W, int nrow, int ncol, int32_t *indptr,
                        int32_t *indices, float *data, int *nnz);
int et_fmt_csr_pattern(int nrow, int ncol, float sparsity, uint64_t seed,
                       int32_t *indptr, int32_t *indices, int *nnz);
/* .csr file reader (mat_type/csr_mat/csr_mat.h:19-35). */
int et_fmt_csr_read(const char *path, int *nrow, int *ncol, int *nnz,
                    int32_t *indptr, int32_t *indices, float *data);

#ifdef __cplusplus
}
#endif
#endif /* ET_ABI_H */
