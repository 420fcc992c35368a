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
int et_memset(void *ptr, int byte, size_t bytes, et_stream stream);
int et_memcpy_h2d(void *dst, const void *src_host, size_t bytes);
int et_memcpy_d2h(void *dst_host, const void *src, size_t bytes);
int et_memcpy_d2d(void *dst, const void *src, size_t bytes, et_stream stream);
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

/* Tuning hook: et_linear_bsr16_f16 with an explicit launch geometry — mt in
 * {1,2,4} 16-token blocks per workgroup strip, stage != 0 keeps the strip of X
 * in LDS, threads per workgroup (multiple of 64, <= 512) and block-rows of W per
 * workgroup.  Same result as et_linear_bsr16_f16; no reference counterpart. */
int et_linear_bsr16_f16_geom(const int32_t *row_ptr, const int32_t *col_idx,
                             const et_f16 *tiles, const et_f16 *bias,
                             const et_f16 *X, et_f16 *Y, int T, int in, int out,
                             int act, int mt, int stage, int threads,
                             int rows_per_wg, et_stream stream);

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
 * both contractions are fp32-accumulated.  S % 16 == 0, hd in {32, 64, 128}.
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

/* ------------------------------------------------------------------------
 * Normalisation and element-wise operators.
 * ------------------------------------------------------------------------ */

/* out[r] = LayerNorm(src[r] + skip[r]) * gamma + beta over H features,
 * statistics in fp32, one pass over HBM.  H % 4 == 0, H <= 8192.
 * Replaces SkipLayerNorm::forward (SkipLayerNorm/SkipLayerNorm.cu:73-82). */
int et_skip_layernorm_f16(et_f16 *out, const et_f16 *src, const et_f16 *skip,
                          const et_f16 *gamma, const et_f16 *beta, int rows,
                          int H, float eps, et_stream stream);

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

#ifdef __cplusplus
}
#endif
#endif /* ET_ABI_H */
