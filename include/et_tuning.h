/*
 * et_tuning.h — entry points for tuning experiments.  Not part of the drop-in
 * boundary (that is et_abi.h): nothing in the class layer calls them and a
 * binding does not need them.  Exported by the same library.
 */
#ifndef ET_TUNING_H
#define ET_TUNING_H

#include "et_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Tuning hook: et_linear_bsr16_f16 with an explicit launch geometry — mt in
 * {1,2,4} 16-token blocks per workgroup strip, stage != 0 keeps the strip of X
 * in LDS, threads per workgroup (multiple of 64, <= 512) and block-rows of W per
 * workgroup.  Same result as et_linear_bsr16_f16; no reference counterpart. */
int et_linear_bsr16_f16_geom(const int32_t *row_ptr, const int32_t *col_idx,
                             const et_f16 *tiles, const et_f16 *bias,
                             const et_f16 *X, et_f16 *Y, int T, int in, int out,
                             int act, int mt, int stage, int threads,
                             int rows_per_wg, et_stream stream);

/* Tuning hook: et_bsr16_pack_create with an explicit geometry — mt 16-row blocks
 * per token strip (1 or 2), block-row groups per strip, waves per workgroup and
 * slots per wave (4, 8, 12, 16, 20 or 24); 0 picks a value as
 * et_bsr16_pack_create does.  No reference counterpart. */
int et_bsr16_pack_create_geom(const int32_t *row_ptr, const int32_t *col_idx,
                              const et_f16 *tiles, int T, int in, int out,
                              int flags, int mt, int ngroups, int nwave, int cap,
                              et_bsr_pack *pack);

/* Tuning hook: et_mha_fuseo_f16 with an explicit number of waves per workgroup
 * (1, 2 or 4: 16, 32 or 64 tokens per attention workgroup and projection strip;
 * 0 picks as et_mha_fuseo_f16 does).  No reference counterpart. */
int et_mha_fuseo_f16_geom(const et_f16 *Q, const et_f16 *K, const et_f16 *V,
                          int ldq, int ldk, int ldv, et_f16 *Z, int ldz,
                          const et_f16 *mask, const int32_t *lens, int B, int S,
                          int nh, int hd, float scale, int flags,
                          const int32_t *o_row_ptr, const int32_t *o_col_idx,
                          const et_f16 *o_tiles, const et_f16 *o_bias,
                          et_f16 *out, int emdim, int waves, et_stream stream);

/* Machine probes (scpaper-2021_amd/kernel_bench.py --set machine): an empty launch of nwg
 * workgroups (what a kernel boundary costs inside a graph), and a launch in which every
 * workgroup requests vec_per_thread (4, 8, 16, 32) 16-byte vectors per thread, all before it
 * uses the first, from a region of src of its own (shared = 0) or from the region of the
 * first workgroup of its XCD (shared != 0: lines that hit that XCD's L2 after the first
 * touch): how fast one compute unit takes bytes in.  sink: nwg words.  No reference
 * counterpart. */
int et_probe_empty(int nwg, int threads, et_stream stream);
int et_probe_read(const void *src, size_t src_bytes, int nwg, int threads,
                  int vec_per_thread, int shared, uint32_t *sink, et_stream stream);

#ifdef __cplusplus
}
#endif

#endif /* ET_TUNING_H */
