/*
 * vaq_tuning.h -- kernel-variant overrides for this library's own tests and benchmarks.  Not part of the drop-in
 * surface (include/vllm_amd_qlinear.h): the reference's kernels take no such argument and the ops never pass one.
 * The struct layout is mirrored by vllm_amd/_lib.py and may change with the kernels.
 */
#ifndef VAQ_TUNING_H_
#define VAQ_TUNING_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

/*
 * Kernel-variant overrides for tests and benchmarks.  No counterpart in the reference (its kernels take no such
 * argument); the drop-in surface never passes one.  A VaqTuning applies to the ONE call it is handed to, on the calling
 * thread only: the library keeps no tuning state between calls.  Every field: 0 = the automatic choice.
 */
typedef struct VaqTuning {
  int decode_impl;      /* W4A16 decode kernel: 1 LDS-staged activations, 2 register-resident activations          */
  int decode2_gs;       /* LDS-staged kernel: weight tiles per wavefront                                             */
  int decode2_wks;      /*   K slices per workgroup                                                                  */
  int decode2_wn;       /*   n-tiles per workgroup                                                                   */
  int decode_tg;        /* register-resident kernel: groups per wavefront                                            */
  int decode_wk;        /*   wavefronts along K per workgroup                                                        */
  int decode_gx;        /*   workgroups along N                                                                      */
  int decode_depth;     /*   prefetch depth                                                                          */
  int prefill_tile;     /* W4A16 tile kernel: tile id + 1                                                            */
  int prefill_split;    /*   K split                                                                                 */
  int fp8_path;         /* FP8 GEMM: 1 weight-streaming kernel, 2 tile kernel                                        */
  int fp8_tile_impl;    /*   1 register-staged tile kernel                                                           */
  int fp8_tile_cfg;     /*   multi-stage tile shape id, -1 = two-stage kernel                                        */
  int fp8_split;        /*   K split of the tile kernel                                                              */
  int fp8_gx;           /*   workgroups of the weight-streaming kernel                                               */
  int fp8_stream_split; /*   -1 = never run the weight-streaming kernel over two halves of K                         */
  int quant_wg_per_row; /* per-token FP8 quant: 1 = one workgroup per row, 2 = one wavefront per row (where it can)    */
  int exp[15];          /* further switches of the same kind, for A/B timing runs: [0] = 1 shared instead of private  */
                        /*   activation fill, [1] = ring variant + 1, [2] rows over workgroups (1 off, 2 forced) of   */
                        /*   the LDS-staged decode kernel, [3] = 1 sixteen staged rows for M = 5 .. 8, [5] = 1 two K   */
                        /*   slabs never merged into one; [4] FP8 streaming through LDS (1 / 2 / 3 = 8 / 4 / 16 steps   */
                        /*   per wavefront, 9 = off); [8] = 1 W4A16 tile kernel: no 128 x 128 tiles for long K parts;   */
                        /*   [9] = 1 both tile kernels: 256-row tiles also when M fills them poorly; [10] = 1 both tile     */
                        /*   kernels: never split only the tiles of a half-empty last round; [11] = 1 W4A16 tile kernel:  */
                        /*   no 128 x 256 tiles; [12] = 1 FP8 tile kernel: every tile starts at the first K step;       */
                        /*   [13] = 1 FP8 tile kernel: no tile row past M; [14] = 1 FP8 tile kernel: no 128 x 64 tiles;  */
                        /*   [7] = 1 LDS-staged decode kernel: n-tiles in launch order, not grouped by XCD             */
} VaqTuning;

/* The entry points of the same name without `_tuned`, with `tuning` (may be NULL) applied to this call. */
int vaq_w4a16_gemm_workspace_tuned(int64_t size_m, int64_t size_n, int64_t size_k, int has_perm, int device,
                                   size_t* c_tmp_bytes, size_t* a_tmp_bytes, size_t* counter_ints,
                                   const VaqTuning* tuning);
int vaq_w4a16_gemm_tuned(const void* a, int64_t lda, const int32_t* b, const void* scales, const int32_t* zeros,
                         const int32_t* perm, const void* bias, void* c, float* c_tmp, int64_t c_tmp_bytes, void* a_tmp,
                         int32_t* counters, int64_t counter_ints, int64_t size_m, int64_t size_n, int64_t size_k,
                         int group_size, int dtype, int wtype, int force_path, void* stream, const VaqTuning* tuning);
int vaq_fp8_scaled_mm_workspace_tuned(int64_t size_m, int64_t size_n, int64_t size_k, size_t* c_tmp_bytes,
                                      size_t* counter_ints, const VaqTuning* tuning);
int vaq_fp8_scaled_mm_ws_tuned(const uint8_t* a, int64_t lda, const uint8_t* b, int64_t ldb, const float* sa,
                               int64_t sa_count, const float* sb, int64_t sb_count, const void* bias, void* out,
                               int64_t ldc, int out_dtype, int64_t size_m, int64_t size_n, int64_t size_k, float* c_tmp,
                               int64_t c_tmp_bytes, int32_t* counters, int64_t counter_ints, void* stream,
                               const VaqTuning* tuning);
int vaq_fp8_quant_per_token_tuned(const void* in, int in_dtype, int64_t in_row_stride, uint8_t* out,
                                  int64_t out_row_stride, float* scales, const float* scale_ub, int64_t rows,
                                  int64_t hidden, void* stream, const VaqTuning* tuning);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* VAQ_TUNING_H_ */
