/*
 * C ABI of libatorch_amd_probes.so: measurement aids for the benchmark and the tests of the FP8
 * grouped-linear MoE expert path on gfx950 (MI355X).  None of this is part of the product library
 * (libatorch_amd_fp8.so, include/atorch_amd_fp8.h) and none of it has a counterpart in the reference.
 *
 * Conventions are those of atorch_amd_fp8.h: device pointers owned by the caller, `stream` a
 * hipStream_t passed as void*, int status (AAMD_OK / AAMD_ERR_ARG / AAMD_ERR_HIP); the text of the
 * last failure on the calling thread comes from aamd_probes_last_error().
 */
#ifndef ATORCH_AMD_PROBES_H
#define ATORCH_AMD_PROBES_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default) /* the entry points are the only symbols the library exports */

const char *aamd_probes_last_error(void);

/*
 * The grouped GEMMs of the product library (same kernels, same arguments as aamd_grouped_gemm_fp8_nt and
 * aamd_grouped_gemm_fp8_wgrad) with the launch choices the library otherwise makes by itself pinned for
 * this one call: opts = {tile, group_r, gl, ls_batch}, each -1 for the library's own choice.
 *   tile: 0 = 128x128 tiles, 1 = the large configuration (wgrad: 256x128 tiles);
 *   group_r: the tile order groups R tiles (1) or L tiles (0); gl: tiles sharing a panel in the tile order;
 *   ls_batch: 0 = scales fetched one contraction block at a time (which the 128x128 tiles do: the large
 *   configuration of the block-scaled GEMM takes its scales in batches only and is then not chosen).
 * Nothing is kept between calls.
 */
int aamd_tuning_grouped_gemm_fp8_nt(const uint8_t *a, int64_t lda, const float *a_s, const uint8_t *b,
                                    const float *b_s, int b_tile_scaled, const int64_t *group_offsets, int E,
                                    int32_t *tile_ws, int64_t M, int64_t N, int64_t K, void *c, int c_dtype,
                                    int64_t ldc, const void *bias, int bias_dtype, const int *opts, void *stream);
int aamd_tuning_grouped_gemm_fp8_wgrad(const uint8_t *dyt, const float *sdyt, const uint8_t *xt, const float *sxt,
                                       int64_t ld_t, int q_t_layout, const int64_t *group_offsets, int E,
                                       int32_t *tile_ws, int64_t N, int64_t K, void *dw, int dw_dtype,
                                       int64_t expert_stride, int accumulate, const int *opts, void *stream);

/*
 * Shader clock probe (no counterpart in the reference; the benchmark reports the clock the GEMMs
 * run at): one wavefront spins for about min_cycles shader cycles (at most 2^31) and writes
 * out[0] = elapsed shader cycles, out[1] = elapsed ticks of the constant 100 MHz clock.
 */
int aamd_clock_probe(uint64_t *out, int64_t min_cycles, void *stream);

/*
 * Matrix-pipe probe (no counterpart in the reference; the benchmark reports what the fp8 MFMA pipes
 * deliver from registers alone, which on this GPU depends on the operand values through the power
 * limit): `workgroups` workgroups of eight waves issue, `iters` times, the sixteen
 * v_mfma_f32_32x32x64_f8f6f4 of one 128-deep step of a 128 x 64 wave tile, with the block-scale fold
 * (16 FMAs per MFMA pair) when fold == 1, or the fold of per-row scales on both operands (16 multiplies and 16 FMAs
 * per MFMA pair, the weight-gradient step) when fold == 2; fold == 3: sixteen multiplies per pair rescale the accumulator
 * the MFMAs then add to directly (no raw-product buffer, no wait for an MFMA result).  FLOP = workgroups * 8 * iters * 16 * 131072.
 *   operands: 64 * 512 * 12 * 32 bytes of fp8 codes (any values), 32-byte aligned
 *   out: workgroups * 512 floats (checksums); cycles[0]: shader cycles one wave spent in the loop.
 */
int aamd_mfma_probe(const void *operands, int fold, int iters, int workgroups, float *out, uint64_t *cycles,
                    void *stream);

/*
 * Loop probe (no counterpart in the reference; the benchmark reports what one 128-deep step of the
 * 256 x 256 GEMM configuration costs as an instruction sequence on private data): 256 workgroups of
 * eight waves run, `iters` times, the step's sixteen MFMAs with their folds, its 24 fragment reads
 * from an LDS tile laid out like the GEMM's and its eight 1 KB direct-to-LDS loads, without scales,
 * barriers, prologue or epilogue.  stream_panels == 0: the loads re-read the first 4 KB of `panels`;
 * != 0: they walk 1 MiB panels (256 rows of 4 KB, 128 bytes per row and step) shared among the
 * workgroups of an XCD the way the GEMM's tiles share operand panels, and move on to the next set of
 * 96 panels every 32 steps (`panels` then holds a multiple of 96 MiB: panel_bytes / 96 MiB sets, wrapped);
 * 2: the same with the GEMM's two barriers per step, the wait for the loads of the step before in front
 * of the second one, and the loads issued where the GEMM issues them.
 * FLOP = 256 * 8 * iters * 16 * 131072; out: 256 * 512 floats; cycles[0]: shader cycles of one wave.
 */
int aamd_loop_probe(const void *panels, int64_t panel_bytes, int stream_panels, int iters, float *out,
                    uint64_t *cycles, void *stream);

/*
 * Streaming probe (no counterpart in the reference; the benchmark prices the memory-bound kernels
 * against what the memory system delivers for their mix of read and written bytes): per 16-byte word
 * of work one word is read from each of `reads` input streams and one written to each of `writes`
 * output streams, all accesses streaming.  Stream i of src / dst starts at byte i * stride_bytes and
 * holds `units` words.  Built mixes: 1:0 0:1 1:1 2:1 1:2 1:4 4:1 8:1 3:2 2:2.
 */
int aamd_stream_probe(const void *src, void *dst, int reads, int writes, int64_t stride_bytes, int64_t units,
                      void *stream);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* ATORCH_AMD_PROBES_H */
