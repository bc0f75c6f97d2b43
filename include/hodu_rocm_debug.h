/*
 * hodu_rocm_debug.h -- test and measurement hooks of libhodu_rocm_debug.so.
 *
 * Nothing here belongs to the drop-in boundary: a hodu_rocm_kernels crate binds include/hodu_rocm_kernels.h only.
 * These hooks exist so that every compiled kernel variant can be exercised at small sizes, and so that launches as
 * short as 3 us can be timed back to back from C with HIP events on the stream they run on.  The library links
 * against libhodu_rocm_kernels.so and calls its public entry points.
 */
#ifndef HODU_ROCM_DEBUG_H
#define HODU_ROCM_DEBUG_H

#include "hodu_rocm_kernels.h"

#ifdef __cplusplus
extern "C" {
#endif

/* testing hook: pin the MFMA tile variant (0 = 256x256 with 8 wavefronts, 1 = 256x256 with 4,
 * 2 = 128x128, 3 = 64x64; 10..13 the same tiles of the software-pipelined kernel; 30 = no row-streaming
 * GEMV kernel, 31/32/34 = that kernel as one-shot wavefronts (4 x 1, 4 x 2, 8 x 2 wavefronts x weight rows per workgroup),
 * 33 = its row-walking form (one wavefront per SIMD, the default from 16 weight rows per compute unit); 14 = the pipelined 256x128 tile,
 * 15 = the pipelined 256x256 tile on the 16x16x32 instruction (two k-dense 16-bit operands; 11 pins the 32x32x16 one),
 * 16 = the same tile with the loop's LDS-DMA and address instructions spaced by issue slots (an even number of stages);
 * 35/36/37 = the one-pass kernel for M <= 16 with 1/2/4 blocks of 16 weight rows per workgroup, 38 = its
 * variant that cuts K across workgroups wherever it applies, 39 = one block per workgroup with the left operand read
 * in place instead of staged in LDS (what a left operand too large for LDS gets); 40 = the small-product f32 kernel at any size; 41 / 42 / 43 = the f64 matrix-core kernel with
 * 128 x 128 / 64 x 64 / 32 x 32 tiles;
 * -1 = automatic) so that every compiled variant
 * can be exercised at small sizes */
int hodu_rocm_debug_force_tile(hodu_rocm_ctx *ctx, int tile);
/* testing hook: what the context itself has allocated for its kernels' scratch -- bytes of its partial-sum workspace
 * (0 = never allocated), whether its arrival counters exist -- and whether it is (still) pointed at the static
 * scratch of the entry point that allocates nothing, which must never be the case between calls */
int hodu_rocm_debug_scratch_state(hodu_rocm_ctx *ctx, size_t *workspace_bytes, int *arrival_allocated, int *in_fixed_mode);
/* testing hook: number of K ranges the pipelined tile kernels cut a product into (each range a workgroup of its
 * own, partial sums added in a fixed order by a second kernel): -1 = automatic (only products too small to
 * fill the machine are cut), 1 = never, n = n ranges wherever the kernel can */
int hodu_rocm_debug_force_splitk(hodu_rocm_ctx *ctx, int splits);
/* measurement hook: issues the same product `iters` times back to back from C (no per-launch
 * interpreter overhead), cycling through `n_rhs` right-hand buffers so a small operand cannot sit
 * in the Infinity Cache, bracketed by HIP events on the context's stream; *elapsed_ms is the total.
 * is_matmul selects the metadata format; kind: 0 = plain `dtype`, 1 = bf16 x f8e4m3, 2 = i8 x i8 -> i32 */
int hodu_rocm_debug_time_product(hodu_rocm_ctx *ctx, int is_matmul, int kind, int dtype, const void *lhs,
                                 const void *const *rhs_list, size_t n_rhs, void *out, const size_t *metadata,
                                 size_t metadata_len, int iters, float *elapsed_ms);
/* the same, with the `iters` launches captured once into a HIP graph (kernel nodes only) and replayed as
 * one graph launch inside the timed region: the per-launch time a caller sees who replays a recorded
 * decode step instead of paying a host round trip per product */
int hodu_rocm_debug_time_product_graph(hodu_rocm_ctx *ctx, int is_matmul, int kind, int dtype, const void *lhs,
                                       const void *const *rhs_list, size_t n_rhs, void *out, const size_t *metadata,
                                       size_t metadata_len, int iters, float *elapsed_ms);

/* measurement hook: the rate and shader clock of a register-only MFMA loop (no LDS, no memory traffic) on
 * caller-supplied operand bits, two workgroups per compute unit.  kind 0: bf16 32x32x16; kind 1: f8e4m3 32x32x64
 * with unit scales; kind 2: bf16 16x16x32; kind 3: f8e4m3 16x16x128.  `operands`: 16 KB of device memory (1024 x 16 bytes: per lane the a and b fragments, twice).
 * *tflops is what the loop sustained, *shader_mhz the clock one wavefront saw (shader-clock counter over the
 * 100 MHz counter).  Under full MFMA load the clock depends on the data, so this is the ceiling a GEMM kernel can
 * approach on that data. */
int hodu_rocm_debug_mfma_clock(hodu_rocm_ctx *ctx, int kind, const void *operands, int iters, float *elapsed_ms,
                               double *tflops, double *shader_mhz);

/* measurement hook: `iters` launches of a flat streaming read (16 bytes per lane, eight loads in flight, nothing
 * else) of `bytes` from each of the `n_src` device buffers in turn, and `iters` launches of an empty kernel, each
 * bracketed by HIP events on the context's stream.  *read_us: time per read launch; *empty_us: time per empty launch
 * (the launch cadence).  What the memory system and the launch path allow a kernel that moves `bytes`. */
int hodu_rocm_debug_read_floor(hodu_rocm_ctx *ctx, const void *const *src_list, size_t n_src, size_t bytes, int iters,
                               float *read_us, float *empty_us);

/* measurement hook: `iters` back-to-back launches of hodu_rocm_cast (src != dst) or hodu_rocm_contiguous (src == dst)
 * on one metadata array, walking through n_buffers input / output pairs (so that a stream larger than the last-level
 * cache comes from memory), HIP-event timed on the context's stream. */
int hodu_rocm_debug_time_cast(hodu_rocm_ctx *ctx, int src_dtype, int dst_dtype, const void *const *in_list,
                              void *const *out_list, size_t n_buffers, const size_t *metadata, size_t metadata_len,
                              int iters, float *elapsed_ms);
/* measurement hook: the same for hodu_rocm_sum */
int hodu_rocm_debug_time_sum(hodu_rocm_ctx *ctx, int dtype, const void *const *in_list, void *const *out_list,
                             size_t n_buffers, const size_t *metadata, size_t metadata_len, int iters, float *elapsed_ms);
/* measurement hook: hodu_rocm_debug_time_product with fused steps */
int hodu_rocm_debug_time_product_ex(hodu_rocm_ctx *ctx, int is_matmul, int kind, int dtype, const void *lhs,
                                    const void *const *rhs_list, size_t n_rhs, void *out, const size_t *metadata,
                                    size_t metadata_len, const hodu_rocm_epilogue_step *steps, size_t n_steps,
                                    int iters, float *elapsed_ms);

/* measurement hook: `iters` calls of hodu_rocm_dot_bf16_f8e4m3w_noalloc, as hodu_rocm_debug_time_product times
 * the allocating entry point; graph != 0 captures the calls into one HIP graph first (the entry point launches
 * kernels only, so it may be captured from its first call on) */
int hodu_rocm_debug_time_noalloc(hodu_rocm_ctx *ctx, const void *lhs, const void *const *rhs_list, size_t n_rhs,
                                 void *out, const size_t *metadata, size_t metadata_len, int iters, int graph,
                                 float *elapsed_ms);

#ifdef __cplusplus
}
#endif
#endif /* HODU_ROCM_DEBUG_H */
