/* noeira_qlinear_diag.h - measurement helpers of libnoeira_qlinear.so.
 *
 * None of these has a counterpart in the reference, and none is part of the operator: they are what bench.py
 * measures the operator's kernels against (the matrix cores alone, a plain read of a layer's bytes) or with (a GEMM
 * call's per-workgroup timeline, the medium-M kernel under a fixed tile shape).  Every one of them acts on its own
 * launch only: there is no switch here that changes what nq_forward does, on any thread.
 */
#ifndef NOEIRA_QLINEAR_DIAG_H
#define NOEIRA_QLINEAR_DIAG_H

#include "noeira_qlinear.h"

#ifdef __cplusplus
extern "C" {
#endif

/* What the matrix cores alone sustain on this GPU (no counterpart in the reference; bench.py reports it
 * beside the 8-bit GEMM so that the GEMM's fraction of the published peak can be read against what the chip's
 * power limit leaves): `workgroups` workgroups of four wavefronts issue MFMAs back to back on register operands
 * taken from `operands` (device, operand_bytes >= 4096; what the bytes are, constant or random codes, is the
 * caller's choice), 256 accumulators per lane as in the GEMM.  kind 0: 16 * iters v_mfma_f32_32x32x64_f8f6f4 on
 * e4m3 codes (131072 operations each), kind 1: 16 * iters v_mfma_i32_32x32x32_i8 (65536 each), kind 2: 64 * iters
 * v_mfma_f32_16x16x128_f8f6f4 (65536 each), kind 3: 64 * iters v_mfma_i32_16x16x64_i8 (32768 each).  stamps:
 * device int64 [workgroups][2] = the loop's duration in shader clocks and in ticks of the constant 100 MHz clock. */
int32_t nq_diag_mfma_rate(int32_t kind, const void* operands, int64_t operand_bytes, int32_t iters, int32_t workgroups,
                          int64_t* stamps, void* stream);

/* The floor of a weight-streaming call (no counterpart in the reference): a kernel that only reads the first
 * nbytes / 1024 KiB of `src` (device, 16-byte aligned) with 1 KiB load instructions and computes nothing.
 * bench.py times it on the bytes of each large GEMV's weight: launch + stream, what no GEMV over those bytes
 * can beat on this GPU. */
int32_t nq_diag_stream_read(const void* src, int64_t nbytes, void* stream);

/* Where the time of a large-tile 8-bit GEMM goes (no counterpart in the reference): the launch nq_forward makes
 * for 8-bit activations and M >= 64 rows over a layer whose IN is a multiple of 128 (NQ_ERR_UNSUPPORTED otherwise),
 * with every workgroup of the 256 x 256 tile kernel reporting four readings of the GPU's constant 100 MHz clock -
 * entry, first K stage landed, K loop done, stores acknowledged - and the shader clock's cycle counter at the second
 * and third of them (so that the K loop can be read in cycles and the clock it ran at follows) into stamps (device
 * uint64 [tiles][6], tiles = ceil(M / 256) * ceil(OUT / 256) <= max_tiles, else NQ_ERR_INVALID).  The kernel is the
 * form nq_forward takes for the operand type (fp8: four wavefronts, int8: eight), on 256 x 256 tiles throughout.  The arguments are nq_forward's for that case
 * (x: int8 with per-row x_scale, or e4m3 codes with one scale; y fp32 or bf16, for int8 also the raw int32
 * accumulators; no bias).  The stamp buffer is an argument of this
 * one launch: no other call, on this or another thread, writes stamps.  Synchronises the stream before it returns. */
int32_t nq_diag_gemm8_timeline(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale, void* y,
                               int32_t y_dtype, int32_t M, uint64_t* stamps, int64_t max_tiles, void* stream);

/* nq_forward for 8-bit activations (int8 with per-row scales over a W8_CHANNEL layer, e4m3 codes with one scale over
 * an FP8_E4M3 layer; M >= 64, IN a multiple of 128) on the GEMM kernel of the caller's choice (no counterpart in the
 * reference): tile = 256, the 256 x 256 tile kernel nq_forward takes from about a round and a half of such tiles on,
 * or 128, the 128 x 128 tile kernel it takes below that where no 16-row tile kernel is estimated faster; 2564 / 2568:
 * the 256 x 256 tile kernel on four / eight wavefronts per workgroup (256 takes eight for int8, four for fp8).  All
 * return the same bits; tests hold each against the oracle on shapes the dispatch would give to the other, and
 * bench.py times them side by side.  Acts on this one launch only. */
int32_t nq_diag_forward_gemm8(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale, void* y, int32_t y_dtype,
                              int32_t M, const void* bias, int32_t bias_dtype, int32_t epilogue, int32_t tile, void* stream);

/* A forward on the 16-row tile kernel that takes 2 .. 511 rows of fp32 / bf16 activations, under a tile shape of
 * the caller's choice (no counterpart in the reference): mw x nw wavefront tiles of 16 x 16 per workgroup, one of
 * 1 x 1, 1 x 2, 1 x 4, 2 x 2, 2 x 4 (2 x 4 not with fp32 activations).  The arguments are nq_forward's without bias and
 * epilogue; the shape holds for this launch only.  nq_forward picks the shape of least estimated time itself;
 * `bench.py --only a16_shapes` times a grid of calls under each shape with this call and re-derives the estimate's
 * constants from them.  The shape never changes a result's bits.  NQ_ERR_UNSUPPORTED where that kernel does not
 * take the layer (8-bit activations, a GLU layer, a row-fused layer, M < 2). */
int32_t nq_diag_forward_a16(nq_handle h, const void* x, int32_t x_dtype, void* y, int32_t y_dtype, int32_t M,
                            int32_t mw, int32_t nw, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* NOEIRA_QLINEAR_DIAG_H */
