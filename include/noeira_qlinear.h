/* noeira_qlinear.h — C ABI of libnoeira_qlinear.so, the MI355X (gfx950)
 * implementation of noeira's quantized-linear inference path.
 *
 * The reference has no C ABI for this operator: its boundary is the Mojo
 * `Module` surface implemented by `QLinear[IN, OUT]`
 * (noeira/nn/quant/qlinear.mojo:208-524).  This header is what a Mojo host
 * binds through the reference's own FFI idiom
 *     var lib = OwnedDLHandle(path); var f = lib.get_function[c_int]("sym")
 * (benchmarks/_test_cuda_ffi.mojo:61-80, noeira/io/serial/native.mojo:44-109).
 * That idiom fixes the rules followed here: every function has a fixed arity
 * (no variadics: noeira/io/serial/native.mojo:6-14), takes only integers,
 * floats and raw addresses, and returns an int32 status (0 = NQ_OK).  Each
 * entry point cites the reference method it stands in for.
 *
 * Conventions
 *   - W is [OUT, IN] row-major (torch's orientation, qlinear.mojo:3), x is
 *     [M, IN] row-major, y is [M, OUT] row-major, dense strides.
 *   - Host pointers are named *_host; every other data pointer is a device
 *     address valid on the current HIP device.
 *   - `stream` is a hipStream_t passed as an address (NULL = the default
 *     stream).  Compute entry points only enqueue: they never synchronise and,
 *     after the first call at a given M, never allocate (the capture rule of
 *     qlinear.mojo:60-68 gated by tests/nn/quant/test_qlinear_gpu.mojo:55-130).
 *   - A layer handle is used by one host thread at a time; different handles
 *     may be used from different threads/streams.  Identical inputs give
 *     bit-identical outputs on every call (test_qlinear_gpu.mojo:96,128).
 *   - On failure a function returns a non-zero status and leaves a sentence
 *     for nq_last_error(); the wording follows the reference's `raise Error`
 *     messages so a wrapper can re-raise them verbatim.
 *   - This table is append-only; nq_abi_version() guards it.
 */
#ifndef NOEIRA_QLINEAR_H
#define NOEIRA_QLINEAR_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NQ_ABI_VERSION 7

/* status codes */
#define NQ_OK 0
#define NQ_ERR_INVALID 1     /* bad argument / shape / dtype combination */
#define NQ_ERR_NOT_LOADED 2  /* forward before set_weight / set_blocks */
#define NQ_ERR_NO_BLOCKS 3   /* logical blocks were dropped (keep_only_repacked) */
#define NQ_ERR_SIZE 4        /* wrong byte count / scratch too small */
#define NQ_ERR_HIP 5         /* a HIP runtime call failed */
#define NQ_ERR_UNSUPPORTED 6

/* weight formats */
#define NQ_FMT_Q4_0 0        /* the reference's format: groups of 32 along IN,
                                18-byte blocks [fp16 d][16 B nibbles], value
                                (q-8)*d  (noeira/nn/quant/q4_0.mojo:1-8) */
#define NQ_FMT_W8_CHANNEL 1  /* int8 [OUT, IN] + fp32 scale per output channel */
#define NQ_FMT_W4_GROUP 2    /* uint4, 2 per byte (low nibble = even k), fp16
                                scale and uint4 zero-point per group along IN */
#define NQ_FMT_FP8_E4M3 3    /* OCP e4m3fn [OUT, IN] + one fp32 scale */

/* element types of x, y, bias */
#define NQ_DT_F32 0
#define NQ_DT_BF16 1
#define NQ_DT_I8 2        /* x only: int8 codes with a per-row fp32 scale */
#define NQ_DT_FP8_E4M3 3  /* x only: e4m3fn codes with one fp32 scale */
#define NQ_DT_I32 4       /* y only: raw int32 accumulators (W8 x I8) */

/* nq_create flags */
#define NQ_FLAG_NO_TILE_COPY 1 /* a layer of 4 M weights and more (Q4_0, W4_GROUP with groups of 128,
                                  W8_CHANNEL) normally keeps a second copy of its codes on the device, ordered
                                  for the matrix cores 16 rows at a time, which its single-row calls with
                                  bf16 / fp32 activations stream 1.2 .. 1.5 times faster than the row-ordered
                                  codes; 4-bit layers with 512 <= IN <= 6144 keep it too, for calls with a
                                  hundred activation rows and more over wide layers; this flag saves that memory
                                  (0.5 or 1 byte per weight) */
#define NQ_FLAG_PREFER_TILE 2  /* take the kernels that read the tile-ordered copy wherever they apply (4-bit layers:
                                  2 .. 512 activation rows, any width; int8 layers: 2 .. 16 rows up to IN = 4096),
                                  not only where they were measured to win: for tuning on other shapes, and for
                                  tests that walk every instantiation */

/* epilogues (LinearAct's, noeira/nn/primitives/linear_act.mojo:81-115) */
#define NQ_EPI_NONE 0
#define NQ_EPI_RELU 1     /* z > 0 ? z : 0  (ops/relu_op.mojo:29-31) */
#define NQ_EPI_SWIGLU 2   /* layers made by nq_fuse_glu only: up * silu(gate)  (primitives/swiglu.mojo:41-60) */

typedef struct nq_layer* nq_handle;

/* ---- library ----------------------------------------------------------- */

/* NQ_ABI_VERSION of the loaded library ("APPEND ONLY" tables are an ABI in
 * the reference: noeira/io/serial/native.mojo LAYOUT_N). */
int32_t nq_abi_version(void);

/* Copies the calling thread's last error sentence (NUL-terminated, truncated
 * to n) and returns its full length.  Stands in for the Mojo `Error` a
 * QLinear method raises (qlinear.mojo:276-281,334-338,358-369). */
int64_t nq_last_error(char* buf, int64_t n);

/* ---- layer lifecycle ---------------------------------------------------- */

/* `QLinear[IN, OUT].make` (qlinear.mojo:253-260): an empty layer.  `group` is
 * 32 for NQ_FMT_Q4_0 (IN % 32 == 0 is required, qlinear.mojo:243-245), the
 * group width for NQ_FMT_W4_GROUP, ignored otherwise.  flags: 0 or an OR of NQ_FLAG_*. */
int32_t nq_create(nq_handle* out, int32_t format, int32_t in_features, int32_t out_features,
                  int32_t group, int32_t flags);

/* Frees the layer's device and host storage. */
int32_t nq_destroy(nq_handle h);

/* `QLinear.set_blocks` (qlinear.mojo:271-320): load Q4_0 blocks
 * [OUT, IN/32*18] from the host.  nbytes must equal OUT*(IN/32)*18, otherwise
 * NQ_ERR_SIZE "... bytes, expected ...".  The bytes are copied (host copy kept
 * for nq_get_blocks), uploaded, and re-laid-out on the device once; the call
 * returns after the upload has completed. */
int32_t nq_set_blocks(nq_handle h, const uint8_t* blocks_host, int64_t nbytes, void* stream);

/* `QLinear.set_weight` (qlinear.mojo:264-269): round-to-nearest quantisation
 * of an fp32 [OUT, IN] weight on the Q4_0 grid (q4_0.mojo:98-154), run on the
 * device, then loaded as by nq_set_blocks.  n_values must be OUT*IN. */
int32_t nq_set_weight_f32(nq_handle h, const float* w_host, int64_t n_values, void* stream);

/* NQ_FMT_W8_CHANNEL: int8 weight [OUT, IN] and fp32 scales [OUT]. */
int32_t nq_set_weight_i8(nq_handle h, const int8_t* w_host, const float* scales_host, void* stream);

/* NQ_FMT_W4_GROUP: codes [OUT, IN/2], fp16 scale bits [OUT, G], packed uint4
 * zero-points [OUT, ceil(G/2)] (low nibble = even group), G = ceil(IN/group). */
int32_t nq_set_weight_w4g(nq_handle h, const uint8_t* codes_host, const uint16_t* scales_f16_host,
                          const uint8_t* zps_host, void* stream);

/* NQ_FMT_FP8_E4M3: e4m3fn codes [OUT, IN] and the per-tensor scale. */
int32_t nq_set_weight_fp8(nq_handle h, const uint8_t* w_host, float scale, void* stream);

/* Bytes of the logical weight (`QLinear.BYTES`, qlinear.mojo:216-217, for
 * Q4_0; the codes' byte count for the other formats). */
int64_t nq_blocks_bytes(nq_handle h);

/* `QLinear.blocks()` (qlinear.mojo:322-324): the Q4_0 blocks back, byte for
 * byte.  NQ_ERR_NOT_LOADED / NQ_ERR_NO_BLOCKS as `_need_blocks` (:358-369). */
int32_t nq_get_blocks(nq_handle h, uint8_t* out_host, int64_t nbytes);

/* `QLinear.keep_only_repacked` (qlinear.mojo:342-356): drop the host copy of
 * the logical blocks; only the device layout the forward reads is kept. */
int32_t nq_keep_only_repacked(nq_handle h);

/* Device memory the layer's weights occupy, in bytes: codes, scales, zero points and every copy of them in another
 * order that a kernel reads (no counterpart in the reference, whose `keep_only_repacked` documents the one-copy rule,
 * qlinear.mojo:342-356; this is how a caller checks it).  0 for an unloaded layer or a null handle.  Q4_0: 0.5625
 * bytes per weight; a 4-bit layer at least 2048 columns wide (or made with NQ_FLAG_PREFER_TILE) and a layer of 4 M
 * weights and more keep a second, tile-ordered copy of their codes unless made with NQ_FLAG_NO_TILE_COPY: 1.06 bytes
 * per weight, 1.16 where IN = 960 pads to 1024 in tile order (int8: 2.0). */
int64_t nq_device_bytes(nq_handle h);

/* ---- compute ------------------------------------------------------------ */

/* `QLinear.forward` (qlinear.mojo:407-477) generalised to the formats above
 * and to `LinearAct`'s bias/activation epilogue:
 *     y[M, OUT] = epi( x[M, IN] @ deq(W)^T  (+ bias[OUT]) )
 * x_dtype: F32 or BF16 for Q4_0 / W8_CHANNEL / W4_GROUP; I8 for W8_CHANNEL
 * (x_scale = fp32 [M], one per row); FP8_E4M3 for FP8_E4M3 weights
 * (x_scale = fp32 [1]).  x_scale is NULL otherwise.
 * y_dtype: F32 or BF16; I32 with x_dtype I8 returns the raw accumulators
 * (no scale, bias or epilogue).  bias may be NULL; bias_dtype F32 or BF16.
 * The dequantised weight is never materialised.
 * Non-finite activations: products and sums follow IEEE, with one exception.
 * A single F32 / BF16 row (M = 1) over W8_CHANNEL weights of 4 M codes and
 * more, or over 4-bit weights (Q4_0, W4_GROUP with groups of 128) of so many
 * rows that every workgroup on the chip gets three tiles of 16 (OUT >= 24576
 * up to IN = 4096, >= 12288 up to 8192; any such layer with
 * NQ_FLAG_PREFER_TILE), is split into int8 terms under the largest magnitude
 * of the row (or of a slice of it; error <= 6e-8 of that magnitude per
 * element); if the row holds a NaN or an infinity, every output of the call
 * is NaN before the epilogue.  The epilogue NQ_EPI_RELU is z > 0 ? z : 0 in every kernel: a NaN
 * pre-activation becomes 0 and -0.0 becomes +0.0 (ops/relu_op.mojo:29-31). */
int32_t nq_forward(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale, void* y,
                   int32_t y_dtype, int32_t M, const void* bias, int32_t bias_dtype,
                   int32_t epilogue, void* stream);

/* One layer made of the rows of up to four loaded layers that share their
 * input (same format, IN, group width; FP8_E4M3: same scale), e.g. q|k|v or
 * gate|up of a decoder layer: the seven projections the reference's caller
 * launches one by one (`DecoderLayerWeights.proj_fwd`,
 * noeira/deep_agents/smolvla/layer_weights.mojo:455-508, called from
 * fused.mojo:287-363) read the same activations three and two at a time.  The
 * weights are copied on the device ([OUT, IN] rows are independent, groups
 * never span rows), so the sources may be destroyed afterwards.  The result
 * is an ordinary layer (nq_forward writes one [M, sum OUT] y) that also
 * remembers its parts for nq_forward_fused. */
int32_t nq_fuse_rows(nq_handle* out, const nq_handle* layers, int32_t n, void* stream);

/* gate | up of a decoder MLP and the SwiGLU between them and `down`, as ONE layer: the reference's caller runs
 * two projections, a concatenation and `SwiGLU.forward` (noeira/deep_agents/smolvla/fused.mojo:337-353:
 * `proj_fwd[LORA_GATE]`, `proj_fwd[LORA_UP]`, `glu_cat`, `glu`; out = up * silu(gate), silu(v) = v / (1 + exp(-v)),
 * noeira/nn/primitives/swiglu.mojo:41-60).  The two loaded layers (same format, IN, OUT, group width; Q4_0,
 * W4_GROUP or W8_CHANNEL) are copied on the device with their rows interleaved, so the sources may be destroyed.
 * The result runs with nq_forward(..., epilogue = NQ_EPI_SWIGLU) only and writes y[M, OUT]: x fp32 or bf16,
 * y fp32 or bf16, no bias; one launch for M = 1 and for M >= 2.  nq_get_blocks and nq_fuse_rows refuse it. */
int32_t nq_fuse_glu(nq_handle* out, nq_handle gate, nq_handle up, void* stream);

/* Number of parts of a layer made by nq_fuse_rows (1 for any other layer). */
int32_t nq_fused_parts(nq_handle h);

/* nq_forward of a fused layer with one dense output per part:
 * ys[t] is [M, OUT_t], what nq_forward of part t alone would write: a row's
 * arithmetic does not depend on its neighbours (bit for bit at 2 <= M < 512;
 * at M = 1 the number of lanes that share a row, and from 512 rows on the
 * kernel, hence the order of a row's sum, may follow the total row count).
 * n_ys must equal nq_fused_parts(h).  bias, if any, is [sum OUT].  One launch
 * where the kernel for the shape can place rows by part (bf16/fp32
 * activations at any M; at 17 .. 511 rows only where all parts take the same
 * kernel on their own), otherwise one launch per part. */
int32_t nq_forward_fused(nq_handle h, const void* x, int32_t x_dtype, const float* x_scale,
                         void* const* ys, int32_t n_ys, int32_t y_dtype, int32_t M, const void* bias,
                         int32_t bias_dtype, int32_t epilogue, void* stream);

/* The device twin of `dequantize_q4_0` (`dequant_q4_0_kernel`,
 * q4_0.mojo:242-266; `QLinear.dequantized`, qlinear.mojo:326-328): deq(W)
 * [OUT, IN] fp32 into out_dev (n_values >= OUT*IN else NQ_ERR_SIZE, the
 * `share_scratch` rule of qlinear.mojo:330-340), or, with out_dev = NULL and
 * n_values = 0, into the workspace shared by nq_set_workspace.  Any format. */
int32_t nq_dequantize(nq_handle h, float* out_dev, int64_t n_values, void* stream);

/* `QLinear.share_scratch` (qlinear.mojo:330-340): the caller's buffer takes the place of the layer's own dequantize
 * scratch; every layer of a model can share one, they run one at a time.  nq_workspace_bytes: the bytes that scratch
 * holds, 4 * OUT * IN, whatever M (no forward of this library dequantizes to memory, so none reads or writes the
 * workspace; M is taken for callers written against a forward that does); 0 for a null handle.  nq_set_workspace:
 * NQ_ERR_SIZE with share_scratch's sentence if nbytes is smaller, NQ_ERR_INVALID for a null or misaligned buffer;
 * (NULL, 0) takes the workspace away again.  The buffer stays the caller's: the library neither frees nor outlives it. */
int64_t nq_workspace_bytes(nq_handle h, int32_t M);
int32_t nq_set_workspace(nq_handle h, void* dev, int64_t nbytes);

/* `QLinear.vjp` (qlinear.mojo:479-518): gx[M, IN] = gy[M, OUT] @ deq(W),
 * fp32 in and out, overwriting gx.  Q4_0 only. */
int32_t nq_grad_input(nq_handle h, const float* gy, float* gx, int32_t M, void* stream);

/* Per-row (token) absmax int8 quantisation of activations [M, K]:
 *     s[m] = absmax(x[m,:]) / 127 (1 where 0);  q = clip(rhe(x / s), -127, 127)
 * divide and ties-to-even, as the RTN grid insists (q4_0.mojo:30-32).
 * x_dtype F32 or BF16. */
int32_t nq_quantize_rows_i8(const void* x, int32_t x_dtype, int8_t* q, float* scales, int32_t M,
                            int32_t K, void* stream);

/* `_cast_pad_kernel` (qlinear.mojo:152-172): fp32 [rows, cols] -> bf16
 * [rows, cols_pad] with a zero tail. */
int32_t nq_cast_pad_bf16(const float* src, uint16_t* dst, int32_t rows, int32_t cols,
                         int32_t cols_pad, void* stream);

/* `_slice_cast_kernel` (qlinear.mojo:175-192): bf16 [rows, cols_pad] -> fp32
 * [rows, cols]. */
int32_t nq_slice_cast_f32(const uint16_t* src, float* dst, int32_t rows, int32_t cols,
                          int32_t cols_pad, void* stream);

/* Three W8_CHANNEL layers run as one launch for batched-env actor inference
 * (SAC/PPO actor MLP; `LinearAct` chain): per token
 *     h1 = relu(L1(q8(x))), h2 = relu(L2(q8(h1))), y = L3(q8(h2)) (+ relu if
 *     final_epilogue), q8 = nq_quantize_rows_i8's rule, int32 accumulation.
 * x fp32 [M, IN1], y fp32 [M, OUT3]; b1..b3 fp32 or NULL.  The layers'
 * shapes must chain (OUT1 == IN2, OUT2 == IN3), IN <= 256, OUT <= 256. */
int32_t nq_mlp3_w8a8_forward(nq_handle l1, nq_handle l2, nq_handle l3, const float* x, float* y,
                             int32_t M, const float* b1, const float* b2, const float* b3,
                             int32_t final_epilogue, void* stream);

/* A frozen LoRA adapter's share, added into the base layer's output right after its forward:
 *     y[T, OUT] += scale * (x[T, IN] @ A[IN, R_PAD]) @ B[R_PAD, OUT]
 * `LoRAAdapter.forward_add` (noeira/nn/peft/lora.mojo:292-349).  a, b: the adapter's device
 * parameters (`lora_A.val`, `lora_B.val`: fp32 row-major, rank-padded with zeros); scale:
 * `LoRAAdapter.scale()` (alpha / R, or alpha / sqrt(R)); x: the base layer's own input, fp32 or
 * bf16; y: its fp32 output.  One launch, no scratch; a merged adapter simply does not call it. */
int32_t nq_lora_forward_add(const float* a, const float* b, int32_t in_features, int32_t out_features,
                            int32_t r_pad, float scale, const void* x, int32_t x_dtype, float* y, int32_t T,
                            void* stream);

/* The base layer's forward and a frozen adapter's share in one call:
 *     y[M, OUT] = x @ deq(W)^T + bias + scale * (x @ A[IN, R_PAD]) @ B[R_PAD, OUT]
 * i.e. `QLinear.forward` followed by `LoRAAdapter.forward_add` (noeira/nn/peft/lora.mojo:292-349; the pair
 * `QLoRALinear.forward` makes, tests/nn/quant/qlora_common.mojo).  Where the base call runs on the kernel that keeps
 * its rows' activations resident (4-bit layers with 512 <= IN <= 4096 whose split of K leaves a wavefront at most two
 * steps of 128: IN <= 1280, 1537..2048 and 3073..4096; fp32 activations: IN <= 2048 - at 2..512 rows when made with
 * NQ_FLAG_PREFER_TILE, else 17 .. 511 rows over layers at least 2048 wide, wherever nq_forward itself takes that
 * kernel: where its estimated time is the lower one, e.g. 960 -> 2560 at 135 rows; R_PAD <= 16)
 * the adapter is folded into that launch: h = x A is formed once per 16 rows from the activations the workgroup
 * already holds, and s * h B is added before the store; y may then be fp32 or bf16.  Elsewhere it is nq_forward
 * followed by nq_lora_forward_add (y fp32).  Either way B = 0 returns the bits of nq_forward on the same arguments. */
int32_t nq_forward_lora(nq_handle h, const void* x, int32_t x_dtype, void* y, int32_t y_dtype, int32_t M,
                        const void* bias, int32_t bias_dtype, const float* lora_a, const float* lora_b, int32_t r_pad,
                        float scale, void* stream);

/* One frozen adapter of a fused call: the device parameters and scale nq_lora_forward_add takes; a = b = NULL: the
 * part has none (the caller's `Optional` adapter slots, noeira/deep_agents/smolvla/layer_weights.mojo:713-739). */
typedef struct nq_lora_part {
    const float* a;   /* [IN, R_PAD] fp32 */
    const float* b;   /* [R_PAD, OUT_t] fp32 */
    int32_t r_pad;
    float scale;
} nq_lora_part;

/* nq_forward_fused of a layer made by nq_fuse_rows, with one adapter per part: what the reference's caller does per
 * projection - `proj_fwd` = base linear, then `LoRAAdapter.forward_add` (layer_weights.mojo:455-508; q | k | v and
 * gate | up read the same activations, fused.mojo:287-363) - as two launches for the whole group:
 *     ys[t][M, OUT_t] = x @ deq(W_t)^T + bias_t + scale_t * (x @ A_t) @ B_t        (fp32)
 * the base call of nq_forward_fused, then ONE launch that adds every part's share (R_PAD = 16, IN a multiple of 32,
 * OUT_t multiples of 4 and 16-byte aligned operands; otherwise one adding launch per part).  B_t = 0, or no adapter,
 * leaves the bits of nq_forward_fused.  x fp32 or bf16; adapters[n_ys].
 * glu_out != NULL: the layer's two parts are gate and up of one MLP (equal widths, no bias).  The adding launch then
 * also writes glu_out[M, OUT] = up * silu(gate) (`SwiGLU.forward`, noeira/nn/primitives/swiglu.mojo:41-60; fp32 or
 * bf16 by glu_dtype) from the sums it formed, and ys[0], ys[1] keep the base projections: they are scratch the caller
 * lends.
 * A layer made by nq_fuse_glu (gate and up interleaved, SwiGLU in the kernel's epilogue) takes the call too, as ONE
 * launch: adapters[0] is the gate projection's, adapters[1] the up projection's, both present with one R_PAD <= 16 (or
 * both absent), glu_out [M, OUT / 2] is the only output and ys is not read.  Both shares enter the accumulators ahead
 * of the activation, which only the kernel for 17 .. 511 rows over rows of at most 4096 codes can do: other shapes
 * return NQ_ERR_UNSUPPORTED before anything is launched (fuse gate and up with nq_fuse_rows then).  B = 0 on both
 * leaves the bits of nq_forward on that layer wherever nq_forward takes the same kernel (by default from a few tens
 * of rows on). */
int32_t nq_forward_fused_lora(nq_handle h, const void* x, int32_t x_dtype, float* const* ys, int32_t n_ys, int32_t M,
                              const void* bias, int32_t bias_dtype, const nq_lora_part* adapters, void* glu_out,
                              int32_t glu_dtype, void* stream);

/* ---- GPTQ onto the Q4_0 grid (load time; noeira/nn/quant/gptq.mojo) ------------------------ */

/* The calibration Hessian of one linear's inputs, H = sum x x^T in fp64, kept on the device:
 * `HessianAccumulator` (noeira/nn/quant/hessian.mojo:24-77). */
typedef struct nq_hessian_s* nq_hessian;

/* An all-zero [n, n] Hessian (hessian.mojo:34-37). */
int32_t nq_hessian_create(nq_hessian* out, int32_t n);
int32_t nq_hessian_destroy(nq_hessian h);

/* H += X^T X over the first `rows` rows of the device slab x [rows, n] (fp32 or bf16), the rows
 * added in ascending order: `HessianAccumulator.add` (hessian.mojo:41-77) without the download. */
int32_t nq_hessian_add(nq_hessian h, const void* x, int32_t x_dtype, int32_t rows, void* stream);

/* Rows added so far (`HessianAccumulator.rows`). */
int64_t nq_hessian_rows(nq_hessian h);

/* Copy H out to / in from host memory ([n, n] fp64 row-major; `count` must be n * n).  `set` also
 * sets the row count (a Hessian computed elsewhere, e.g. read from a fixture). */
int32_t nq_hessian_get(nq_hessian h, double* out_host, int64_t count);
int32_t nq_hessian_set(nq_hessian h, const double* h_host, int64_t count, int64_t rows);

/* U, upper triangular with U^T U = h^-1, for h symmetric positive definite ([n, n] fp64 on the
 * host, not modified), computed on the device: `hinv_upper_f64` (noeira/nn/quant/dense.mojo:355-363).
 * Fails with NQ_ERR_INVALID and the pivot's index when h is not positive definite
 * (dense.mojo:229-236). */
int32_t nq_hinv_upper_f64(const double* h_host, int32_t n, double* u_host, void* stream);

/* nq_hinv_upper_f64 for callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  h_dev and u_dev are [n, n] fp64
 * on the device (h_dev is not modified), pivot_dev a device int32 that is set to INT32_MAX, or to the index of
 * the first non-positive pivot (of the index-reversed matrix) when h is not positive definite, in which case
 * u_dev holds no result.  The call only enqueues on `stream`: it allocates nothing, frees nothing and does not
 * synchronise; its working copy of h lives in a fixed device array of the library, which limits n to 1024
 * (NQ_ERR_SIZE beyond) and is shared by every call on the same GPU: calls that overlap on one GPU race. */
int32_t nq_hinv_upper_f64_dev(const double* h_dev, int32_t n, double* u_dev, int32_t* pivot_dev, void* stream);

/* `gptq_q4_0` (noeira/nn/quant/gptq.mojo:62-150) followed by `pack_q4_0` and the upload: quantizes
 * the host fp32 weight w [OUT, IN] of a Q4_0 layer column by column against the Hessian of the
 * layer's inputs (not modified), and loads the layer with the result, as nq_set_weight_f32 does
 * with round-to-nearest.  damp_frac: the damping as a fraction of mean(diag H) (the reference's
 * default is 0.01).  dead_out / damp_out (may be NULL): `GPTQStats`. */
int32_t nq_set_weight_gptq(nq_handle h, const float* w_host, int64_t n_values, nq_hessian hess,
                           double damp_frac, int64_t* dead_out, double* damp_out, void* stream);

/* `q4_0_objective` (gptq.mojo:152-189): tr((W - What) H (W - What)^T) in fp64 for the layer's
 * current weights What against the host fp32 weight w [OUT, IN] they were quantized from. */
int32_t nq_q4_0_objective(nq_handle h, const float* w_host, int64_t n_values, nq_hessian hess,
                          double* out, void* stream);

/* (The measurement helpers bench.py uses - the matrix cores alone, a plain read, a GEMM call's timeline, a forward
 * under a given tile shape - are declared in noeira_qlinear_diag.h: a caller of the operator needs none of them, and
 * none of them changes what any other call does.) */

#ifdef __cplusplus
}
#endif
#endif /* NOEIRA_QLINEAR_H */
