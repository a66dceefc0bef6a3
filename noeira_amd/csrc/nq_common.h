// Internal declarations shared by the translation units of libnoeira_qlinear.so.
// Nothing here crosses the C ABI (include/noeira_qlinear.h does).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/noeira_qlinear.h"
#include "../../include/noeira_qlinear_diag.h"

namespace nq {

constexpr int Q4_GROUP = 32;  // weights per Q4_0 group (noeira/nn/quant/q4_0.mojo:49)
constexpr int Q4_BLOCK = 18;  // bytes per Q4_0 block   (noeira/nn/quant/q4_0.mojo:51)
constexpr int CHUNK = 16;     // bytes one lane loads per weight fetch (128-bit)

// Sets the calling thread's error sentence and returns `code`.
int32_t fail(int32_t code, const std::string& msg);
int32_t fail_hip(hipError_t e, const char* what);

#define NQ_HIP(expr)                                        \
    do {                                                    \
        hipError_t _e = (expr);                             \
        if (_e != hipSuccess) return nq::fail_hip(_e, #expr); \
    } while (0)

// nq_diag.hip: the matrix cores' own rate (a diagnostic)
int32_t launch_stream_read(const void* src, int64_t kib, hipStream_t s);
int32_t launch_mfma_rate(int kind, const int* seed, int seed_words, int iters, int blocks, int64_t* stamps, float* sink,
                         hipStream_t s);

// hipFuncAttributeMaxDynamicSharedMemorySize is a per-device setting of a kernel: set once per (kernel, device)
struct LdsAttrOnce {
    bool done[64] = {};
};
hipError_t set_max_lds_once(LdsAttrOnce& st, const void* kernel, size_t bytes);

}  // namespace nq

// One quantized linear layer.  Device layouts (all row-major over OUT):
//   Q4_0        codes  [OUT][G][16 B]   the nibble bytes of each block, so that
//                                        every group is one aligned 128-bit load
//               scales [OUT][G] fp16    the block scales, split off the blocks
//   W8_CHANNEL  codes  [OUT][IN] int8,  scales [OUT] fp32
//   W4_GROUP    codes  [OUT][IN/2]      (low nibble = even k)
//               scales [OUT][G] fp16,   zps [OUT][G] uint8 (unpacked)
//   FP8_E4M3    codes  [OUT][IN],       scale = one fp32
struct nq_layer {
    int32_t format = 0;
    int32_t in = 0;
    int32_t out = 0;
    int32_t group = 0;
    int32_t groups = 0;        // G = ceil(IN / group) for the grouped formats
    bool loaded = false;
    bool has_host_blocks = false;
    std::vector<uint8_t> host_blocks;  // logical bytes as handed to set_* (Q4_0: the blocks)
    int device = -1;
    uint8_t* d_codes = nullptr;
    void* d_scales = nullptr;
    uint8_t* d_zps = nullptr;
    // W8_CHANNEL layers of at most 256 x 256: a second copy of the codes as MFMA operand tiles for the fused MLP
    // (tile (j, s) = rows 16 j .., k = 64 s .. is 1 KiB, lane l's 16 bytes at 16 l; zeros beyond OUT and IN)
    uint8_t* d_tiled = nullptr;
    int64_t tiled_bytes = 0;
    // large layers (nq_gemv_tile.hip): a second copy of the codes in the matrix core's operand order for 16 rows
    // at a time, and (4-bit) of the group records in the same order; tile_nj = steps of K per row tile
    uint8_t* d_tile16 = nullptr;
    void* d_tile16_scales = nullptr;
    float* workspace = nullptr;     // caller-owned dequantize scratch (nq_set_workspace), never read by a forward
    int64_t workspace_bytes = 0;
    int32_t tile_nj = 0;
    bool no_tile_copy = false;  // NQ_FLAG_NO_TILE_COPY
    bool prefer_tile = false;   // NQ_FLAG_PREFER_TILE
    float scale = 1.0f;
    int64_t row_bytes = 0;     // bytes of one row of d_codes
    std::vector<int32_t> seg_end;  // a row-fused layer: the end row of each fused part (else empty)
    // nq_fuse_glu: rows 2 n and 2 n + 1 are row n of the gate and of the up projection; the forward writes
    // [M, OUT / 2] = up * silu(gate) (epilogue NQ_EPI_SWIGLU) and nothing else
    bool glu = false;
};

namespace nq {

// Where the rows of a launch go: part t covers rows [end[t-1], end[t]) and is written dense to
// y[t] as [M, end[t] - end[t-1]].  An ordinary layer is one part.
struct SegTable {
    int32_t nseg;
    int32_t end[4];
    void* y[4];
};

// `SwiGLU`'s forward as the reference writes it (noeira/nn/primitives/swiglu.mojo:41-60): s = 1 / (1 + exp(-v)),
// out = u * (v * s), with u the up projection and v the gate, in fp32.
__device__ __forceinline__ float swiglu_f32(float up, float gate) {
    const float sg = 1.0f / (1.0f + expf(-gate));
    return up * (gate * sg);
}

// the value the neighbouring lane (lane ^ 1) holds: in the matrix core's result layout adjacent lanes are adjacent
// output columns, i.e. the gate and the up row of one pair
__device__ __forceinline__ float lane_xor1(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false));
}

// row n -> (part's y, its width, the column in it).  Every table entry is read with a constant index, so the
// table stays in scalar registers (a run-time index would turn into a load from the argument buffer, a round
// trip to memory at the end of the kernel).
__device__ __forceinline__ void seg_lookup(const SegTable& sg, int n, void*& y, int& width, int& col) {
    int base = 0, end = sg.end[0];
    void* yy = sg.y[0];
#pragma unroll
    for (int t = 0; t < 3; t++)
        if (t + 1 < sg.nseg && n >= sg.end[t]) base = sg.end[t], end = sg.end[t + 1], yy = sg.y[t + 1];
    y = yy, width = end - base, col = n - base;
}

struct ForwardArgs {
    const nq_layer* L;
    const void* x;
    int32_t x_dtype;
    const float* x_scale;
    void* y;
    int32_t y_dtype;
    int32_t M;
    const void* bias;
    int32_t bias_dtype;
    int32_t epilogue;
    hipStream_t stream;
    SegTable seg;  // seg.y[0] == y and seg.end[0] == OUT for an ordinary call
    // nq_forward_lora: the adapter folded into the launch (only the M-tile kernel reads these)
    const float* lora_a = nullptr;
    const float* lora_b = nullptr;
    int32_t lora_r = 0;
    float lora_s = 0.0f;
    const float* lora_a2 = nullptr;  // a gate | up layer's second adapter (the up projection's; lora_a / lora_b: the gate's)
    const float* lora_b2 = nullptr;
    float lora_s2 = 0.0f;
    // nq_diag_gemm8_timeline: where the large-tile GEMM writes its per-tile clock readings (null: none)
    unsigned long long* diag_stamps = nullptr;
    int diag_gemm8_waves = 0;  // 0: the library's choice; 4 / 8: the 256 x 256 tile GEMM with that many wavefronts; 12: its 128 x 256 tile form
    // nq_diag_forward_a16: the 16-row tile kernel's shape for this launch, mw << 4 | nw (0: the library's choice)
    int32_t diag_a16_shape = 0;
};

// nq_q4_0.hip
int32_t launch_q4_0_repack(const uint8_t* raw_dev, uint8_t* codes, uint16_t* scales, int64_t nblocks,
                           hipStream_t s);
int32_t launch_q4_0_rtn(const float* w_dev, uint8_t* blocks_dev, int64_t n, int64_t k, hipStream_t s);
int32_t launch_dequantize(const nq_layer* L, float* out, hipStream_t s);
int32_t launch_grad_input_q4_0(const nq_layer* L, const float* gy, float* gx, int32_t M, hipStream_t s);
int32_t launch_w4g_unpack_zps(const uint8_t* packed, uint8_t* out, int64_t rows, int64_t groups,
                              hipStream_t s);

int32_t launch_w4g_repack(uint8_t* codes, int64_t nchunks, hipStream_t s);

// nq_gemm_a16.hip: medium-M dequant GEMM on the bf16 matrix cores
bool gemm_a16_applicable(const ForwardArgs& a);
int32_t launch_gemm_a16(const ForwardArgs& a);
// the medium-M kernel's tile shape for a call (M >= 2, below the many-rows kernel's range) and its estimated time
float gemm_a16_estimate_us(int32_t format, bool xf32, int M, int N, int K, int* mw_out, int* nw_out);
// ... the lower of that and the many-rows kernel's estimate (from 256 rows on)
float gemm_a16_best_estimate_us(int32_t format, bool xf32, int M, int N, int K);
// a row-fused layer of 256 .. 511 rows whose parts differ in which of the two kernels they take: part by part
bool gemm_a16_splits_parts(const ForwardArgs& a);

// nq_gemv.hip: dequant-GEMV for small M (also the any-M fallback)
int32_t launch_gemv(const ForwardArgs& a);
int32_t launch_gemv_i8(const ForwardArgs& a);

// nq_gemv_m1.hip: register-resident GEMV for a single activation row
bool gemv_m1_applicable(const ForwardArgs& a);
int32_t launch_gemv_m1(const ForwardArgs& a);

// nq_gemv_row4.hip: 4-bit GEMV for one activation row over a large weight, on the bf16 matrix cores
bool gemv_row4_applicable(const ForwardArgs& a);
int32_t launch_gemv_row4(const ForwardArgs& a);

// nq_gemv_row8.hip: 8-bit GEMV for one bf16 / fp32 activation row over a large weight, x staged in LDS
bool gemv_row8_applicable(const ForwardArgs& a);
int32_t launch_gemv_row8(const ForwardArgs& a);

// nq_gemv_split.hip: int8 weights under one bf16 / fp32 row, x split into int8 terms for the int8 matrix cores
bool gemv_split8_applicable(const ForwardArgs& a);
int32_t launch_gemv_split8(const ForwardArgs& a);

// nq_gemv_tile.hip: one bf16 / fp32 row over a large 4-bit or int8 weight, from the tile-ordered copy of the codes
bool tile_copy_wanted(const nq_layer* L);
int32_t build_tile_copy(nq_layer* L, hipStream_t s);
bool gemv_tile_applicable(const ForwardArgs& a);
bool gemv_tile_rows_applicable(const ForwardArgs& a);
bool gemv_tile8_rows_applicable(const ForwardArgs& a);
int32_t launch_gemv_tile8_rows(const ForwardArgs& a);
bool gemm_tile_mt_applicable(const ForwardArgs& a);
bool gemm_tile_mt_splits_parts(const ForwardArgs& a);
bool gemm_tile_mt_lora_foldable(const ForwardArgs& a);
bool gemm_tile_mt_takes_shape(const ForwardArgs& a);
int32_t launch_gemm_tile_mt(const ForwardArgs& a);
int32_t launch_gemv_tile_rows(const ForwardArgs& a);
int32_t launch_gemv_tile(const ForwardArgs& a);

// nq_gemv_fp8.hip: fp8 x fp8 and int8 x int8 on the matrix cores for one row (fp8) and for as many
// activation rows as the large-tile GEMM would leave most of the chip idle with
bool gemv_fp8_applicable(const ForwardArgs& a);
int32_t launch_gemv_fp8(const ForwardArgs& a);
bool tile8_i8_applicable(const ForwardArgs& a);
int32_t launch_tile8_i8(const ForwardArgs& a);

// nq_gemm8.hip: LDS-tiled fp8 / int8 MFMA GEMM for large M
double gemm8_estimate_us(int M, int N, int K, bool i8);  // what launch_gemm8 is expected to take, on the tile form it picks
bool gemm8_applicable(const ForwardArgs& a);
int32_t launch_gemm8(const ForwardArgs& a);

// nq_mlp.hip: three W8A8 layers in one launch
int32_t launch_mlp3_w8a8(const nq_layer* l1, const nq_layer* l2, const nq_layer* l3, const float* x, float* y,
                         int32_t M, const float* b1, const float* b2, const float* b3, int32_t final_relu,
                         hipStream_t s);

// nq_quant.hip
int32_t launch_quantize_rows_i8(const void* x, int32_t x_dtype, int8_t* q, float* scales, int32_t M,
                                int32_t K, hipStream_t s);
int32_t launch_cast_pad_bf16(const float* src, uint16_t* dst, int32_t rows, int32_t cols,
                             int32_t cols_pad, hipStream_t s);
int32_t launch_slice_cast_f32(const uint16_t* src, float* dst, int32_t rows, int32_t cols,
                              int32_t cols_pad, hipStream_t s);

// nq_lora.hip: y += s (x A) B
int32_t launch_lora_add(const void* x, int32_t x_dtype, const float* A, const float* B, float* y, int32_t T, int32_t IN,
                        int32_t OUT, int32_t R, float s, hipStream_t stream);
// the adapters of a row-fused layer's parts, added into the parts' fp32 outputs in one launch (b null: the part has
// none); glu_out non-null: two parts of equal width, gate and up - their sums go through SwiGLU into glu_out
struct LoraPartArgs {
    const float* a;
    const float* b;
    float* y;
    int32_t out;
    int32_t r;
    float s;
};
int32_t launch_lora_multi(const void* x, int32_t x_dtype, int32_t T, int32_t IN, int32_t n, const LoraPartArgs* parts, void* glu_out,
                          int32_t glu_dtype, hipStream_t stream);

// nq_gptq.hip: the calibration Hessian, the factor of its inverse, GPTQ's column loop, its objective
int32_t launch_hessian_add(double* H, int n, const void* x, int32_t x_dtype, int rows, hipStream_t s);
int32_t launch_hinv_upper_f64(double* h, int n, double* u, int* status_dev, hipStream_t s);
int32_t run_hinv_upper_f64_dev(const double* h_dev, int n, double* u_dev, int* pivot_dev, hipStream_t s);
int32_t hinv_dev_max_n();
void hinv_dev_setup();
int32_t run_gptq_q4_0(float* w_dev, int64_t n, int k, double* h_dev, double damp_frac, uint8_t* blocks_dev,
                      double* stats_host, hipStream_t s);
int32_t run_q4_0_objective(const float* w_dev, const float* deq_dev, int64_t n, int k, const double* h_dev,
                           double* out_host, hipStream_t s);

// nq_diag.hip: the matrix cores' own rate (a diagnostic)
int32_t launch_stream_read(const void* src, int64_t kib, hipStream_t s);
int32_t launch_mfma_rate(int kind, const int* seed, int seed_words, int iters, int blocks, int64_t* stamps, float* sink,
                         hipStream_t s);

}  // namespace nq
