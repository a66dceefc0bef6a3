// Activation-side helpers: per-row absmax int8 quantisation, and the two cast
// kernels of the reference's NVIDIA forward.
#include "nq_common.h"

namespace nq {

namespace {

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {
    // round to nearest even, NaN -> 0x7FC0 (noeira/io/safetensors.mojo:578-588)
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ float4 load4(const void* x, int x_dtype, int64_t idx4) {
    if (x_dtype == NQ_DT_F32) return reinterpret_cast<const float4*>(x)[idx4];
    uint2 v = reinterpret_cast<const uint2*>(x)[idx4];
    return make_float4(bf16_bits_to_f32(v.x & 0xFFFFu), bf16_bits_to_f32(v.x >> 16),
                       bf16_bits_to_f32(v.y & 0xFFFFu), bf16_bits_to_f32(v.y >> 16));
}

__device__ __forceinline__ int q8(float x, float s) {
    float t = rintf(__fdiv_rn(x, s));  // a true division, ties to even
    t = t > -127.0f ? t : -127.0f;
    t = t < 127.0f ? t : 127.0f;
    return (int)t;
}

// One wavefront per row: s = absmax / 127 (1 where 0), q = clip(rhe(x / s)).
__global__ __launch_bounds__(256) void quantize_rows_i8_kernel(const void* __restrict__ x, int x_dtype,
                                                               int8_t* __restrict__ q,
                                                               float* __restrict__ scales, int M, int K) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const int n4 = K / 4;
    const int64_t base4 = (int64_t)row * n4;
    float amax = 0.0f;
    for (int i = lane; i < n4; i += 64) {
        float4 v = load4(x, x_dtype, base4 + i);
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));
    float s = amax / 127.0f;
    if (s == 0.0f) s = 1.0f;
    if (lane == 0) scales[row] = s;
    uint32_t* dst = reinterpret_cast<uint32_t*>(q) + base4;
    for (int i = lane; i < n4; i += 64) {
        float4 v = load4(x, x_dtype, base4 + i);
        uint32_t packed = ((uint32_t)q8(v.x, s) & 0xFFu) | (((uint32_t)q8(v.y, s) & 0xFFu) << 8) |
                          (((uint32_t)q8(v.z, s) & 0xFFu) << 16) | (((uint32_t)q8(v.w, s) & 0xFFu) << 24);
        dst[i] = packed;
    }
}

// fp32 [rows, cols] -> bf16 [rows, cols_pad], zero tail (qlinear.mojo:152-172)
__global__ __launch_bounds__(256) void cast_pad_kernel(const float* __restrict__ src,
                                                       uint16_t* __restrict__ dst, int64_t rows, int cols,
                                                       int cols_pad) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * cols_pad) return;
    int64_t r = i / cols_pad;
    int c = (int)(i % cols_pad);
    dst[i] = c < cols ? f32_to_bf16_bits(src[r * cols + c]) : (uint16_t)0;
}

// bf16 [rows, cols_pad] -> fp32 [rows, cols] (qlinear.mojo:175-192)
__global__ __launch_bounds__(256) void slice_cast_kernel(const uint16_t* __restrict__ src,
                                                         float* __restrict__ dst, int64_t rows, int cols,
                                                         int cols_pad) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * cols) return;
    int64_t r = i / cols;
    int c = (int)(i % cols);
    dst[i] = bf16_bits_to_f32(src[r * cols_pad + c]);
}

}  // namespace

int32_t launch_quantize_rows_i8(const void* x, int32_t x_dtype, int8_t* q, float* scales, int32_t M,
                                int32_t K, hipStream_t s) {
    if (M == 0) return NQ_OK;
    hipLaunchKernelGGL(quantize_rows_i8_kernel, dim3((M + 3) / 4), dim3(256), 0, s, x, x_dtype, q, scales, M, K);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

int32_t launch_cast_pad_bf16(const float* src, uint16_t* dst, int32_t rows, int32_t cols, int32_t cols_pad,
                             hipStream_t s) {
    int64_t n = (int64_t)rows * cols_pad;
    if (n == 0) return NQ_OK;
    hipLaunchKernelGGL(cast_pad_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, src, dst,
                       (int64_t)rows, cols, cols_pad);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

int32_t launch_slice_cast_f32(const uint16_t* src, float* dst, int32_t rows, int32_t cols, int32_t cols_pad,
                              hipStream_t s) {
    int64_t n = (int64_t)rows * cols;
    if (n == 0) return NQ_OK;
    hipLaunchKernelGGL(slice_cast_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, src, dst,
                       (int64_t)rows, cols, cols_pad);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace nq
