// A diagnostic, not part of the forward path: what the matrix cores alone sustain on this GPU.
// Every wavefront issues v_mfma back to back on register operands (no memory, no LDS in the loop), 16
// independent accumulators of 32 x 32 as in the 8-bit GEMM's inner loop, one wavefront per SIMD and one
// workgroup per CU.  The operands come from a caller's buffer, so the caller chooses what the multipliers
// see (constant bytes, random e4m3 codes ...): on data that toggles them the chip runs at its power limit and
// the clock, hence the rate, drops.  The kernel stamps the shader clock and the constant 100 MHz clock
// around its loop, from which the effective shader clock follows.
#include <type_traits>

#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(16))) int i32x16;

// KIND 0: v_mfma_f32_32x32x64_f8f6f4 (e4m3 x e4m3), 1: v_mfma_i32_32x32x32_i8
template <int KIND>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void mfma_rate_kernel(const int* __restrict__ seed, int seed_words, int iters, int64_t* __restrict__ stamps, float* sink) {
    // four A fragments and four B fragments per wavefront, as one k-step of the GEMM's 4 x 4 register tile
    i32x8 a[4], b[4];
#pragma unroll
    for (int o = 0; o < 4; o++)
#pragma unroll
        for (int i = 0; i < 8; i++) {
            a[o][i] = seed[(threadIdx.x * 8 + i + 2048 * o) % seed_words];
            b[o][i] = seed[(threadIdx.x * 8 + i + 2048 * o + 1024) % seed_words];
        }
    typedef typename std::conditional<KIND == 0, f32x16, i32x16>::type acc_t;
    acc_t acc[16];
#pragma unroll
    for (int j = 0; j < 16; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[j][r] = 0;
    const int64_t c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            if constexpr (KIND == 0)
                acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[j % 4], a[j / 4], acc[j], 0, 0, 0, 0, 0, 0);
            else
                acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8((i32x4){b[j % 4][0], b[j % 4][1], b[j % 4][2], b[j % 4][3]},
                                                               (i32x4){a[j / 4][0], a[j / 4][1], a[j / 4][2], a[j / 4][3]},
                                                               acc[j], 0, 0, 0);
        }
    }
    const int64_t c1 = clock64(), w1 = wall_clock64();
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; j++) s += (float)acc[j][0];
    if (s == 12345.678f) sink[0] = s;  // (keeps the accumulators alive)
    if (threadIdx.x == 0) stamps[2 * blockIdx.x] = c1 - c0, stamps[2 * blockIdx.x + 1] = w1 - w0;
}

// The same yardstick for the 16 x 16 shapes: KIND 2: v_mfma_f32_16x16x128_f8f6f4, 3: v_mfma_i32_16x16x64_i8.  Eight A and
// eight B fragments per wavefront (a 128 x 128 register tile as 8 x 8 results of 16 x 16): 64 MFMAs per iteration, twice
// the operations of the 32 x 32 kernels' 16.
typedef __attribute__((ext_vector_type(4))) float f32x4;
template <int KIND>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void mfma16_rate_kernel(const int* __restrict__ seed, int seed_words, int iters, int64_t* __restrict__ stamps, float* sink) {
    i32x8 a[8], b[8];
#pragma unroll
    for (int o = 0; o < 8; o++)
#pragma unroll
        for (int i = 0; i < 8; i++) {
            a[o][i] = seed[(threadIdx.x * 8 + i + 2048 * o) % seed_words];
            b[o][i] = seed[(threadIdx.x * 8 + i + 2048 * o + 1024) % seed_words];
        }
    typedef typename std::conditional<KIND == 2, f32x4, i32x4>::type acc_t;
    acc_t acc[64];
#pragma unroll
    for (int j = 0; j < 64; j++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[j][r] = 0;
    const int64_t c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int j = 0; j < 64; j++) {
            if constexpr (KIND == 2)
                acc[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[j % 8], a[j / 8], acc[j], 0, 0, 0, 0, 0, 0);
            else
                acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8((i32x4){b[j % 8][0], b[j % 8][1], b[j % 8][2], b[j % 8][3]},
                                                               (i32x4){a[j / 8][0], a[j / 8][1], a[j / 8][2], a[j / 8][3]},
                                                               acc[j], 0, 0, 0);
        }
    }
    const int64_t c1 = clock64(), w1 = wall_clock64();
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 64; j++) s += (float)acc[j][0];
    if (s == 12345.678f) sink[0] = s;  // (keeps the accumulators alive)
    if (threadIdx.x == 0) stamps[2 * blockIdx.x] = c1 - c0, stamps[2 * blockIdx.x + 1] = w1 - w0;
}

// A second yardstick: a kernel that only READS `kib` KiB (one 1 KiB load instruction per wavefront and KiB, four
// in flight per wavefront, eight wavefronts per workgroup) and computes nothing.  What it takes for the bytes
// of a GEMV's weight is the floor of that GEMV on this GPU: launch + the stream.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
// (written only: `used` and a volatile store keep the compiler from deleting it, and with it the loads)
__device__ __attribute__((used)) uint32_t g_read_sink;
// `never`: a value the XOR of the data is not expected to take, from the host, so that the compiler must keep the loads
__global__ __launch_bounds__(512) void stream_read_kernel(const u32x4* __restrict__ src, int64_t kib, uint32_t never) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t b0 = ((int64_t)blockIdx.x * 8 + wave) * 4;
    u32x4 v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = __builtin_nontemporal_load(src + min(b0 + j, kib - 1) * 64 + lane);
    uint32_t x = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) x ^= v[j][0] ^ v[j][1] ^ v[j][2] ^ v[j][3];
    if (x == never) *(volatile uint32_t*)&g_read_sink = x;
}

}  // namespace

int32_t launch_stream_read(const void* src, int64_t kib, hipStream_t s) {
    hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)((kib + 31) / 32)), dim3(512), 0, s,
                       reinterpret_cast<const u32x4*>(src), kib, 0x9E3779B9u);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

int32_t launch_mfma_rate(int kind, const int* seed, int seed_words, int iters, int blocks, int64_t* stamps, float* sink,
                         hipStream_t s) {
    if (kind == 2)
        hipLaunchKernelGGL(mfma16_rate_kernel<2>, dim3(blocks), dim3(256), 0, s, seed, seed_words, iters, stamps, sink);
    else if (kind == 3)
        hipLaunchKernelGGL(mfma16_rate_kernel<3>, dim3(blocks), dim3(256), 0, s, seed, seed_words, iters, stamps, sink);
    else if (kind == 0)
        hipLaunchKernelGGL(mfma_rate_kernel<0>, dim3(blocks), dim3(256), 0, s, seed, seed_words, iters, stamps, sink);
    else
        hipLaunchKernelGGL(mfma_rate_kernel<1>, dim3(blocks), dim3(256), 0, s, seed, seed_words, iters, stamps, sink);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace nq
