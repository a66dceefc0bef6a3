// Load-time and auxiliary kernels: Q4_0 block split, device RTN quantiser,
// dequantise-to-fp32 for every format, and Q4_0 grad_input.
#include <hip/hip_fp16.h>

#include "nq_common.h"
#include "nq_nib.h"

namespace nq {

// ---------------------------------------------------------------------------
// Q4_0 blocks [nblocks][18] -> device chunks [nblocks][16] + fp16 scale bits.
// The 18-byte block is only 2-byte aligned; splitting the scale off makes each
// group one aligned 128-bit load for the forward kernels, and the nibbles are
// re-ordered from the block's split-half order (byte j = element j | element
// j+16 << 4) to the device order of nq_nib.h.  Scale bytes are moved, never
// reinterpreted, so NaN/inf/subnormal scales survive unchanged.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void q4_0_repack_kernel(const uint8_t* __restrict__ raw,
                                                          uint8_t* __restrict__ codes,
                                                          uint16_t* __restrict__ scales,
                                                          int64_t nblocks) {
    int64_t b = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) return;
    const uint16_t* src = reinterpret_cast<const uint16_t*>(raw + b * Q4_BLOCK);  // 2-byte aligned
    uint16_t h[9];
#pragma unroll
    for (int i = 0; i < 9; i++) h[i] = src[i];
    scales[b] = h[0];
    uint8_t e[Q4_GROUP];
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const uint8_t byte = (uint8_t)(h[1 + (j >> 1)] >> (8 * (j & 1)));
        e[j] = byte & 0xF;
        e[j + 16] = byte >> 4;
    }
    uint4 v;
    v.x = nib_pack8(e), v.y = nib_pack8(e + 8), v.z = nib_pack8(e + 16), v.w = nib_pack8(e + 24);
    reinterpret_cast<uint4*>(codes)[b] = v;
}

int32_t launch_q4_0_repack(const uint8_t* raw_dev, uint8_t* codes, uint16_t* scales, int64_t nblocks,
                           hipStream_t s) {
    if (nblocks == 0) return NQ_OK;
    dim3 grid((unsigned)((nblocks + 255) / 256));
    hipLaunchKernelGGL(q4_0_repack_kernel, grid, dim3(256), 0, s, raw_dev, codes, scales, nblocks);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// ---------------------------------------------------------------------------
// Round-to-nearest on the Q4_0 grid, one thread per group of 32
// (noeira/nn/quant/q4_0.mojo:97-154):
//   d = (FIRST element of largest magnitude) / -8;  1e-8 where that is 0;
//   d rounded to bf16 (ties to even, NaN -> 0x7FC0: io/safetensors.mojo:578);
//   q = clip(round_half_even(w / d) + 8, 0, 15) with a true division;
//   stored scale = fp16(d), round to nearest even.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bf16_round_dev(float x) {
    uint32_t bits = __float_as_uint(x);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return __uint_as_float(0x7FC00000u);
    uint32_t bias = 0x7FFFu + ((bits >> 16) & 1u);
    return __uint_as_float((bits + bias) & 0xFFFF0000u);
}

__global__ __launch_bounds__(256) void q4_0_rtn_kernel(const float* __restrict__ w,
                                                       uint8_t* __restrict__ blocks,
                                                       int64_t ngroups) {
    int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= ngroups) return;
    const float4* src = reinterpret_cast<const float4*>(w + g * Q4_GROUP);
    float v[Q4_GROUP];
#pragma unroll
    for (int i = 0; i < Q4_GROUP / 4; i++) {
        float4 t = src[i];
        v[4 * i] = t.x, v[4 * i + 1] = t.y, v[4 * i + 2] = t.z, v[4 * i + 3] = t.w;
    }
    float best = v[0];
    float best_abs = fabsf(v[0]);
#pragma unroll
    for (int j = 1; j < Q4_GROUP; j++) {
        float a = fabsf(v[j]);
        if (a > best_abs) {
            best_abs = a;
            best = v[j];
        }
    }
    float d = best / -8.0f;  // exact: a power-of-two divisor
    if (d == 0.0f) d = 1e-8f;
    d = bf16_round_dev(d);
    uint8_t q[Q4_GROUP];
#pragma unroll
    for (int j = 0; j < Q4_GROUP; j++) {
        float t = rintf(__fdiv_rn(v[j], d)) + 8.0f;  // rintf: ties to even
        t = t > 0.0f ? t : 0.0f;
        t = t < 15.0f ? t : 15.0f;
        q[j] = (uint8_t)(int)t;
    }
    uint16_t hb = __half_as_ushort(__float2half_rn(d));
    uint16_t* dst = reinterpret_cast<uint16_t*>(blocks + g * Q4_BLOCK);
    dst[0] = hb;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        uint32_t b0 = q[2 * i] | (q[2 * i + 16] << 4);
        uint32_t b1 = q[2 * i + 1] | (q[2 * i + 17] << 4);
        dst[1 + i] = (uint16_t)(b0 | (b1 << 8));
    }
}

int32_t launch_q4_0_rtn(const float* w_dev, uint8_t* blocks_dev, int64_t n, int64_t k, hipStream_t s) {
    int64_t ngroups = n * (k / Q4_GROUP);
    if (ngroups == 0) return NQ_OK;
    dim3 grid((unsigned)((ngroups + 255) / 256));
    hipLaunchKernelGGL(q4_0_rtn_kernel, grid, dim3(256), 0, s, w_dev, blocks_dev, ngroups);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// packed uint4 zero-points [rows][ceil(G/2)] -> bytes [rows][G]
__global__ __launch_bounds__(256) void w4g_unpack_zps_kernel(const uint8_t* __restrict__ packed,
                                                             uint8_t* __restrict__ out, int64_t rows,
                                                             int64_t groups) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * groups) return;
    int64_t r = i / groups, g = i % groups;
    uint8_t b = packed[r * ((groups + 1) / 2) + g / 2];
    out[i] = (g & 1) ? (b >> 4) : (b & 0xF);
}

int32_t launch_w4g_unpack_zps(const uint8_t* packed, uint8_t* out, int64_t rows, int64_t groups,
                              hipStream_t s) {
    int64_t n = rows * groups;
    if (n == 0) return NQ_OK;
    hipLaunchKernelGGL(w4g_unpack_zps_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                       packed, out, rows, groups);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// W4_GROUP codes, in place: logical bytes (byte i = element 2i | element 2i+1 << 4) -> device order
__global__ __launch_bounds__(256) void w4g_repack_kernel(uint8_t* __restrict__ codes, int64_t nchunks) {
    int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= nchunks) return;
    uint4 v = reinterpret_cast<uint4*>(codes)[c];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint8_t e[32];
#pragma unroll
    for (int j = 0; j < 16; j++) {
        const uint8_t byte = (uint8_t)(w[j >> 2] >> (8 * (j & 3)));
        e[2 * j] = byte & 0xF;
        e[2 * j + 1] = byte >> 4;
    }
    v.x = nib_pack8(e), v.y = nib_pack8(e + 8), v.z = nib_pack8(e + 16), v.w = nib_pack8(e + 24);
    reinterpret_cast<uint4*>(codes)[c] = v;
}

int32_t launch_w4g_repack(uint8_t* codes, int64_t nchunks, hipStream_t s) {
    if (nchunks == 0) return NQ_OK;
    hipLaunchKernelGGL(w4g_repack_kernel, dim3((unsigned)((nchunks + 255) / 256)), dim3(256), 0, s, codes, nchunks);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// ---------------------------------------------------------------------------
// deq(W) [OUT, IN] fp32.  The device twin of dequantize_q4_0
// (`dequant_q4_0_kernel`, q4_0.mojo:242-266), one thread per 128-bit chunk of
// codes (32 four-bit or 16 eight-bit weights), writing whole float4s.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float e4m3_to_f32(uint32_t byte) {
    // OCP e4m3fn decode through the hardware converter (exact).
    typedef __attribute__((ext_vector_type(2))) float f32x2;
    f32x2 p = __builtin_amdgcn_cvt_pk_f32_fp8((int)byte, false);
    return p[0];
}

template <int FMT>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ codes,
                                                         const void* __restrict__ scales,
                                                         const uint8_t* __restrict__ zps,
                                                         float* __restrict__ out, int64_t rows,
                                                         int32_t K, int32_t group, int32_t groups,
                                                         float tscale) {
    constexpr int EPC = (FMT == NQ_FMT_Q4_0 || FMT == NQ_FMT_W4_GROUP) ? 32 : 16;
    const int nch = K / EPC;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * nch) return;
    int64_t r = i / nch;
    int c = (int)(i % nch);
    uint4 v = reinterpret_cast<const uint4*>(codes)[i];
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float* dst = out + r * (int64_t)K + (int64_t)c * EPC;
    float o[EPC];
    if (FMT == NQ_FMT_Q4_0 || FMT == NQ_FMT_W4_GROUP) {
        float d, z;
        if (FMT == NQ_FMT_Q4_0) {
            d = __half2float(__ushort_as_half(reinterpret_cast<const uint16_t*>(scales)[i]));
            z = 8.0f;
        } else {
            const int g = (c * EPC) / group;
            d = __half2float(__ushort_as_half(reinterpret_cast<const uint16_t*>(scales)[r * groups + g]));
            z = (float)zps[r * groups + g];
        }
        float q[EPC];
#pragma unroll
        for (int t = 0; t < 4; t++) nib_unpack8(w[t], q + 8 * t);
#pragma unroll
        for (int j = 0; j < EPC; j++) o[j] = (q[j] - z) * d;
    } else if (FMT == NQ_FMT_W8_CHANNEL) {
        float s = reinterpret_cast<const float*>(scales)[r];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            int8_t q = (int8_t)((w[j >> 2] >> (8 * (j & 3))) & 0xFFu);
            o[j] = (float)q * s;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 16; j++)
            o[j] = e4m3_to_f32((w[j >> 2] >> (8 * (j & 3))) & 0xFFu) * tscale;
    }
#pragma unroll
    for (int j = 0; j < EPC / 4; j++)
        reinterpret_cast<float4*>(dst)[j] = make_float4(o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]);
}

int32_t launch_dequantize(const nq_layer* L, float* out, hipStream_t s) {
    const int epc = (L->format == NQ_FMT_Q4_0 || L->format == NQ_FMT_W4_GROUP) ? 32 : 16;
    int64_t n = (int64_t)L->out * (L->in / epc);
    if (n == 0) return NQ_OK;
    dim3 grid((unsigned)((n + 255) / 256)), block(256);
#define NQ_DEQ(F)                                                                              \
    hipLaunchKernelGGL(dequantize_kernel<F>, grid, block, 0, s, L->d_codes, L->d_scales, L->d_zps, \
                       out, (int64_t)L->out, L->in, L->group, L->groups, L->scale)
    switch (L->format) {
        case NQ_FMT_Q4_0: NQ_DEQ(NQ_FMT_Q4_0); break;
        case NQ_FMT_W8_CHANNEL: NQ_DEQ(NQ_FMT_W8_CHANNEL); break;
        case NQ_FMT_W4_GROUP: NQ_DEQ(NQ_FMT_W4_GROUP); break;
        case NQ_FMT_FP8_E4M3: NQ_DEQ(NQ_FMT_FP8_E4M3); break;
        default: return fail(NQ_ERR_INVALID, "nq_dequantize: unknown format");
    }
#undef NQ_DEQ
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// ---------------------------------------------------------------------------
// grad_input for a Q4_0 layer (QLinear.vjp, qlinear.mojo:479-518):
//   gx[m, i] = sum_o gy[m, o] * deq(W)[o, i]
// One lane owns one group (32 consecutive i) for MT rows of gy; the four waves
// of a block split the OUT rows and are combined through LDS in wave order, so
// the result does not depend on scheduling.
// ---------------------------------------------------------------------------
constexpr int GI_MT = 2;

__global__ __launch_bounds__(256) void grad_input_q4_0_kernel(const uint8_t* __restrict__ codes,
                                                              const uint16_t* __restrict__ scales,
                                                              const float* __restrict__ gy,
                                                              float* __restrict__ gx, int32_t M,
                                                              int32_t K, int32_t N) {
    __shared__ float part[3][GI_MT][64][33];
    const int G = K / Q4_GROUP;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = blockIdx.x * 64 + lane;
    const int m0 = blockIdx.y * GI_MT;
    const bool active = g < G;
    float acc[GI_MT][Q4_GROUP];
#pragma unroll
    for (int m = 0; m < GI_MT; m++)
#pragma unroll
        for (int j = 0; j < Q4_GROUP; j++) acc[m][j] = 0.0f;
    const int rows_per_wave = (N + 3) / 4;
    const int o0 = wave * rows_per_wave;
    const int o1 = min(N, o0 + rows_per_wave);
    if (active) {
        for (int o = o0; o < o1; o++) {
            uint4 v = reinterpret_cast<const uint4*>(codes)[(int64_t)o * G + g];
            float d = __half2float(__ushort_as_half(scales[(int64_t)o * G + g]));
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
            float gv[GI_MT];
#pragma unroll
            for (int m = 0; m < GI_MT; m++) gv[m] = (m0 + m < M) ? gy[(int64_t)(m0 + m) * N + o] : 0.0f;
            float q[Q4_GROUP];
#pragma unroll
            for (int t = 0; t < 4; t++) nib_unpack8(w[t], q + 8 * t);
#pragma unroll
            for (int j = 0; j < Q4_GROUP; j++) {
                const float wv = (q[j] - 8.0f) * d;
#pragma unroll
                for (int m = 0; m < GI_MT; m++) acc[m][j] = fmaf(gv[m], wv, acc[m][j]);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int m = 0; m < GI_MT; m++)
#pragma unroll
            for (int j = 0; j < Q4_GROUP; j++) part[wave - 1][m][lane][j] = acc[m][j];
    }
    __syncthreads();
    if (wave == 0 && active) {
#pragma unroll
        for (int m = 0; m < GI_MT; m++) {
            if (m0 + m >= M) continue;
            float* dst = gx + (int64_t)(m0 + m) * K + (int64_t)g * Q4_GROUP;
#pragma unroll
            for (int j = 0; j < Q4_GROUP; j++) {
                float t = acc[m][j];
                t += part[0][m][lane][j];
                t += part[1][m][lane][j];
                t += part[2][m][lane][j];
                dst[j] = t;
            }
        }
    }
}

int32_t launch_grad_input_q4_0(const nq_layer* L, const float* gy, float* gx, int32_t M, hipStream_t s) {
    if (M == 0) return NQ_OK;
    const int G = L->in / Q4_GROUP;
    dim3 grid((G + 63) / 64, (M + GI_MT - 1) / GI_MT);
    hipLaunchKernelGGL(grad_input_q4_0_kernel, grid, dim3(256), 0, s, L->d_codes,
                       reinterpret_cast<const uint16_t*>(L->d_scales), gy, gx, M, L->in, L->out);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace nq
