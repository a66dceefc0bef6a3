// Dequant-GEMV: y[M, N] = epi(x[M, K] @ deq(W)^T + bias) for small M.
//
// HBM-bound: the packed weights are streamed exactly once with 128-bit loads,
// dequantised in registers and reduced across lanes; deq(W) is never written.
// (The reference's AMD path writes deq(W) as fp32 and reads it back,
// noeira/nn/quant/qlinear.mojo:464-477: 8.5 B per weight against 0.5625 here.)
//
// Work split.  A row of W is `nch` chunks of 16 bytes (32 four-bit or 16
// eight-bit weights).  `lpr` consecutive lanes (a power of two) share a row:
// lane j of the group takes chunks j, j+lpr, ...  so a group's loads are
// contiguous.  Each lane group walks RPL rows at once (RPL independent loads
// in flight, one read of x shared by the RPL rows) and RI such row sets in
// sequence.  x is staged once per block into LDS as fp32, quad-interleaved
// (all first float4s of every chunk, then all second ones, ...) so that lanes
// holding consecutive chunks read consecutive 16-byte words: conflict free.
//
// Zero points are folded out of the inner loop: with xsum[c] the sum of x over
// chunk c, sum_k x_k (q_k - z) = sum_k x_k q_k - z * xsum[c].
//
// Reductions run in a fixed order (per lane over chunks, then a butterfly over
// the lane group), so a repeated call returns identical bits
// (tests/nn/quant/test_qlinear_gpu.mojo:96,128).
#include <hip/hip_fp16.h>

#include <algorithm>

#include "nq_common.h"

namespace nq {

namespace {

struct GemvParams {
    const uint8_t* codes;
    const void* scales;
    const uint8_t* zps;
    const void* x;
    const float* x_scale;
    void* y;
    const void* bias;
    int32_t M, N, K;
    int32_t group, groups;
    float tscale;
    int32_t nch;       // chunks per row
    int32_t lpr;       // lanes per row (power of two, <= 64)
    int32_t ri;        // row sets per lane group
    int32_t psq;       // LDS plane stride in float4s
    int32_t x_dtype, y_dtype, bias_dtype, epilogue;
};

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

// four consecutive activations of row m starting at element 4*f, as fp32
__device__ __forceinline__ float4 load_x4(const void* x, int x_dtype, int64_t row_off, int f) {
    if (x_dtype == NQ_DT_F32) {
        return reinterpret_cast<const float4*>(reinterpret_cast<const float*>(x) + row_off)[f];
    } else if (x_dtype == NQ_DT_BF16) {
        uint2 v = reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(x) + row_off)[f];
        return make_float4(bf16_to_f32(v.x & 0xFFFFu), bf16_to_f32(v.x >> 16), bf16_to_f32(v.y & 0xFFFFu),
                           bf16_to_f32(v.y >> 16));
    } else {  // NQ_DT_FP8_E4M3
        uint32_t v = reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(x) + row_off)[f];
        f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)v, false);
        f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)v, true);
        return make_float4(lo[0], lo[1], hi[0], hi[1]);
    }
}

__device__ __forceinline__ float dot4(float4 a, float b0, float b1, float b2, float b3, float acc) {
    acc = fmaf(a.x, b0, acc);
    acc = fmaf(a.y, b1, acc);
    acc = fmaf(a.z, b2, acc);
    acc = fmaf(a.w, b3, acc);
    return acc;
}

__device__ __forceinline__ float ub0(uint32_t t) { return (float)(t & 0xFFu); }
__device__ __forceinline__ float ub1(uint32_t t) { return (float)((t >> 8) & 0xFFu); }
__device__ __forceinline__ float ub2(uint32_t t) { return (float)((t >> 16) & 0xFFu); }
__device__ __forceinline__ float ub3(uint32_t t) { return (float)(t >> 24); }

template <int FMT, int MT, int RPL>
__global__ __launch_bounds__(256) void gemv_kernel(const GemvParams p) {
    constexpr bool FOUR_BIT = (FMT == NQ_FMT_Q4_0 || FMT == NQ_FMT_W4_GROUP);
    constexpr int EPC = FOUR_BIT ? 32 : 16;  // weights per 16-byte chunk
    constexpr int QPC = EPC / 4;             // float4s of x per chunk
    constexpr bool HAS_ZP = (FMT != NQ_FMT_FP8_E4M3);

    extern __shared__ float4 smem[];
    float4* xs = smem;                                                    // [MT][QPC][psq]
    float* xsum = reinterpret_cast<float*>(smem + MT * QPC * p.psq);      // [MT][nch]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * MT;

    // ---- row assignment and the first weight fetch, issued before staging x
    const int lpr = p.lpr;
    const int rg_per_wave = 64 / lpr;
    const int rg = lane / lpr, lj = lane % lpr;
    const int set_rows = 4 * rg_per_wave * RPL;  // rows one pass of the block covers
    const int64_t block_row0 = (int64_t)blockIdx.x * set_rows * p.ri;

    // ---- stage x (rows m0 .. m0+MT-1, zero beyond M) into LDS, fp32, quad-interleaved
    const int nf4 = p.K / 4;
    for (int m = 0; m < MT; m++) {
        const bool live = (m0 + m) < p.M;
        for (int f0 = 0; f0 < nf4; f0 += 256) {
            const int f = f0 + tid;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (live && f < nf4) v = load_x4(p.x, p.x_dtype, (int64_t)(m0 + m) * p.K, f);
            if (HAS_ZP) {
                float s = (v.x + v.y) + (v.z + v.w);
                s += __shfl_xor(s, 1);
                s += __shfl_xor(s, 2);
                if (QPC == 8) s += __shfl_xor(s, 4);
                if (f < nf4 && (f % QPC) == 0) xsum[m * p.nch + f / QPC] = s;
            }
            if (f < nf4) xs[(m * QPC + (f % QPC)) * p.psq + f / QPC] = v;
        }
    }
    __syncthreads();

    const u32x4* wq = reinterpret_cast<const u32x4*>(p.codes);

    for (int it = 0; it < p.ri; it++) {
        const int64_t row0 = block_row0 + (int64_t)it * set_rows + (int64_t)(wave * rg_per_wave + rg) * RPL;
        if (row0 >= p.N) break;  // uniform per lane group; later sets are further out
        int64_t rows[RPL];
#pragma unroll
        for (int r = 0; r < RPL; r++) rows[r] = min(row0 + r, (int64_t)p.N - 1);

        // the epilogue's operands are requested before the K loop, not after the reduction
        float ep_scale[RPL], ep_bias[RPL];
#pragma unroll
        for (int r = 0; r < RPL; r++) {
            ep_scale[r] = 1.0f, ep_bias[r] = 0.0f;
            if (FMT == NQ_FMT_W8_CHANNEL) ep_scale[r] = reinterpret_cast<const float*>(p.scales)[rows[r]];
            if (FMT == NQ_FMT_FP8_E4M3) ep_scale[r] = p.tscale * (p.x_scale ? p.x_scale[0] : 1.0f);
            if (p.bias)
                ep_bias[r] = (p.bias_dtype == NQ_DT_F32)
                                 ? reinterpret_cast<const float*>(p.bias)[rows[r]]
                                 : bf16_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[rows[r]]);
        }
        float acc[RPL][MT];
#pragma unroll
        for (int r = 0; r < RPL; r++)
#pragma unroll
            for (int m = 0; m < MT; m++) acc[r][m] = 0.0f;

        for (int c = lj; c < p.nch; c += lpr) {
            u32x4 wv[RPL];
#pragma unroll
            for (int r = 0; r < RPL; r++) wv[r] = __builtin_nontemporal_load(&wq[rows[r] * p.nch + c]);

            float cs[RPL], cz[RPL];
#pragma unroll
            for (int r = 0; r < RPL; r++) {
                if (FMT == NQ_FMT_Q4_0) {
                    cs[r] = __half2float(__ushort_as_half(
                        reinterpret_cast<const uint16_t*>(p.scales)[rows[r] * p.nch + c]));
                    cz[r] = 8.0f;
                } else if (FMT == NQ_FMT_W4_GROUP) {
                    const int g = (c * EPC) / p.group;
                    cs[r] = __half2float(__ushort_as_half(
                        reinterpret_cast<const uint16_t*>(p.scales)[rows[r] * p.groups + g]));
                    cz[r] = (float)p.zps[rows[r] * p.groups + g];
                } else {
                    cs[r] = 1.0f;
                    cz[r] = 128.0f;  // W8: codes are biased to unsigned below
                }
            }

            float dot[RPL][MT];
#pragma unroll
            for (int r = 0; r < RPL; r++)
#pragma unroll
                for (int m = 0; m < MT; m++) dot[r][m] = 0.0f;

#pragma unroll
            for (int jw = 0; jw < 4; jw++) {
                // the x quads this 32-bit word of codes multiplies
                float4 xa[MT], xb[MT];
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    if (FOUR_BIT) {                    // word jw: elements 8jw .. 8jw+7
                        xa[m] = xs[(m * QPC + 2 * jw) * p.psq + c];
                        xb[m] = xs[(m * QPC + 2 * jw + 1) * p.psq + c];
                    } else {                           // word jw: elements 4jw .. 4jw+3
                        xa[m] = xs[(m * QPC + jw) * p.psq + c];
                    }
                }
#pragma unroll
                for (int r = 0; r < RPL; r++) {
                    const uint32_t word = wv[r][jw];
                    if (FOUR_BIT) {
                        // device nibble order (nq_nib.h): low nibbles of the four bytes are elements
                        // 0, 4, 1, 5; high nibbles are elements 2, 6, 3, 7
                        const uint32_t lo = word & 0x0F0F0F0Fu, hi = (word >> 4) & 0x0F0F0F0Fu;
                        const float e0 = ub0(lo), e4 = ub1(lo), e1 = ub2(lo), e5 = ub3(lo);
                        const float e2 = ub0(hi), e6 = ub1(hi), e3 = ub2(hi), e7 = ub3(hi);
#pragma unroll
                        for (int m = 0; m < MT; m++) {
                            dot[r][m] = dot4(xa[m], e0, e1, e2, e3, dot[r][m]);
                            dot[r][m] = dot4(xb[m], e4, e5, e6, e7, dot[r][m]);
                        }
                    } else if (FMT == NQ_FMT_W8_CHANNEL) {
                        const uint32_t t = word ^ 0x80808080u;  // int8 + 128 as unsigned bytes
                        const float b0 = ub0(t), b1 = ub1(t), b2 = ub2(t), b3 = ub3(t);
#pragma unroll
                        for (int m = 0; m < MT; m++) dot[r][m] = dot4(xa[m], b0, b1, b2, b3, dot[r][m]);
                    } else {
                        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)word, false);
                        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)word, true);
#pragma unroll
                        for (int m = 0; m < MT; m++) dot[r][m] = dot4(xa[m], a[0], a[1], b[0], b[1], dot[r][m]);
                    }
                }
            }
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const float xsm = HAS_ZP ? xsum[m * p.nch + c] : 0.0f;
#pragma unroll
                for (int r = 0; r < RPL; r++) {
                    if (FMT == NQ_FMT_FP8_E4M3)
                        acc[r][m] += dot[r][m];
                    else if (FMT == NQ_FMT_W8_CHANNEL)
                        acc[r][m] += fmaf(-cz[r], xsm, dot[r][m]);
                    else
                        acc[r][m] = fmaf(cs[r], fmaf(-cz[r], xsm, dot[r][m]), acc[r][m]);
                }
            }
        }

        // ---- butterfly over the lane group, then the epilogue on its first lane
#pragma unroll
        for (int r = 0; r < RPL; r++)
#pragma unroll
            for (int m = 0; m < MT; m++) {
                float v = acc[r][m];
                for (int off = lpr >> 1; off > 0; off >>= 1) v += __shfl_xor(v, off);
                acc[r][m] = v;
            }
        if (lj == 0) {
#pragma unroll
            for (int r = 0; r < RPL; r++) {
                const int64_t n = row0 + r;
                if (n >= p.N) continue;
                const float rs = ep_scale[r], b = ep_bias[r];
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    if (m0 + m >= p.M) continue;
                    float z = acc[r][m];
                    if (FMT == NQ_FMT_W8_CHANNEL || FMT == NQ_FMT_FP8_E4M3) z *= rs;
                    if (p.bias) z += b;
                    if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
                    const int64_t o = (int64_t)(m0 + m) * p.N + n;
                    if (p.y_dtype == NQ_DT_F32)
                        reinterpret_cast<float*>(p.y)[o] = z;
                    else
                        reinterpret_cast<uint16_t*>(p.y)[o] = f32_to_bf16(z);
                }
            }
        }
    }
}

// int8 activations x int8 weights -> exact int32 accumulators (v_dot4_i32_i8),
// then either the raw accumulators or epi(acc * sx[m] * sw[n] + bias).
template <int MT>
__global__ __launch_bounds__(256) void gemv_i8_kernel(const GemvParams p) {
    extern __shared__ float4 smem[];
    uint4* xs = reinterpret_cast<uint4*>(smem);  // [MT][nch] 16 int8 each
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * MT;
    for (int m = 0; m < MT; m++)
        for (int c = tid; c < p.nch; c += 256) {
            uint4 v = make_uint4(0, 0, 0, 0);
            if (m0 + m < p.M)
                v = reinterpret_cast<const uint4*>(reinterpret_cast<const int8_t*>(p.x) + (int64_t)(m0 + m) * p.K)[c];
            xs[m * p.nch + c] = v;
        }
    __syncthreads();
    const int lpr = p.lpr, rg_per_wave = 64 / lpr, rg = lane / lpr, lj = lane % lpr;
    const int set_rows = 4 * rg_per_wave;
    const uint4* wq = reinterpret_cast<const uint4*>(p.codes);
    for (int it = 0; it < p.ri; it++) {
        const int64_t n = ((int64_t)blockIdx.x * p.ri + it) * set_rows + wave * rg_per_wave + rg;
        if (n >= p.N) break;
        int32_t acc[MT];
#pragma unroll
        for (int m = 0; m < MT; m++) acc[m] = 0;
        for (int c = lj; c < p.nch; c += lpr) {
            const uint4 wv = wq[n * p.nch + c];
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const uint4 xv = xs[m * p.nch + c];
                acc[m] = __builtin_amdgcn_sdot4((int)xv.x, (int)wv.x, acc[m], false);
                acc[m] = __builtin_amdgcn_sdot4((int)xv.y, (int)wv.y, acc[m], false);
                acc[m] = __builtin_amdgcn_sdot4((int)xv.z, (int)wv.z, acc[m], false);
                acc[m] = __builtin_amdgcn_sdot4((int)xv.w, (int)wv.w, acc[m], false);
            }
        }
#pragma unroll
        for (int m = 0; m < MT; m++)
            for (int off = lpr >> 1; off > 0; off >>= 1) acc[m] += __shfl_xor(acc[m], off);
        if (lj == 0) {
            const float sw = reinterpret_cast<const float*>(p.scales)[n];
            float b = 0.0f;
            if (p.bias)
                b = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const float*>(p.bias)[n]
                                                : bf16_to_f32(reinterpret_cast<const uint16_t*>(p.bias)[n]);
#pragma unroll
            for (int m = 0; m < MT; m++) {
                if (m0 + m >= p.M) continue;
                const int64_t o = (int64_t)(m0 + m) * p.N + n;
                if (p.y_dtype == NQ_DT_I32) {
                    reinterpret_cast<int32_t*>(p.y)[o] = acc[m];
                    continue;
                }
                float z = (float)acc[m] * (p.x_scale[m0 + m] * sw);
                if (p.bias) z += b;
                if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(p.y)[o] = z;
                else
                    reinterpret_cast<uint16_t*>(p.y)[o] = f32_to_bf16(z);
            }
        }
    }
}

// lanes per row: the power of two that wastes the fewest lane slots, larger
// (more rows in flight per byte) on ties broken towards more parallel waves.
void choose_split(int nch, int N, int rpl_max, int* lpr_out, int* rpl_out, int* ri_out) {
    int best_lpr = 64, best_rpl = 1;
    long best_cost = -1;
    for (int lpr = 64; lpr >= 1; lpr >>= 1) {
        if (lpr > 1 && lpr / 2 >= nch) continue;  // a smaller group already covers the row
        for (int rpl = rpl_max; rpl >= 1; rpl >>= 1) {
            const long iters = (nch + lpr - 1) / lpr;
            const long rows_per_wave = (64 / lpr) * rpl;
            const long waves = (N + rows_per_wave - 1) / rows_per_wave;
            const long rounds = (waves + 2047) / 2048;  // 256 CUs x 8 resident waves
            const long cost = rounds * iters * rpl;
            if (best_cost < 0 || cost < best_cost) {
                best_cost = cost, best_lpr = lpr, best_rpl = rpl;
            }
        }
    }
    *lpr_out = best_lpr;
    *rpl_out = best_rpl;
    // several row sets per block amortise the staging of x when the matrix is large
    const long rows_per_set = 4L * (64 / best_lpr) * best_rpl;
    long sets = (N + rows_per_set - 1) / rows_per_set;
    int ri = 1;
    while (ri < 8 && sets / (ri * 2) >= 1024) ri *= 2;
    *ri_out = ri;
}

template <int FMT, int MT>
int32_t launch_gemv_rpl(const GemvParams& p, int rpl, dim3 grid, size_t lds, hipStream_t s) {
    switch (rpl) {
        case 1: hipLaunchKernelGGL((gemv_kernel<FMT, MT, 1>), grid, dim3(256), lds, s, p); break;
        case 2: hipLaunchKernelGGL((gemv_kernel<FMT, MT, 2>), grid, dim3(256), lds, s, p); break;
        default: hipLaunchKernelGGL((gemv_kernel<FMT, MT, 4>), grid, dim3(256), lds, s, p); break;
    }
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

template <int FMT>
int32_t launch_gemv_fmt(const GemvParams& p, int mt, int rpl, dim3 grid, size_t lds, hipStream_t s) {
    switch (mt) {
        case 1: return launch_gemv_rpl<FMT, 1>(p, rpl, grid, lds, s);
        case 2: return launch_gemv_rpl<FMT, 2>(p, rpl, grid, lds, s);
        default: return launch_gemv_rpl<FMT, 4>(p, rpl, grid, lds, s);
    }
}

}  // namespace

int32_t launch_gemv(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    const bool four_bit = (L->format == NQ_FMT_Q4_0 || L->format == NQ_FMT_W4_GROUP);
    const int epc = four_bit ? 32 : 16;
    GemvParams p{};
    p.codes = L->d_codes, p.scales = L->d_scales, p.zps = L->d_zps;
    p.x = a.x, p.x_scale = a.x_scale, p.y = a.y, p.bias = a.bias;
    p.M = a.M, p.N = L->out, p.K = L->in;
    p.group = L->group, p.groups = L->groups, p.tscale = L->scale;
    p.nch = L->in / epc;
    p.x_dtype = a.x_dtype, p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;

    // x tile held in LDS: MT rows of K fp32 (+ chunk sums), at most 64 KiB
    int mt = a.M >= 4 ? 4 : (a.M >= 2 ? 2 : 1);
    while (mt > 1 && (size_t)mt * L->in * 4 > 48 * 1024) mt >>= 1;
    if ((size_t)L->in * 4 > 60 * 1024)
        return fail(NQ_ERR_UNSUPPORTED, "nq_forward: IN = " + std::to_string(L->in) +
                                            " exceeds the GEMV kernel's LDS tile (15360)");
    int lpr, rpl, ri;
    choose_split(p.nch, p.N, mt == 1 ? 4 : (mt == 2 ? 2 : 2), &lpr, &rpl, &ri);
    p.lpr = lpr, p.ri = ri;
    const int qpc = epc / 4;
    p.psq = p.nch + ((9 - (p.nch % 8)) % 8);  // plane stride = 1 (mod 8) float4s: conflict-free staging
    const size_t lds = (size_t)mt * qpc * p.psq * 16 + (size_t)mt * p.nch * 4;
    const int rows_per_block = 4 * (64 / lpr) * rpl * ri;
    dim3 grid((p.N + rows_per_block - 1) / rows_per_block, (a.M + mt - 1) / mt);
    switch (L->format) {
        case NQ_FMT_Q4_0: return launch_gemv_fmt<NQ_FMT_Q4_0>(p, mt, rpl, grid, lds, a.stream);
        case NQ_FMT_W8_CHANNEL: return launch_gemv_fmt<NQ_FMT_W8_CHANNEL>(p, mt, rpl, grid, lds, a.stream);
        case NQ_FMT_W4_GROUP: return launch_gemv_fmt<NQ_FMT_W4_GROUP>(p, mt, rpl, grid, lds, a.stream);
        case NQ_FMT_FP8_E4M3: return launch_gemv_fmt<NQ_FMT_FP8_E4M3>(p, mt, rpl, grid, lds, a.stream);
    }
    return fail(NQ_ERR_INVALID, "nq_forward: unknown format");
}

int32_t launch_gemv_i8(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    GemvParams p{};
    p.codes = L->d_codes, p.scales = L->d_scales;
    p.x = a.x, p.x_scale = a.x_scale, p.y = a.y, p.bias = a.bias;
    p.M = a.M, p.N = L->out, p.K = L->in;
    p.nch = L->in / 16;
    p.x_dtype = a.x_dtype, p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    int mt = a.M >= 4 ? 4 : (a.M >= 2 ? 2 : 1);
    if ((size_t)L->in > 60 * 1024)
        return fail(NQ_ERR_UNSUPPORTED, "nq_forward: IN exceeds the int8 GEMV kernel's LDS tile");
    while (mt > 1 && (size_t)mt * L->in > 48 * 1024) mt >>= 1;
    int lpr, rpl, ri;
    choose_split(p.nch, p.N, 1, &lpr, &rpl, &ri);
    p.lpr = lpr, p.ri = ri;
    const size_t lds = (size_t)mt * p.nch * 16;
    const int rows_per_block = 4 * (64 / lpr) * ri;
    dim3 grid((p.N + rows_per_block - 1) / rows_per_block, (a.M + mt - 1) / mt);
    switch (mt) {
        case 1: hipLaunchKernelGGL(gemv_i8_kernel<1>, grid, dim3(256), lds, a.stream, p); break;
        case 2: hipLaunchKernelGGL(gemv_i8_kernel<2>, grid, dim3(256), lds, a.stream, p); break;
        default: hipLaunchKernelGGL(gemv_i8_kernel<4>, grid, dim3(256), lds, a.stream, p); break;
    }
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace nq
