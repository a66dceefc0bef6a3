// Medium-M dequant GEMM on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16):
//     y[M, N] = epi( x[M, K] @ deq(W)^T + bias ),  x bf16 or fp32,
//     W in Q4_0, W4_GROUP or W8_CHANNEL codes.
// This is the regime of the reference's real caller, the SmolVLA prefill at
// T = 135 tokens (noeira/deep_agents/smolvla/fused.mojo:255-384), and of
// BASELINE's M = 100 / 256 configs: the weights are ~1 MB, so the call is
// latency- and occupancy-bound, not MFMA-bound.  The kernel therefore has no
// LDS staging and no block-wide barrier in its K loop: every wavefront pulls
// its own operand fragments straight from global memory (x is L2-resident, W
// is read exactly once per M tile) and the only synchronisation is the final
// fixed-order reduction of the four K-slices through LDS.
//
// Exactness.  Weights enter the MFMA as the integer codes, converted to bf16
// exactly: a 4-bit code q becomes 16 + q by OR-ing it into the mantissa of
// bf16 16.0 (one shift and one and-or per pair), an int8 code becomes q + 128.
// The offset is removed in fp32 with X = sum_k x_k, which a second MFMA against
// an all-ones operand provides in the same lane layout:
//     sum_k x_k (q_k - z) = P - (offset + z) X.
// Scales are applied in fp32 after the MFMA, per 32-wide chunk for the 4-bit
// formats (one chunk = one Q4_0 group = one MFMA), once at the end for W8.
// bf16 activations are exact operands; fp32 activations are split into three
// bf16 terms hi + mid + lo that add up to the fp32 value exactly, so every
// product the matrix core forms is exact and only the fp32 accumulation rounds
// (the reference's own AMD path is an fp32 GEMM over deq(W), gate 1e-5).
//
// 4-bit device layout (see nq_q4_0.hip): a 16-byte chunk holds 32 consecutive
// k as four words of eight; lane (n, kb) loads the whole chunk c0 + kb of its
// row with one 128-bit load, and two lane-swap stages (v_permlane32_swap,
// v_permlane16_swap) transpose the 4 x 4 words among the four lanes of a row so
// that lane kb ends up with word kb of chunks c0 .. c0+3: exactly its share of
// the B operand of four MFMAs.
#include <hip/hip_fp16.h>

#include <cstdlib>

#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

struct A16Params {
    const uint8_t* codes;
    const void* scales;
    const uint8_t* zps;
    const void* x;
    void* y;
    const void* bias;
    int32_t M, N, K;
    int32_t group, groups;
    int32_t nch;      // 16-byte chunks per weight row
    int32_t y_dtype, bias_dtype, epilogue;
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// eight 4-bit codes of one word (pair s = elements 2s, 2s+1 in nibbles s and s+4) -> bf16 16+q
__device__ __forceinline__ u32x4 nib_word_to_bf16(uint32_t w) {
    u32x4 r;
    r[0] = ((w << 3) & 0x00780078u) | 0x41804180u;
    r[1] = ((w >> 1) & 0x00780078u) | 0x41804180u;
    r[2] = ((w >> 5) & 0x00780078u) | 0x41804180u;
    r[3] = ((w >> 9) & 0x00780078u) | 0x41804180u;
    return r;
}

// four int8 codes of one word -> two bf16 pairs holding q + 128 (exact)
__device__ __forceinline__ void i8_word_to_bf16(uint32_t w, uint32_t& p0, uint32_t& p1) {
    const uint32_t t = w ^ 0x80808080u;
    const float f0 = (float)(t & 0xFFu), f1 = (float)((t >> 8) & 0xFFu);
    const float f2 = (float)((t >> 16) & 0xFFu), f3 = (float)(t >> 24);
    // values <= 255 have at most 8 significant bits: the high half of the fp32 is the exact bf16
    p0 = (__float_as_uint(f0) >> 16) | (__float_as_uint(f1) & 0xFFFF0000u);
    p1 = (__float_as_uint(f2) >> 16) | (__float_as_uint(f3) & 0xFFFF0000u);
}

// A-operand terms for 8 consecutive activations.  NT = 1 (bf16 input) or 3 (fp32 split).
template <bool XF32>
__device__ __forceinline__ void load_a(const void* x, int64_t elem_off, bool valid, u32x4 (&t)[XF32 ? 3 : 1]) {
    if constexpr (!XF32) {
        t[0] = valid ? *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(x) + elem_off)
                     : (u32x4){0, 0, 0, 0};
    } else {
        float v[8];
        if (valid) {
            const float4 a = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(x) + elem_off)[0];
            const float4 b = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(x) + elem_off)[1];
            v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = 0.0f;
        }
        uint32_t h[8], m[8], l[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            // truncating splits: each residual is exact in fp32, the third term is exact in bf16
            const uint32_t hb = __float_as_uint(v[i]) & 0xFFFF0000u;
            const float r1 = v[i] - __uint_as_float(hb);
            const uint32_t mb = __float_as_uint(r1) & 0xFFFF0000u;
            const float r2 = r1 - __uint_as_float(mb);
            h[i] = hb, m[i] = mb, l[i] = __float_as_uint(r2) & 0xFFFF0000u;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            t[0][i] = (h[2 * i] >> 16) | h[2 * i + 1];
            t[1][i] = (m[2 * i] >> 16) | m[2 * i + 1];
            t[2][i] = (l[2 * i] >> 16) | l[2 * i + 1];
        }
    }
}

template <int FMT, bool XF32, int MW, int NW>
__global__ __launch_bounds__(512) void gemm_a16_kernel(const A16Params p) {
    constexpr bool FOUR_BIT = (FMT != NQ_FMT_W8_CHANNEL);
    constexpr int NT = XF32 ? 3 : 1;
    constexpr int KSTEP = FOUR_BIT ? 128 : 64;  // k covered by one 16-byte weight load per lane x 4 lanes
    constexpr int NMF = FOUR_BIT ? 4 : 2;       // MFMAs (32 k each) per k-step
    constexpr int RED = MW * NW * 4 * 64;       // floats one wavefront contributes to the reduction
    extern __shared__ float red[];              // [KW - 1][RED]
    const int KW = blockDim.x >> 6;             // wavefronts splitting K

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ln = lane & 15, kb = lane >> 4;
    const int n_base = blockIdx.x * (16 * NW);
    const int m_base = blockIdx.y * (16 * MW);

    const u32x4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};

    f32x4 acc[MW][NW];
    f32x4 xacc[MW];  // W8 only: sum_k x_k over the wave's k-steps
#pragma unroll
    for (int i = 0; i < MW; i++) {
        xacc[i] = (f32x4){0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < NW; j++) acc[i][j] = (f32x4){0, 0, 0, 0};
    }

    int64_t xrow[MW];
#pragma unroll
    for (int i = 0; i < MW; i++) xrow[i] = (int64_t)min(m_base + 16 * i + ln, p.M - 1) * p.K;
    int64_t wrow[NW];
    int nrow[NW];
#pragma unroll
    for (int j = 0; j < NW; j++) {
        nrow[j] = min(n_base + 16 * j + ln, p.N - 1);
        wrow[j] = (int64_t)nrow[j] * p.nch;
    }
    const u32x4* wq = reinterpret_cast<const u32x4*>(p.codes);

    // the epilogue's operands are requested up front: nothing is loaded after the reduction
    float ep_scale[NW], ep_bias[NW];
#pragma unroll
    for (int j = 0; j < NW; j++) {
        ep_scale[j] = (FMT == NQ_FMT_W8_CHANNEL) ? reinterpret_cast<const float*>(p.scales)[nrow[j]] : 1.0f;
        ep_bias[j] = 0.0f;
        if (p.bias)
            ep_bias[j] = (p.bias_dtype == NQ_DT_F32)
                             ? reinterpret_cast<const float*>(p.bias)[nrow[j]]
                             : __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[nrow[j]] << 16);
    }

    const int nsteps = (p.K + KSTEP - 1) / KSTEP;
    auto load_w = [&](int ks, u32x4 (&dst)[NW]) {
        const int c = ks * 4 + kb;  // the 16-byte chunk this lane loads
        const bool cvalid = ks < nsteps && c < p.nch;
#pragma unroll
        for (int j = 0; j < NW; j++) dst[j] = cvalid ? wq[wrow[j] + c] : (u32x4){0, 0, 0, 0};
    };
    u32x4 wv[NW], wnext[NW];
    load_w(wave, wv);
    for (int ks = wave; ks < nsteps; ks += KW) {
        load_w(ks + KW, wnext);  // in flight while this k-step is multiplied

        if constexpr (FOUR_BIT) {
            // per-chunk scale and zero point for chunks 4ks .. 4ks+3 of row n (lane's own column)
            float cs[NW][4], cz[NW][4];
#pragma unroll
            for (int j = 0; j < NW; j++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const int cc = ks * 4 + q;
                    if (cc < p.nch) {
                        if (FMT == NQ_FMT_Q4_0) {
                            cs[j][q] = __half2float(__ushort_as_half(
                                reinterpret_cast<const uint16_t*>(p.scales)[(int64_t)nrow[j] * p.nch + cc]));
                            cz[j][q] = 24.0f;  // 16 (conversion offset) + 8 (Q4_0's implicit zero point)
                        } else {
                            const int g = (cc * 32) / p.group;
                            cs[j][q] = __half2float(__ushort_as_half(
                                reinterpret_cast<const uint16_t*>(p.scales)[(int64_t)nrow[j] * p.groups + g]));
                            cz[j][q] = 16.0f + (float)p.zps[(int64_t)nrow[j] * p.groups + g];
                        }
                    } else {
                        cs[j][q] = 0.0f, cz[j][q] = 0.0f;
                    }
                }
            // ---- transpose words among the four lanes (kb = 0..3) that share a row
#pragma unroll
            for (int j = 0; j < NW; j++) {
                auto s02 = __builtin_amdgcn_permlane32_swap(wv[j][0], wv[j][2], false, false);
                auto s13 = __builtin_amdgcn_permlane32_swap(wv[j][1], wv[j][3], false, false);
                wv[j][0] = s02[0], wv[j][2] = s02[1], wv[j][1] = s13[0], wv[j][3] = s13[1];
                auto t01 = __builtin_amdgcn_permlane16_swap(wv[j][0], wv[j][1], false, false);
                auto t23 = __builtin_amdgcn_permlane16_swap(wv[j][2], wv[j][3], false, false);
                wv[j][0] = t01[0], wv[j][1] = t01[1], wv[j][2] = t23[0], wv[j][3] = t23[1];
            }
#pragma unroll
            for (int q = 0; q < NMF; q++) {
                const int k0 = ks * KSTEP + q * 32 + kb * 8;
                const bool kvalid = k0 < p.K;
                u32x4 bop[NW];
#pragma unroll
                for (int j = 0; j < NW; j++) bop[j] = nib_word_to_bf16(wv[j][q]);
#pragma unroll
                for (int i = 0; i < MW; i++) {
                    u32x4 at[NT];
                    load_a<XF32>(p.x, xrow[i] + k0, kvalid, at);
                    f32x4 xs = {0, 0, 0, 0};
#pragma unroll
                    for (int t = 0; t < NT; t++)
                        xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(ones), xs, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < NW; j++) {
                        f32x4 pp = {0, 0, 0, 0};
#pragma unroll
                        for (int t = 0; t < NT; t++)
                            pp = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(bop[j]), pp, 0, 0,
                                                                          0);
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            acc[i][j][r] = fmaf(cs[j][q], fmaf(-cz[j][q], xs[r], pp[r]), acc[i][j][r]);
                    }
                }
            }
        } else {
#pragma unroll
            for (int q = 0; q < NMF; q++) {
                const int k0 = ks * KSTEP + kb * 16 + q * 8;
                const bool kvalid = k0 < p.K;
                u32x4 bop[NW];
#pragma unroll
                for (int j = 0; j < NW; j++) {
                    uint32_t b0, b1, b2, b3;
                    i8_word_to_bf16(wv[j][2 * q], b0, b1);
                    i8_word_to_bf16(wv[j][2 * q + 1], b2, b3);
                    bop[j] = (u32x4){b0, b1, b2, b3};
                }
#pragma unroll
                for (int i = 0; i < MW; i++) {
                    u32x4 at[NT];
                    load_a<XF32>(p.x, xrow[i] + k0, kvalid, at);
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        xacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(ones), xacc[i], 0,
                                                                          0, 0);
#pragma unroll
                        for (int j = 0; j < NW; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(bop[j]),
                                                                                acc[i][j], 0, 0, 0);
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < NW; j++) wv[j] = wnext[j];
    }

    if constexpr (!FOUR_BIT) {
#pragma unroll
        for (int i = 0; i < MW; i++)
#pragma unroll
            for (int j = 0; j < NW; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[i][j][r] = fmaf(-128.0f, xacc[i][r], acc[i][j][r]);
    }

    // ---- combine the four K-slices in wave order (fixed, so results repeat bit for bit)
    if (wave > 0) {
#pragma unroll
        for (int i = 0; i < MW; i++)
#pragma unroll
            for (int j = 0; j < NW; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) red[(wave - 1) * RED + ((i * NW + j) * 4 + r) * 64 + lane] = acc[i][j][r];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int j = 0; j < NW; j++) {
        const int n = n_base + 16 * j + ln;
        if (n >= p.N) continue;
        const float rs = ep_scale[j], b = ep_bias[j];
#pragma unroll
        for (int i = 0; i < MW; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int m = m_base + 16 * i + 4 * kb + r;  // D layout: row 4*(lane/16) + r, column lane%16
                if (m >= p.M) continue;
                const int ri = ((i * NW + j) * 4 + r) * 64 + lane;
                float z = acc[i][j][r];
                for (int w = 0; w < KW - 1; w++) z += red[w * RED + ri];
                if (FMT == NQ_FMT_W8_CHANNEL) z *= rs;
                z += b;
                if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
                const int64_t o = (int64_t)m * p.N + n;
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(p.y)[o] = z;
                else
                    reinterpret_cast<uint16_t*>(p.y)[o] = f32_to_bf16_rne(z);
            }
    }
}

template <int FMT, bool XF32, int MW>
int32_t launch_nw(const A16Params& p, int nw, int kw, dim3 grid, hipStream_t s) {
    const size_t lds = (size_t)(kw - 1) * MW * nw * 4 * 64 * sizeof(float);
    if (nw == 1)
        hipLaunchKernelGGL((gemm_a16_kernel<FMT, XF32, MW, 1>), grid, dim3(64 * kw), lds, s, p);
    else
        hipLaunchKernelGGL((gemm_a16_kernel<FMT, XF32, MW, 2>), grid, dim3(64 * kw), lds, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

template <int FMT, bool XF32>
int32_t launch_mw(const A16Params& p, int mw, int nw, int kw, dim3 grid, hipStream_t s) {
    switch (mw) {
        case 1: return launch_nw<FMT, XF32, 1>(p, nw, kw, grid, s);
        case 2: return launch_nw<FMT, XF32, 2>(p, nw, kw, grid, s);
        case 3: return launch_nw<FMT, XF32, 3>(p, nw, kw, grid, s);
        default: return launch_nw<FMT, XF32, 4>(p, nw, kw, grid, s);
    }
}

template <int FMT>
int32_t launch_x(const A16Params& p, bool xf32, int mw, int nw, int kw, dim3 grid, hipStream_t s) {
    return xf32 ? launch_mw<FMT, true>(p, mw, nw, kw, grid, s) : launch_mw<FMT, false>(p, mw, nw, kw, grid, s);
}

int env_int(const char* name, int dflt) {
    const char* v = std::getenv(name);
    return v ? std::atoi(v) : dflt;
}

}  // namespace

bool gemm_a16_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (a.x_dtype != NQ_DT_F32 && a.x_dtype != NQ_DT_BF16) return false;
    if (L->format == NQ_FMT_FP8_E4M3) return false;
    if (L->format != NQ_FMT_W8_CHANNEL && L->in % 32 != 0) return false;
    if (L->format == NQ_FMT_W8_CHANNEL && L->in % 16 != 0) return false;
    return a.M >= 5;
}

int32_t launch_gemm_a16(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    const bool four_bit = L->format != NQ_FMT_W8_CHANNEL;
    A16Params p{};
    p.codes = L->d_codes, p.scales = L->d_scales, p.zps = L->d_zps;
    p.x = a.x, p.y = a.y, p.bias = a.bias;
    p.M = a.M, p.N = L->out, p.K = L->in;
    p.group = L->group, p.groups = L->groups;
    p.nch = L->in / (four_bit ? 32 : 16);
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    // M tile: the smallest multiple of 16 rows (<= 64) that wastes the least padding
    int mw = 4;
    if (a.M <= 16) mw = 1;
    else if (a.M <= 32) mw = 2;
    else if (a.M <= 48) mw = 3;
    else {
        int best_tiles = 1 << 30;
        for (int c = 4; c >= 2; c--) {
            const int tiles = (a.M + 16 * c - 1) / (16 * c) * c;  // 16-row MFMA tiles computed
            if (tiles < best_tiles) best_tiles = tiles, mw = c;
        }
    }
    int nw = (L->out >= 1024) ? 2 : 1;
    if (mw * nw > 6) nw = 1;  // 4 x 2 MFMA tiles per wavefront would spill under the 256-register budget
    // wavefronts along K: as many as it takes to leave each one at most two k-steps (the call is
    // latency-bound: a k-step is one dependent round trip to memory), within the LDS the
    // fixed-order reduction needs
    const int kstep = four_bit ? 128 : 64;
    const int nsteps = (L->in + kstep - 1) / kstep;
    int kw = 4;
    while (kw < 8 && (nsteps + kw - 1) / kw > 2) kw *= 2;
    while ((size_t)(kw - 1) * mw * nw * 1024 > 60 * 1024) {
        if (nw > 1) nw = 1;
        else if (mw > 1) mw--;
        else kw /= 2;
    }
    kw = env_int("NQ_A16_KW", kw);
    dim3 grid((L->out + 16 * nw - 1) / (16 * nw), (a.M + 16 * mw - 1) / (16 * mw));
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    switch (L->format) {
        case NQ_FMT_Q4_0: return launch_x<NQ_FMT_Q4_0>(p, xf32, mw, nw, kw, grid, a.stream);
        case NQ_FMT_W4_GROUP: return launch_x<NQ_FMT_W4_GROUP>(p, xf32, mw, nw, kw, grid, a.stream);
        case NQ_FMT_W8_CHANNEL: return launch_x<NQ_FMT_W8_CHANNEL>(p, xf32, mw, nw, kw, grid, a.stream);
    }
    return fail(NQ_ERR_INVALID, "nq_forward: unknown format");
}

}  // namespace nq
