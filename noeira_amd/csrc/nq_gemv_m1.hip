// Dequant-GEMV for one activation row (M = 1): y[N] = epi(deq(W) x + bias).
//
// The regime is HBM- or latency-bound: the only large operand is the packed
// weight, read exactly once with 128-bit non-temporal loads.  x is small and
// shared by every row, so each lane keeps the slice of x it needs IN REGISTERS
// for the whole kernel: `lpr` lanes (a power of two) share a row, lane j owns
// the 16-byte chunks j, j + lpr, ... (CPL of them), and the x values under
// those chunks are loaded once, up front, together with the first weights -
// one round trip to memory, no LDS, no barrier (one exception: fp32 x under
// 4-bit weights in a launch of a thousand wavefronts, STAGE_X below).  A lane
// group then walks its rows RPL at a time (RPL x CPL independent loads in flight per lane); the
// host picks one row per lane group and as many lanes per row as it takes to
// launch ~1k wavefronts, which measured best from 68 KB to 45 MB of weights.
// Every load is unconditional from a clamped address (a predicated load
// becomes a branch and serialises the batch); the product of a chunk past the
// end of a row is dropped with one select.
//
//   8-bit weights (int8, fp8):  x held as fp32, one v_cvt per code (for int8
//       the sign-extending byte form of v_cvt_f32_i32) + one FMA.  fp8
//       weights with fp8 activations go to nq_gemv_fp8.hip instead.
//   4-bit weights, bf16 x:      x held as packed bf16 pairs; a word of eight
//       codes becomes four bf16 pairs (16 + q) with a shift and an and-or each
//       (device nibble order, nq_nib.h) and goes through v_dot2_f32_bf16:
//       1.5 VALU ops per weight instead of 2.25.
//   4-bit weights, fp32 x:      x held as fp32, v_cvt + FMA (exact fp32
//       products, the reference's 1e-5 band).
// Offsets and zero points leave the inner loop through xsum, the sum of x
// under a chunk: sum x (q - z) = sum x q - z xsum.
//
// The cross-lane sum is a fixed butterfly, so a repeated call returns the same
// bits (tests/nn/quant/test_qlinear_gpu.mojo:96,128).
#include <hip/hip_fp16.h>


#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

struct M1Params {
    const uint8_t* codes;
    const void* scales;
    const uint8_t* zps;
    const void* x;
    const float* x_scale;
    void* y;
    const void* bias;
    int32_t N, K;
    int32_t group, groups;
    float tscale;
    int32_t nch;   // 16-byte chunks per row
    int32_t lpr;   // lanes per row (a power of two)
    int32_t lpr_log2;
    int32_t rpw;   // rows per lane group (a multiple of RPL)
    int32_t x_dtype, y_dtype, bias_dtype, epilogue;
    SegTable seg;
};

__device__ __forceinline__ float bf16lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16hi(uint32_t pair) { return __uint_as_float(pair & 0xFFFF0000u); }

__device__ __forceinline__ uint16_t to_bf16(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

// Sum over a group of `lpr` consecutive lanes (a power of two); every lane of the group ends with
// the total.  Butterfly in a fixed order: quad swaps, half-row and row mirrors (DPP), then the
// 16- and 32-lane swaps (v_permlane16_swap / v_permlane32_swap).  No LDS traffic.
__device__ __forceinline__ float group_sum(float v, int lpr) {
    int t;
    if (lpr > 1) {
        t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false);  // quad_perm [1,0,3,2]
        v += __int_as_float(t);
    }
    if (lpr > 2) {
        t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false);  // quad_perm [2,3,0,1]
        v += __int_as_float(t);
    }
    if (lpr > 4) {
        t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, false);  // row_half_mirror
        v += __int_as_float(t);
    }
    if (lpr > 8) {
        t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, false);  // row_mirror
        v += __int_as_float(t);
    }
    if (lpr > 16) {
        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
    if (lpr > 32) {
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        v = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
    return v;
}

template <int FMT, int XDT, bool DOT2, int CPL, int RPL, bool STAGE_X>
__global__ __launch_bounds__(256) void gemv_m1_kernel(const M1Params p) {
    constexpr bool FOUR_BIT = (FMT == NQ_FMT_Q4_0 || FMT == NQ_FMT_W4_GROUP);
    constexpr int EPC = FOUR_BIT ? 32 : 16;
    constexpr int XR = DOT2 ? EPC / 2 : EPC;  // registers of x per chunk
    static_assert(!DOT2 || FOUR_BIT, "the bf16 dot path is for 4-bit weights");
    // STAGE_X (4-bit weights with fp32 x, launches of a thousand wavefronts and more): a lane's chunk of x is
    // 128 bytes, and eight loads whose lanes sit 128 bytes apart cost the L1 as much as eight times the cache
    // lines they touch.  The workgroup fetches x once, adjacent lanes adjacent pieces, and hands it round
    // through LDS instead.  (With fewer wavefronts the extra barrier costs more than the loads: measured.)
    static_assert(!STAGE_X || (FOUR_BIT && !DOT2), "x is staged for 4-bit weights with fp32 x only");
    extern __shared__ __attribute__((aligned(16))) uint8_t xstage[];  // STAGE_X: nch x 128 bytes

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lpr = p.lpr;
    const int rg = lane >> p.lpr_log2, lj = lane & (lpr - 1);

    const u32x4* wq = reinterpret_cast<const u32x4*>(p.codes);
    const int64_t group_id = (((int64_t)blockIdx.x * 4 + wave) << (6 - p.lpr_log2)) + rg;
    const int64_t row_begin = group_id * p.rpw;
    bool cval[CPL];
#pragma unroll
    for (int i = 0; i < CPL; i++) cval[i] = (lj + i * lpr) < p.nch;

    // One batch = RPL rows x CPL chunks of codes (+ their scales) for this lane.  The first batch is
    // requested before x so that both arrive in one round trip; afterwards batch b+1 is in flight
    // while batch b is multiplied.
    auto fetch = [&](int64_t row0, u32x4 (&wv)[RPL][CPL], float (&cs)[RPL][CPL], float (&cz)[RPL][CPL],
                     float (&rs)[RPL], uint32_t (&rbias)[RPL]) {
#pragma unroll
        for (int r = 0; r < RPL; r++) {
            const int64_t row = min(row0 + r, (int64_t)p.N - 1);
            // the epilogue's operands travel with the codes, so nothing is loaded after the reduction
            rs[r] = (FMT == NQ_FMT_W8_CHANNEL) ? reinterpret_cast<const float*>(p.scales)[row] : 1.0f;
            // (the bias stays raw until the epilogue: widening a bf16 bias here would make the wavefront
            // wait for it before the codes and x are requested)
            rbias[r] = 0;
            if (p.bias)
                rbias[r] = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[row]
                                                       : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[row];
#pragma unroll
            for (int i = 0; i < CPL; i++) {
                // Unconditional loads from clamped addresses: a lane whose chunk index runs past the
                // row re-reads the last chunk, and its partial product is dropped (one select per chunk).
                // (A predicated load would become a branch around the load and serialise the batch.)
                const int c = min(lj + i * lpr, p.nch - 1);
                wv[r][i] = __builtin_nontemporal_load(&wq[row * p.nch + c]);
                cs[r][i] = 0.0f, cz[r][i] = 0.0f;
                if constexpr (FMT == NQ_FMT_Q4_0) {
                    cs[r][i] = __half2float(
                        __ushort_as_half(reinterpret_cast<const uint16_t*>(p.scales)[row * p.nch + c]));
                    cz[r][i] = 8.0f;
                } else if constexpr (FMT == NQ_FMT_W4_GROUP) {
                    const int g = (c * EPC) / p.group;
                    cs[r][i] = __half2float(
                        __ushort_as_half(reinterpret_cast<const uint16_t*>(p.scales)[row * p.groups + g]));
                    cz[r][i] = (float)p.zps[row * p.groups + g];
                }
            }
        }
    };
    u32x4 wv[RPL][CPL], wn[RPL][CPL];
    float cs[RPL][CPL], cz[RPL][CPL], csn[RPL][CPL], czn[RPL][CPL];
    float rs[RPL], rsn[RPL];
    uint32_t rbias[RPL], rbiasn[RPL];
    const float tscale = (FMT == NQ_FMT_FP8_E4M3) ? p.tscale * (p.x_scale ? p.x_scale[0] : 1.0f) : 1.0f;

    // ---- this lane's slice of x, loaded once
    uint32_t xr[CPL][XR];  // fp32 bits, or bf16 pairs when DOT2
    float xsum[CPL];
    // piece v (16 bytes) of chunk c sits at c * 128 + (v ^ (c / 2) % 8) * 16: 16 lanes reading the same piece
    // of 16 consecutive chunks then touch every LDS bank once
    auto xslot = [](int c, int v) { return c * 128 + ((v ^ ((c >> 1) & 7)) << 4); };
    // Every load of the first batch is issued before anything waits, x first: it comes from L2 and is widened and
    // summed while the weights are still on their way from memory (loads return in the order of issue, so with the
    // weights first the wait for x would be the wait for them).  The scheduling barrier below keeps the loads
    // above it and their uses beneath: left to itself the compiler put the weights' loads after the wait for x in
    // about half of the variants - a second, and with a scale in between a third, round trip to memory per call.
    constexpr int XRAW = STAGE_X ? 2 * CPL : DOT2 ? EPC / 8 : XDT == NQ_DT_F32 ? EPC / 4 : XDT == NQ_DT_BF16 ? EPC / 8 : EPC / 16;
    u32x4 xraw[STAGE_X ? 1 : CPL][XRAW];
    if constexpr (STAGE_X) {
        // (at most 64 CPL chunks of 8 pieces: 2 CPL per thread)
        const int npieces = p.nch * 8;
#pragma unroll
        for (int v = 0; v < XRAW; v++) {
            const int e = min((int)threadIdx.x + 256 * v, npieces - 1);
            xraw[0][v] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(p.x) + (size_t)e * 16);
        }
    } else {
#pragma unroll
        for (int i = 0; i < CPL; i++) {
            // clamped, unconditional loads; the product of a chunk past the end of the row is dropped below
            const int64_t k0 = (int64_t)min(lj + i * lpr, p.nch - 1) * EPC;
            const char* xb = reinterpret_cast<const char*>(p.x) + k0 * (XDT == NQ_DT_F32 ? 4 : XDT == NQ_DT_BF16 ? 2 : 1);
#pragma unroll
            for (int v = 0; v < XRAW; v++) xraw[i][v] = *reinterpret_cast<const u32x4*>(xb + 16 * v);
        }
    }
    fetch(row_begin, wv, cs, cz, rs, rbias);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (STAGE_X) {
        const int npieces = p.nch * 8;
#pragma unroll
        for (int v = 0; v < XRAW; v++) {
            const int e = (int)threadIdx.x + 256 * v;
            if (e < npieces) *reinterpret_cast<u32x4*>(xstage + xslot(e >> 3, e & 7)) = xraw[0][v];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < CPL; i++) {
        float s = 0.0f;
        if constexpr (DOT2) {
#pragma unroll
            for (int v = 0; v < EPC / 8; v++) {
                const u32x4 t = xraw[i][v];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    xr[i][4 * v + e] = t[e];
                    s += bf16lo(xr[i][4 * v + e]) + bf16hi(xr[i][4 * v + e]);
                }
            }
        } else {
            float f[EPC];
            if constexpr (STAGE_X) {
                const int cc = min(lj + i * lpr, p.nch - 1);
#pragma unroll
                for (int v = 0; v < 8; v++) {
                    const float4 t = *reinterpret_cast<const float4*>(xstage + xslot(cc, v));
                    f[4 * v] = t.x, f[4 * v + 1] = t.y, f[4 * v + 2] = t.z, f[4 * v + 3] = t.w;
                }
            } else if constexpr (XDT == NQ_DT_F32) {
#pragma unroll
                for (int v = 0; v < EPC / 4; v++) {
                    const u32x4 t = xraw[i][v];
#pragma unroll
                    for (int e = 0; e < 4; e++) f[4 * v + e] = __uint_as_float(t[e]);
                }
            } else if constexpr (XDT == NQ_DT_BF16) {
#pragma unroll
                for (int v = 0; v < EPC / 8; v++) {
                    const u32x4 t = xraw[i][v];
#pragma unroll
                    for (int e = 0; e < 4; e++) f[8 * v + 2 * e] = bf16lo(t[e]), f[8 * v + 2 * e + 1] = bf16hi(t[e]);
                }
            } else {  // fp8 e4m3
#pragma unroll
                for (int v = 0; v < EPC / 16; v++) {
                    const u32x4 t = xraw[i][v];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)t[e], false);
                        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)t[e], true);
                        f[16 * v + 4 * e] = a[0], f[16 * v + 4 * e + 1] = a[1];
                        f[16 * v + 4 * e + 2] = b[0], f[16 * v + 4 * e + 3] = b[1];
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < EPC; e++) {
                xr[i][e] = __float_as_uint(f[e]);
                s += f[e];
            }
        }
        xsum[i] = s;
    }

#define XF(i, e) __uint_as_float(xr[(i)][(e)])
    // (p.rpw is RPL in every launch; with the trip count a compile-time 1 the compiler orders the
    // prologue differently and most calls are 2 - 8 % slower: measured, with and without a scheduling
    // barrier after the first loads)
    for (int rb = 0; rb < p.rpw; rb += RPL) {
        const int64_t row0 = row_begin + rb;
        if (row0 >= p.N) break;
        if (rb + RPL < p.rpw) fetch(row0 + RPL, wn, csn, czn, rsn, rbiasn);

        float acc[RPL];
#pragma unroll
        for (int r = 0; r < RPL; r++) {
            acc[r] = 0.0f;
#pragma unroll
            for (int i = 0; i < CPL; i++) {
                float dot = 0.0f;
                if constexpr (FOUR_BIT) {
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const uint32_t w = wv[r][i][t];
                        if constexpr (DOT2) {
                            // pair s of the word = elements 2s, 2s+1 -> bf16 (16 + q, 16 + q')
                            const uint32_t w0 = ((w << 3) & 0x00780078u) | 0x41804180u;
                            const uint32_t w1 = ((w >> 1) & 0x00780078u) | 0x41804180u;
                            const uint32_t w2 = ((w >> 5) & 0x00780078u) | 0x41804180u;
                            const uint32_t w3 = ((w >> 9) & 0x00780078u) | 0x41804180u;
                            dot = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, xr[i][4 * t]),
                                                                  __builtin_bit_cast(bf16x2, w0), dot, false);
                            dot = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, xr[i][4 * t + 1]),
                                                                  __builtin_bit_cast(bf16x2, w1), dot, false);
                            dot = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, xr[i][4 * t + 2]),
                                                                  __builtin_bit_cast(bf16x2, w2), dot, false);
                            dot = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, xr[i][4 * t + 3]),
                                                                  __builtin_bit_cast(bf16x2, w3), dot, false);
                        } else {
                            // low nibbles of the four bytes: elements 0, 4, 1, 5; high nibbles: 2, 6, 3, 7
                            const uint32_t lo = w & 0x0F0F0F0Fu, hi = (w >> 4) & 0x0F0F0F0Fu;
                            dot = fmaf(XF(i, 8 * t + 0), (float)(lo & 0xFFu), dot);
                            dot = fmaf(XF(i, 8 * t + 4), (float)((lo >> 8) & 0xFFu), dot);
                            dot = fmaf(XF(i, 8 * t + 1), (float)((lo >> 16) & 0xFFu), dot);
                            dot = fmaf(XF(i, 8 * t + 5), (float)(lo >> 24), dot);
                            dot = fmaf(XF(i, 8 * t + 2), (float)(hi & 0xFFu), dot);
                            dot = fmaf(XF(i, 8 * t + 6), (float)((hi >> 8) & 0xFFu), dot);
                            dot = fmaf(XF(i, 8 * t + 3), (float)((hi >> 16) & 0xFFu), dot);
                            dot = fmaf(XF(i, 8 * t + 7), (float)(hi >> 24), dot);
                        }
                    }
                    const float zoff = DOT2 ? cz[r][i] + 16.0f : cz[r][i];
                    acc[r] += cval[i] ? cs[r][i] * fmaf(-zoff, xsum[i], dot) : 0.0f;
                } else if constexpr (FMT == NQ_FMT_W8_CHANNEL) {
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        // sign-extending byte -> fp32 conversions (v_cvt_f32_i32 with a byte select)
                        const uint32_t u = wv[r][i][t];
                        dot = fmaf(XF(i, 4 * t + 0), (float)(int)(int8_t)(u & 0xFFu), dot);
                        dot = fmaf(XF(i, 4 * t + 1), (float)(int)(int8_t)((u >> 8) & 0xFFu), dot);
                        dot = fmaf(XF(i, 4 * t + 2), (float)(int)(int8_t)((u >> 16) & 0xFFu), dot);
                        dot = fmaf(XF(i, 4 * t + 3), (float)((int)u >> 24), dot);
                    }
                    acc[r] += cval[i] ? dot : 0.0f;
                } else {
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv[r][i][t], false);
                        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)wv[r][i][t], true);
                        dot = fmaf(XF(i, 4 * t + 0), a[0], dot);
                        dot = fmaf(XF(i, 4 * t + 1), a[1], dot);
                        dot = fmaf(XF(i, 4 * t + 2), b[0], dot);
                        dot = fmaf(XF(i, 4 * t + 3), b[1], dot);
                    }
                    acc[r] += cval[i] ? dot : 0.0f;
                }
            }
        }

#pragma unroll
        for (int r = 0; r < RPL; r++) acc[r] = group_sum(acc[r], lpr);

        if (p.epilogue == NQ_EPI_SWIGLU) {
            // (uniform) rows 2 n and 2 n + 1 are the gate and the up row of output n: adjacent lane groups
            // (every lane of a group holds its row's sum), or adjacent wavefronts when a row takes all 64 lanes
            float z = acc[0];
            if (FMT == NQ_FMT_W8_CHANNEL) z *= rs[0];
            if (FMT == NQ_FMT_FP8_E4M3) z *= tscale;
            float other;
            if (lpr < 64) {
                other = __shfl_xor(z, lpr);
            } else {
                __shared__ float pair[4];
                if (lane == 0) pair[wave] = z;
                __syncthreads();
                other = pair[wave ^ 1];
            }
            const int64_t n = row0;
            if (lj == 0 && (n & 1) == 0 && n + 1 < p.N) {
                const float g = swiglu_f32(other, z);
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(p.y)[n >> 1] = g;
                else
                    reinterpret_cast<uint16_t*>(p.y)[n >> 1] = to_bf16(g);
            }
            continue;  // (one row per lane group in every launch: the loop runs once)
        }
        if (lj == 0) {
#pragma unroll
            for (int r = 0; r < RPL; r++) {
                const int64_t n = row0 + r;
                if (n >= p.N) continue;
                float z = acc[r];
                if (FMT == NQ_FMT_W8_CHANNEL) z *= rs[r];
                if (FMT == NQ_FMT_FP8_E4M3) z *= tscale;
                z += p.bias_dtype == NQ_DT_F32 ? __uint_as_float(rbias[r]) : __uint_as_float(rbias[r] << 16);
                if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
                void* yp;
                int width, col;
                seg_lookup(p.seg, (int)n, yp, width, col);  // M = 1: the part's row is its only row
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(yp)[col] = z;
                else
                    reinterpret_cast<uint16_t*>(yp)[col] = to_bf16(z);
            }
        }
        if (rb + RPL < p.rpw) {
#pragma unroll
            for (int r = 0; r < RPL; r++)
#pragma unroll
                for (int i = 0; i < CPL; i++) wv[r][i] = wn[r][i], cs[r][i] = csn[r][i], cz[r][i] = czn[r][i];
#pragma unroll
            for (int r = 0; r < RPL; r++) rs[r] = rsn[r], rbias[r] = rbiasn[r];
        }
    }
}

#undef XF

// Only the combinations the host picks are instantiated: one row per lane group (RPL = 1: more rows per
// lane measured slower at every size, see launch_gemv_m1), and at most 96 registers of x (CPL <= 3 when a
// chunk of x takes 32 registers).
template <int FMT, int XDT, bool DOT2, int CPL, bool STAGE_X>
int32_t launch_one(const M1Params& p, dim3 grid, hipStream_t s) {
    const size_t lds = STAGE_X ? (size_t)p.nch * 128 : 0;  // at most 3 x 64 chunks: 24 KiB
    hipLaunchKernelGGL((gemv_m1_kernel<FMT, XDT, DOT2, CPL, 1, STAGE_X>), grid, dim3(256), lds, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

template <int FMT, int XDT, bool DOT2>
int32_t launch_cpl(const M1Params& p, int cpl, dim3 grid, hipStream_t s) {
    constexpr bool WIDE_X = (FMT == NQ_FMT_Q4_0 || FMT == NQ_FMT_W4_GROUP) && !DOT2;
    if constexpr (WIDE_X) {
        if ((int64_t)grid.x * 4 >= 1024) {  // x through LDS
            switch (cpl) {
                case 1: return launch_one<FMT, XDT, DOT2, 1, true>(p, grid, s);
                case 2: return launch_one<FMT, XDT, DOT2, 2, true>(p, grid, s);
                case 3: return launch_one<FMT, XDT, DOT2, 3, true>(p, grid, s);
            }
        }
    }
    switch (cpl) {
        case 1: return launch_one<FMT, XDT, DOT2, 1, false>(p, grid, s);
        case 2: return launch_one<FMT, XDT, DOT2, 2, false>(p, grid, s);
        case 3: return launch_one<FMT, XDT, DOT2, 3, false>(p, grid, s);
    }
    if constexpr (!WIDE_X) {
        switch (cpl) {
            case 4: return launch_one<FMT, XDT, DOT2, 4, false>(p, grid, s);
            case 5: return launch_one<FMT, XDT, DOT2, 5, false>(p, grid, s);
            case 6: return launch_one<FMT, XDT, DOT2, 6, false>(p, grid, s);
        }
    }
    return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no single-row GEMV variant for this IN");
}

// (lanes per row, chunks per lane) covering nch chunks with the fewest idle slots
bool pick_split(int nch, int cpl_max, int* lpr_out, int* cpl_out) {
    int best = -1;
    for (int lpr = 64; lpr >= 1; lpr >>= 1) {
        const int cpl = (nch + lpr - 1) / lpr;
        if (cpl > cpl_max) break;
        const int slots = lpr * cpl;
        if (best < 0 || slots < best) best = slots, *lpr_out = lpr, *cpl_out = cpl;
    }
    return best >= 0;
}

}  // namespace

bool gemv_m1_applicable(const ForwardArgs& a) {
    if (a.M != 1) return false;
    const nq_layer* L = a.L;
    if (a.x_dtype == NQ_DT_I8) return false;
    const bool four_bit = (L->format == NQ_FMT_Q4_0 || L->format == NQ_FMT_W4_GROUP);
    const bool dot2 = four_bit && a.x_dtype == NQ_DT_BF16;
    const int nch = L->in / (four_bit ? 32 : 16);
    int lpr, cpl;
    // x registers per chunk: 16 (8-bit, or 4-bit through the bf16 dot) or 32 (4-bit with fp32 x)
    return pick_split(nch, (four_bit && !dot2) ? 3 : 6, &lpr, &cpl);
}

int32_t launch_gemv_m1(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    const bool four_bit = (L->format == NQ_FMT_Q4_0 || L->format == NQ_FMT_W4_GROUP);
    const bool dot2 = four_bit && a.x_dtype == NQ_DT_BF16;
    M1Params p{};
    p.codes = L->d_codes, p.scales = L->d_scales, p.zps = L->d_zps;
    p.x = a.x, p.x_scale = a.x_scale, p.y = a.y, p.bias = a.bias, p.seg = a.seg;
    p.N = L->out, p.K = L->in, p.group = L->group, p.groups = L->groups, p.tscale = L->scale;
    p.nch = L->in / (four_bit ? 32 : 16);
    p.x_dtype = a.x_dtype, p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    int lpr = 64, cpl = 1;
    pick_split(p.nch, (four_bit && !dot2) ? 3 : 6, &lpr, &cpl);
    // a small matrix wants wavefronts more than it wants busy lanes: widen the lane group until the
    // launch has ~1k wavefronts (idle lanes cost nothing, a short dependency chain is the point)
    while (lpr < 64 && (int64_t)L->out * lpr / 64 < 1024) {
        lpr *= 2;
        cpl = (p.nch + lpr - 1) / lpr;
    }
    // One row per lane group and one batch per wavefront: the most wavefronts, the shortest
    // dependency chain.  Measured best from 68 KB to 45 MB of weights (memory-level parallelism
    // comes from occupancy, not from rows per lane).
    cpl = (p.nch + lpr - 1) / lpr;
    p.lpr = lpr;
    p.lpr_log2 = 0;
    while ((1 << p.lpr_log2) < lpr) p.lpr_log2++;
    p.rpw = 1;
    const int64_t groups = ((int64_t)L->out + p.rpw - 1) / p.rpw;
    const int64_t groups_per_block = 4 * (64 / lpr);
    dim3 grid((unsigned)((groups + groups_per_block - 1) / groups_per_block));
    const int xd = a.x_dtype;
    switch (L->format) {
        case NQ_FMT_Q4_0:
            if (dot2) return launch_cpl<NQ_FMT_Q4_0, NQ_DT_BF16, true>(p, cpl, grid, a.stream);
            return launch_cpl<NQ_FMT_Q4_0, NQ_DT_F32, false>(p, cpl, grid, a.stream);
        case NQ_FMT_W4_GROUP:
            if (dot2) return launch_cpl<NQ_FMT_W4_GROUP, NQ_DT_BF16, true>(p, cpl, grid, a.stream);
            return launch_cpl<NQ_FMT_W4_GROUP, NQ_DT_F32, false>(p, cpl, grid, a.stream);
        case NQ_FMT_W8_CHANNEL:
            if (xd == NQ_DT_BF16) return launch_cpl<NQ_FMT_W8_CHANNEL, NQ_DT_BF16, false>(p, cpl, grid, a.stream);
            return launch_cpl<NQ_FMT_W8_CHANNEL, NQ_DT_F32, false>(p, cpl, grid, a.stream);
        case NQ_FMT_FP8_E4M3:
            if (xd == NQ_DT_FP8_E4M3)
                return launch_cpl<NQ_FMT_FP8_E4M3, NQ_DT_FP8_E4M3, false>(p, cpl, grid, a.stream);
            if (xd == NQ_DT_BF16) return launch_cpl<NQ_FMT_FP8_E4M3, NQ_DT_BF16, false>(p, cpl, grid, a.stream);
            return launch_cpl<NQ_FMT_FP8_E4M3, NQ_DT_F32, false>(p, cpl, grid, a.stream);
    }
    return fail(NQ_ERR_INVALID, "nq_forward: unknown format");
}

}  // namespace nq
