// int8 weights under ONE bf16 / fp32 activation row (M = 1) over a large weight, on the int8 matrix cores:
//     y[N] = epi( (W[N, K] x) * s_w[n] + bias ),  W int8 with per-channel scales.
//
// A streaming kernel that converts each code on the vector ALU spends one to two instructions per
// weight, which is more instruction issue than the loads of a 45 MB weight leave room for.  The int8
// MFMA takes the codes as they lie in memory; what it cannot take is x.  So x is split, once per
// workgroup, into three int8 terms under one scale,
//     x[k] = (absmax / 127) * (q1[k] + q2[k] / 254 + q3[k] / 254^2) + e,   |e| <= absmax / (127 * 254^2 * 2),
// (each q the round-to-nearest-even of what the terms before it left over, so |q| <= 127), and the row's
// dot product is three exact int32 sums combined in fp32.  The error of the split is 6e-8 of the row's
// absmax per element, the size of an fp32 rounding of the products themselves.
//   - one wavefront owns one weight row and reads it as 1 KiB contiguous per load instruction, all loads
//     requested before x is touched;
//   - each thread converts 4, 8 or 16 elements of x, so that all 512 take part (absmax: integer max over the
//     bit patterns, so a NaN or an infinity in x is seen and turns every output into NaN), and leaves one word
//     per term and four elements in LDS;
//   - the MFMA is used "diagonally" as in the 8-bit x 8-bit row kernel (nq_gemv_fp8.hip): the 16 B columns
//     are 16 segments of the row, the 16 A rows the matching segments of the leading term of x, and the dot
//     product is the trace of the tile: one v_mfma_i32_16x16x64_i8 per KiB of codes; the two small terms go
//     through v_dot4_i32_i8 into per-lane sums, so that the matrix core and the vector ALU share the work;
//   - the lanes' shares meet in a fixed butterfly (a repeated call returns the same bits).

#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

struct SplitParams {
    const uint8_t* w;
    const void* x;
    const float* col_scale;
    const void* bias;
    int32_t N, K;
    int32_t y_dtype, bias_dtype, epilogue;
    SegTable seg;
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

constexpr float MAGIC = 12582912.0f;  // 1.5 * 2^23: the low byte of (t + MAGIC)'s bits is rne(t) as an int8

// the low bytes of four words, packed in order
__device__ __forceinline__ uint32_t pack_low_bytes(uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3) {
    return __builtin_amdgcn_perm(a1, a0, 0x0c0c0400u) | __builtin_amdgcn_perm(a3, a2, 0x04000c0cu);
}

#define NQ_DPP_F32(v, ctrl) __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), ctrl, 0xF, 0xF, false))
__device__ __forceinline__ float butterfly_sum(float v) {
    v += NQ_DPP_F32(v, 0xB1);
    v += NQ_DPP_F32(v, 0x4E);
    v += NQ_DPP_F32(v, 0x141);
    v += NQ_DPP_F32(v, 0x140);
    {
        const uint32_t b = __float_as_uint(v);
        const auto sw = __builtin_amdgcn_permlane16_swap(b, b, false, false);
        v = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
    {
        const uint32_t b = __float_as_uint(v);
        const auto sw = __builtin_amdgcn_permlane32_swap(b, b, false, false);
        v = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
    return v;
}

template <bool XF32, int CPL, int WAVES, int RPW, int EPT>
__global__ __launch_bounds__(64 * WAVES, 4) void gemv_split8_kernel(const SplitParams p) {
    constexpr int NTHR = 64 * WAVES;
    constexpr int NUNIT = CPL * 1024 / EPT;  // a thread splits one unit of EPT consecutive elements of x
    static_assert(NUNIT <= NTHR && (EPT == 4 || EPT == 8 || EPT == 16), "one unit per thread");
    constexpr int NW = XF32 ? EPT : EPT / 2;  // words of x per unit
    __shared__ u32x4 xs[3][CPL * 64];
    __shared__ uint32_t wmax[WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // a wavefront owns RPW adjacent rows (the split of x is paid once per workgroup: WAVES * RPW rows share it)
    const int64_t row0 = ((int64_t)blockIdx.x * WAVES + wave) * RPW;
    const int nch = p.K >> 4;
    const int nunit = p.K / EPT;

    // every load is unconditional from a clamped index; a unit past K counts as x = 0
    uint32_t xg[NW];
    {
        const int u = min(tid, nunit - 1);
        if constexpr (NW == 2) {
            const uint2 v = reinterpret_cast<const uint2*>(p.x)[u];
            xg[0] = v.x, xg[1] = v.y;
        } else {
            const u32x4* xr = reinterpret_cast<const u32x4*>(p.x) + (int64_t)u * (NW / 4);
#pragma unroll
            for (int q = 0; q < NW / 4; q++) {
                const u32x4 v = xr[q];
                xg[4 * q] = v[0], xg[4 * q + 1] = v[1], xg[4 * q + 2] = v[2], xg[4 * q + 3] = v[3];
            }
        }
    }
    u32x4 wv[RPW][CPL];
    float csraw[RPW];
    uint32_t braw[RPW];
#pragma unroll
    for (int rr = 0; rr < RPW; rr++) {
        const int64_t rowc = min(row0 + rr, (int64_t)p.N - 1);
        const u32x4* wr = reinterpret_cast<const u32x4*>(p.w + rowc * p.K);
#pragma unroll
        for (int j = 0; j < CPL; j++) wv[rr][j] = __builtin_nontemporal_load(wr + min(j * 64 + lane, nch - 1));
        csraw[rr] = p.col_scale[rowc];
        braw[rr] = 0;
        if (p.bias)
            braw[rr] = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[rowc]
                                                   : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[rowc];
    }

    // ---- x as fp32, and the largest magnitude of the row (as a bit pattern: NaN > inf > finite)
    float xf[EPT];
    uint32_t mbits = 0;
    {
        const bool live = tid < nunit;
#pragma unroll
        for (int e = 0; e < EPT; e++) {
            uint32_t b;
            if constexpr (XF32) b = xg[e];
            else b = (e & 1) ? (xg[e >> 1] & 0xFFFF0000u) : (xg[e >> 1] << 16);
            if (!live) b = 0;
            xf[e] = __uint_as_float(b);
            mbits = max(mbits, b & 0x7FFFFFFFu);
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mbits = max(mbits, (uint32_t)__shfl_xor((int)mbits, off));
    if (lane == 0) wmax[wave] = mbits;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < WAVES; w++) mbits = max(mbits, wmax[w]);
    const bool finite = mbits < 0x7F800000u;
    // (a row below 2^-60 is lifted by 2^64 first, exactly: 127 / absmax then stays finite and the row keeps its terms)
    const float lift = mbits < 0x21800000u ? 0x1p64f : 1.0f;
    const float absmax = __uint_as_float(mbits) * lift;
    const float inv_s = (finite && absmax > 0.0f) ? 127.0f / absmax : 0.0f;
    const float s_x = inv_s != 0.0f ? (absmax * (1.0f / 127.0f)) / lift : 0.0f;

    if (tid < NUNIT) {
        uint32_t* const x0 = reinterpret_cast<uint32_t*>(xs[0]) + tid * (EPT / 4);
        uint32_t* const x1 = reinterpret_cast<uint32_t*>(xs[1]) + tid * (EPT / 4);
        uint32_t* const x2 = reinterpret_cast<uint32_t*>(xs[2]) + tid * (EPT / 4);
        if (tid - lane >= nunit) {  // uniform over the wavefront: nothing of x here, only the padding of the last load
#pragma unroll
            for (int q = 0; q < EPT / 4; q++) x0[q] = x1[q] = x2[q] = 0;
        } else {
            // four elements at a time, one word per term
#pragma unroll
            for (int q = 0; q < EPT / 4; q++) {
                uint32_t a1[4], a2[4], a3[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    // Round by adding 1.5 * 2^23 (the sum's low byte is the int8), and take every leftover against
                    // the very integer that was packed: the second and third term round the exact product
                    // (one fma each), so that no leftover exceeds a half and no term leaves the int8 range.
                    const float t = (xf[4 * q + e] * lift) * inv_s;
                    const float b1 = t + MAGIC;
                    a1[e] = __float_as_uint(b1);
                    const float r1 = t - (b1 - MAGIC);
                    const float b2 = __builtin_fmaf(r1, 254.0f, MAGIC);
                    a2[e] = __float_as_uint(b2);
                    const float r2 = __builtin_fmaf(r1, 254.0f, MAGIC - b2);
                    a3[e] = __float_as_uint(__builtin_fmaf(r2, 254.0f, MAGIC));
                }
                x0[q] = pack_low_bytes(a1[0], a1[1], a1[2], a1[3]);
                x1[q] = pack_low_bytes(a2[0], a2[1], a2[2], a2[3]);
                x2[q] = pack_low_bytes(a3[0], a3[1], a3[2], a3[3]);
            }
        }
    }
    __syncthreads();

    // lane holds D[4 (lane / 16) + r][lane % 16]: its diagonal entry, if any, is r = c % 4 where
    // c = lane % 16 and c / 4 == lane / 16.  |acc| <= 128 * 127 * 64 * 8 < 2^24: exact as fp32.
    const int c16 = lane & 15, r = c16 & 3;
    const bool holder = (c16 >> 2) == (lane >> 4);
    auto pick = [&](const i32x4& a) { return r == 0 ? a[0] : r == 1 ? a[1] : r == 2 ? a[2] : a[3]; };
    // a term of x is read from LDS once per chunk and meets every row of the wavefront: the leading term on the
    // matrix core, the two small ones on the vector ALU (v_dot4_i32_i8, per-lane sums), so that both pipes work
    i32x4 acc[RPW];
    int d1[RPW], d2[RPW];
#pragma unroll
    for (int rr = 0; rr < RPW; rr++) acc[rr] = (i32x4){0, 0, 0, 0}, d1[rr] = 0, d2[rr] = 0;
#pragma unroll
    for (int j = 0; j < CPL; j++) {
        const i32x4 x0 = __builtin_bit_cast(i32x4, xs[0][j * 64 + lane]);
        const i32x4 x1 = __builtin_bit_cast(i32x4, xs[1][j * 64 + lane]);
        const i32x4 x2 = __builtin_bit_cast(i32x4, xs[2][j * 64 + lane]);
#pragma unroll
        for (int rr = 0; rr < RPW; rr++) {
            const i32x4 w = __builtin_bit_cast(i32x4, wv[rr][j]);
            acc[rr] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, w, acc[rr], 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                d1[rr] = __builtin_amdgcn_sdot4(x1[e], w[e], d1[rr], false);
                d2[rr] = __builtin_amdgcn_sdot4(x2[e], w[e], d2[rr], false);
            }
        }
    }
#pragma unroll
    for (int rr = 0; rr < RPW; rr++) {
        const float lead = holder ? (float)pick(acc[rr]) : 0.0f;
        float v = lead + (float)d1[rr] * (1.0f / 254.0f) + (float)d2[rr] * (1.0f / 64516.0f);
        v = butterfly_sum(v);
        const int64_t row = row0 + rr;
        if (lane == 0 && row < p.N) {
            const float bias = p.bias_dtype == NQ_DT_F32 ? __uint_as_float(braw[rr]) : __uint_as_float(braw[rr] << 16);
            float z = v * (s_x * csraw[rr]) + bias;
            if (!finite) z = __uint_as_float(0x7FC00000u);
            if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
            void* y;
            int width, col;
            seg_lookup(p.seg, (int)row, y, width, col);
            if (p.y_dtype == NQ_DT_F32)
                reinterpret_cast<float*>(y)[col] = z;
            else
                reinterpret_cast<uint16_t*>(y)[col] = f32_to_bf16_rne(z);
        }
    }
}

template <bool XF32, int CPL>
int32_t launch_split8(const SplitParams& p, hipStream_t s) {
    // one row per wavefront: two and four rows per wavefront (the split of x is then paid once per 16 or 32 rows)
    // were measured and are slower, 4096 -> 11008 in 10.5 / 11.4 / 14.8 us, 8192 -> 8192 in 14.6 / 16.1 us
    // (likewise 16 wavefronts per workgroup: 12.6 / 27.2 us on 4096 -> 11008 / 28672 against 10.6 / 22 .. 24)
    constexpr int EPT = CPL <= 2 ? 4 : CPL <= 4 ? 8 : 16;  // all 512 threads take part in the split of x
    hipLaunchKernelGGL((gemv_split8_kernel<XF32, CPL, 8, 1, EPT>), dim3((unsigned)((p.N + 7) / 8)), dim3(512), 0, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

template <bool XF32>
int32_t launch_split8_cpl(const SplitParams& p, hipStream_t s) {
    // (rows of 4096 codes and more: four to eight loads per lane)
    switch ((p.K / 16 + 63) / 64) {
        case 4: return launch_split8<XF32, 4>(p, s);
        case 5: return launch_split8<XF32, 5>(p, s);
        case 6: return launch_split8<XF32, 6>(p, s);
        case 7: return launch_split8<XF32, 7>(p, s);
        default: return launch_split8<XF32, 8>(p, s);
    }
}

}  // namespace

// One bf16 / fp32 row over int8 weights with rows of 4096 .. 8192 codes (a multiple of 16) and 16 MB and more.
// Measured against the kernels that convert every code on the vector ALU (us, cold): 4096 -> 4096 5.3 / 5.4,
// 4096 -> 6144 6.6 / 7.7, 4096 -> 11008 10.3 / 11.5, 4096 -> 28672 21 .. 23 / 27.8, 5120 -> 5120 7.2 / 8.3,
// 8192 -> 8192 14.1 / 14.7.  Shorter rows lose (3072 -> 9216 8.2 / 7.8, 2048 -> 16384 9.7 / 8.4, 1024 -> 16384
// 7.5 / 6.5): the split and its two barriers are paid per 8 rows whatever their length.
bool gemv_split8_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (a.M != 1 || L->format != NQ_FMT_W8_CHANNEL || ((uintptr_t)a.x & 15)) return false;
    if (a.x_dtype != NQ_DT_BF16 && a.x_dtype != NQ_DT_F32) return false;
    if (a.y_dtype != NQ_DT_F32 && a.y_dtype != NQ_DT_BF16) return false;
    if (L->in % 16 != 0 || L->in < 4096 || L->in > 8192) return false;
    return (int64_t)L->in * L->out >= ((int64_t)16 << 20);
}

int32_t launch_gemv_split8(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    SplitParams p{};
    p.w = L->d_codes, p.x = a.x, p.col_scale = reinterpret_cast<const float*>(L->d_scales), p.bias = a.bias;
    p.N = L->out, p.K = L->in;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    p.seg = a.seg;
    if (a.x_dtype == NQ_DT_F32) return launch_split8_cpl<true>(p, a.stream);
    return launch_split8_cpl<false>(p, a.stream);
}

}  // namespace nq
