// 4-bit dequant-GEMV for one activation row over a LARGE weight (M = 1, megabytes of codes):
//     y[N] = epi( deq(W)[N, K] x + bias ),   Q4_0 (group 32) or W4_GROUP (groups of 128 k), x bf16 or fp32.
//
// At this size the call is bound by the weight stream, and what keeps a vector-ALU kernel from
// it is instruction issue: at 70 % of HBM a SIMD must take in 1 KiB of codes (2048 weights)
// every ~450 cycles, a wavefront instruction occupies it for 4, and unpack + convert + multiply
// on the vector ALU is 1.5 .. 2.25 instructions for every 64 weights.  Here the multiplies run
// on the bf16 matrix core and the vector ALU only unpacks nibbles:
//   - one wavefront owns one weight row and reads it as 1 KiB contiguous per load instruction:
//     lane (c = l % 16, q = l / 16) takes the 16-byte chunk 64 j + 4 c + q, one group of 32
//     codes as four words of 8;
//   - a 4 x 4 transpose between the four 16-lane rows of the wavefront (two v_permlane32_swap,
//     two v_permlane16_swap) leaves lane (c, q) with word q of the chunks 4 c .. 4 c + 3: MFMA m
//     then has the 32 codes of chunk 4 c + m spread over the four lanes that
//     v_mfma_f32_16x16x32_bf16 sums for column c;
//   - the A operand is x under the same chunk (lane (c, q): 8 consecutive values from LDS), so
//     D[c][c] is that group's dot product; 15/16 of the tile is unused, which costs nothing
//     (64 .. 192 MFMA cycles per 1 KiB against the 450 available);
//   - the four lanes of column c all fetch the four group scales of chunks 4 c .. 4 c + 3 with
//     one 8-byte load; the lane holding the diagonal (q = c / 4, register c % 4) picks its
//     entry and adds d (D - (16 + z) xsum): the 16 comes from the nibble -> bf16 trick (bits
//     0x4180 | code << 3 are exactly 16 + code), xsum = the sum of x under the chunk, kept in
//     LDS.  A W4_GROUP group of 128 k is the four chunks of one column: the MFMAs accumulate
//     and scale and zero point are applied once;
//   - x is staged once per workgroup into LDS as bf16: bf16 input as it is, fp32 input as the
//     three-term split hi + mid + lo (each term exact, together the fp32 value), one MFMA per
//     term, so the products are the exact fp32 x times the exact code (the 1e-5 band of the
//     reference's fp32 path).  Within a block of 64 chunks the eight values lane (c, q) needs
//     for MFMA m sit at byte 1024 m + 16 (c + 16 q): an MFMA's operand read is one KiB with lane l
//     at byte 16 l, the pattern a 128-bit LDS read serves without bank conflicts.
//     Chunks past K read zeros of x; their scale is forced to 0.
// Every load is unconditional from a clamped address and is requested before x is staged.  The cross-lane
// sum is a fixed butterfly.
#include <hip/hip_fp16.h>


#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

struct Row4Params {
    const uint8_t* codes;
    const uint16_t* scales;
    const uint8_t* zps;
    const void* x;
    void* y;
    const void* bias;
    int32_t N, K, nch;
    int32_t groups;
    int32_t y_dtype, bias_dtype, epilogue;
    SegTable seg;
};

__device__ __forceinline__ bf16x8 as_bf16x8(const u32x4& v) { return __builtin_bit_cast(bf16x8, v); }

// eight nibbles of a word -> four packed bf16 pairs holding 16 + code, in k order (nq_nib.h).  `magic` is
// 0x41804180 held in a vector register the compiler cannot see through: with two literal constants it emits
// an and and an or (an instruction takes one literal), with one a single v_and_or_b32.
__device__ __forceinline__ u32x4 nib_word_to_bf16(uint32_t w, uint32_t magic) {
    u32x4 r;
    r[0] = ((w << 3) & 0x00780078u) | magic;
    r[1] = ((w >> 1) & 0x00780078u) | magic;
    r[2] = ((w >> 5) & 0x00780078u) | magic;
    r[3] = ((w >> 9) & 0x00780078u) | magic;
    return r;
}

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

template <int FMT, bool XF32, int CPL, int WAVES, int RPW>
__global__ __launch_bounds__(64 * WAVES) void gemv_row4_kernel(const Row4Params p) {
    constexpr bool G128 = FMT == NQ_FMT_W4_GROUP;  // one scale and zero point per column and load
    constexpr int NT = XF32 ? 3 : 1;               // bf16 terms of x
    constexpr int KPAD = CPL * 2048;               // k covered by CPL loads of a wavefront
    constexpr int NTHR = 64 * WAVES;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t* const plane = lds;                                         // [NT][KPAD] bf16, chunk slots permuted
    float* const xsum = reinterpret_cast<float*>(lds + NT * KPAD * 2);  // [KPAD / 32], or [KPAD / 128] sums of four

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, kq = lane >> 4;
    const u32x4* wq = reinterpret_cast<const u32x4*>(p.codes);
    const int64_t row_first = ((int64_t)blockIdx.x * WAVES + wave) * RPW;

    // a row's codes and group records for this lane.  Codes: chunk 64 j + 4 c + q, clamped.  Records, the
    // same for the four lanes of a column: Q4_0 the four fp16 scales of chunks 4 c .. 4 c + 3 (8 bytes);
    // W4_GROUP the group's fp16 scale | zero point << 16.  A chunk past the row gets scale 0.
    auto fetch = [&](int64_t row, u32x4 (&wv)[CPL], uint2 (&meta)[CPL]) {
        const int64_t r = min(row, (int64_t)p.N - 1);
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            const int chunk = j * 64 + 4 * c + kq;
            wv[j] = __builtin_nontemporal_load(&wq[r * p.nch + min(chunk, p.nch - 1)]);
            const int c4 = j * 64 + 4 * c, c4c = min(c4, p.nch - 4);  // nch is a multiple of 4
            if constexpr (!G128) {
                uint2 rec = *reinterpret_cast<const uint2*>(p.scales + r * p.nch + c4c);
                const uint32_t keep = c4 < p.nch ? ~0u : 0u;
                rec.x &= keep, rec.y &= keep;
                meta[j] = rec;
            } else {
                const int g = c4c >> 2;  // groups of four chunks
                const uint32_t keep = c4 < p.nch ? ~0u : 0u;
                meta[j].x = (uint32_t)p.scales[r * p.groups + g] & keep;
                meta[j].y = (uint32_t)p.zps[r * p.groups + g];
            }
        }
    };

    // x first (it is staged first, and loads return in the order of issue), then all of this wavefront's rows: their
    // latency is paid once, under the staging of x.  The scheduling barrier keeps every load above the first wait.
    constexpr int XIT = (KPAD / 8 + NTHR - 1) / NTHR;  // staging steps per thread
    u32x4 xraw[XIT][XF32 ? 2 : 1];
#pragma unroll
    for (int it = 0; it < XIT; it++) {
        const int kc = min(min(tid + it * NTHR, KPAD / 8 - 1) * 8, p.K - 8);
        if constexpr (XF32) {
            xraw[it][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(p.x) + kc);
            xraw[it][XF32 ? 1 : 0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(p.x) + kc + 4);
        } else {
            xraw[it][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + kc);
        }
    }
    u32x4 wv[RPW][CPL];
    uint2 meta[RPW][CPL];
#pragma unroll
    for (int rr = 0; rr < RPW; rr++) fetch(row_first + rr, wv[rr], meta[rr]);
    // the epilogue's operand travels with the codes (raw: widening a bf16 bias here would wait for it)
    uint32_t braw[RPW];
#pragma unroll
    for (int rr = 0; rr < RPW; rr++) {
        braw[rr] = 0;
        if (p.bias) {
            const int64_t n = min(row_first + rr, (int64_t)p.N - 1);
            braw[rr] = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[n]
                                                   : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n];
        }
    }

    __builtin_amdgcn_sched_barrier(0);

    // ---- x -> LDS: 8 values per thread and step; 4 consecutive threads cover one chunk
#pragma unroll
    for (int it = 0; it < XIT; it++) {
        const int e = tid + it * NTHR;
        if (e >= KPAD / 8) break;  // (uniform over a wavefront)
        const int k0 = e * 8;
        const uint32_t keep = k0 < p.K ? ~0u : 0u;
        const int ch = e >> 2, blk = ch >> 6, cin = ch & 63;
        // byte offset in a plane: MFMA m = cin % 4 of the block reads one KiB, lane (c = cin / 4, q = e % 4) its 16 bytes
        const int at = blk * 4096 + (cin & 3) * 1024 + ((cin >> 2) + 16 * (e & 3)) * 16;
        float part;
        if constexpr (XF32) {
            const u32x4 r0 = xraw[it][0], r1 = xraw[it][XF32 ? 1 : 0];
            uint32_t v[8];
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = r0[i] & keep, v[4 + i] = r1[i] & keep;
            // hi + mid + lo = the fp32 value: each split truncates, so each residual is exact in fp32
            u32x4 t0, t1, t2;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t a = v[2 * i], b = v[2 * i + 1];
                const float ra = __uint_as_float(a) - __uint_as_float(a & 0xFFFF0000u);
                const float rb = __uint_as_float(b) - __uint_as_float(b & 0xFFFF0000u);
                const float sa = ra - __uint_as_float(__float_as_uint(ra) & 0xFFFF0000u);
                const float sb = rb - __uint_as_float(__float_as_uint(rb) & 0xFFFF0000u);
                t0[i] = __builtin_amdgcn_perm(b, a, 0x07060302u);
                t1[i] = __builtin_amdgcn_perm(__float_as_uint(rb), __float_as_uint(ra), 0x07060302u);
                t2[i] = __builtin_amdgcn_perm(__float_as_uint(sb), __float_as_uint(sa), 0x07060302u);
            }
            *reinterpret_cast<u32x4*>(plane + 0 * KPAD * 2 + at) = t0;
            *reinterpret_cast<u32x4*>(plane + 1 * KPAD * 2 + at) = t1;
            *reinterpret_cast<u32x4*>(plane + 2 * KPAD * 2 + at) = t2;
            part = ((__uint_as_float(v[0]) + __uint_as_float(v[1])) + (__uint_as_float(v[2]) + __uint_as_float(v[3]))) +
                   ((__uint_as_float(v[4]) + __uint_as_float(v[5])) + (__uint_as_float(v[6]) + __uint_as_float(v[7])));
        } else {
            u32x4 r0 = xraw[it][0];
#pragma unroll
            for (int i = 0; i < 4; i++) r0[i] &= keep;
            *reinterpret_cast<u32x4*>(plane + at) = r0;
            part = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; i++)
                part += __uint_as_float(r0[i] << 16) + __uint_as_float(r0[i] & 0xFFFF0000u);
        }
        // the chunk's sum over its four threads, then (groups of 128) over four chunks: butterflies in a fixed order
        part += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(part), 0xB1, 0xF, 0xF, false));
        part += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(part), 0x4E, 0xF, 0xF, false));
        if constexpr (G128) {
            part += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(part), 0x141, 0xF, 0xF, false));
            part += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(part), 0x140, 0xF, 0xF, false));
            if ((e & 15) == 0) xsum[e >> 4] = part;
        } else {
            if ((e & 3) == 0) xsum[ch] = part;
        }
    }
    __syncthreads();

    // lane-constant bit masks that pick the diagonal entry out of the MFMA's four registers (and-or, so that
    // the pick cannot become a branch around the MFMA's result)
    const int rsel = c & 3;
    const uint32_t k0 = rsel == 0 ? ~0u : 0u, k1 = rsel == 1 ? ~0u : 0u, k2 = rsel == 2 ? ~0u : 0u,
                   k3 = rsel == 3 ? ~0u : 0u;
    const bool holder = (c >> 2) == kq;
    uint32_t magic = 0x41804180u;
    asm volatile("" : "+v"(magic));  // kept in a vector register
    auto diag = [&](const f32x4& d) -> float {
        return __uint_as_float((__float_as_uint(d[0]) & k0) | (__float_as_uint(d[1]) & k1) |
                               (__float_as_uint(d[2]) & k2) | (__float_as_uint(d[3]) & k3));
    };

#pragma unroll
    for (int rr = 0; rr < RPW; rr++) {
        const int64_t row = row_first + rr;
        const float bias = __uint_as_float(p.bias_dtype == NQ_DT_F32 ? braw[rr] : braw[rr] << 16);
        const u32x4(&w)[CPL] = wv[rr];
        const uint2(&mt)[CPL] = meta[rr];
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < CPL; j++) {
            // words (registers) <-> 16-lane rows: a 4 x 4 transpose in two swap stages
            uint32_t w0 = w[j][0], w1 = w[j][1], w2 = w[j][2], w3 = w[j][3];
            {
                const auto s02 = __builtin_amdgcn_permlane32_swap(w0, w2, false, false);
                const auto s13 = __builtin_amdgcn_permlane32_swap(w1, w3, false, false);
                w0 = s02[0], w2 = s02[1], w1 = s13[0], w3 = s13[1];
                const auto s01 = __builtin_amdgcn_permlane16_swap(w0, w1, false, false);
                const auto s23 = __builtin_amdgcn_permlane16_swap(w2, w3, false, false);
                w0 = s01[0], w1 = s01[1], w2 = s23[0], w3 = s23[1];
            }
            const uint32_t tw[4] = {w0, w1, w2, w3};
            f32x4 dd = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const u32x4 bop = nib_word_to_bf16(tw[m], magic);
                if constexpr (!G128) dd = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    // x under chunk 64 j + 4 c + m, values 8 q .. 8 q + 7: lane l reads bytes 16 l of the MFMA's KiB
                    const u32x4 aop = *reinterpret_cast<const u32x4*>(plane + t * KPAD * 2 + j * 4096 + m * 1024 + lane * 16);
                    dd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop), as_bf16x8(bop), dd, 0, 0, 0);
                }
                if constexpr (!G128) {
                    const uint32_t sbits = (m < 2 ? mt[j].x : mt[j].y) >> (16 * (m & 1));
                    const float d = __half2float(__ushort_as_half((uint16_t)(sbits & 0xFFFFu)));
                    const float dsel = diag(dd);
                    acc = fmaf(d, fmaf(-24.0f, xsum[j * 64 + 4 * c + m], dsel), acc);
                }
            }
            if constexpr (G128) {
                const float d = __half2float(__ushort_as_half((uint16_t)(mt[j].x & 0xFFFFu)));
                const float zoff = 16.0f + (float)mt[j].y;
                const float dsel = diag(dd);
                acc = fmaf(d, fmaf(-zoff, xsum[j * 16 + c], dsel), acc);
            }
        }
        float v = holder ? acc : 0.0f;
        int t;
        t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, false);
        v += __int_as_float(t);
        t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, false);
        v += __int_as_float(t);
        t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xF, 0xF, false);
        v += __int_as_float(t);
        t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xF, 0xF, false);
        v += __int_as_float(t);
        {
            const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
            v = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
        }
        {
            const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
            v = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
        }
        if (lane == 0 && row < p.N) {
            float z = v + bias;
            if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
            void* yp;
            int width, col;
            seg_lookup(p.seg, (int)row, yp, width, col);  // M = 1: the part's row is its only row
            if (p.y_dtype == NQ_DT_F32)
                reinterpret_cast<float*>(yp)[col] = z;
            else
                reinterpret_cast<uint16_t*>(yp)[col] = f32_to_bf16_rne(z);
        }
    }
}

template <int FMT, bool XF32, int CPL, int WAVES, int RPW>
int32_t launch_one(const Row4Params& p, hipStream_t s) {
    constexpr int NT = XF32 ? 3 : 1;
    constexpr size_t lds = (size_t)NT * CPL * 2048 * 2 + (size_t)CPL * 64 * 4;
    auto kernel = gemv_row4_kernel<FMT, XF32, CPL, WAVES, RPW>;
    static LdsAttrOnce attr;
    if (lds > 48 * 1024) NQ_HIP(set_max_lds_once(attr, reinterpret_cast<const void*>(kernel), lds));
    const int rows_per_wg = WAVES * RPW;
    hipLaunchKernelGGL(kernel, dim3((unsigned)((p.N + rows_per_wg - 1) / rows_per_wg)), dim3(64 * WAVES), lds, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// One row per wavefront measured best on every shape tried (more rows per wavefront amortise the staging
// of x but leave fewer wavefronts to hide each other's waits); 8 wavefronts per workgroup, 16 for fp32 x.
template <int FMT, bool XF32, int CPL>
int32_t launch_rpw(const Row4Params& p, hipStream_t s) {
    if constexpr (XF32) return launch_one<FMT, XF32, CPL, 16, 1>(p, s);  // the three-term split of x: 16 rows share it
    return launch_one<FMT, XF32, CPL, 8, 1>(p, s);
}

template <int FMT, bool XF32>
int32_t launch_cpl(const Row4Params& p, int cpl, hipStream_t s) {
    switch (cpl) {
        case 1: return launch_rpw<FMT, XF32, 1>(p, s);
        case 2: return launch_rpw<FMT, XF32, 2>(p, s);
        case 3: return launch_rpw<FMT, XF32, 3>(p, s);
        case 4: return launch_rpw<FMT, XF32, 4>(p, s);
        case 5: return launch_rpw<FMT, XF32, 5>(p, s);
        case 6: return launch_rpw<FMT, XF32, 6>(p, s);
        case 7: return launch_rpw<FMT, XF32, 7>(p, s);
        case 8: return launch_rpw<FMT, XF32, 8>(p, s);
    }
    return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no 4-bit row GEMV for this IN");
}

}  // namespace

// a 4-bit weight of at least 2 MB whose rows are 1 .. 8 KiB of codes (2048 <= K <= 16384, K a multiple of
// 128; W4_GROUP: groups of exactly 128 k), one activation row in bf16 or fp32
bool gemv_row4_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (a.M != 1) return false;
    if (L->format != NQ_FMT_Q4_0 && !(L->format == NQ_FMT_W4_GROUP && L->group == 128)) return false;
    if (a.x_dtype != NQ_DT_BF16 && a.x_dtype != NQ_DT_F32) return false;
    if (L->in % 128 != 0 || L->in < 2048 || L->in > 16384) return false;
    return (int64_t)L->in * L->out >= ((int64_t)4 << 20);
}

int32_t launch_gemv_row4(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    Row4Params p{};
    p.codes = L->d_codes, p.scales = reinterpret_cast<const uint16_t*>(L->d_scales), p.zps = L->d_zps;
    p.x = a.x, p.y = a.y, p.bias = a.bias, p.seg = a.seg;
    p.N = L->out, p.K = L->in, p.nch = L->in / 32, p.groups = L->groups;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    const int cpl = (p.nch + 63) / 64;
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    if (L->format == NQ_FMT_Q4_0)
        return xf32 ? launch_cpl<NQ_FMT_Q4_0, true>(p, cpl, a.stream) : launch_cpl<NQ_FMT_Q4_0, false>(p, cpl, a.stream);
    return xf32 ? launch_cpl<NQ_FMT_W4_GROUP, true>(p, cpl, a.stream) : launch_cpl<NQ_FMT_W4_GROUP, false>(p, cpl, a.stream);
}

}  // namespace nq
