// Medium-M dequant GEMM on the bf16 matrix cores (v_mfma_f32_16x16x32_bf16):
//     y[M, N] = epi( x[M, K] @ deq(W)^T + bias ),  x bf16 or fp32,
//     W in Q4_0, W4_GROUP or W8_CHANNEL codes.
// This is the regime of the reference's real caller, the SmolVLA prefill at
// T = 135 tokens (noeira/deep_agents/smolvla/fused.mojo:255-384), and of
// BASELINE's M = 100 / 256 configs: the weights are ~1 MB, so the call is
// bound by instruction issue per wavefront and by what its loads cost in the
// L1, not by MFMA or bytes.  The medium-M kernel has no block-wide barrier in
// its K loop: every wavefront fetches its own operands (row-contiguous loads,
// x is L2-resident, W is read once per M tile), turns them into MFMA fragments
// through a private piece of LDS, and the only synchronisation is the final
// fixed-order reduction of the K-slices through LDS.  From 512 rows on a second
// kernel stages tiles per workgroup (below).
//
// Exactness.  Weights enter the MFMA as the integer codes, converted to bf16
// exactly: a 4-bit code q becomes 16 + q by OR-ing it into the mantissa of
// bf16 16.0 (one shift and one and-or per pair), an int8 code becomes q + 128.
// The offset is removed in fp32 with X = sum_k x_k, which a second MFMA against
// an all-ones operand provides in the same lane layout:
//     sum_k x_k (q_k - z) = P - (offset + z) X,
// and -(offset + z) X is handed to the product MFMA as its C operand.  Scales
// are applied in fp32 after the MFMA: per 32-wide chunk (one chunk = one Q4_0
// group = one MFMA), per 128-wide k-step where a k-step lies in one group
// (W4_GROUP with a group width that is a multiple of 128), once at the end for
// W8.
// bf16 activations are exact operands; fp32 activations are split into three
// bf16 terms hi + mid + lo that add up to the fp32 value exactly, so every
// product the matrix core forms is exact and only the fp32 accumulation rounds
// (the reference's own AMD path is an fp32 GEMM over deq(W), gate 1e-5).
//
// 4-bit device layout (see nq_q4_0.hip): a 16-byte chunk holds 32 consecutive
// k as four words of eight; lane (n, kb) takes the whole chunk c0 + kb of its
// row from the staging area with one 128-bit read, and two lane-swap stages
// (v_permlane32_swap, v_permlane16_swap) transpose the 4 x 4 words among the
// four lanes of a row so that lane kb ends up with word kb of chunks
// c0 .. c0+3: exactly its share of the B operand of four MFMAs.
#include <hip/hip_fp16.h>

#include <algorithm>


#include <atomic>

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
    int32_t groups;
    float inv_cpg;    // W4_GROUP: 1 / (16-byte chunks per group)
    float tscale;     // FP8_E4M3: the weight's per-tensor scale
    int32_t s_pairs;  // Q4_0: scale rows are 4-byte (1) or 8-byte (2) aligned, else 0
    int32_t nch;      // 16-byte chunks per weight row
    int32_t y_dtype, bias_dtype, epilogue;
    SegTable seg;
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// loads at a uniform base plus a 32-bit byte offset (one address register per lane)
__device__ __forceinline__ u32x4 ld16(const void* base, uint32_t off) {
    return *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(base) + off);
}
__device__ __forceinline__ uint32_t ld4(const void* base, uint32_t off) {
    return *reinterpret_cast<const uint32_t*>(reinterpret_cast<const char*>(base) + off);
}
__device__ __forceinline__ uint32_t ld2(const void* base, uint32_t off) {
    return *reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(base) + off);
}
__device__ __forceinline__ uint32_t ld1(const void* base, uint32_t off) {
    return *reinterpret_cast<const uint8_t*>(reinterpret_cast<const char*>(base) + off);
}

// LDS slot swizzles.  A 128-bit LDS read of a wavefront is served in four passes of 16 lanes, and a pass is
// not 16 consecutive lanes: within each half of the wavefront it takes the quads (groups of four lanes) whose
// index has even parity, then those with odd parity, i.e. lanes {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19,
// 28-31}, and the same + 32 (measured with the bank-conflict counter on single-wavefront access patterns).
// A pass is free of bank conflicts when its 16 lanes touch 16 different 16-byte slots modulo 256 bytes.
//   64-byte rows (weights): row r keeps piece p at slot p ^ wswz(r); with lane (row ln, piece kb) reading,
//     wswz = -(r / 4) mod 4 separates the four quads of every pass.
//   128-byte rows (activations, two pieces per lane-row apart by D slots between kb and kb + 1): slot
//     p ^ xswz128(r, D); rows two apart differ by r / 2, and the quads that a pass takes from kb + 1 get D more.
__device__ __forceinline__ int wswz(int r) { return (0 - (r >> 2)) & 3; }
__device__ __forceinline__ int xswz128(int r, int d) { return ((r >> 1) ^ ((((r >> 2) ^ (r >> 3)) & 1) * d)) & 7; }

// eight 4-bit codes of one word (pair s = elements 2s, 2s+1 in nibbles s and s+4) -> bf16 16+q.
// `magic` is 0x41804180 (bf16 16.0 twice) held in a vector register whose value the compiler
// cannot see, which makes it fuse the mask and the OR into one v_and_or_b32.
__device__ __forceinline__ u32x4 nib_word_to_bf16(uint32_t w, uint32_t magic) {
    u32x4 r;
    r[0] = ((w << 3) & 0x00780078u) | magic;
    r[1] = ((w >> 1) & 0x00780078u) | magic;
    r[2] = ((w >> 5) & 0x00780078u) | magic;
    r[3] = ((w >> 9) & 0x00780078u) | magic;
    return r;
}

// four int8 codes of one word -> two bf16 pairs holding q + 128 (exact)
__device__ __forceinline__ void i8_word_to_bf16(uint32_t w, uint32_t& p0, uint32_t& p1) {
    const uint32_t t = w ^ 0x80808080u;
    const float f0 = (float)(t & 0xFFu), f1 = (float)((t >> 8) & 0xFFu);
    const float f2 = (float)((t >> 16) & 0xFFu), f3 = (float)(t >> 24);
    // values <= 255 have at most 8 significant bits: the high half of the fp32 is the exact bf16
    p0 = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
    p1 = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
}

// four fp8 e4m3 codes of one word -> two bf16 pairs holding the decoded values (exact: 4 significant bits;
// the hardware converter decodes OCP e4m3fn, NaN codes included)
__device__ __forceinline__ void fp8_word_to_bf16(uint32_t w, uint32_t& p0, uint32_t& p1) {
    typedef __attribute__((ext_vector_type(2))) float f32x2;
    const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    p0 = __builtin_amdgcn_perm(__float_as_uint(a[1]), __float_as_uint(a[0]), 0x07060302u);
    p1 = __builtin_amdgcn_perm(__float_as_uint(b[1]), __float_as_uint(b[0]), 0x07060302u);
}

template <int FMT>
__device__ __forceinline__ void byte_word_to_bf16(uint32_t w, uint32_t& p0, uint32_t& p1) {
    if constexpr (FMT == NQ_FMT_FP8_E4M3)
        fp8_word_to_bf16(w, p0, p1);
    else
        i8_word_to_bf16(w, p0, p1);
}

// A-operand terms of 8 consecutive activations held raw in registers: one term for bf16
// input, three for fp32 (hi + mid + lo = the fp32 value exactly: each split truncates, so
// each residual is exact in fp32 and the third has at most 8 significant bits).  A term pair
// is the two high halves, gathered with one byte permute.
template <bool XF32>
__device__ __forceinline__ void make_terms(const u32x4 (&raw)[XF32 ? 2 : 1], u32x4 (&t)[XF32 ? 3 : 1]) {
    if constexpr (!XF32) {
        t[0] = raw[0];
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t a = raw[i >> 1][(2 * i) & 3], b = raw[i >> 1][(2 * i + 1) & 3];
            const float ra = __uint_as_float(a) - __uint_as_float(a & 0xFFFF0000u);
            const float rb = __uint_as_float(b) - __uint_as_float(b & 0xFFFF0000u);
            const float sa = ra - __uint_as_float(__float_as_uint(ra) & 0xFFFF0000u);
            const float sb = rb - __uint_as_float(__float_as_uint(rb) & 0xFFFF0000u);
            t[0][i] = __builtin_amdgcn_perm(b, a, 0x07060302u);
            t[1][i] = __builtin_amdgcn_perm(__float_as_uint(rb), __float_as_uint(ra), 0x07060302u);
            t[2][i] = __builtin_amdgcn_perm(__float_as_uint(sb), __float_as_uint(sa), 0x07060302u);
        }
    }
}

// One workgroup computes a [16 MW] x [16 NW] output tile; its KW wavefronts split K by
// k-steps (wave w takes k-steps w, w + KW, ...).  Calls of this size are bound by how many
// instructions one wavefront executes back to back and by what its loads cost in the L1
// (a load instruction is priced by the number of separate pieces of cache line its lanes
// touch, not by its bytes: 64 lanes reading 16 bytes each from 16 rows, the four lanes of a
// row 16 lanes apart, take about 100 cycles of the L1; the same bytes with a row's lanes
// adjacent about 45; two-byte loads cost as much as 16-byte ones), which shapes the kernel:
//   - operands are loaded row-contiguously (a run of lanes per row) into registers one k-step
//     ahead, and reach the MFMA operand layout through a private piece of LDS per wavefront:
//     one 128-bit store and one 128-bit read per register quad, both free of bank conflicts
//     (XOR swizzle of the 16-byte slot by the row), no barrier (LDS executes one wavefront's
//     accesses in order);
//   - a wavefront's activations are the large operand (2 or 4 bytes an element against half
//     a byte or one byte of weight), so the tile is wide in N: every activation fragment,
//     and for fp32 input its three-term split, is formed once for NW weight tiles;
//   - scale records come in as few loads as their alignment allows;
//   - the zero-point term enters the MFMA as its C operand, and where a whole k-step lies in
//     one group (WHOLE) the scale is applied once per k-step instead of once per chunk.
template <int FMT, bool XF32, int MW, int NW, int KW, bool WHOLE>
__global__ __launch_bounds__(64 * KW) void gemm_a16_kernel(const A16Params p) {
    constexpr bool FOUR_BIT = (FMT != NQ_FMT_W8_CHANNEL && FMT != NQ_FMT_FP8_E4M3);
    constexpr int NT = XF32 ? 3 : 1;            // bf16 terms per activation
    constexpr int NL = XF32 ? 2 : 1;            // 16-byte pieces per activation fragment
    constexpr int ES = XF32 ? 4 : 2;            // bytes per activation
    constexpr int KSTEP = FOUR_BIT ? 128 : 64;  // k covered by 64 bytes of a weight row
    constexpr int NMF = FOUR_BIT ? 4 : 2;       // MFMAs (32 k each) per k-step
    constexpr int NS = WHOLE ? 1 : 4;           // scale records per k-step and weight row
    constexpr int TA = MW * NW * 4;             // accumulator registers per lane
    constexpr int RED = TA * 64;                // floats one wavefront contributes to the reduction
    constexpr int EPW = (TA + KW - 1) / KW;     // accumulators one wavefront finishes
    // activations travel in units of 16 rows x XB bytes: NI loads, each RPI rows x XB bytes
    constexpr int XB = (!FOUR_BIT && !XF32) ? 128 : 256;
    constexpr int NU = KSTEP * ES / XB;  // units per k-step
    constexpr int QU = NMF / NU;         // MFMA fragments per unit
    constexpr int PPR = XB / 16;         // 16-byte pieces per row of a unit
    constexpr int RPI = 64 / PPR;        // rows per load instruction
    constexpr int NI = 16 / RPI;         // load instructions per unit
    constexpr int KU = XB / ES;          // k per unit
    constexpr int XS = 16 * XB;          // bytes of the activation staging area
    constexpr int SCR = XS + NW * 1024;  // staging bytes per wavefront
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // max(KW SCR, KW RED floats)
    float* red = reinterpret_cast<float*>(smem);                    // [KW][RED], after the K loop

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ln = lane & 15, kb = lane >> 4;
    const int n_base = blockIdx.x * (16 * NW);
    const int m_base = blockIdx.y * (16 * MW);
    uint8_t* scr = smem + wave * SCR;

    const u32x4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    uint32_t magic = 0x41804180u;
    asm volatile("" : "+v"(magic));

    // ---- the lane's place in a load: weights, row lane/4 of a 16-row tile and 16-byte piece lane%4 of the
    // k-step's 64 bytes; activations, row lane/PPR of the instruction's RPI rows and piece lane%PPR
    const int wrow = lane >> 2, wpc = lane & 3;
    const int trow = lane / PPR, tpc = lane % PPR;

    // byte offsets of the rows this lane loads (the host has checked that every operand is < 4 GiB)
    uint32_t xoff[MW][NI], woff[NW], soff[NW];
#pragma unroll
    for (int i = 0; i < MW; i++)
#pragma unroll
        for (int ii = 0; ii < NI; ii++)
            xoff[i][ii] = (uint32_t)min(m_base + 16 * i + ii * RPI + trow, p.M - 1) * (uint32_t)p.K * ES;
#pragma unroll
    for (int j = 0; j < NW; j++) {
        woff[j] = (uint32_t)min(n_base + 16 * j + wrow, p.N - 1) * (uint32_t)p.nch * 16u;
        const uint32_t n = (uint32_t)min(n_base + 16 * j + ln, p.N - 1);
        soff[j] = n * (uint32_t)(FMT == NQ_FMT_Q4_0 ? p.nch : p.groups);  // in elements
    }

    const int nsteps = (p.K + KSTEP - 1) / KSTEP;

    // ---- loaders: unconditional, from clamped addresses; what lies past K is multiplied by a
    // zero scale (4-bit formats) and meets zero activations
    auto load_w = [&](int ks, u32x4 (&dst)[NW]) {
        const uint32_t c = (uint32_t)min(ks * 4 + wpc, p.nch - 1) * 16u;  // the 16-byte chunk this lane loads
#pragma unroll
        for (int j = 0; j < NW; j++) dst[j] = ld16(p.codes, woff[j] + c);
    };
    // Scale records.  A load instruction costs the same whether its lanes fetch 2 bytes or 16, and the
    // four lanes (kb = 0..3) that share a weight row would all fetch the same record: instead lane
    // (row, kb) fetches the record of the wavefront's k-step ks + kb KW, so one set of loads serves
    // four consecutive k-steps of the wavefront ("a quad"), and each k-step picks its record out of
    // the lane that holds it with a lane permute (ds_bpermute).  The loads return raw registers and
    // nothing is computed from them here: an instruction that uses a loaded value right away would
    // make the wavefront wait out the whole memory latency at the point of the prefetch.  decode_s
    // turns them into fp16 scale | zero point << 16 when the k-step is consumed.
    constexpr int NR = FMT == NQ_FMT_Q4_0 ? 4 : FMT == NQ_FMT_W4_GROUP ? 2 * NS : 1;
    auto load_s = [&](int ks0, uint32_t (&dst)[NW][NR]) {
        const int ks = ks0 + kb * KW;  // this lane's k-step of the quad
        if constexpr (FMT == NQ_FMT_Q4_0) {
            if (p.s_pairs) {  // rows are 4- or 8-byte aligned (the last load may run 4 bytes past a row)
                const uint32_t c0 = (uint32_t)min(ks, nsteps - 1) * 8u;
#pragma unroll
                for (int j = 0; j < NW; j++) {
                    if (p.s_pairs == 2) {
                        const u32x2 v = *reinterpret_cast<const u32x2*>(reinterpret_cast<const char*>(p.scales) +
                                                                        (soff[j] * 2u + c0));
                        dst[j][0] = v[0], dst[j][1] = v[1];
                    } else {
                        dst[j][0] = ld4(p.scales, soff[j] * 2u + c0), dst[j][1] = ld4(p.scales, soff[j] * 2u + c0 + 4u);
                    }
                    dst[j][2] = 0, dst[j][3] = 0;
                }
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t cc = (uint32_t)min(ks * 4 + q, p.nch - 1);
#pragma unroll
                    for (int j = 0; j < NW; j++) dst[j][q] = ld2(p.scales, (soff[j] + cc) * 2u);
                }
            }
        } else if constexpr (FMT == NQ_FMT_W4_GROUP) {
#pragma unroll
            for (int q = 0; q < NS; q++) {
                const int cc = min(ks * 4 + q, p.nch - 1);
                const uint32_t g = (uint32_t)(((float)cc + 0.5f) * p.inv_cpg);  // cc / chunks per group
#pragma unroll
                for (int j = 0; j < NW; j++) {
                    dst[j][2 * q] = ld2(p.scales, (soff[j] + g) * 2u);
                    dst[j][2 * q + 1] = ld1(p.zps, soff[j] + g);
                }
            }
        }
    };
    // t: the k-step's place in its quad (0..3); its records sit in the lanes kb = t of each row
    auto decode_s = [&](const uint32_t (&raw)[NW][NR], int t, uint32_t (&sc)[NW][NS]) {
        const int src = (ln + 16 * t) * 4;
        auto pick = [&](uint32_t v) { return (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)v); };
#pragma unroll
        for (int j = 0; j < NW; j++) {
            if constexpr (FMT == NQ_FMT_Q4_0) {
                if (p.s_pairs) {
                    const uint32_t v0 = pick(raw[j][0]), v1 = pick(raw[j][1]);
                    sc[j][0] = v0 & 0xFFFFu, sc[j][1] = v0 >> 16;
                    sc[j][2] = v1 & 0xFFFFu, sc[j][3] = v1 >> 16;
                } else {
#pragma unroll
                    for (int q = 0; q < 4; q++) sc[j][q] = pick(raw[j][q]);
                }
            } else if constexpr (FMT == NQ_FMT_W4_GROUP) {
#pragma unroll
                for (int q = 0; q < NS; q++) sc[j][q] = pick(raw[j][2 * q] | (raw[j][2 * q + 1] << 16));
            }
        }
    };
    // (a piece can lie past K only in a k-step that K cuts short: its address is clamped here
    // and its value replaced by zero when the registers are staged)
    auto load_x = [&](int ks, int i, int u, u32x4 (&dst)[NI]) {
        int k0 = ks * KSTEP + u * KU + tpc * (16 / ES);
        if (k0 >= p.K) k0 = 0;
#pragma unroll
        for (int ii = 0; ii < NI; ii++) dst[ii] = ld16(p.x, xoff[i][ii] + (uint32_t)k0 * ES);
    };
    auto scale_of = [&](uint32_t rec, bool valid) {
        return valid ? __half2float(__ushort_as_half((uint16_t)(rec & 0xFFFFu))) : 0.0f;
    };
    auto zero_of = [&](uint32_t rec) {  // 16 (the conversion offset) + the zero point
        return (FMT == NQ_FMT_Q4_0) ? 24.0f : 16.0f + (float)(rec >> 16);
    };
    auto lds16 = [&](uint32_t off) -> u32x4& { return *reinterpret_cast<u32x4*>(scr + off); };

    u32x4 wv[NW];
    uint32_t sv[NW][NR];
    u32x4 xr[MW][NU][NI];
    load_w(wave, wv);
#pragma unroll
    for (int u = 0; u < NU; u++)
#pragma unroll
        for (int i = 0; i < MW; i++) load_x(wave, i, u, xr[i][u]);
    load_s(wave, sv);

    // (everything from here to the loop is set up while the first loads are in flight)
    f32x4 acc[MW][NW];
    f32x4 xacc[MW];  // W8 only: sum_k x_k over the wave's k-steps
#pragma unroll
    for (int i = 0; i < MW; i++) {
        xacc[i] = (f32x4){0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < NW; j++) acc[i][j] = (f32x4){0, 0, 0, 0};
    }

    // ---- where a loaded register goes in the staging area and where a fragment (MFMA layout) comes from
    // weights: staged at row * 64 + (piece ^ wswz(row)) * 16 and read back as (row ln, piece kb)
    const uint32_t w_st = XS + wrow * 64 + ((wpc ^ wswz(wrow)) & 3) * 16;
    const uint32_t w_rd = XS + ln * 64 + ((kb ^ wswz(ln)) & 3) * 16;
    // activations: staged at row * XB + (piece ^ f(row)) * 16 with f(row) = row (XB = 256) or xswz128 (XB = 128)
    auto swz = [](int row) {
        if (XB == 128) return xswz128(row, 2);
        // 256-byte rows: lane (row ln, kb) reads piece c + D kb, and piece ^ row separates the quads of a pass
        // for D = 1 and 2 (the 4-bit formats); int8 weights with fp32 x have D = 4 and need it added for rows 4 .. 11
        return (!FOUR_BIT && XF32) ? (row ^ ((((row >> 2) ^ (row >> 3)) & 1) * 4)) : row;
    };
    uint32_t x_st[NI], x_rd[QU][NL];
#pragma unroll
    for (int ii = 0; ii < NI; ii++) {
        const int row = ii * RPI + trow;
        x_st[ii] = row * XB + ((tpc ^ swz(row)) & (PPR - 1)) * 16;
    }
#pragma unroll
    for (int qq = 0; qq < QU; qq++)
#pragma unroll
        for (int h = 0; h < NL; h++) {
            // the piece that holds the first 8 k of fragment q of this lane (second half: + 4) within its unit
            const int piece = FOUR_BIT ? (XF32 ? 8 * qq + 2 * kb + h : 4 * qq + kb)
                                       : (XF32 ? 4 * kb + 2 * qq + h : 2 * kb + qq);
            x_rd[qq][h] = ln * XB + ((piece ^ swz(ln)) & (PPR - 1)) * 16;
        }

    // the accumulators this wavefront finishes after the reduction are idx = wave + t KW; their
    // per-channel operands are requested now so that nothing is loaded after the reduction
    // (raw: a bf16 bias is widened where it is used; a shift here would make the wavefront wait for
    // the load before its operands are even requested)
    float ep_scale[EPW];
    uint32_t ep_bias[EPW];
#pragma unroll
    for (int t = 0; t < EPW; t++) {
        const int idx = min(wave + t * KW, TA - 1);
        const int n = min(n_base + 16 * ((idx >> 2) % NW) + ln, p.N - 1);
        ep_scale[t] = (FMT == NQ_FMT_W8_CHANNEL) ? reinterpret_cast<const float*>(p.scales)[n]
                      : (FMT == NQ_FMT_FP8_E4M3)  ? p.tscale
                                                   : 1.0f;
        ep_bias[t] = 0;
        if (p.bias)
            ep_bias[t] = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[n]
                                                     : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n];
    }

    int t4 = 0;  // the k-step's place in its quad of scale records
    for (int ks = wave; ks < nsteps; ks += KW, t4 = (t4 + 1) & 3) {
        const int kn = ks + KW;  // the k-step the registers are refilled for, if there is one
        const bool more = kn < nsteps;
        u32x4 wc[NW];
        uint32_t sc[NW][NS];
#pragma unroll
        for (int j = 0; j < NW; j++) lds16(w_st + j * 1024) = wv[j];
        decode_s(sv, t4, sc);
        if (more) {
            load_w(kn, wv);
            if (t4 == 3) load_s(kn, sv);  // the next quad (this one's last record has just been taken)
        }
#pragma unroll
        for (int j = 0; j < NW; j++) wc[j] = lds16(w_rd + j * 1024);

        if constexpr (FOUR_BIT) {
            // ---- transpose words among the four lanes (kb = 0..3) that share a row
#pragma unroll
            for (int j = 0; j < NW; j++) {
                auto s02 = __builtin_amdgcn_permlane32_swap(wc[j][0], wc[j][2], false, false);
                auto s13 = __builtin_amdgcn_permlane32_swap(wc[j][1], wc[j][3], false, false);
                wc[j][0] = s02[0], wc[j][2] = s02[1], wc[j][1] = s13[0], wc[j][3] = s13[1];
                auto t01 = __builtin_amdgcn_permlane16_swap(wc[j][0], wc[j][1], false, false);
                auto t23 = __builtin_amdgcn_permlane16_swap(wc[j][2], wc[j][3], false, false);
                wc[j][0] = t01[0], wc[j][1] = t01[1], wc[j][2] = t23[0], wc[j][3] = t23[1];
            }
        }

        // WHOLE: one group for the whole k-step, the four chunks are summed in the MFMA accumulator
        f32x4 xs_w[MW], pp_w[MW][NW];
        if constexpr (FOUR_BIT && WHOLE) {
#pragma unroll
            for (int i = 0; i < MW; i++) {
                xs_w[i] = (f32x4){0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < NW; j++) pp_w[i][j] = (f32x4){0, 0, 0, 0};
            }
        }

#pragma unroll
        for (int u = 0; u < NU; u++) {
            // ---- the unit's activations: registers -> staging -> fragments; refill the registers
            u32x4 fr[MW][QU][NL];
#pragma unroll
            for (int i = 0; i < MW; i++) {
                if ((ks + 1) * KSTEP > p.K) {  // uniform over the wavefront
                    const bool in = ks * KSTEP + u * KU + tpc * (16 / ES) < p.K;
#pragma unroll
                    for (int ii = 0; ii < NI; ii++) xr[i][u][ii] = in ? xr[i][u][ii] : (u32x4){0, 0, 0, 0};
                }
#pragma unroll
                for (int ii = 0; ii < NI; ii++) lds16(x_st[ii]) = xr[i][u][ii];
                if (more) load_x(kn, i, u, xr[i][u]);
#pragma unroll
                for (int qq = 0; qq < QU; qq++)
#pragma unroll
                    for (int h = 0; h < NL; h++) fr[i][qq][h] = lds16(x_rd[qq][h]);
            }
#pragma unroll
            for (int qq = 0; qq < QU; qq++) {
                const int q = u * QU + qq;
                u32x4 bop[NW];
                if constexpr (FOUR_BIT) {
#pragma unroll
                    for (int j = 0; j < NW; j++) bop[j] = nib_word_to_bf16(wc[j][q], magic);
                } else {
#pragma unroll
                    for (int j = 0; j < NW; j++) {
                        uint32_t b0, b1, b2, b3;
                        byte_word_to_bf16<FMT>(wc[j][2 * q], b0, b1);
                        byte_word_to_bf16<FMT>(wc[j][2 * q + 1], b2, b3);
                        bop[j] = (u32x4){b0, b1, b2, b3};
                    }
                }
                const bool cvalid = ks * 4 + q < p.nch;  // (activations past K arrive as zeros)
#pragma unroll
                for (int i = 0; i < MW; i++) {
                    u32x4 at[NT];
                    make_terms<XF32>(fr[i][qq], at);
                    if constexpr (FOUR_BIT && WHOLE) {
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            xs_w[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(ones),
                                                                               xs_w[i], 0, 0, 0);
#pragma unroll
                            for (int j = 0; j < NW; j++)
                                pp_w[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                    as_bf16x8(at[t]), as_bf16x8(bop[j]), pp_w[i][j], 0, 0, 0);
                        }
                    } else if constexpr (FOUR_BIT) {
                        f32x4 xs = {0, 0, 0, 0};
#pragma unroll
                        for (int t = 0; t < NT; t++)
                            xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(ones), xs, 0, 0,
                                                                          0);
#pragma unroll
                        for (int j = 0; j < NW; j++) {
                            // the zero-point term -(16 + z) sum_k x_k is the MFMA's C operand
                            const float cz = zero_of(sc[j][q]);
                            f32x4 pp;
#pragma unroll
                            for (int r = 0; r < 4; r++) pp[r] = -cz * xs[r];
#pragma unroll
                            for (int t = 0; t < NT; t++)
                                pp = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(bop[j]), pp,
                                                                              0, 0, 0);
                            const float cs = scale_of(sc[j][q], cvalid);
#pragma unroll
                            for (int r = 0; r < 4; r++) acc[i][j][r] = fmaf(cs, pp[r], acc[i][j][r]);
                        }
                    } else {
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            if constexpr (FMT == NQ_FMT_W8_CHANNEL)
                                xacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(ones),
                                                                                  xacc[i], 0, 0, 0);
#pragma unroll
                            for (int j = 0; j < NW; j++)
                                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(bop[j]),
                                                                                    acc[i][j], 0, 0, 0);
                        }
                    }
                }
            }
        }

        if constexpr (FOUR_BIT && WHOLE) {
#pragma unroll
            for (int j = 0; j < NW; j++) {
                const float cs = scale_of(sc[j][0], true), cz = zero_of(sc[j][0]);
#pragma unroll
                for (int i = 0; i < MW; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        acc[i][j][r] = fmaf(cs, fmaf(-cz, xs_w[i][r], pp_w[i][j][r]), acc[i][j][r]);
            }
        }
    }

    if constexpr (FMT == NQ_FMT_W8_CHANNEL) {
#pragma unroll
        for (int i = 0; i < MW; i++)
#pragma unroll
            for (int j = 0; j < NW; j++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[i][j][r] = fmaf(-128.0f, xacc[i][r], acc[i][j][r]);
    }

    // ---- combine the K-slices: every wavefront posts its partial tile, then wavefront w sums
    // accumulators w, w + KW, ... over the slices in wave order (fixed, so results repeat bit
    // for bit) and stores them
    __syncthreads();  // the reduction area overlays the staging areas
#pragma unroll
    for (int i = 0; i < MW; i++)
#pragma unroll
        for (int j = 0; j < NW; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) red[wave * RED + ((i * NW + j) * 4 + r) * 64 + lane] = acc[i][j][r];
    __syncthreads();
#pragma unroll
    for (int t = 0; t < EPW; t++) {
        const int idx = wave + t * KW;
        if (TA % KW != 0 && idx >= TA) break;
        float part[KW];
#pragma unroll
        for (int w = 0; w < KW; w++) part[w] = red[w * RED + idx * 64 + lane];
        float z = part[0];
#pragma unroll
        for (int w = 1; w < KW; w++) z += part[w];
        const int r = idx & 3, j = (idx >> 2) % NW, i = (idx >> 2) / NW;
        const int n = n_base + 16 * j + ln;
        const int m = m_base + 16 * i + 4 * kb + r;  // D layout: row 4*(lane/16) + r, column lane%16
        if (!FOUR_BIT) z *= ep_scale[t];
        z += p.bias_dtype == NQ_DT_F32 ? __uint_as_float(ep_bias[t]) : __uint_as_float(ep_bias[t] << 16);
        if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
        if (p.epilogue == NQ_EPI_SWIGLU) {
            // (uniform) even columns are gate rows, the odd column next to each its up row, one lane over
            const float other = lane_xor1(z);
            if ((n & 1) == 0 && n + 1 < p.N && m < p.M) {
                const float g = swiglu_f32(other, z);
                const int64_t o = (int64_t)m * (p.N >> 1) + (n >> 1);
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(p.y)[o] = g;
                else
                    reinterpret_cast<uint16_t*>(p.y)[o] = f32_to_bf16_rne(g);
            }
            continue;
        }
        if (n < p.N && m < p.M) {
            void* yp;
            int width, col;
            seg_lookup(p.seg, n, yp, width, col);
            const int64_t o = (int64_t)m * width + col;
            if (p.y_dtype == NQ_DT_F32)
                reinterpret_cast<float*>(yp)[o] = z;
            else
                reinterpret_cast<uint16_t*>(yp)[o] = f32_to_bf16_rne(z);
        }
    }
}

// ---- Many rows (hundreds and more).  The kernel above re-reads and re-unpacks a weight tile for
// every 16 or 32 rows of activations; here one workgroup of four wavefronts (2 x 2) owns a
// [32 MT] x 128 tile of y and walks all of K, so a weight is unpacked once per 32 MT rows:
//   - per k-step the workgroup stages its activation rows (32 MT x KSTEP) and its 128 weight
//     rows (64 bytes each) in LDS, row-contiguous loads into registers one k-step ahead, one
//     128-bit store per register quad, XOR-swizzled slots as above; two buffers, one barrier
//     per k-step;
//   - a wavefront reads its MT x 4 fragments per MFMA k-extent and its four weight tiles from
//     LDS and multiplies MT x 4 output tiles of 16 x 16 (4 MT accumulator quads per lane);
//   - scale records: one set of loads per four k-steps, as above;
//   - the arithmetic per MFMA (exact codes, zero point through the C operand, scale in fp32 per
//     chunk or per k-step, exact three-term split of fp32 activations) is the kernel above's.
template <int FMT, bool XF32, int MT, int NW, bool WHOLE>
__global__ __launch_bounds__(128 * (8 / NW)) void gemm_a16_big_kernel(const A16Params p) {
    constexpr bool FOUR_BIT = (FMT != NQ_FMT_W8_CHANNEL && FMT != NQ_FMT_FP8_E4M3);
    constexpr int NT = XF32 ? 3 : 1;
    constexpr int NL = XF32 ? 2 : 1;
    constexpr int ES = XF32 ? 4 : 2;
    constexpr int KSTEP = FOUR_BIT ? 128 : 64;
    constexpr int NMF = FOUR_BIT ? 4 : 2;
    constexpr int NS = WHOLE ? 1 : 4;
    constexpr int WN = 8 / NW;             // wavefronts along N (NW weight tiles of 16 rows each): 2 x WN wavefronts
    constexpr int NTHR = 128 * WN;
    constexpr int BM = 32 * MT, BN = 128;  // the workgroup's tile
    constexpr int XB = KSTEP * ES;         // bytes of an activation row per k-step (128, 256 or 512)
    constexpr int PPR = XB / 16;           // 16-byte pieces of it
    constexpr int XTILE = BM * XB, WTILE = BN * 64, STAGE = XTILE + WTILE;
    constexpr int XI = BM * PPR / NTHR;    // activation pieces per thread and k-step
    constexpr int WI = 512 / NTHR;         // weight pieces per thread and k-step
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];  // [2][STAGE]

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ln = lane & 15, kb = lane >> 4;
    const int wm = wave / WN, wn = wave % WN;
    const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;

    const u32x4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    uint32_t magic = 0x41804180u;
    asm volatile("" : "+v"(magic));
    auto swz = [](int row) {
        if (XB < 256) return xswz128(row, 2);
        return ((!FOUR_BIT && XF32) ? (row ^ ((((row >> 2) ^ (row >> 3)) & 1) * 4)) : row) & 15;
    };

    // ---- staging: piece g = i NTHR + tid of the tile -> row g / PPR, piece g % PPR
    uint32_t xsrc[XI], xdst[XI];
    int xpc[XI];
#pragma unroll
    for (int i = 0; i < XI; i++) {
        const int g = i * NTHR + tid, row = g / PPR, pc = g % PPR;
        xsrc[i] = (uint32_t)min(m0 + row, p.M - 1) * (uint32_t)p.K * ES + pc * 16;
        xdst[i] = row * XB + ((pc ^ swz(row)) & (PPR - 1)) * 16;
        xpc[i] = pc;
    }
    uint32_t wsrc[WI], wdst[WI];
#pragma unroll
    for (int i = 0; i < WI; i++) {
        const int g = i * NTHR + tid, row = g >> 2, pc = g & 3;
        wsrc[i] = (uint32_t)min(n0 + row, p.N - 1) * (uint32_t)p.nch * 16u;
        wdst[i] = XTILE + row * 64 + ((pc ^ wswz(row)) & 3) * 16;
    }
    const int wpc = tid & 3;
    // ---- fragments
    uint32_t a_rd[MT][NMF][NL], b_rd[NW];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int q = 0; q < NMF; q++)
#pragma unroll
            for (int h = 0; h < NL; h++) {
                const int piece = FOUR_BIT ? (XF32 ? 8 * q + 2 * kb + h : 4 * q + kb) : (XF32 ? 4 * kb + 2 * q + h : 2 * kb + q);
                a_rd[i][q][h] = (wm * 16 * MT + 16 * i + ln) * XB + ((piece ^ swz(ln)) & (PPR - 1)) * 16;
            }
#pragma unroll
    for (int j = 0; j < NW; j++) b_rd[j] = XTILE + (wn * 16 * NW + 16 * j + ln) * 64 + ((kb ^ wswz(ln)) & 3) * 16;

    uint32_t soff[NW];
#pragma unroll
    for (int j = 0; j < NW; j++) {
        const uint32_t n = (uint32_t)min(n0 + wn * 16 * NW + 16 * j + ln, p.N - 1);
        soff[j] = n * (uint32_t)(FMT == NQ_FMT_Q4_0 ? p.nch : p.groups);
    }
    const int nsteps = (p.K + KSTEP - 1) / KSTEP;

    u32x4 xv[XI], wv[WI];
    auto load_tiles = [&](int ks) {
        const int k0 = ks * KSTEP;
#pragma unroll
        for (int i = 0; i < XI; i++) {
            int k = k0 + xpc[i] * (16 / ES);
            if (k >= p.K) k = 0;
            xv[i] = ld16(p.x, xsrc[i] + (uint32_t)(k - xpc[i] * (16 / ES)) * ES);
        }
        const uint32_t c = (uint32_t)min(ks * 4 + wpc, p.nch - 1) * 16u;
#pragma unroll
        for (int i = 0; i < WI; i++) wv[i] = ld16(p.codes, wsrc[i] + c);
    };
    // scale records: lane (row, kb) fetches those of k-step ks0 + kb (one set of loads per four k-steps)
    constexpr int NR = FMT == NQ_FMT_Q4_0 ? 4 : FMT == NQ_FMT_W4_GROUP ? 2 * NS : 1;
    uint32_t sv[NW][NR];
    auto load_s = [&](int ks0) {
        const int ks = ks0 + kb;
        if constexpr (FMT == NQ_FMT_Q4_0) {
            if (p.s_pairs) {
                const uint32_t c0 = (uint32_t)min(ks, nsteps - 1) * 8u;
#pragma unroll
                for (int j = 0; j < NW; j++) {
                    if (p.s_pairs == 2) {
                        const u32x2 v = *reinterpret_cast<const u32x2*>(reinterpret_cast<const char*>(p.scales) +
                                                                        (soff[j] * 2u + c0));
                        sv[j][0] = v[0], sv[j][1] = v[1];
                    } else {
                        sv[j][0] = ld4(p.scales, soff[j] * 2u + c0), sv[j][1] = ld4(p.scales, soff[j] * 2u + c0 + 4u);
                    }
                }
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t cc = (uint32_t)min(ks * 4 + q, p.nch - 1);
#pragma unroll
                    for (int j = 0; j < NW; j++) sv[j][q] = ld2(p.scales, (soff[j] + cc) * 2u);
                }
            }
        } else if constexpr (FMT == NQ_FMT_W4_GROUP) {
#pragma unroll
            for (int q = 0; q < NS; q++) {
                const int cc = min(ks * 4 + q, p.nch - 1);
                const uint32_t g = (uint32_t)(((float)cc + 0.5f) * p.inv_cpg);
#pragma unroll
                for (int j = 0; j < NW; j++) {
                    sv[j][2 * q] = ld2(p.scales, (soff[j] + g) * 2u);
                    sv[j][2 * q + 1] = ld1(p.zps, soff[j] + g);
                }
            }
        }
    };
    auto decode_s = [&](int t, uint32_t (&sc)[NW][NS]) {
        const int src = (ln + 16 * t) * 4;
        auto pick = [&](uint32_t v) { return (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)v); };
#pragma unroll
        for (int j = 0; j < NW; j++) {
            if constexpr (FMT == NQ_FMT_Q4_0) {
                if (p.s_pairs) {
                    const uint32_t v0 = pick(sv[j][0]), v1 = pick(sv[j][1]);
                    sc[j][0] = v0 & 0xFFFFu, sc[j][1] = v0 >> 16, sc[j][2] = v1 & 0xFFFFu, sc[j][3] = v1 >> 16;
                } else {
#pragma unroll
                    for (int q = 0; q < 4; q++) sc[j][q] = pick(sv[j][q]);
                }
            } else if constexpr (FMT == NQ_FMT_W4_GROUP) {
#pragma unroll
                for (int q = 0; q < NS; q++) sc[j][q] = pick(sv[j][2 * q] | (sv[j][2 * q + 1] << 16));
            }
        }
    };
    auto scale_of = [&](uint32_t rec, bool valid) {
        return valid ? __half2float(__ushort_as_half((uint16_t)(rec & 0xFFFFu))) : 0.0f;
    };
    auto zero_of = [&](uint32_t rec) { return (FMT == NQ_FMT_Q4_0) ? 24.0f : 16.0f + (float)(rec >> 16); };

    f32x4 acc[MT][NW], xacc[MT];
#pragma unroll
    for (int i = 0; i < MT; i++) {
        xacc[i] = (f32x4){0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < NW; j++) acc[i][j] = (f32x4){0, 0, 0, 0};
    }

    load_tiles(0);
    load_s(0);
    for (int ks = 0; ks < nsteps; ks++) {
        uint8_t* buf = smem + (ks & 1) * STAGE;
        auto lds16 = [&](uint32_t off) -> u32x4& { return *reinterpret_cast<u32x4*>(buf + off); };
        // registers -> LDS (what lies past K arrives as zeros), then the next k-step's loads
        if ((ks + 1) * KSTEP > p.K) {  // uniform
#pragma unroll
            for (int i = 0; i < XI; i++)
                if (ks * KSTEP + xpc[i] * (16 / ES) >= p.K) xv[i] = (u32x4){0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < XI; i++) lds16(xdst[i]) = xv[i];
#pragma unroll
        for (int i = 0; i < WI; i++) lds16(wdst[i]) = wv[i];
        uint32_t sc[NW][NS];
        decode_s(ks & 3, sc);
        if (ks + 1 < nsteps) {
            load_tiles(ks + 1);
            if ((ks & 3) == 3) load_s(ks + 1);
        }
        __syncthreads();

        u32x4 wc[NW];
#pragma unroll
        for (int j = 0; j < NW; j++) wc[j] = lds16(b_rd[j]);
        if constexpr (FOUR_BIT) {
#pragma unroll
            for (int j = 0; j < NW; j++) {
                auto s02 = __builtin_amdgcn_permlane32_swap(wc[j][0], wc[j][2], false, false);
                auto s13 = __builtin_amdgcn_permlane32_swap(wc[j][1], wc[j][3], false, false);
                wc[j][0] = s02[0], wc[j][2] = s02[1], wc[j][1] = s13[0], wc[j][3] = s13[1];
                auto t01 = __builtin_amdgcn_permlane16_swap(wc[j][0], wc[j][1], false, false);
                auto t23 = __builtin_amdgcn_permlane16_swap(wc[j][2], wc[j][3], false, false);
                wc[j][0] = t01[0], wc[j][1] = t01[1], wc[j][2] = t23[0], wc[j][3] = t23[1];
            }
        }
        f32x4 xs_w[MT], pp_w[MT][NW];
        if constexpr (FOUR_BIT && WHOLE) {
#pragma unroll
            for (int i = 0; i < MT; i++) {
                xs_w[i] = (f32x4){0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < NW; j++) pp_w[i][j] = (f32x4){0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int q = 0; q < NMF; q++) {
            u32x4 bop[NW];
            if constexpr (FOUR_BIT) {
#pragma unroll
                for (int j = 0; j < NW; j++) bop[j] = nib_word_to_bf16(wc[j][q], magic);
            } else {
#pragma unroll
                for (int j = 0; j < NW; j++) {
                    uint32_t b0, b1, b2, b3;
                    byte_word_to_bf16<FMT>(wc[j][2 * q], b0, b1);
                    byte_word_to_bf16<FMT>(wc[j][2 * q + 1], b2, b3);
                    bop[j] = (u32x4){b0, b1, b2, b3};
                }
            }
            const bool cvalid = ks * 4 + q < p.nch;
#pragma unroll
            for (int i = 0; i < MT; i++) {
                u32x4 raw[NL], at[NT];
#pragma unroll
                for (int h = 0; h < NL; h++) raw[h] = lds16(a_rd[i][q][h]);
                make_terms<XF32>(raw, at);
                if constexpr (FOUR_BIT && WHOLE) {
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        xs_w[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(ones), xs_w[i], 0,
                                                                           0, 0);
#pragma unroll
                        for (int j = 0; j < NW; j++)
                            pp_w[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(bop[j]),
                                                                                 pp_w[i][j], 0, 0, 0);
                    }
                } else if constexpr (FOUR_BIT) {
                    f32x4 xs = {0, 0, 0, 0};
#pragma unroll
                    for (int t = 0; t < NT; t++)
                        xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(ones), xs, 0, 0, 0);
#pragma unroll
                    for (int j = 0; j < NW; j++) {
                        const float cz = zero_of(sc[j][q]);
                        f32x4 pp;
#pragma unroll
                        for (int r = 0; r < 4; r++) pp[r] = -cz * xs[r];
#pragma unroll
                        for (int t = 0; t < NT; t++)
                            pp = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(bop[j]), pp, 0, 0, 0);
                        const float cs = scale_of(sc[j][q], cvalid);
#pragma unroll
                        for (int r = 0; r < 4; r++) acc[i][j][r] = fmaf(cs, pp[r], acc[i][j][r]);
                    }
                } else {
#pragma unroll
                    for (int t = 0; t < NT; t++) {
                        if constexpr (FMT == NQ_FMT_W8_CHANNEL)
                            xacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(ones), xacc[i],
                                                                              0, 0, 0);
#pragma unroll
                        for (int j = 0; j < NW; j++)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(at[t]), as_bf16x8(bop[j]),
                                                                                acc[i][j], 0, 0, 0);
                    }
                }
            }
        }
        if constexpr (FOUR_BIT && WHOLE) {
#pragma unroll
            for (int j = 0; j < NW; j++) {
                const float cs = scale_of(sc[j][0], true), cz = zero_of(sc[j][0]);
#pragma unroll
                for (int i = 0; i < MT; i++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        acc[i][j][r] = fmaf(cs, fmaf(-cz, xs_w[i][r], pp_w[i][j][r]), acc[i][j][r]);
            }
        }
    }

    // ---- epilogue: lane holds column n = ln of tile j, rows 4 kb + r of tile i
#pragma unroll
    for (int j = 0; j < NW; j++) {
        const int n = n0 + wn * 16 * NW + 16 * j + ln;
        const int nc = min(n, p.N - 1);
        const float cscale = (FMT == NQ_FMT_W8_CHANNEL) ? reinterpret_cast<const float*>(p.scales)[nc]
                             : (FMT == NQ_FMT_FP8_E4M3)  ? p.tscale
                                                          : 1.0f;
        float cbias = 0.0f;
        if (p.bias)
            cbias = (p.bias_dtype == NQ_DT_F32)
                        ? reinterpret_cast<const float*>(p.bias)[nc]
                        : __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[nc] << 16);
        void* yp = nullptr;
        int width = 0, col = 0;
        if (n < p.N) seg_lookup(p.seg, n, yp, width, col);
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int m = m0 + wm * 16 * MT + 16 * i + 4 * kb + r;
                float z = acc[i][j][r];
                if constexpr (FMT == NQ_FMT_W8_CHANNEL) z = fmaf(-128.0f, xacc[i][r], z);
                if constexpr (!FOUR_BIT) z *= cscale;
                z += cbias;
                if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
                if (p.epilogue == NQ_EPI_SWIGLU) {  // (uniform) gate in the even column, up one lane over
                    const float other = lane_xor1(z);
                    if ((n & 1) == 0 && n + 1 < p.N && m < p.M) {
                        const float g = swiglu_f32(other, z);
                        const int64_t o = (int64_t)m * (p.N >> 1) + (n >> 1);
                        if (p.y_dtype == NQ_DT_F32)
                            reinterpret_cast<float*>(p.y)[o] = g;
                        else
                            reinterpret_cast<uint16_t*>(p.y)[o] = f32_to_bf16_rne(g);
                    }
                    continue;
                }
                if (n < p.N && m < p.M) {
                    const int64_t o = (int64_t)m * width + col;
                    if (p.y_dtype == NQ_DT_F32)
                        reinterpret_cast<float*>(yp)[o] = z;
                    else
                        reinterpret_cast<uint16_t*>(yp)[o] = f32_to_bf16_rne(z);
                }
            }
    }
}

template <int FMT, bool XF32, bool WHOLE>
int32_t launch_big(const A16Params& p, int mt, int nw, hipStream_t s) {
    const bool four_bit = FMT != NQ_FMT_W8_CHANNEL && FMT != NQ_FMT_FP8_E4M3;
    const int xb = (four_bit ? 128 : 64) * (XF32 ? 4 : 2);
    const size_t lds = 2 * ((size_t)32 * mt * xb + 128 * 64);
    const dim3 grid((unsigned)((p.N + 127) / 128), (unsigned)((p.M + 32 * mt - 1) / (32 * mt)));
#define NQ_BIG_CASE(MT_, NW_)                                                                     \
    if (mt == MT_ && nw == NW_) {                                                                 \
        auto kernel = gemm_a16_big_kernel<FMT, XF32, MT_, NW_, WHOLE>;                            \
        static LdsAttrOnce attr;                                                                  \
        if (lds > 48 * 1024) NQ_HIP(set_max_lds_once(attr, reinterpret_cast<const void*>(kernel), lds)); \
        hipLaunchKernelGGL(kernel, grid, dim3(128 * (8 / NW_)), lds, s, p);                       \
        NQ_HIP(hipGetLastError());                                                                \
        return NQ_OK;                                                                             \
    }
    NQ_BIG_CASE(2, 4)
    NQ_BIG_CASE(2, 2)
    if constexpr (!XF32) { NQ_BIG_CASE(4, 4) NQ_BIG_CASE(4, 2) }
#undef NQ_BIG_CASE
    return fail(NQ_ERR_INVALID, "nq_forward: no large-M kernel of that tile shape");
}

template <int FMT, bool XF32, bool WHOLE>
int32_t launch_tile(const A16Params& p, int mw, int nw, int kw, dim3 grid, hipStream_t s) {
    const bool four_bit = FMT != NQ_FMT_W8_CHANNEL && FMT != NQ_FMT_FP8_E4M3;
    const size_t staging = (size_t)kw * (16 * ((!four_bit && !XF32) ? 128 : 256) + nw * 1024);
    const size_t lds = std::max(staging, (size_t)kw * mw * nw * 4 * 64 * sizeof(float));
    const dim3 block(64 * kw);
#define NQ_A16_CASE(MW_, NW_, KW_)                                                                         \
    if (mw == MW_ && nw == NW_ && kw == KW_) {                                                             \
        hipLaunchKernelGGL((gemm_a16_kernel<FMT, XF32, MW_, NW_, KW_, WHOLE>), grid, block, lds, s, p);    \
        NQ_HIP(hipGetLastError());                                                                         \
        return NQ_OK;                                                                                      \
    }
#define NQ_A16_TILE(MW_, NW_) NQ_A16_CASE(MW_, NW_, 4) NQ_A16_CASE(MW_, NW_, 8)
    NQ_A16_TILE(1, 1)
    NQ_A16_TILE(1, 2)
    NQ_A16_TILE(1, 4)
    NQ_A16_TILE(2, 2)
    if constexpr (!XF32) { NQ_A16_TILE(2, 4) }
#undef NQ_A16_TILE
#undef NQ_A16_CASE
    return fail(NQ_ERR_INVALID, "nq_forward: no medium-M kernel of that tile shape");
}

}  // namespace


// Tile shape of the medium-M kernel (wavefront tiles of 16 rows x 16 columns: mw x nw of them per workgroup) and what
// the call will take.  One workgroup of any shape fits a CU at a time, so a call runs in ceil(workgroups / 256)
// rounds, and a round costs a fixed part and a part per k-step that both grow with the tile: measured over K = 512 ..
// 6144, N = 320 .. 4096 and M = 17 .. 500 for each format and activation type (five shapes each, 3000 calls), a call
// takes
//     t = F + rounds * (p0 + p1 * k-steps)   microseconds
// within 3 - 6 % on average, with the constants below.  The shape with the least estimate is taken: over those calls
// that is within 1 % of always taking the fastest shape (the rules it replaces - the widest tile that still gave 128
// workgroups, none with two M tiles for an odd count of them - were 5 - 18 % off: with fp32 activations two M tiles
// per wavefront are never worth their registers, 4096 x 4096 int8 codes at M = 256 67 -> 47 us, and with bf16 ones an
// odd count of M tiles is worth padding, 2048 x 2048 at M = 135 9.4 -> 7.9 us).  The shape changes which workgroup
// computes an output, not the order of its sum.
float gemm_a16_estimate_us(int32_t format, bool xf32, int M, int N, int K, int* mw_out, int* nw_out) {
    struct ShapeCost {
        int mw, nw;
        float f, p0, p1;
    };
    static const ShapeCost costs[6][5] = {
        // 8-bit codes (int8, e4m3), bf16 activations
        {{2, 4, 1.18f, 2.773f, 0.1292f}, {2, 2, 2.56f, 0.495f, 0.0795f}, {1, 4, 2.52f, 0.579f, 0.0972f},
         {1, 2, 2.41f, 0.256f, 0.0518f}, {1, 1, 2.36f, 0.205f, 0.0318f}},
        // 8-bit codes, fp32 activations (the 2 x 4 shape does not fit the registers)
        {{2, 4, 0, 0, 0}, {2, 2, 1.10f, 1.796f, 0.1967f}, {1, 4, 2.55f, 0.536f, 0.1604f},
         {1, 2, 2.44f, 0.232f, 0.1084f}, {1, 1, 2.53f, 0.133f, 0.0788f}},
        // Q4_0, bf16 activations
        {{2, 4, 1.68f, 2.926f, 0.2849f}, {2, 2, 1.70f, 1.690f, 0.1809f}, {1, 4, 1.90f, 1.621f, 0.2214f},
         {1, 2, 2.82f, 0.333f, 0.1093f}, {1, 1, 2.59f, 0.190f, 0.0722f}},
        // Q4_0, fp32 activations
        {{2, 4, 0, 0, 0}, {2, 2, 2.03f, 1.825f, 0.3953f}, {1, 4, 1.99f, 1.759f, 0.3347f},
         {1, 2, 2.17f, 0.711f, 0.2540f}, {1, 1, 2.80f, 0.198f, 0.1620f}},
        // 4-bit codes in groups with zero points, bf16 activations
        {{2, 4, 1.69f, 2.576f, 0.2536f}, {2, 2, 1.75f, 1.402f, 0.1698f}, {1, 4, 2.08f, 1.169f, 0.2006f},
         {1, 2, 2.69f, 0.302f, 0.0984f}, {1, 1, 2.54f, 0.162f, 0.0667f}},
        // 4-bit codes in groups with zero points, fp32 activations
        {{2, 4, 0, 0, 0}, {2, 2, 2.03f, 1.446f, 0.3875f}, {1, 4, 1.96f, 1.469f, 0.3212f},
         {1, 2, 2.15f, 0.562f, 0.2366f}, {1, 1, 2.70f, 0.142f, 0.1565f}},
    };
    const bool four_bit = format != NQ_FMT_W8_CHANNEL && format != NQ_FMT_FP8_E4M3;
    const int mt = (M + 15) / 16;
    const int kstep = four_bit ? 128 : 64;
    const int nsteps = (K + kstep - 1) / kstep;
    const ShapeCost* row = costs[(!four_bit ? 0 : format == NQ_FMT_Q4_0 ? 2 : 4) + (xf32 ? 1 : 0)];
    int mw = 1, nw = 1;
    float least = 0.0f;
    for (int c = 0; c < 5; c++) {
        const ShapeCost& sc = row[c];
        if (sc.mw * sc.nw == 8 && xf32) continue;
        if (sc.mw == 2 && mt == 1) continue;  // a second M tile of padding only
        const int64_t wgs = (int64_t)((mt + sc.mw - 1) / sc.mw) * ((N + 16 * sc.nw - 1) / (16 * sc.nw));
        const float t = sc.f + (float)((wgs + 255) / 256) * (sc.p0 + sc.p1 * (float)nsteps);
        if (least == 0.0f || t < least) least = t, mw = sc.mw, nw = sc.nw;
    }
    if (mw_out) *mw_out = mw;
    if (nw_out) *nw_out = nw;
    return least;
}

bool gemm_a16_applicable(const ForwardArgs& a);

// What the many-rows kernel (a weight unpacked once per 64 or 128 rows) will take, in microseconds, or 0 where it
// does not apply: below 256 rows, or with fewer than 64 workgroups of 64 rows.  Measured against the medium-M kernel
// over K = 512 .. 4096, N = 1024 .. 11008 and M = 256 .. 1024 for each format and activation type (960 pairs of calls):
// t = F + rounds * (c0 + c1 * k-steps), rounds of 256 workgroups, twice the cost per round with 128 rows per
// workgroup, within 5 - 9 % on average.  Taking this kernel where its estimate is below the medium-M kernel's is
// within 1 - 3 % of always taking the faster of the two; the thresholds before (512 rows and 192 such workgroups, 256
// with fp32 activations) were 6 - 13 % off over those calls.  mt_out: 32-row tiles per workgroup (2 or 4).
static float big_estimate_us(int32_t format, bool xf32, int M, int N, int K, int* mt_out) {
    static const float consts[6][3] = {
        {5.64f, 0.684f, 0.3934f}, {12.26f, -2.602f, 1.0247f},   // 8-bit codes: bf16, fp32 activations
        {6.49f, -0.439f, 1.1383f}, {14.01f, -3.669f, 2.6569f},  // Q4_0
        {5.46f, 0.237f, 0.9032f}, {10.55f, -1.821f, 2.1478f},   // 4-bit codes in groups with zero points
    };
    const bool four_bit = format != NQ_FMT_W8_CHANNEL && format != NQ_FMT_FP8_E4M3;
    const int64_t wgs64 = (int64_t)((N + 127) / 128) * ((M + 63) / 64);
    const int mt = (!xf32 && K >= 4096 && wgs64 >= 384) ? 4 : 2;  // 128 rows per workgroup over a long K
    if (mt_out) *mt_out = mt;
    if (M < 256 || wgs64 < 64) return 0.0f;
    const float* c = consts[(!four_bit ? 0 : format == NQ_FMT_Q4_0 ? 2 : 4) + (xf32 ? 1 : 0)];
    const int64_t wgs = (int64_t)((N + 127) / 128) * ((M + 32 * mt - 1) / (32 * mt));
    const int nsteps = (K + (four_bit ? 128 : 64) - 1) / (four_bit ? 128 : 64);
    return c[0] + (float)((wgs + 255) / 256) * (float)(mt / 2) * (c[1] + c[2] * (float)nsteps);
}

// the many-rows kernel for a layer (or a part of a row-fused one) `width` columns wide
static bool big_wins(const ForwardArgs& a, int width) {
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    const float big = big_estimate_us(a.L->format, xf32, a.M, width, a.L->in, nullptr);
    return big > 0.0f && big < gemm_a16_estimate_us(a.L->format, xf32, a.M, width, a.L->in, nullptr, nullptr);
}

static int big_parts(const ForwardArgs& a) {
    int n = 0;
    for (int i = 0, prev = 0; i < a.seg.nseg; prev = a.seg.end[i], i++) n += big_wins(a, a.seg.end[i] - prev);
    return n;
}

// Below 512 rows a part of a row-fused layer gets the kernel - and so the bits - of its own layer's forward: all
// parts on the many-rows kernel, none, or (this) part by part.  From 512 rows on the whole layer's width decides.
bool gemm_a16_splits_parts(const ForwardArgs& a) {
    if (a.seg.nseg < 2 || a.M < 256 || a.M >= 512 || !gemm_a16_applicable(a)) return false;
    const int n = big_parts(a);
    return n > 0 && n < a.seg.nseg;
}

// the lower of the two kernels' estimates (what the M-tile kernel's estimate is held against)
float gemm_a16_best_estimate_us(int32_t format, bool xf32, int M, int N, int K) {
    const float medium = gemm_a16_estimate_us(format, xf32, M, N, K, nullptr, nullptr);
    const float big = big_estimate_us(format, xf32, M, N, K, nullptr);
    return big > 0.0f && big < medium ? big : medium;
}

bool gemm_a16_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (a.x_dtype != NQ_DT_F32 && a.x_dtype != NQ_DT_BF16) return false;
    const bool bytes = L->format == NQ_FMT_W8_CHANNEL || L->format == NQ_FMT_FP8_E4M3;
    if (L->in % (bytes ? 16 : 32) != 0) return false;
    // the kernel addresses each operand with 32-bit byte offsets
    const int64_t lim = (int64_t)1 << 32;
    if ((int64_t)a.M * L->in * 4 >= lim || (int64_t)L->out * L->in >= lim) return false;
    return a.M >= 2;  // (measured: from two rows on, a padded 16-row MFMA tile beats the LDS GEMV)
}

int32_t launch_gemm_a16(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    const bool four_bit = L->format != NQ_FMT_W8_CHANNEL && L->format != NQ_FMT_FP8_E4M3;
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    A16Params p{};
    p.codes = L->d_codes, p.scales = L->d_scales, p.zps = L->d_zps;
    p.x = a.x, p.y = a.y, p.bias = a.bias, p.seg = a.seg;
    p.M = a.M, p.N = L->out, p.K = L->in;
    p.groups = L->groups;
    p.inv_cpg = L->group ? 32.0f / (float)L->group : 1.0f;
    p.tscale = L->scale;
    p.s_pairs = L->format != NQ_FMT_Q4_0 ? 0 : (L->in / 32) % 4 == 0 ? 2 : (L->in / 32) % 2 == 0 ? 1 : 0;
    p.nch = L->in / (four_bit ? 32 : 16);
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    // Many rows: the kernel that unpacks a weight once per 64 or 128 rows, from 256 rows on wherever its estimated
    // time is the lower one.  Its sums are formed in another order than the medium-M kernel's.  Below 512 rows a
    // row-fused layer takes it only when every part would on its own (a mix runs part by part:
    // gemm_a16_splits_parts); from 512 rows on the whole layer's width decides, and a row's bits in a row-fused
    // layer may differ from those in its own layer.
    const bool use_big = !a.diag_a16_shape && ((a.M >= 512 || a.seg.nseg < 2) ? big_wins(a, L->out) : big_parts(a) == a.seg.nseg);
    if (use_big) {
        int big = 2;
        big_estimate_us(L->format, xf32, a.M, L->out, L->in, &big);
        const int bnw = xf32 ? 4 : 2;                                      // four or eight wavefronts
        switch (L->format) {
            case NQ_FMT_Q4_0:
                return xf32 ? launch_big<NQ_FMT_Q4_0, true, false>(p, 2, bnw, a.stream)
                            : launch_big<NQ_FMT_Q4_0, false, false>(p, big, bnw, a.stream);
            case NQ_FMT_W4_GROUP:
                if (L->group % 128 == 0)
                    return xf32 ? launch_big<NQ_FMT_W4_GROUP, true, true>(p, 2, bnw, a.stream)
                                : launch_big<NQ_FMT_W4_GROUP, false, true>(p, big, bnw, a.stream);
                return xf32 ? launch_big<NQ_FMT_W4_GROUP, true, false>(p, 2, bnw, a.stream)
                            : launch_big<NQ_FMT_W4_GROUP, false, false>(p, big, bnw, a.stream);
            case NQ_FMT_W8_CHANNEL:
                return xf32 ? launch_big<NQ_FMT_W8_CHANNEL, true, false>(p, 2, bnw, a.stream)
                            : launch_big<NQ_FMT_W8_CHANNEL, false, false>(p, big, bnw, a.stream);
            case NQ_FMT_FP8_E4M3:
                return xf32 ? launch_big<NQ_FMT_FP8_E4M3, true, false>(p, 2, bnw, a.stream)
                            : launch_big<NQ_FMT_FP8_E4M3, false, false>(p, big, bnw, a.stream);
        }
    }
    int mw = 1, nw = 1;
    gemm_a16_estimate_us(L->format, xf32, a.M, L->out, L->in, &mw, &nw);
    if (const int forced = a.diag_a16_shape) mw = forced >> 4, nw = forced & 15;  // nq_diag_forward_a16
    const int kstep = four_bit ? 128 : 64;
    const int nsteps = (L->in + kstep - 1) / kstep;
    // K split: 8 wavefronts when there are more than 4 k-steps.  It follows K alone: the K split fixes
    // the order in which an output's sum is formed, and a row must get the same bits whichever
    // layer (its own, or a row-fused one) it is computed in.
    int kw = nsteps > 4 ? 8 : 4;
    dim3 grid((L->out + 16 * nw - 1) / (16 * nw), (a.M + 16 * mw - 1) / (16 * mw));
    switch (L->format) {
        case NQ_FMT_Q4_0:
            return xf32 ? launch_tile<NQ_FMT_Q4_0, true, false>(p, mw, nw, kw, grid, a.stream)
                        : launch_tile<NQ_FMT_Q4_0, false, false>(p, mw, nw, kw, grid, a.stream);
        case NQ_FMT_W4_GROUP:
            // a k-step (128 k) lies in one group when the group width is a multiple of 128
            if (L->group % 128 == 0)
                return xf32 ? launch_tile<NQ_FMT_W4_GROUP, true, true>(p, mw, nw, kw, grid, a.stream)
                            : launch_tile<NQ_FMT_W4_GROUP, false, true>(p, mw, nw, kw, grid, a.stream);
            return xf32 ? launch_tile<NQ_FMT_W4_GROUP, true, false>(p, mw, nw, kw, grid, a.stream)
                        : launch_tile<NQ_FMT_W4_GROUP, false, false>(p, mw, nw, kw, grid, a.stream);
        case NQ_FMT_W8_CHANNEL:
            return xf32 ? launch_tile<NQ_FMT_W8_CHANNEL, true, false>(p, mw, nw, kw, grid, a.stream)
                        : launch_tile<NQ_FMT_W8_CHANNEL, false, false>(p, mw, nw, kw, grid, a.stream);
        case NQ_FMT_FP8_E4M3:
            return xf32 ? launch_tile<NQ_FMT_FP8_E4M3, true, false>(p, mw, nw, kw, grid, a.stream)
                        : launch_tile<NQ_FMT_FP8_E4M3, false, false>(p, mw, nw, kw, grid, a.stream);
    }
    return fail(NQ_ERR_INVALID, "nq_forward: unknown format");
}

}  // namespace nq
