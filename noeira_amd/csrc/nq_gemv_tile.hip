// Dequant-GEMV for ONE activation row (M = 1) over a LARGE weight, from a second, tile-ordered copy of the codes:
//     y[N] = epi( deq(W)[N, K] x + bias ),   x bf16 or fp32,
//     W: Q4_0 (group 32), W4_GROUP with groups of 128 k, or W8_CHANNEL (int8 + per-channel scale).
//
// What holds a streaming kernel for 4-bit codes below the weight stream is instruction issue, and most of
// what the row-ordered kernels issue is not arithmetic: with one weight row per wavefront the matrix core
// can only be used "diagonally" (16 columns = 16 segments of the row, one useful entry per column, picked
// out per group), every wavefront stages x again, and the codes must be transposed between lanes.  Here
// the codes are laid out at load time the way the matrix core wants them for 16 weight rows at once:
//
//   4-bit   tile[R][J][lane l = c + 16 q][word m]  (16 bytes per lane, 1 KiB per (R, J))
//             = word q (codes 8 q .. 8 q + 7, device nibble order of nq_nib.h) of the 32-code chunk
//               4 J + m of row 16 R + c:  MFMA m of step J (v_mfma_f32_16x16x32_bf16) takes word m as
//               its B operand, so column c is one chunk of row 16 R + c, i.e. one Q4_0 group, and the
//               four MFMAs of a step are one group of 128;
//           scales[R][J][c][m] fp16 (Q4_0) or [R][J][c] = fp16 scale | zero point << 16 (groups of 128)
//   int8    tile[R][J][lane][16 B] = codes 64 J + 16 q .. + 15 of row 16 R + c: the B operand of
//           v_mfma_i32_16x16x64_i8 as it lies in memory
//
// so a load instruction is 1 KiB contiguous, nothing is transposed or picked, and the 16 results of a
// step sit in the same register of lanes 0 .. 15.  A workgroup owns one tile of 16 rows; its KW
// wavefronts split K (JPW steps each; all of a wavefront's loads are requested before anything else)
// and meet in LDS in wave order (fixed: a repeated call returns the same bits).
//
// The A operand is x, and its 16 rows are free: a lane's A row is lane % 16, and only the rows that hold
// something are read back.  bf16 x is row 0.  fp32 x is the exact three-term bf16 split hi + mid + lo in
// rows 0, 1, 2 of the SAME MFMA (so fp32 activations cost the one MFMA bf16 activations cost; the three
// partial dot products are added in fp32).  For int8 weights x is split, per wavefront and slice of K, into
// three int8 terms under the slice's largest magnitude,
//     x[k] = (absmax / 127) (q1[k] + q2[k] / 254 + q3[k] / 254^2) + e,  |e| <= 6e-8 absmax,
// again rows 0, 1, 2 of one MFMA: three exact int32 sums per slice, combined in fp32.  A wavefront stages
// its own slice of x in its own piece of LDS (LDS runs one wavefront's accesses in order: no barrier).
// 4-bit codes become the exact bf16 values 16 + q (bits 0x4180 | q << 3); the zero point leaves the
// inner loop through the slice's group sums of x, which stay in registers and are read with v_readlane.
//
// Steps past K (K is a multiple of the step; the last round of a wavefront may be short) load from a
// clamped address, meet x = 0 and get scale 0.
#include <hip/hip_fp16.h>

#include <algorithm>

#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

struct TileParams {
    const u32x4* tile;
    const void* tscales;      // 4-bit: the tile-ordered group records
    const float* col_scale;   // int8: per output channel [N]
    const void* x;
    const void* bias;
    int32_t N, K, NJ;         // NJ steps per row tile (128 k for 4-bit, 64 k for int8)
    int32_t y_dtype, bias_dtype, epilogue;
    int32_t prefer;           // NQ_FLAG_PREFER_TILE: the int8-matrix-core route for 4-bit codes whatever the layer's size
    SegTable seg;
};

__device__ __forceinline__ bf16x8 as_bf16x8(const u32x4& v) { return __builtin_bit_cast(bf16x8, v); }

// eight nibbles of a word -> four packed bf16 pairs holding 16 + code, in k order (nq_nib.h); `magic` is
// 0x41804180 in a vector register the compiler cannot see through (one v_and_or_b32 per pair)
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

#define NQ_DPP(v, ctrl) __builtin_amdgcn_update_dpp(0, (int)(v), ctrl, 0xF, 0xF, false)
#define NQ_DPP_F32(v, ctrl) __int_as_float(NQ_DPP(__float_as_int(v), ctrl))

// The epilogue's operands of row 16 R + lane % 16, requested at kernel start (raw: nothing is computed from them
// before the end, so their latency hides under the weight stream instead of following the barrier).
struct RowTail {
    float cs;
    uint32_t braw;
};

__device__ __forceinline__ RowTail fetch_tail(const TileParams& p, int64_t R, int lane) {
    RowTail t;
    const int64_t n = min(R * 16 + (lane & 15), (int64_t)p.N - 1);
    t.cs = p.col_scale ? p.col_scale[n] : 1.0f;
    t.braw = 0;
    if (p.bias)
        t.braw = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[n]
                                             : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n];
    return t;
}

// the workgroup's 16 rows: the wavefronts' shares summed in wave order, bias, epilogue, placement by part
template <int KW>
__device__ __forceinline__ void finish_rows(const TileParams& p, const float (&red)[KW][16], int64_t R, const RowTail& t) {
    if (threadIdx.x < 16) {
        float z = red[0][threadIdx.x];
#pragma unroll
        for (int w = 1; w < KW; w++) z += red[w][threadIdx.x];
        const int64_t n = R * 16 + threadIdx.x;
        if (n < p.N) {
            if (p.col_scale) z *= t.cs;
            if (p.bias) z += __uint_as_float(p.bias_dtype == NQ_DT_F32 ? t.braw : t.braw << 16);
            if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
            void* yp;
            int width, col;
            seg_lookup(p.seg, (int)n, yp, width, col);  // M = 1: the part's row is its only row
            if (p.y_dtype == NQ_DT_F32)
                reinterpret_cast<float*>(yp)[col] = z;
            else
                reinterpret_cast<uint16_t*>(yp)[col] = f32_to_bf16_rne(z);
        }
    }
}

// ---- 4-bit codes ----------------------------------------------------------------------------------
// EXACT: K is exactly KW * JPW steps (one round, no step past K): the clamps and masks below fall away
template <int FMT, bool XF32, int KW, int JPW, bool EXACT>
__global__ __launch_bounds__(64 * KW) void gemv_tile4_kernel(const TileParams p) {
    constexpr bool G128 = FMT == NQ_FMT_W4_GROUP;
    constexpr int NT = XF32 ? 3 : 1;
    constexpr int NP = JPW * 16;         // 16-byte pieces (8 values) of x per wavefront and term
    constexpr int PPL = (NP + 63) / 64;  // pieces per lane
    __shared__ __attribute__((aligned(16))) uint8_t xs[KW][NT][NP * 16];
    __shared__ float red[KW][16];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, q = lane >> 4;
    const int64_t R = blockIdx.x;
    uint32_t magic = 0x41804180u;
    asm volatile("" : "+v"(magic));
    // A row = lane % 16: rows 0 .. NT - 1 are the terms of x, the others repeat the last (their results are unused)
    const uint8_t* const arow = &xs[wave][XF32 ? min(c, 2) : 0][q * 16];
    float acc = 0.0f;

    RowTail tail{};
    if (wave == 0) tail = fetch_tail(p, R, lane);

    for (int J0 = wave * JPW; J0 < p.NJ; J0 += EXACT ? p.NJ : KW * JPW) {
        // Every load of the round is requested here, x first (it is needed first, and waiting for it leaves the
        // codes in flight), from clamped addresses, and nothing loaded is touched before it is needed: an
        // instruction on a loaded value makes the wavefront wait for that load and every load before it.
        // The slice of x under this round: lane l holds the 8-value pieces l, l + 64.
        u32x4 xr[PPL][XF32 ? 2 : 1];
#pragma unroll
        for (int h = 0; h < PPL; h++) {
            const int kx = J0 * 128 + (lane + 64 * h) * 8;
            const int kc = (EXACT && NP % 64 == 0) ? kx : min(kx, p.K - 8);
            if constexpr (XF32) {
                const float* xf = reinterpret_cast<const float*>(p.x) + kc;
                xr[h][0] = *reinterpret_cast<const u32x4*>(xf), xr[h][1] = *reinterpret_cast<const u32x4*>(xf + 4);
            } else {
                xr[h][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + kc);
            }
        }
        u32x4 wv[JPW];
        uint2 sc[JPW];
        // (32-bit offsets from the tile's base: a layer's tile copy is below 4 GB)
        const u32x4* const wbase = p.tile + R * p.NJ * 64;
        const uint32_t* const sbase = reinterpret_cast<const uint32_t*>(p.tscales) + R * p.NJ * (G128 ? 16 : 32);
#pragma unroll
        for (int j = 0; j < JPW; j++) wv[j] = __builtin_nontemporal_load(wbase + ((EXACT ? J0 + j : min(J0 + j, p.NJ - 1)) * 64 + lane));
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            const int at = (EXACT ? J0 + j : min(J0 + j, p.NJ - 1)) * 16 + c;
            if constexpr (!G128) sc[j] = reinterpret_cast<const uint2*>(sbase)[at];
            else sc[j].x = sbase[at], sc[j].y = 0;
        }
        // x -> this wavefront's piece of LDS, and the sums of x under every chunk / group; a piece past K is zero
        float part[PPL];
#pragma unroll
        for (int h = 0; h < PPL; h++) {
            const int pc = lane + 64 * h;               // piece of the slice
            const uint32_t keep = (EXACT || J0 * 128 + pc * 8 < p.K) ? ~0u : 0u;
            const bool mine = pc < NP;
            if constexpr (XF32) {
                uint32_t v[8];
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = xr[h][0][i] & keep, v[4 + i] = xr[h][1][i] & keep;
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
                if (mine) {
                    *reinterpret_cast<u32x4*>(&xs[wave][0][pc * 16]) = t0;
                    *reinterpret_cast<u32x4*>(&xs[wave][1][pc * 16]) = t1;
                    *reinterpret_cast<u32x4*>(&xs[wave][2][pc * 16]) = t2;
                }
                part[h] = ((__uint_as_float(v[0]) + __uint_as_float(v[1])) + (__uint_as_float(v[2]) + __uint_as_float(v[3]))) +
                          ((__uint_as_float(v[4]) + __uint_as_float(v[5])) + (__uint_as_float(v[6]) + __uint_as_float(v[7])));
            } else {
                u32x4 r0 = xr[h][0];
#pragma unroll
                for (int i = 0; i < 4; i++) r0[i] &= keep;
                if (mine) *reinterpret_cast<u32x4*>(&xs[wave][0][pc * 16]) = r0;
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; i++) sum += __uint_as_float(r0[i] << 16) + __uint_as_float(r0[i] & 0xFFFF0000u);
                part[h] = sum;
            }
            // the sum of x under a chunk (four lanes), under a group of 128 (sixteen): fixed butterflies
            part[h] += NQ_DPP_F32(part[h], 0xB1);
            part[h] += NQ_DPP_F32(part[h], 0x4E);
            if constexpr (G128) {
                part[h] += NQ_DPP_F32(part[h], 0x141);
                part[h] += NQ_DPP_F32(part[h], 0x140);
            }
        }
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            // a step past K (its loads were clamped, its x is zero) gets scale 0; the choice is uniform over the
            // wavefront and made here, not where the record was loaded
            const bool live = EXACT || J0 + j < p.NJ;
            f32x4 dd[G128 ? 1 : 4];
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const u32x4 bop = nib_word_to_bf16(wv[j][m], magic);
                const u32x4 aop = *reinterpret_cast<const u32x4*>(arow + (16 * j + 4 * m) * 16);
                if (!G128 || m == 0) dd[G128 ? 0 : m] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
                dd[G128 ? 0 : m] =
                    __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop), as_bf16x8(bop), dd[G128 ? 0 : m], 0, 0, 0);
            }
            auto rowsum = [](const f32x4& d) -> float { return XF32 ? (d[0] + d[1]) + d[2] : d[0]; };
            if constexpr (!G128) {
#pragma unroll
                for (int m = 0; m < 4; m++) {
                    const uint32_t sbits = (m < 2 ? sc[j].x : sc[j].y) >> (16 * (m & 1));
                    const float d = live ? __half2float(__ushort_as_half((uint16_t)(sbits & 0xFFFFu))) : 0.0f;
                    const int g4 = 4 * (4 * j + m);  // the chunk's sum sits in lanes g4 .. g4 + 3 of part[g4 / 64]
                    const float xsg = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(part[g4 / 64]), g4 % 64));
                    acc = fmaf(d, fmaf(-24.0f, xsg, rowsum(dd[m])), acc);
                }
            } else {
                const float d = live ? __half2float(__ushort_as_half((uint16_t)(sc[j].x & 0xFFFFu))) : 0.0f;
                const float zoff = 16.0f + (float)(sc[j].x >> 16);
                const int g16 = 16 * j;
                const float xsg = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(part[g16 / 64]), g16 % 64));
                acc = fmaf(d, fmaf(-zoff, xsg, rowsum(dd[0])), acc);
            }
        }
    }
    if (q == 0) red[wave][c] = acc;
    __syncthreads();
    finish_rows<KW>(p, red, R, tail);
}


// ---- a few activation rows (2 <= M <= 16) over 4-bit codes ---------------------------------------------
// The tile of 16 weight rows is the same; the A operand now holds real rows: bf16 x row i is A row i
// (M <= 16), fp32 x row i is A rows 3 i, 3 i + 1, 3 i + 2 (its three bf16 terms; M <= 5).  One workgroup of 16
// wavefronts per CU visits tiles blockIdx.x, blockIdx.x + gridDim.x, ...; wavefront w takes the same steps
// 16-byte pieces of K in every tile, so its A operands are fetched from memory once, straight into registers (a
// lane's 16 bytes of row lane % 16), and stay there, and so do the zero-point terms: the sum of x under a
// chunk, per row, comes out of the matrix core in the product's own register layout when the B operand is all
// ones (Q4_0: times -24 and used as the product MFMA's C operand; groups of 128: times -(16 + z) first).  The
// next tile's codes are requested before the current tile is multiplied - by hand: loads in inline assembly into two
// register slots in turn and an explicit wait, see the kernel - and the biases of all of a workgroup's tiles are
// staged in LDS before the loop, so that its only loads are the codes.  The 16 wavefronts' [16 x 16] shares
// meet in LDS in wave order (two buffers, one barrier per tile); thread (row, column) adds bias and epilogue.
struct TileMrParams {
    TileParams t;
    int32_t M;
    // a frozen LoRA adapter folded into the call (the M-tile kernel only; null = none): y += ls * (x la) lb
    const float* la;  // [IN][lr] fp32
    const float* lb;  // [lr][OUT] fp32
    int32_t lr;       // rank as stored (padded), <= 16
    float ls;
    // a second adapter, for a gate | up layer (nq_fuse_glu: gate in the even columns, up in the odd ones): la / lb are
    // the gate projection's adapter, la2 / lb2 the up projection's, each B [lr][OUT / 2]; null = none
    const float* la2;
    const float* lb2;
    float ls2;
};

constexpr int TR_MAXT = 64;  // row tiles per workgroup of the rows kernels: its 1024 threads stage one tile column each

template <int FMT, bool XF32, int JPW>
__global__ __launch_bounds__(1024) void gemv_tile4_rows_kernel(const TileMrParams pm) {
    const TileParams& p = pm.t;
    constexpr bool G128 = FMT == NQ_FMT_W4_GROUP;
    constexpr int KW = 16;
    constexpr int NT = XF32 ? 3 : 1;
    constexpr bool XS_REGS = G128 || JPW <= 2;  // Q4_0 keeps 4 JPW row-sum tiles: beyond 2 steps they no longer fit
    __shared__ __attribute__((aligned(16))) float red[2][KW][256];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, q = lane >> 4;
    const int ntiles = (p.N + 15) / 16;
    const int J0 = wave * JPW;
    const int vrow = c / NT, vterm = c % NT;   // this lane's A row: activation row and term
    const int xrow = min(vrow, pm.M - 1);
    uint32_t magic = 0x41804180u;
    asm volatile("" : "+v"(magic));

    const int g = gridDim.x;
    const int fr = threadIdx.x >> 4, fc = threadIdx.x & 15;  // threads 0 .. 255 finish a tile: row fr, column fc
    // ---- the biases of all of this workgroup's tiles at once (at most TR_MAXT tiles): thread i stages that of column
    // i % 16 of its tile i / 16.  The oldest load; then the activations, then the first tile.
    __shared__ float fin_bias[TR_MAXT * 16];
    uint32_t st_bias = 0;
    if (p.bias) {  // (as loaded: a shift here would wait for the load)
        const int64_t n = min(((int64_t)blockIdx.x + (int64_t)fr * g) * 16 + fc, (int64_t)p.N - 1);
        st_bias = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[n]
                                              : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n];
    }
    // The tiles' loads and the waits for them are written out: the compiler's own wait counts are exact in straight
    // code only, and across the loop's back edge they drain the tile requested ahead together with the one about to
    // be multiplied.  A fetch is 2 JPW loads (codes and scales of every step), so with the next tile under way "all
    // but the youngest 2 JPW" is the tile about to be multiplied; loads and stores the compiler issues in between
    // only make that wait longer.  The waits name no registers (nothing is copied ahead of them); the hand-over that
    // follows them on every path does, so that nothing reads a slot before its wait.  One tile ahead, two register
    // slots in turn: two tiles ahead measured slower wherever a workgroup has three tiles and more.
    struct Slot {
        u32x4 wv[JPW];
        uint2 sc[JPW];  // (groups of 128: .x only)
    };
    auto fetch = [&](int tile, Slot& s) {
        if (tile >= ntiles) return;
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            const int64_t at = (int64_t)tile * p.NJ + min(J0 + j, p.NJ - 1);
            const u32x4* const src = p.tile + at * 64 + lane;
            asm volatile("global_load_dwordx4 %0, %1, off nt ; pf" : "=v"(s.wv[j]) : "v"(src));
            if constexpr (!G128) {
                const uint2* const ssrc = reinterpret_cast<const uint2*>(p.tscales) + at * 16 + c;
                asm volatile("global_load_dwordx2 %0, %1, off ; pf" : "=v"(s.sc[j]) : "v"(ssrc));
            } else {
                const uint32_t* const ssrc = reinterpret_cast<const uint32_t*>(p.tscales) + at * 16 + c;
                asm volatile("global_load_dword %0, %1, off ; pf" : "=v"(s.sc[j].x) : "v"(ssrc));
                s.sc[j].y = 0;
            }
        }
    };
    auto arrived = [&](int tile, Slot& s) {  // (the next tile is under way if there is one)
        if (tile + g < ntiles) {
            if constexpr (JPW == 1) asm volatile("s_waitcnt vmcnt(2)");
            if constexpr (JPW == 2) asm volatile("s_waitcnt vmcnt(4)");
            if constexpr (JPW == 3) asm volatile("s_waitcnt vmcnt(6)");
        } else {
            asm volatile("s_waitcnt vmcnt(0)");
        }
        if constexpr (G128) {
            if constexpr (JPW == 1) asm volatile("; pfh %0 %1" : "+v"(s.wv[0]), "+v"(s.sc[0].x));
            if constexpr (JPW == 2) asm volatile("; pfh %0 %1 %2 %3" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.sc[0].x), "+v"(s.sc[1].x));
            if constexpr (JPW == 3)
                asm volatile("; pfh %0 %1 %2 %3 %4 %5" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.wv[2]), "+v"(s.sc[0].x), "+v"(s.sc[1].x), "+v"(s.sc[2].x));
        } else {
            if constexpr (JPW == 1) asm volatile("; pfh %0 %1" : "+v"(s.wv[0]), "+v"(s.sc[0]));
            if constexpr (JPW == 2) asm volatile("; pfh %0 %1 %2 %3" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.sc[0]), "+v"(s.sc[1]));
            if constexpr (JPW == 3)
                asm volatile("; pfh %0 %1 %2 %3 %4 %5" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.wv[2]), "+v"(s.sc[0]), "+v"(s.sc[1]), "+v"(s.sc[2]));
        }
    };

    // (Q4_0 under fp32 rows at three steps: the first tile is requested after the operands are built, or the
    // registers run out while both are under way)
    constexpr bool LATE_FIRST = !G128 && XF32 && JPW == 3;
    // ---- the activations first (older than the tiles' loads: waiting for them leaves the tiles under way)
    u32x4 xraw[JPW][4][XF32 ? 2 : 1];
#pragma unroll
    for (int j = 0; j < JPW; j++)
#pragma unroll
        for (int m = 0; m < 4; m++) {
            const int k = min((J0 + j) * 128 + 32 * m + 8 * q, p.K - 8);
            if constexpr (XF32) {
                const float* xf = reinterpret_cast<const float*>(p.x) + (int64_t)xrow * p.K + k;
                xraw[j][m][0] = *reinterpret_cast<const u32x4*>(xf), xraw[j][m][XF32 ? 1 : 0] = *reinterpret_cast<const u32x4*>(xf + 4);
            } else {
                xraw[j][m][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + (int64_t)xrow * p.K + k);
            }
        }
    Slot s0, s1;
    if constexpr (!LATE_FIRST) fetch(blockIdx.x, s0);

    // ---- A operands, once: 16 bytes of bf16 per (step, MFMA); rows past M and steps past K are zero
    u32x4 aop[JPW][4];
#pragma unroll
    for (int j = 0; j < JPW; j++)
#pragma unroll
        for (int m = 0; m < 4; m++) {
            u32x4 t;
            if constexpr (XF32) {
                const u32x4 r0 = xraw[j][m][0], r1 = xraw[j][m][XF32 ? 1 : 0];
                uint32_t v[8];
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = r0[i], v[4 + i] = r1[i];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    // hi + mid + lo = the fp32 value (each split truncates: every residual is exact); this lane keeps one
                    const uint32_t a = v[2 * i], b = v[2 * i + 1];
                    const float ra = __uint_as_float(a) - __uint_as_float(a & 0xFFFF0000u);
                    const float rb = __uint_as_float(b) - __uint_as_float(b & 0xFFFF0000u);
                    const float sa = ra - __uint_as_float(__float_as_uint(ra) & 0xFFFF0000u);
                    const float sb = rb - __uint_as_float(__float_as_uint(rb) & 0xFFFF0000u);
                    const uint32_t ta = vterm == 0 ? a : vterm == 1 ? __float_as_uint(ra) : __float_as_uint(sa);
                    const uint32_t tb = vterm == 0 ? b : vterm == 1 ? __float_as_uint(rb) : __float_as_uint(sb);
                    t[i] = __builtin_amdgcn_perm(tb, ta, 0x07060302u);
                }
            } else {
                t = xraw[j][m][0];
            }
            const uint32_t keep = (vrow < pm.M && J0 + j < p.NJ) ? ~0u : 0u;
#pragma unroll
            for (int i = 0; i < 4; i++) t[i] &= keep;
            aop[j][m] = t;
        }
    // ---- the rows' sums of x under every chunk (Q4_0, times -24) or group of 128, in the product's layout
    const u32x4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    f32x4 xs[XS_REGS ? JPW : 1][G128 ? 1 : 4];
    if constexpr (XS_REGS) {
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            if constexpr (G128) {
                xs[j][0] = zero4;
#pragma unroll
                for (int m = 0; m < 4; m++)
                    xs[j][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[j][m]), as_bf16x8(ones), xs[j][0], 0, 0, 0);
            } else {
#pragma unroll
                for (int m = 0; m < 4; m++) {
                    xs[j][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[j][m]), as_bf16x8(ones), zero4, 0, 0, 0);
#pragma unroll
                    for (int t = 0; t < 4; t++) xs[j][m][t] *= -24.0f;
                }
            }
        }
    }
    fin_bias[threadIdx.x] = __uint_as_float(p.bias_dtype == NQ_DT_F32 ? st_bias : st_bias << 16);  // (read after a barrier)
    if constexpr (LATE_FIRST) {
#pragma unroll
        for (int j = 0; j < JPW; j++)
#pragma unroll
            for (int m = 0; m < 4; m++) asm volatile("" : "+v"(aop[j][m]));  // (built before the request below)
        fetch(blockIdx.x, s0);
    }

    int buf = 0, nth = 0;  // nth: the tile's place among this workgroup's
    auto multiply = [&](int tile, Slot& s) {
        arrived(tile, s);
        const u32x4(&wv)[JPW] = s.wv;
        const uint2(&sc)[JPW] = s.sc;
        f32x4 acc = zero4;
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            const bool live = J0 + j < p.NJ;  // (a step past K: its A operand is zero; its scale is set to zero too)
            if constexpr (!G128) {
#pragma unroll
                for (int m = 0; m < 4; m++) {
                    const u32x4 bop = nib_word_to_bf16(wv[j][m], magic);
                    f32x4 cin;
                    if constexpr (XS_REGS) {
                        cin = xs[j][m];
                    } else {
                        cin = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[j][m]), as_bf16x8(ones), zero4, 0, 0, 0);
#pragma unroll
                        for (int t = 0; t < 4; t++) cin[t] *= -24.0f;
                    }
                    const f32x4 dd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[j][m]), as_bf16x8(bop), cin, 0, 0, 0);
                    const uint32_t sbits = (m < 2 ? sc[j].x : sc[j].y) >> (16 * (m & 1));
                    const float d = live ? __half2float(__ushort_as_half((uint16_t)(sbits & 0xFFFFu))) : 0.0f;
#pragma unroll
                    for (int t = 0; t < 4; t++) acc[t] = fmaf(d, dd[t], acc[t]);
                }
            } else {
                const float d = live ? __half2float(__ushort_as_half((uint16_t)(sc[j].x & 0xFFFFu))) : 0.0f;
                const float zoff = -(16.0f + (float)(sc[j].x >> 16));
                f32x4 dd;
#pragma unroll
                for (int t = 0; t < 4; t++) dd[t] = zoff * xs[j][0][t];
#pragma unroll
                for (int m = 0; m < 4; m++) {
                    const u32x4 bop = nib_word_to_bf16(wv[j][m], magic);
                    dd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[j][m]), as_bf16x8(bop), dd, 0, 0, 0);
                }
#pragma unroll
                for (int t = 0; t < 4; t++) acc[t] = fmaf(d, dd[t], acc[t]);
            }
        }
        *reinterpret_cast<f32x4*>(&red[buf][wave][lane * 4]) = acc;
        __syncthreads();
        // D[v][cc] sits in lane cc + 16 (v / 4), register v % 4.  Thread (row fr, column fc) sums its row's terms'
        // shares, each over the wavefronts in wave order.
        if (threadIdx.x < 256 && fr < pm.M && (!XF32 || fr < 5)) {
            float z = 0.0f;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int v = NT * fr + t;
                const int at = (fc + 16 * (v >> 2)) * 4 + (v & 3);
                float zt = red[buf][0][at];
#pragma unroll
                for (int w = 1; w < KW; w++) zt += red[buf][w][at];
                z = t == 0 ? zt : z + zt;
            }
            const int64_t n = (int64_t)tile * 16 + fc;
            if (n < p.N) {
                z += fin_bias[nth * 16 + fc];
                if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
                void* yp;
                int width, col;
                seg_lookup(p.seg, (int)n, yp, width, col);
                const int64_t o = (int64_t)fr * width + col;
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(yp)[o] = z;
                else
                    reinterpret_cast<uint16_t*>(yp)[o] = f32_to_bf16_rne(z);
            }
        }
        buf ^= 1, nth++;
    };
    for (int tile = blockIdx.x; tile < ntiles;) {
        fetch(tile + g, s1);
        multiply(tile, s0);
        if ((tile += g) >= ntiles) break;
        fetch(tile + g, s0);
        multiply(tile, s1);
        tile += g;
    }
}

// ---- tens to hundreds of activation rows over 4-bit codes ------------------------------------------------
// The same scheme over tiles of M: workgroup (x, y) owns the 16 activation rows of M tile y - their A operands for
// all of K sit in its wavefronts' registers for the whole call - and walks a share of the 16-row weight tiles.
// KW wavefronts split K (JPW steps of 128 k each) and the 16 / KW groups of them take different weight tiles at the
// same time; a group's [16 x 16] shares meet in LDS in wave order and 256 of its threads finish the tile (bias,
// ReLU or SwiGLU, part placement).  fp32 activations are three exact bf16 terms per value, i.e. three A operands
// and three MFMAs per chunk into one accumulator (JPW = 1 only: beyond, the operands no longer fit the registers).
// A weight tile is read once per M tile (from L2 after the first), an activation once per workgroup; K, the group
// count and the sum order follow IN alone, so a row gets the same bits in its own layer and in a row-fused one.
// LORA: `y += s (x A) B` of a frozen adapter (noeira/nn/peft/lora.mojo:292-349) in the same launch.  The workgroup
// holds its rows' x for all of K already, so h = x A [16 x rank] costs it a handful of MFMAs once (A's fp32 values as
// three exact bf16 terms against the one or three terms of x, products below 2^-24 of the largest left out), summed
// over the K split through LDS; s * h . B[:, columns] then enters each tile as four fp32 MFMAs, one each in the
// accumulators of the group's first four wavefronts (ranks 4 w .. 4 w + 3), whose shares meet in LDS with the K split's.
// With B = 0 that adds exact zeros and the base result keeps its bits.  A gate | up layer takes two adapters, the gate
// projection's on its even columns and the up projection's on the odd ones: two such MFMAs per wavefront, each with the
// other projection's columns of B set to zero.
// the sum of N wavefronts' shares of one output (256 floats apart), in wave order: all reads issued, then the additions
template <int N>
__device__ __forceinline__ float sum_shares(const float* r0) {
    float v[N];
#pragma unroll
    for (int w = 0; w < N; w++) v[w] = r0[w * 256];
    float z = v[0];
#pragma unroll
    for (int w = 1; w < N; w++) z += v[w];
    return z;
}
// (n = 4 .. 16, uniform: a loop over a run-time count would wait for every read before the next)
__device__ __forceinline__ float sum_shares_n(const float* r0, int n) {
    switch (n) {
        case 4: return sum_shares<4>(r0);
        case 5: return sum_shares<5>(r0);
        case 6: return sum_shares<6>(r0);
        case 7: return sum_shares<7>(r0);
        case 8: return sum_shares<8>(r0);
        case 9: return sum_shares<9>(r0);
        case 10: return sum_shares<10>(r0);
        case 11: return sum_shares<11>(r0);
        case 12: return sum_shares<12>(r0);
        case 13: return sum_shares<13>(r0);
        case 14: return sum_shares<14>(r0);
        case 15: return sum_shares<15>(r0);
        default: return sum_shares<16>(r0);
    }
}

// LORA: 0 none, 1 one adapter over the layer's columns, 2 a gate | up layer's pair of adapters (both added before SwiGLU)
template <int FMT, bool XF32, int JPW, int TB, int LORA>
__global__ __launch_bounds__(1024) void gemm_tile4_mt_kernel(const TileMrParams pm, const int kw) {
    const TileParams& p = pm.t;
    constexpr int LN = LORA == 2 ? 2 : 1;  // adapters
    constexpr bool G128 = FMT == NQ_FMT_W4_GROUP;
    constexpr int NT = XF32 ? 3 : 1;
    constexpr bool XS_REGS = (G128 || JPW <= 2) && !(LORA && !G128 && JPW >= 2);  // (registers: the adapter's operands need them)
    __shared__ __attribute__((aligned(16))) float red[2][16][256];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, q = lane >> 4;
    const int ng = 16 / kw;                      // groups of wavefronts, each on its own weight tile
    const int grp = wave / kw, kwi = wave - grp * kw;
    const bool active = grp < ng;
    const int ntiles = (p.N + 15) / 16;
    const int J0 = kwi * JPW;
    const int m0 = blockIdx.y * 16;
    const int rows = min(16, pm.M - m0);
    const int xrow = m0 + min(c, rows - 1);
    uint32_t magic = 0x41804180u;
    asm volatile("" : "+v"(magic));

    // a group's tiles: first, first + stride, ...; fetched TB at a time, a batch ahead of their use.  (TB = 1 is
    // what is launched: with 2 or 4 tiles in flight the same calls measured 3 - 10 % slower, and the hand-written
    // request and wait of the rows kernels, which keeps exactly one tile under way across the loop's back edge,
    // changed nothing here (960 -> 2560 at 256 rows: 9.35 against 9.48 us): a pass is not waiting for its codes.
    // Of that call's 8.9 us, finishing is 2.0 - 1.2 of them the stores of y in 64-byte row segments - the rest is the
    // launch, the operands' set-up and five passes of unpack, MFMA, LDS and barrier.)
    const int stride = gridDim.x * ng;
    const int first = blockIdx.x * ng + min(grp, ng - 1);
    auto fetch = [&](int it0, u32x4 (&wv)[TB][JPW], uint2 (&sc)[TB][JPW]) {
#pragma unroll
        for (int t = 0; t < TB; t++) {
            const int64_t R = min(first + (it0 + t) * stride, ntiles - 1);
#pragma unroll
            for (int j = 0; j < JPW; j++) {
                const int64_t at = R * p.NJ + min(J0 + j, p.NJ - 1);
                wv[t][j] = p.tile[at * 64 + lane];
                if constexpr (!G128) sc[t][j] = reinterpret_cast<const uint2*>(p.tscales)[at * 16 + c];
                else sc[t][j].x = reinterpret_cast<const uint32_t*>(p.tscales)[at * 16 + c], sc[t][j].y = 0;
            }
        }
    };
    u32x4 wv[TB][JPW], wn[TB][JPW];
    uint2 sc[TB][JPW], sn[TB][JPW];
    fetch(0, wv, sc);

    // ---- A operands, once: 16 bytes of bf16 per (term, step, MFMA); rows past M and k past K are zero
    u32x4 aop[NT][JPW][4];
#pragma unroll
    for (int j = 0; j < JPW; j++)
#pragma unroll
        for (int m = 0; m < 4; m++) {
            const int k0 = (J0 + j) * 128 + 32 * m + 8 * q;
            const int k = min(k0, p.K - 8);
            const uint32_t keep = (c < rows && k0 < p.K && active) ? ~0u : 0u;
            if constexpr (XF32) {
                const float* xf = reinterpret_cast<const float*>(p.x) + (int64_t)xrow * p.K + k;
                const u32x4 r0 = *reinterpret_cast<const u32x4*>(xf), r1 = *reinterpret_cast<const u32x4*>(xf + 4);
                uint32_t v[8];
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = r0[i] & keep, v[4 + i] = r1[i] & keep;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    // hi + mid + lo = the fp32 value (each split truncates: every residual is exact)
                    const uint32_t a = v[2 * i], b = v[2 * i + 1];
                    const float ra = __uint_as_float(a) - __uint_as_float(a & 0xFFFF0000u);
                    const float rb = __uint_as_float(b) - __uint_as_float(b & 0xFFFF0000u);
                    const float sa = ra - __uint_as_float(__float_as_uint(ra) & 0xFFFF0000u);
                    const float sb = rb - __uint_as_float(__float_as_uint(rb) & 0xFFFF0000u);
                    aop[0][j][m][i] = __builtin_amdgcn_perm(b, a, 0x07060302u);
                    aop[1][j][m][i] = __builtin_amdgcn_perm(__float_as_uint(rb), __float_as_uint(ra), 0x07060302u);
                    aop[2][j][m][i] = __builtin_amdgcn_perm(__float_as_uint(sb), __float_as_uint(sa), 0x07060302u);
                }
            } else {
                u32x4 t = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + (int64_t)xrow * p.K + k);
#pragma unroll
                for (int i = 0; i < 4; i++) t[i] &= keep;
                aop[0][j][m] = t;
            }
        }
    // ---- the rows' sums of x under every chunk (Q4_0, times -24) or group of 128, in the product's layout
    const u32x4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    const f32x4 zero4 = {0.0f, 0.0f, 0.0f, 0.0f};
    auto chunk_sum = [&](int j, int m, f32x4 into) {
#pragma unroll
        for (int t = NT - 1; t >= 0; t--)  // (smallest term first)
            into = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[t][j][m]), as_bf16x8(ones), into, 0, 0, 0);
        return into;
    };
    f32x4 xs[XS_REGS ? JPW : 1][G128 ? 1 : 4];
    if constexpr (XS_REGS) {
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            if constexpr (G128) {
                xs[j][0] = zero4;
#pragma unroll
                for (int m = 0; m < 4; m++) xs[j][0] = chunk_sum(j, m, xs[j][0]);
            } else {
#pragma unroll
                for (int m = 0; m < 4; m++) {
                    xs[j][m] = chunk_sum(j, m, zero4);
#pragma unroll
                    for (int t = 0; t < 4; t++) xs[j][m][t] *= -24.0f;
                }
            }
        }
    }
    // this thread's place in its group's finished tile: token row fr, weight row (column of y) fc.  (Finishing the
    // groups' neighbouring tiles side by side, a wavefront's stores covering whole 128-byte lines of y instead of
    // 64-byte halves, measured slower: 9.4 against 8.9 us on 960 -> 2560 at 256 rows.)
    const int f = threadIdx.x - grp * kw * 64;
    const bool finisher = active && f < 256;
    const int fr = (f >> 4) & 15, fc = f & 15;

    __shared__ float hfin[LN][LORA ? 4 : 1][16][17];
    if constexpr (LORA != 0) {
#pragma unroll
      for (int ad = 0; ad < LN; ad++) {
        const float* const lap = ad ? pm.la2 : pm.la;
        // h = x A over this wavefront's share of K: the MFMA's B operand is A[k][r] for 8 consecutive k of column
        // r = lane % 16 (ranks past lr, and k past K, are zero)
        // (the groups of a workgroup hold the same x: each forms h over every ng-th chunk and all sixteen shares
        // are summed, so that the splitting of A into bf16 terms - the vector ALU's work here - is done once)
        const int rc = min(c, pm.lr - 1);
        f32x4 hacc = zero4;
#pragma unroll
        for (int j = 0; j < JPW; j++)
#pragma unroll
            for (int m = 0; m < 4; m++) {
                const int ci = j * 4 + m;
                const bool mine = active && (ng == 1 || (ng == 2 && ((ci ^ grp) & 1) == 0) || (ng == 3 && ci % 3 == grp) ||
                                             (ng == 4 && (ci & 3) == grp));
                if (!mine) continue;  // (uniform)
                const int k0 = (J0 + j) * 128 + 32 * m + 8 * q;
                const uint32_t keep = (c < pm.lr && k0 < p.K && active) ? ~0u : 0u;
                uint32_t av[8];
#pragma unroll
                for (int i = 0; i < 8; i++)
                    av[i] = reinterpret_cast<const uint32_t*>(lap)[(int64_t)min(k0 + i, p.K - 1) * pm.lr + rc];
                u32x4 pl[3];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t a0 = av[2 * i] & keep, b0 = av[2 * i + 1] & keep;
                    const float ra = __uint_as_float(a0) - __uint_as_float(a0 & 0xFFFF0000u);
                    const float rb = __uint_as_float(b0) - __uint_as_float(b0 & 0xFFFF0000u);
                    const float sa = ra - __uint_as_float(__float_as_uint(ra) & 0xFFFF0000u);
                    const float sb = rb - __uint_as_float(__float_as_uint(rb) & 0xFFFF0000u);
                    pl[0][i] = __builtin_amdgcn_perm(b0, a0, 0x07060302u);
                    pl[1][i] = __builtin_amdgcn_perm(__float_as_uint(rb), __float_as_uint(ra), 0x07060302u);
                    pl[2][i] = __builtin_amdgcn_perm(__float_as_uint(sb), __float_as_uint(sa), 0x07060302u);
                }
                auto mm = [&](int xt, int at) {
                    hacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[xt][j][m]), as_bf16x8(pl[at]), hacc, 0, 0, 0);
                };
                if constexpr (XF32) {  // smallest products first
                    mm(1, 1), mm(2, 0), mm(0, 2), mm(1, 0), mm(0, 1), mm(0, 0);
                } else {
                    mm(0, 2), mm(0, 1), mm(0, 0);
                }
            }
        *reinterpret_cast<f32x4*>(&red[0][wave][lane * 4]) = hacc;
        __syncthreads();
        if (finisher) {
            const int at = (fc + 16 * (fr >> 2)) * 4 + (fr & 3);  // D[token fr][rank fc]
            const float hv = sum_shares_n(&red[0][0][at], ng * kw);
            hfin[ad][grp][fr][fc] = hv;
        }
        __syncthreads();
      }
    }
    // The adapter's share of a tile, s h B[:, columns], is four fp32 MFMAs of 16x16x4 (rank 16 as four k-extents)
    // before the K split's shares meet: the A operand is s h (token lane % 16, rank 4 m + lane / 16), kept in registers
    // for the whole call; the B operand B[rank][column lane % 16], one load per lane, tile and k-extent.  (The threads
    // that finish a tile used to do it: sixteen loads of B, sixteen LDS reads of h and sixteen FMAs per output; then
    // the group's first wavefront alone, all four MFMAs: on a tile of twelve bf16 MFMAs per wavefront that made the
    // group wait for it - 3 us on a 9 us call, 9 us with two adapters.)
    // (one of the four k-extents per wavefront: the first four wavefronts of a group take ranks 4 kwi .. 4 kwi + 3
    // each, so that no wavefront's tile is more than one such MFMA per adapter longer than the others')
    float hA[LN];
    const int lrank = 4 * kwi + q;
    if constexpr (LORA != 0) {
#pragma unroll
        for (int ad = 0; ad < LN; ad++)
            hA[ad] = (kwi < 4 && active && lrank < pm.lr) ? (ad ? pm.ls2 : pm.ls) * hfin[ad][grp][c][min(lrank, 15)] : 0.0f;
    }

    const int iters = (ntiles + stride - 1) / stride;
    int buf = 0;
    for (int it0 = 0; it0 < iters; it0 += TB) {
      const bool more = it0 + TB < iters;
      if (more) fetch(it0 + TB, wn, sn);  // the next batch is on its way while this one is multiplied
#pragma unroll
      for (int tb = 0; tb < TB; tb++) {
        const int it = it0 + tb;
        if (it >= iters) break;  // (uniform)
        const int tile = first + it * stride;
        const bool have = active && tile < ntiles;
        uint32_t braw = 0;
        const int64_t fn = min((int64_t)tile * 16 + fc, (int64_t)p.N - 1);
        if (p.bias && finisher)
            braw = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[fn]
                                               : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[fn];
        float lbf[LN];
        if constexpr (LORA == 1) {
            if (kwi < 4 && active) {  // (uniform per wavefront)
                const int64_t nb = min((int64_t)tile * 16 + c, (int64_t)p.N - 1);
                lbf[0] = pm.lb[(int64_t)min(lrank, pm.lr - 1) * p.N + nb];
            }
        } else if constexpr (LORA == 2) {
            // the lane's column is a gate column (even) or an up column (odd) of projection row nb / 2: one adapter's B
            // is loaded, the other's operand is zero there
            if (kwi < 4 && active) {
                const int64_t nb = min((int64_t)tile * 16 + c, (int64_t)p.N - 1);
                const bool up = (nb & 1) != 0;
                const float v = (up ? pm.lb2 : pm.lb)[(int64_t)min(lrank, pm.lr - 1) * (p.N >> 1) + (nb >> 1)];
                lbf[0] = up ? 0.0f : v, lbf[1] = up ? v : 0.0f;
            }
        }
        if (have) {
            f32x4 acc = zero4;
#pragma unroll
            for (int j = 0; j < JPW; j++) {
                const bool live = J0 + j < p.NJ;  // (a step past K: its A operand is zero; its scale is set to zero too)
                if constexpr (!G128) {
#pragma unroll
                    for (int m = 0; m < 4; m++) {
                        const u32x4 bop = nib_word_to_bf16(wv[tb][j][m], magic);
                        f32x4 dd;
                        if constexpr (XS_REGS) {
                            dd = xs[j][m];
                        } else {
                            dd = chunk_sum(j, m, zero4);
#pragma unroll
                            for (int t = 0; t < 4; t++) dd[t] *= -24.0f;
                        }
#pragma unroll
                        for (int t = NT - 1; t >= 0; t--)
                            dd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[t][j][m]), as_bf16x8(bop), dd, 0, 0, 0);
                        const uint32_t sbits = (m < 2 ? sc[tb][j].x : sc[tb][j].y) >> (16 * (m & 1));
                        const float d = live ? __half2float(__ushort_as_half((uint16_t)(sbits & 0xFFFFu))) : 0.0f;
#pragma unroll
                        for (int t = 0; t < 4; t++) acc[t] = fmaf(d, dd[t], acc[t]);
                    }
                } else {
                    const float d = live ? __half2float(__ushort_as_half((uint16_t)(sc[tb][j].x & 0xFFFFu))) : 0.0f;
                    const float zoff = -(16.0f + (float)(sc[tb][j].x >> 16));
                    f32x4 dd;
#pragma unroll
                    for (int t = 0; t < 4; t++) dd[t] = zoff * xs[j][0][t];
#pragma unroll
                    for (int m = 0; m < 4; m++) {
                        const u32x4 bop = nib_word_to_bf16(wv[tb][j][m], magic);
#pragma unroll
                        for (int t = NT - 1; t >= 0; t--)
                            dd = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[t][j][m]), as_bf16x8(bop), dd, 0, 0, 0);
                    }
#pragma unroll
                    for (int t = 0; t < 4; t++) acc[t] = fmaf(d, dd[t], acc[t]);
                }
            }
            if constexpr (LORA != 0) {
                if (kwi < 4) {
#pragma unroll
                    for (int ad = 0; ad < LN; ad++) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(hA[ad], lbf[ad], acc, 0, 0, 0);
                }
            }
            *reinterpret_cast<f32x4*>(&red[buf][wave][lane * 4]) = acc;
        }
        __syncthreads();
        // D[v][cc] sits in lane cc + 16 (v / 4), register v % 4: v the token row, cc the weight row
        if (finisher && have) {
            const int at = (fc + 16 * (fr >> 2)) * 4 + (fr & 3);
            const float* r0 = &red[buf][grp * kw][at];  // the group's shares, in wave order
            float z = sum_shares_n(r0, kw);
            const int n = tile * 16 + fc;
            if (p.bias) z += __uint_as_float(p.bias_dtype == NQ_DT_F32 ? braw : braw << 16);
            if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
            if (p.epilogue == NQ_EPI_SWIGLU) {  // (uniform) gate in the even column, up one lane over
                const float other = lane_xor1(z);
                if ((n & 1) == 0 && n + 1 < p.N && fr < rows) {
                    const float g = swiglu_f32(other, z);
                    const int64_t o = (int64_t)(m0 + fr) * (p.N >> 1) + (n >> 1);
                    if (p.y_dtype == NQ_DT_F32)
                        reinterpret_cast<float*>(p.seg.y[0])[o] = g;
                    else
                        reinterpret_cast<uint16_t*>(p.seg.y[0])[o] = f32_to_bf16_rne(g);
                }
            } else if (n < p.N && fr < rows) {
                void* yp;
                int width, col;
                seg_lookup(p.seg, n, yp, width, col);
                const int64_t o = (int64_t)(m0 + fr) * width + col;
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(yp)[o] = z;
                else
                    reinterpret_cast<uint16_t*>(yp)[o] = f32_to_bf16_rne(z);
            }
        }
        buf ^= 1;
      }
      if (more) {
#pragma unroll
        for (int t = 0; t < TB; t++)
#pragma unroll
            for (int j = 0; j < JPW; j++) wv[t][j] = wn[t][j], sc[t][j] = sn[t][j];
      }
    }
}

// ---- int8 codes -----------------------------------------------------------------------------------
constexpr float MAGIC = 12582912.0f;  // 1.5 * 2^23: the low byte of (t + MAGIC)'s bits is rne(t) as an int8

__device__ __forceinline__ uint32_t pack_low_bytes(uint32_t a0, uint32_t a1, uint32_t a2, uint32_t a3) {
    return __builtin_amdgcn_perm(a1, a0, 0x0c0c0400u) | __builtin_amdgcn_perm(a3, a2, 0x04000c0cu);
}

// ---- 4-bit codes on the int8 matrix cores ----------------------------------------------------------------
// The same tile, read as int8: a word of the tile holds eight codes as nibbles, and `w & 0x0F0F0F0F`,
// `(w >> 4) & 0x0F0F0F0F` are each four of them as bytes (elements 0, 4, 1, 5 and 2, 6, 3, 7 of the word's eight
// k), so a lane's 16 bytes become the B operands of two v_mfma_i32_16x16x64_i8 with 12 instructions, where the bf16
// route spends 32 on its four.  x is split per wavefront slice into three int8 terms under one scale, as for int8
// weights (x = (absmax / 127) (q1 + q2 / 254 + q3 / 254^2) + e, |e| <= 6e-8 absmax; a NaN or infinity in x makes
// every output NaN), written to LDS in the bytes' own order, and sits in the MFMA's A rows - once per slice, in
// registers.  Which rows: a word of a lane belongs to ONE chunk of 32 k (word m = chunk m of the tile), so with
// Q4_0, whose every chunk has its own scale, A row 4 G + t carries term t in word G only and zeros elsewhere: the
// MFMA's result row 4 G + t is then chunk G's sum for term t, and it lands in lane n + 16 G, register t - each of a
// weight row's four lanes finishes one chunk: three conversions, the three terms' weights, -8 times the chunk's sum
// of x (fp32, from the x stage), the chunk's scale.  Groups of 128: rows 0 .. 2 carry the terms in every word, lane
// n finishes the tile.  A workgroup takes RT row tiles, which share the x stage.
constexpr int T4I_MAXT = 8;  // row tiles a workgroup walks at most
template <int FMT, bool XF32, int KW, int JPW>
__global__ __launch_bounds__(64 * KW) void gemv_tile4i_kernel(const TileParams p) {
    constexpr bool EXACT = false;
    constexpr bool G128 = FMT == NQ_FMT_W4_GROUP;
    constexpr int NO = JPW * 16;  // octets (8 consecutive k) of x per wavefront and round: one per lane
    static_assert(JPW >= 1 && JPW <= 4, "a lane holds one octet of the slice");
    __shared__ __attribute__((aligned(16))) uint32_t xq[KW][3][2][NO];  // [term][lo / hi bytes][16 j + 4 q + m]
    __shared__ float xsum[KW][G128 ? JPW : JPW * 4];
    __shared__ float red[T4I_MAXT][KW][16];
    __shared__ RowTail tails[T4I_MAXT][16];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, q = lane >> 4;
    const int NR = (p.N + 15) / 16;
    // The workgroup walks row tiles blockIdx.x, blockIdx.x + gridDim.x, ... (at most T4I_MAXT); wavefront w keeps the
    // same slice of K in all of them, so x is split once and its A operands stay in registers, and the next
    // tile's codes are requested before the current one is multiplied.
    // That request and the wait for the current tile are written out (two register slots in turn, no copies): the
    // compiler's own counts would drain the tile requested ahead at the end of every pass through the loop.  A
    // fetch is 2 JPW loads (codes and records of every step), so with the next tile under way "all but the youngest
    // 2 JPW" is the tile about to be multiplied; loads and stores the compiler issues in between only make that wait
    // longer.  The waits name no registers (nothing is copied ahead of them); the hand-over that follows them on
    // every path does, so that nothing reads a slot before its wait.
    const int J0 = wave * JPW;
    const int g = gridDim.x;
    struct Slot {
        u32x4 wv[JPW];
        uint32_t sc[JPW];
    };
    auto fetch = [&](int64_t R, Slot& s) {
        const u32x4* const wbase = p.tile + R * p.NJ * 64;
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            const u32x4* const src = wbase + (min(J0 + j, p.NJ - 1) * 64 + lane);
            asm volatile("global_load_dwordx4 %0, %1, off nt ; pf" : "=v"(s.wv[j]) : "v"(src));
        }
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            const int64_t at = (R * p.NJ + min(J0 + j, p.NJ - 1)) * 16 + c;
            if constexpr (!G128) {
                const uint16_t* const src = reinterpret_cast<const uint16_t*>(p.tscales) + (at * 4 + q);  // chunk q's scale
                asm volatile("global_load_ushort %0, %1, off ; pf" : "=v"(s.sc[j]) : "v"(src));
            } else {
                const uint32_t* const src = reinterpret_cast<const uint32_t*>(p.tscales) + at;
                asm volatile("global_load_dword %0, %1, off ; pf" : "=v"(s.sc[j]) : "v"(src));
            }
        }
    };
    auto arrived = [&](bool next_under_way, Slot& s) {
        if (next_under_way) {
            if constexpr (JPW == 1) asm volatile("s_waitcnt vmcnt(2)");
            if constexpr (JPW == 2) asm volatile("s_waitcnt vmcnt(4)");
            if constexpr (JPW == 3) asm volatile("s_waitcnt vmcnt(6)");
            if constexpr (JPW == 4) asm volatile("s_waitcnt vmcnt(8)");
        } else {
            asm volatile("s_waitcnt vmcnt(0)");
        }
        if constexpr (JPW == 1) asm volatile("; pfh %0 %1" : "+v"(s.wv[0]), "+v"(s.sc[0]));
        if constexpr (JPW == 2) asm volatile("; pfh %0 %1 %2 %3" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.sc[0]), "+v"(s.sc[1]));
        if constexpr (JPW == 3)
            asm volatile("; pfh %0 %1 %2 %3 %4 %5" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.wv[2]), "+v"(s.sc[0]), "+v"(s.sc[1]), "+v"(s.sc[2]));
        if constexpr (JPW == 4)
            asm volatile("; pfh %0 %1 %2 %3 %4 %5 %6 %7" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.wv[2]), "+v"(s.wv[3]), "+v"(s.sc[0]), "+v"(s.sc[1]),
                         "+v"(s.sc[2]), "+v"(s.sc[3]));
    };
    // what finishing needs, for all of this workgroup's tiles: thread (tile i, row r) requests it first of all
    RowTail my_tail{};
    if ((int)threadIdx.x < 16 * T4I_MAXT) {
        const int64_t Rt = (int64_t)blockIdx.x + (int64_t)(threadIdx.x >> 4) * g;
        if (Rt < NR) my_tail = fetch_tail(p, Rt, threadIdx.x & 15);
    }
    Slot s0, s1;
    i32x4 aq[JPW][2];
    float xz[JPW];
    float s_x;
    {
        // x first, then the first tile's codes and their records, every load from a clamped address
        const int k0 = J0 * 128 + min(lane, NO - 1) * 8;
        const int kc = EXACT ? k0 : min(k0, p.K - 8);
        const bool live = EXACT || k0 < p.K;
        u32x4 xr[XF32 ? 2 : 1];
        if constexpr (XF32) {
            const float* xf = reinterpret_cast<const float*>(p.x) + kc;
            xr[0] = *reinterpret_cast<const u32x4*>(xf), xr[1] = *reinterpret_cast<const u32x4*>(xf + 4);
        } else {
            xr[0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + kc);
        }
        fetch(blockIdx.x, s0);
        float xf[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if constexpr (XF32) xf[i] = __uint_as_float(xr[i / 4][i % 4]);
            else xf[i] = (i & 1) ? __uint_as_float(xr[0][i / 2] & 0xFFFF0000u) : __uint_as_float(xr[0][i / 2] << 16);
            if (!live) xf[i] = 0.0f;
        }
        // the slice's largest magnitude as a bit pattern (NaN > inf > finite), over the wavefront
        uint32_t mbits = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) mbits = max(mbits, __float_as_uint(xf[i]) & 0x7FFFFFFFu);
        mbits = max(mbits, (uint32_t)NQ_DPP(mbits, 0xB1));
        mbits = max(mbits, (uint32_t)NQ_DPP(mbits, 0x4E));
        mbits = max(mbits, (uint32_t)NQ_DPP(mbits, 0x141));
        mbits = max(mbits, (uint32_t)NQ_DPP(mbits, 0x140));
        {
            const auto sw = __builtin_amdgcn_permlane16_swap(mbits, mbits, false, false);
            mbits = max(sw[0], sw[1]);
        }
        {
            const auto sw = __builtin_amdgcn_permlane32_swap(mbits, mbits, false, false);
            mbits = max(sw[0], sw[1]);
        }
        const bool finite = mbits < 0x7F800000u;
        // a slice whose largest magnitude is below 2^-60 is lifted by 2^64 first (exact), so that 127 / absmax stays
        // finite and the slice keeps its three terms (an all-tiny x is still a vector with a direction)
        const float lift = mbits < 0x21800000u ? 0x1p64f : 1.0f;
        const float absmax = __uint_as_float(mbits) * lift;
        const float inv_s = (finite && absmax > 0.0f) ? 127.0f / absmax : 0.0f;
        s_x = finite ? (absmax * (1.0f / 127.0f)) / lift : __uint_as_float(0x7FC00000u);
        uint32_t a1[8], a2[8], a3[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            // round by adding 1.5 * 2^23 (the sum's low byte is the int8) and take every leftover against the very
            // integer that was packed: no leftover exceeds a half, no term leaves the int8 range
            const float t = (xf[e] * lift) * inv_s;
            const float b1 = t + MAGIC;
            a1[e] = __float_as_uint(b1);
            const float r1 = t - (b1 - MAGIC);
            const float b2 = __builtin_fmaf(r1, 254.0f, MAGIC);
            a2[e] = __float_as_uint(b2);
            const float r2 = __builtin_fmaf(r1, 254.0f, MAGIC - b2);
            a3[e] = __float_as_uint(__builtin_fmaf(r2, 254.0f, MAGIC));
        }
        // the sum of x under a chunk (four lanes), under a group of 128 (sixteen): fixed butterflies
        float ps = ((xf[0] + xf[1]) + (xf[2] + xf[3])) + ((xf[4] + xf[5]) + (xf[6] + xf[7]));
        ps += NQ_DPP_F32(ps, 0xB1);
        ps += NQ_DPP_F32(ps, 0x4E);
        if constexpr (G128) {
            ps += NQ_DPP_F32(ps, 0x141);
            ps += NQ_DPP_F32(ps, 0x140);
        }
        if (lane < NO) {
            // octet l of the slice is k = 8 l ..: tile j = l / 16, chunk m = (l / 4) % 4, piece q = l % 4
            const int at = (lane & ~15) + (lane & 3) * 4 + ((lane >> 2) & 3);
            xq[wave][0][0][at] = pack_low_bytes(a1[0], a1[4], a1[1], a1[5]), xq[wave][0][1][at] = pack_low_bytes(a1[2], a1[6], a1[3], a1[7]);
            xq[wave][1][0][at] = pack_low_bytes(a2[0], a2[4], a2[1], a2[5]), xq[wave][1][1][at] = pack_low_bytes(a2[2], a2[6], a2[3], a2[7]);
            xq[wave][2][0][at] = pack_low_bytes(a3[0], a3[4], a3[1], a3[5]), xq[wave][2][1][at] = pack_low_bytes(a3[2], a3[6], a3[3], a3[7]);
            if constexpr (!G128) {
                if ((lane & 3) == 0) xsum[wave][lane >> 2] = -8.0f * ps;
            } else {
                if ((lane & 15) == 0) xsum[wave][lane >> 4] = ps;
            }
        }
        // (the region is this wavefront's own and a wavefront's LDS accesses execute in order)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // the A operands of the slice's tiles, and this lane's zero-point terms
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            if constexpr (!G128) {
                const int G = c >> 2, t = c & 3;  // A row c = 4 G + t
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    uint32_t v = xq[wave][min(t, 2)][h][j * 16 + q * 4 + G];
                    v = t < 3 ? v : 0u;
                    aq[j][h] = (i32x4){(int)(G == 0 ? v : 0u), (int)(G == 1 ? v : 0u), (int)(G == 2 ? v : 0u), (int)(G == 3 ? v : 0u)};
                }
                xz[j] = xsum[wave][j * 4 + q];
            } else {
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    i32x4 v = *reinterpret_cast<const i32x4*>(&xq[wave][min(c, 2)][h][j * 16 + q * 4]);
                    if (c >= 3) v = (i32x4){0, 0, 0, 0};
                    aq[j][h] = v;
                }
                xz[j] = xsum[wave][j];
            }
        }
    }
    if ((int)threadIdx.x < 16 * T4I_MAXT) tails[threadIdx.x >> 4][threadIdx.x & 15] = my_tail;  // (read after the barrier)
    auto multiply = [&](int nt, bool next_under_way, Slot& s) {
        arrived(next_under_way, s);
        const u32x4(&wv)[JPW] = s.wv;
        const uint32_t(&sc)[JPW] = s.sc;
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            const bool live_j = J0 + j < p.NJ;  // (a step past K: its x is zero; its scale is set to zero too)
            const u32x4 w = wv[j];
            i32x4 lo, hi;
#pragma unroll
            for (int m = 0; m < 4; m++) lo[m] = (int)(w[m] & 0x0F0F0F0Fu), hi[m] = (int)((w[m] >> 4) & 0x0F0F0F0Fu);
            i32x4 d = {0, 0, 0, 0};
            d = __builtin_amdgcn_mfma_i32_16x16x64_i8(aq[j][0], lo, d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_i32_16x16x64_i8(aq[j][1], hi, d, 0, 0, 0);
            // |sum| <= 15 * 127 * 128 < 2^24: exact as fp32
            const float f = fmaf((float)d[2], 1.0f / 64516.0f, fmaf((float)d[1], 1.0f / 254.0f, (float)d[0]));
            if constexpr (!G128) {
                const float ds = live_j ? __half2float(__ushort_as_half((uint16_t)sc[j])) : 0.0f;
                acc = fmaf(ds, fmaf(s_x, f, xz[j]), acc);
            } else {
                const float ds = (live_j && q == 0) ? __half2float(__ushort_as_half((uint16_t)(sc[j] & 0xFFFFu))) : 0.0f;
                const float z = (float)(sc[j] >> 16);
                acc = fmaf(ds, fmaf(s_x, f, -z * xz[j]), acc);
            }
        }
        // a row's four lanes (its chunks' shares); the wavefronts' shares meet once, after the last tile
        acc += __shfl_xor(acc, 16);
        acc += __shfl_xor(acc, 32);
        if (q == 0) red[nt][wave][c] = acc;
    };
    int nt = 0;
    // (one tile ahead: requesting the tile after next as well measured slower, here as in the rows kernels)
    for (int64_t R = blockIdx.x;;) {
        bool more = R + g < NR && nt + 1 < T4I_MAXT;
        if (more) fetch(R + g, s1);
        multiply(nt++, more, s0);
        if (!more) break;
        R += g;
        more = R + g < NR && nt + 1 < T4I_MAXT;
        if (more) fetch(R + g, s0);
        multiply(nt++, more, s1);
        if (!more) break;
        R += g;
    }
    __syncthreads();
    // thread (tile i, row r): the wavefronts' shares in wave order, bias, epilogue, placement by part
    if ((int)threadIdx.x < 16 * nt) {
        const int i = threadIdx.x >> 4, r = threadIdx.x & 15;
        float z = red[i][0][r];
#pragma unroll
        for (int w = 1; w < KW; w++) z += red[i][w][r];
        const int64_t n = ((int64_t)blockIdx.x + (int64_t)i * gridDim.x) * 16 + r;
        if (n < p.N) {
            const RowTail t = tails[i][r];
            if (p.bias) z += __uint_as_float(p.bias_dtype == NQ_DT_F32 ? t.braw : t.braw << 16);
            if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
            void* yp;
            int width, col;
            seg_lookup(p.seg, (int)n, yp, width, col);  // M = 1: the part's row is its only row
            if (p.y_dtype == NQ_DT_F32)
                reinterpret_cast<float*>(yp)[col] = z;
            else
                reinterpret_cast<uint16_t*>(yp)[col] = f32_to_bf16_rne(z);
        }
    }
}

template <bool XF32, int KW, int JPW, bool EXACT>
__global__ __launch_bounds__(64 * KW) void gemv_tile8_kernel(const TileParams p) {
    constexpr int SL = JPW * 64;  // k per wavefront and round
    constexpr int VPL = SL > 256 ? 8 : 4;  // values of x per lane (one or two words of int8 per term)
    constexpr int NL = SL / VPL;           // lanes that hold a piece of the slice (16 .. 64)
    __shared__ __attribute__((aligned(16))) uint8_t xq[KW][3][SL];
    __shared__ float red[KW][16];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, q = lane >> 4;
    const int64_t R = blockIdx.x;
    const uint8_t* const arow = &xq[wave][min(c, 2)][q * 16];
    float accf = 0.0f;

    RowTail tail{};
    if (wave == 0) tail = fetch_tail(p, R, lane);

    for (int J0 = wave * JPW; J0 < p.NJ; J0 += EXACT ? p.NJ : KW * JPW) {
        // x first (it is needed first, and waiting for it leaves the codes in flight), every load from a clamped
        // address.  The slice of x under this round: lane l < NL holds values VPL l .. ; past K they are zero.
        const int k0 = J0 * 64 + min(lane, NL - 1) * VPL;
        const int kc = EXACT ? k0 : min(k0, p.K - VPL);
        const bool live = EXACT || k0 < p.K;
        uint32_t xraw[XF32 ? VPL : VPL / 2];
        if constexpr (XF32) {
            const float* xr = reinterpret_cast<const float*>(p.x) + kc;
#pragma unroll
            for (int i = 0; i < VPL; i += 4) {
                const u32x4 t = *reinterpret_cast<const u32x4*>(xr + i);
                xraw[i] = t[0], xraw[i + 1] = t[1], xraw[i + 2] = t[2], xraw[i + 3] = t[3];
            }
        } else {
            const uint32_t* xr = reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(p.x) + kc);
            if constexpr (VPL == 8) {
                const u32x4 v = *reinterpret_cast<const u32x4*>(xr);
                xraw[0] = v[0], xraw[1] = v[1], xraw[2] = v[2], xraw[3] = v[3];
            } else {
                const uint2 v = *reinterpret_cast<const uint2*>(xr);
                xraw[0] = v.x, xraw[1] = v.y;
            }
        }
        u32x4 wv[JPW];
        const u32x4* const wbase = p.tile + R * p.NJ * 64;  // (32-bit offsets from the tile's base)
#pragma unroll
        for (int j = 0; j < JPW; j++) wv[j] = __builtin_nontemporal_load(wbase + ((EXACT ? J0 + j : min(J0 + j, p.NJ - 1)) * 64 + lane));
        float xf[VPL];
#pragma unroll
        for (int i = 0; i < VPL; i++) {
            if constexpr (XF32) xf[i] = __uint_as_float(xraw[i]);
            else xf[i] = (i & 1) ? __uint_as_float(xraw[i / 2] & 0xFFFF0000u) : __uint_as_float(xraw[i / 2] << 16);
        }
        // the slice's largest magnitude as a bit pattern (NaN > inf > finite), over the wavefront
        uint32_t mbits = 0;
#pragma unroll
        for (int i = 0; i < VPL; i++) {
            if (!live) xf[i] = 0.0f;
            mbits = max(mbits, __float_as_uint(xf[i]) & 0x7FFFFFFFu);
        }
        mbits = max(mbits, (uint32_t)NQ_DPP(mbits, 0xB1));
        mbits = max(mbits, (uint32_t)NQ_DPP(mbits, 0x4E));
        mbits = max(mbits, (uint32_t)NQ_DPP(mbits, 0x141));
        mbits = max(mbits, (uint32_t)NQ_DPP(mbits, 0x140));
        {
            const auto sw = __builtin_amdgcn_permlane16_swap(mbits, mbits, false, false);
            mbits = max(sw[0], sw[1]);
        }
        {
            const auto sw = __builtin_amdgcn_permlane32_swap(mbits, mbits, false, false);
            mbits = max(sw[0], sw[1]);
        }
        const bool finite = mbits < 0x7F800000u;
        // (a slice below 2^-60 is lifted by 2^64 first, exactly: 127 / absmax then stays finite)
        const float lift = mbits < 0x21800000u ? 0x1p64f : 1.0f;
        const float absmax = __uint_as_float(mbits) * lift;
        const float inv_s = (finite && absmax > 0.0f) ? 127.0f / absmax : 0.0f;
        // a NaN or an infinity in the slice makes the slice's share, hence every output, NaN
        const float s_x = finite ? (absmax * (1.0f / 127.0f)) / lift : __uint_as_float(0x7FC00000u);
        uint32_t pk[3][VPL / 4];
#pragma unroll
        for (int i = 0; i < VPL; i += 4) {
            uint32_t a1[4], a2[4], a3[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                // round by adding 1.5 * 2^23 (the sum's low byte is the int8) and take every leftover against the
                // very integer that was packed: no leftover exceeds a half, no term leaves the int8 range
                const float t = (xf[i + e] * lift) * inv_s;
                const float b1 = t + MAGIC;
                a1[e] = __float_as_uint(b1);
                const float r1 = t - (b1 - MAGIC);
                const float b2 = __builtin_fmaf(r1, 254.0f, MAGIC);
                a2[e] = __float_as_uint(b2);
                const float r2 = __builtin_fmaf(r1, 254.0f, MAGIC - b2);
                a3[e] = __float_as_uint(__builtin_fmaf(r2, 254.0f, MAGIC));
            }
            pk[0][i / 4] = pack_low_bytes(a1[0], a1[1], a1[2], a1[3]);
            pk[1][i / 4] = pack_low_bytes(a2[0], a2[1], a2[2], a2[3]);
            pk[2][i / 4] = pack_low_bytes(a3[0], a3[1], a3[2], a3[3]);
        }
        if (lane < NL) {
#pragma unroll
            for (int t = 0; t < 3; t++) {
                if constexpr (VPL == 8)
                    *reinterpret_cast<uint2*>(&xq[wave][t][lane * 8]) = make_uint2(pk[t][0], pk[t][1]);
                else
                    *reinterpret_cast<uint32_t*>(&xq[wave][t][lane * 4]) = pk[t][0];
            }
        }
        i32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            const i32x4 aop = *reinterpret_cast<const i32x4*>(arow + 64 * j);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, __builtin_bit_cast(i32x4, wv[j]), acc, 0, 0, 0);
        }
        // |sum| <= 128 * 127 * 512 < 2^24: exact as fp32
        accf += s_x * fmaf((float)acc[2], 1.0f / 64516.0f, fmaf((float)acc[1], 1.0f / 254.0f, (float)acc[0]));
    }
    if (q == 0) red[wave][c] = accf;
    __syncthreads();
    finish_rows<KW>(p, red, R, tail);
}

// ---- a few activation rows (2 <= M <= 16, fp32 rows 2 <= M <= 5) over int8 codes -----------------------------
// As over 4-bit codes: the activation rows are the MFMA's A rows (a bf16 row as it is, an fp32 row as the three bf16
// rows that sum to it), loaded once per workgroup into registers; the tile's codes become bf16 exactly (one
// sign-extending conversion per code, one byte permute per pair) and a step of 64 k is two 16x16x32 MFMAs: a lane's 16
// codes are k = 64 J + 16 q .. + 15 of weight row c, and the first MFMA takes the first eight under the name
// "k slot (q, i)", the second the other eight, the A operands following the same naming.  One workgroup of 16
// wavefronts per CU walks the row tiles with the next tile requested ahead of the one being multiplied (two register
// slots in turn, no copies); the column scales and biases of all its tiles are staged in LDS before the loop, so that
// nothing a tile needs is requested after younger loads (a wait counts loads in order of issue).  Sums over the
// wavefronts in wave order: the same bits on every call.
template <bool XF32, int JPW>
__global__ __launch_bounds__(1024) void gemv_tile8_rows_kernel(const TileMrParams pm) {
    const TileParams& p = pm.t;
    constexpr int KW = 16;
    constexpr int NT = XF32 ? 3 : 1;
    __shared__ __attribute__((aligned(16))) float red[2][KW][256];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15, q = lane >> 4;
    const int ntiles = (p.N + 15) / 16;
    const int J0 = wave * JPW;
    const int vrow = c / NT, vterm = c % NT;  // this lane's A row: activation row and term
    const int xrow = min(vrow, pm.M - 1);
    const int fr = threadIdx.x >> 4, fc = threadIdx.x & 15;  // threads 0 .. 255 finish a tile: row fr, column fc

    // ---- what finishing needs, for all of this workgroup's tiles at once (at most TR_MAXT of them): thread i stages
    // the scale and the bias of column i % 16 of its tile i / 16.  These are the oldest loads; then the activations,
    // then the first tile: the loop's only loads are tiles' codes.
    __shared__ float fin_scale[TR_MAXT * 16], fin_bias[TR_MAXT * 16];
    const int g = gridDim.x;
    float st_scale = 0.0f;
    uint32_t st_bias = 0;
    {
        const int64_t n = min(((int64_t)blockIdx.x + (int64_t)fr * g) * 16 + fc, (int64_t)p.N - 1);
        st_scale = p.col_scale[n];
        if (p.bias)  // (as loaded: a shift here would wait for the load)
            st_bias = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[n]
                                                  : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n];
    }
    struct Slot {
        u32x4 wv[JPW];
    };
    // The tiles' loads and the waits for them are written out: the compiler's own wait counts are exact in straight
    // code only, and across the loop's back edge they drain the tile requested ahead together with the one about to
    // be multiplied.  A fetch is JPW loads, so with the next tile under way "all but the youngest JPW" is the tile
    // about to be multiplied; loads and stores the compiler issues in between only make that wait longer.  arrived()
    // hands the registers on: nothing reads them before the wait.
    auto fetch = [&](int tile, Slot& s) {
        if (tile >= ntiles) return;
#pragma unroll
        for (int j = 0; j < JPW; j++) {
            const u32x4* const src = p.tile + (((int64_t)tile * p.NJ + min(J0 + j, p.NJ - 1)) * 64 + lane);
            asm volatile("global_load_dwordx4 %0, %1, off nt ; pf" : "=v"(s.wv[j]) : "v"(src));
        }
    };
    auto arrived = [&](int tile, Slot& s) {  // (the next tile is under way if there is one)
        // (the waits name no registers, so that nothing is copied ahead of them; the hand-over follows on every path)
        if (tile + g < ntiles) {
            if constexpr (JPW == 1) asm volatile("s_waitcnt vmcnt(1)");
            if constexpr (JPW == 2) asm volatile("s_waitcnt vmcnt(2)");
            if constexpr (JPW == 3) asm volatile("s_waitcnt vmcnt(3)");
            if constexpr (JPW == 4) asm volatile("s_waitcnt vmcnt(4)");
        } else {
            asm volatile("s_waitcnt vmcnt(0)");
        }
        if constexpr (JPW == 1) asm volatile("; pfh %0" : "+v"(s.wv[0]));
        if constexpr (JPW == 2) asm volatile("; pfh %0 %1" : "+v"(s.wv[0]), "+v"(s.wv[1]));
        if constexpr (JPW == 3) asm volatile("; pfh %0 %1 %2" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.wv[2]));
        if constexpr (JPW == 4) asm volatile("; pfh %0 %1 %2 %3" : "+v"(s.wv[0]), "+v"(s.wv[1]), "+v"(s.wv[2]), "+v"(s.wv[3]));
    };
    // ---- the activations first (the oldest loads: waiting for them leaves the tiles' loads under way), then two tiles
    u32x4 xraw[JPW][2][XF32 ? 2 : 1];
#pragma unroll
    for (int j = 0; j < JPW; j++)
#pragma unroll
        for (int m = 0; m < 2; m++) {
            const int k = min((J0 + j) * 64 + 16 * q + 8 * m, p.K - 8);
            if constexpr (XF32) {
                const float* xf = reinterpret_cast<const float*>(p.x) + (int64_t)xrow * p.K + k;
                xraw[j][m][0] = *reinterpret_cast<const u32x4*>(xf), xraw[j][m][XF32 ? 1 : 0] = *reinterpret_cast<const u32x4*>(xf + 4);
            } else {
                xraw[j][m][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + (int64_t)xrow * p.K + k);
            }
        }
    Slot s0, s1;
    fetch(blockIdx.x, s0);

    // ---- A operands, once: 16 bytes of bf16 per (step, MFMA); rows past M and steps past K are zero
    u32x4 aop[JPW][2];
#pragma unroll
    for (int j = 0; j < JPW; j++)
#pragma unroll
        for (int m = 0; m < 2; m++) {
            u32x4 t;
            if constexpr (XF32) {
                const u32x4 r0 = xraw[j][m][0], r1 = xraw[j][m][XF32 ? 1 : 0];
                uint32_t v[8];
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = r0[i], v[4 + i] = r1[i];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    // hi + mid + lo = the fp32 value (each split truncates: every residual is exact); this lane keeps one
                    const uint32_t a = v[2 * i], b = v[2 * i + 1];
                    const float ra = __uint_as_float(a) - __uint_as_float(a & 0xFFFF0000u);
                    const float rb = __uint_as_float(b) - __uint_as_float(b & 0xFFFF0000u);
                    const float sa = ra - __uint_as_float(__float_as_uint(ra) & 0xFFFF0000u);
                    const float sb = rb - __uint_as_float(__float_as_uint(rb) & 0xFFFF0000u);
                    const uint32_t ta = vterm == 0 ? a : vterm == 1 ? __float_as_uint(ra) : __float_as_uint(sa);
                    const uint32_t tb = vterm == 0 ? b : vterm == 1 ? __float_as_uint(rb) : __float_as_uint(sb);
                    t[i] = __builtin_amdgcn_perm(tb, ta, 0x07060302u);
                }
            } else {
                t = xraw[j][m][0];
            }
            const uint32_t keep = (vrow < pm.M && J0 + j < p.NJ) ? ~0u : 0u;
#pragma unroll
            for (int i = 0; i < 4; i++) t[i] &= keep;
            aop[j][m] = t;
        }

    fin_scale[threadIdx.x] = st_scale;  // (read after a tile's barrier)
    fin_bias[threadIdx.x] = __uint_as_float(p.bias_dtype == NQ_DT_F32 ? st_bias : st_bias << 16);

    int buf = 0, nth = 0;  // nth: the tile's place among this workgroup's
    auto multiply = [&](int tile, Slot& s) {
        arrived(tile, s);
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < JPW; j++)
#pragma unroll
            for (int m = 0; m < 2; m++) {
                u32x4 bop;
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const uint32_t w = s.wv[j][2 * m + h];
                    const float f0 = (float)(int8_t)w, f1 = (float)(int8_t)(w >> 8), f2 = (float)(int8_t)(w >> 16),
                                f3 = (float)((int32_t)w >> 24);
                    bop[2 * h] = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
                    bop[2 * h + 1] = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
                }
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(aop[j][m]), as_bf16x8(bop), acc, 0, 0, 0);
            }
        *reinterpret_cast<f32x4*>(&red[buf][wave][lane * 4]) = acc;
        __syncthreads();
        // D[v][cc] sits in lane cc + 16 (v / 4), register v % 4.  Thread (row fr, column fc) sums its row's terms'
        // shares, each over the wavefronts in wave order.
        if (threadIdx.x < 256 && fr < pm.M && (!XF32 || fr < 5)) {
            float z = 0.0f;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int v = NT * fr + t;
                const int at = (fc + 16 * (v >> 2)) * 4 + (v & 3);
                float zt = red[buf][0][at];
#pragma unroll
                for (int w = 1; w < KW; w++) zt += red[buf][w][at];
                z = t == 0 ? zt : z + zt;
            }
            const int64_t n = (int64_t)tile * 16 + fc;
            if (n < p.N) {
                z = z * fin_scale[nth * 16 + fc] + fin_bias[nth * 16 + fc];
                if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
                void* yp;
                int width, col;
                seg_lookup(p.seg, (int)n, yp, width, col);
                const int64_t o = (int64_t)fr * width + col;
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(yp)[o] = z;
                else
                    reinterpret_cast<uint16_t*>(yp)[o] = f32_to_bf16_rne(z);
            }
        }
        buf ^= 1, nth++;
    };
    for (int tile = blockIdx.x; tile < ntiles;) {
        fetch(tile + g, s1);
        multiply(tile, s0);
        if ((tile += g) >= ntiles) break;
        fetch(tile + g, s0);
        multiply(tile, s1);
        tile += g;
    }
}

// ---- load time: the tile-ordered copies -------------------------------------------------------------
// codes [N][nch][4 words] (row order) -> tile[R][J][lane][4 words]; one thread per lane slot
// (nch: 16-byte chunks per row; a row's last tile may hold fewer than four: the rest is zero codes under zero scales)
__global__ __launch_bounds__(256) void tile4_repack_kernel(const uint32_t* __restrict__ codes, u32x4* __restrict__ tile,
                                                           int64_t N, int64_t NJ, int64_t nch, int64_t slots) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= slots) return;
    const int l = (int)(t & 63), c = l & 15, q = l >> 4;
    const int64_t J = (t >> 6) % NJ, R = (t >> 6) / NJ, row = R * 16 + c;
    u32x4 v = {0, 0, 0, 0};
    if (row < N) {
        const uint32_t* src = codes + (row * nch + J * 4) * 4 + q;  // chunk 4 J of the row, word q
#pragma unroll
        for (int m = 0; m < 4; m++)
            if (J * 4 + m < nch) v[m] = src[m * 4];
    }
    tile[t] = v;
}

// Q4_0 scales [N][nch] fp16 -> [R][J][c][4]; groups of 128: scales [N][G] fp16, zps [N][G] -> [R][J][c] u32
__global__ __launch_bounds__(256) void tile4_scales_kernel(const uint16_t* __restrict__ scales, const uint8_t* __restrict__ zps,
                                                           uint32_t* __restrict__ out, int64_t N, int64_t NJ, int64_t nch,
                                                           int64_t count, int g128) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= count) return;
    const int c = (int)(t & 15);
    const int64_t J = (t >> 4) % NJ, R = (t >> 4) / NJ, row = R * 16 + c;
    if (g128) {
        out[t] = row < N ? ((uint32_t)scales[row * NJ + J] | ((uint32_t)zps[row * NJ + J] << 16)) : 0u;
    } else {
        uint32_t lo = 0, hi = 0;
        if (row < N) {
            const uint16_t* s = scales + row * nch + J * 4;
            uint32_t v[4];
#pragma unroll
            for (int m = 0; m < 4; m++) v[m] = J * 4 + m < nch ? (uint32_t)s[m] : 0u;
            lo = v[0] | (v[1] << 16), hi = v[2] | (v[3] << 16);
        }
        out[2 * t] = lo, out[2 * t + 1] = hi;
    }
}

// int8 codes [N][K] -> tile[R][J][lane][16 B]
__global__ __launch_bounds__(256) void tile8_repack_kernel(const uint8_t* __restrict__ codes, u32x4* __restrict__ tile,
                                                           int64_t N, int64_t K, int64_t NJ, int64_t slots) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= slots) return;
    const int l = (int)(t & 63), c = l & 15, q = l >> 4;
    const int64_t J = (t >> 6) % NJ, R = (t >> 6) / NJ, row = R * 16 + c;
    u32x4 v = {0, 0, 0, 0};
    if (row < N) v = *reinterpret_cast<const u32x4*>(codes + row * K + J * 64 + q * 16);
    tile[t] = v;
}

template <int FMT, bool XF32, int KW>
int32_t launch4_jpw(const TileParams& p, int jpw, dim3 grid, hipStream_t s) {
    const bool exact = p.NJ == KW * jpw;
#define NQ_T4(J_)                                                                                                 \
    case J_:                                                                                                      \
        if (exact) hipLaunchKernelGGL((gemv_tile4_kernel<FMT, XF32, KW, J_, true>), grid, dim3(64 * KW), 0, s, p); \
        else hipLaunchKernelGGL((gemv_tile4_kernel<FMT, XF32, KW, J_, false>), grid, dim3(64 * KW), 0, s, p);      \
        break;
    switch (jpw) {
        NQ_T4(1) NQ_T4(2) NQ_T4(3) NQ_T4(4) NQ_T4(5) NQ_T4(6) NQ_T4(7) NQ_T4(8)
        default: return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no tile GEMV for this IN");
    }
#undef NQ_T4
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

template <int FMT, bool XF32, int KW>
int32_t launch4i_jpw(const TileParams& p, int jpw, dim3 grid, hipStream_t s) {
#define NQ_T4I(J_) \
    case J_: hipLaunchKernelGGL((gemv_tile4i_kernel<FMT, XF32, KW, J_>), grid, dim3(64 * KW), 0, s, p); break;
    switch (jpw) {
        NQ_T4I(1) NQ_T4I(2) NQ_T4I(3) NQ_T4I(4)
        default: return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no tile GEMV for this IN");
    }
#undef NQ_T4I
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// The int8-matrix-core route, K <= 8192: four steps per wavefront at most, 8 wavefronts up to K = 4096, 16 beyond.
// It is launched where every resident workgroup (1024 threads: one per CU; 512: two) gets three row tiles and more:
// the workgroups are then persistent and split x once.  (With fewer tiles a static share per workgroup balances
// worse than the hardware's own hand-out of one workgroup per tile, and launch4 keeps the bf16 route.)
inline int t4i_resident_wgs(int nj) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        cus = 256;
    return std::max(cus, 1) * (nj <= 32 ? 2 : 1);
}
template <int FMT, bool XF32>
int32_t launch4i(const TileParams& p, hipStream_t s) {
    const int kw = p.NJ <= 32 ? 8 : 16;
    const int jpw = (p.NJ + kw - 1) / kw;
    const int nr = (p.N + 15) / 16, res = t4i_resident_wgs(p.NJ);
    const int gridx = std::min(nr, std::max(res, (nr + T4I_MAXT - 1) / T4I_MAXT));
    const dim3 grid((unsigned)gridx);
    return kw == 8 ? launch4i_jpw<FMT, XF32, 8>(p, jpw, grid, s) : launch4i_jpw<FMT, XF32, 16>(p, jpw, grid, s);
}

template <int FMT, bool XF32>
int32_t launch4(const TileParams& p, hipStream_t s) {
    // Which route (measured at 4096 -> 11008 and 8192 -> 28672, cold): the int8 one where its workgroups are persistent
    // (three row tiles and more each: 24.4 -> 21.3 us for groups of 128, 26.3 -> 22.3 for Q4_0); with a workgroup
    // per tile it has no x stage to share and is no faster than the bf16 route (6.4 - 7.5 against 6.2 - 6.9 us)
    if (p.NJ <= 64 && (p.prefer || (p.N + 15) / 16 >= 3 * t4i_resident_wgs(p.NJ))) return launch4i<FMT, XF32>(p, s);
    // about four steps (4 KiB of codes) per wavefront measured best: 8 wavefronts up to K = 4096, 16 beyond
    const int kw = p.NJ <= 32 ? 8 : 16;
    const int jpw = std::min(8, (p.NJ + kw - 1) / kw);
    const dim3 grid((unsigned)((p.N + 15) / 16));
    return kw == 8 ? launch4_jpw<FMT, XF32, 8>(p, jpw, grid, s) : launch4_jpw<FMT, XF32, 16>(p, jpw, grid, s);
}

template <bool XF32, int KW>
int32_t launch8_jpw(const TileParams& p, int jpw, dim3 grid, hipStream_t s) {
    const bool exact = p.NJ == KW * jpw;
#define NQ_T8(J_)                                                                                            \
    case J_:                                                                                                 \
        if (exact) hipLaunchKernelGGL((gemv_tile8_kernel<XF32, KW, J_, true>), grid, dim3(64 * KW), 0, s, p); \
        else hipLaunchKernelGGL((gemv_tile8_kernel<XF32, KW, J_, false>), grid, dim3(64 * KW), 0, s, p);      \
        break;
    switch (jpw) {
        NQ_T8(1) NQ_T8(2) NQ_T8(3) NQ_T8(4) NQ_T8(5) NQ_T8(6) NQ_T8(7) NQ_T8(8)
        default: return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no tile GEMV for this IN");
    }
#undef NQ_T8
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

template <bool XF32>
int32_t launch8(const TileParams& p, hipStream_t s) {
    // eight steps (8 KiB of codes) per wavefront: 8 wavefronts up to K = 4096, 16 beyond; longer rows take rounds
    const int kw = p.NJ <= 64 ? 8 : 16;
    const int jpw = std::min(8, (p.NJ + kw - 1) / kw);
    const dim3 grid((unsigned)((p.N + 15) / 16));
    return kw == 8 ? launch8_jpw<XF32, 8>(p, jpw, grid, s) : launch8_jpw<XF32, 16>(p, jpw, grid, s);
}

template <int FMT, bool XF32>
int32_t launch4_rows(const TileMrParams& pm, hipStream_t s) {
    const int jpw = (pm.t.NJ + 15) / 16;
    int dev = 0, cus = 0;
    NQ_HIP(hipGetDevice(&dev));
    NQ_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int ntiles = (pm.t.N + 15) / 16;
    const dim3 grid((unsigned)std::min(ntiles, std::max(std::max(cus, 1), (ntiles + TR_MAXT - 1) / TR_MAXT)));
    switch (jpw) {
        case 1: hipLaunchKernelGGL((gemv_tile4_rows_kernel<FMT, XF32, 1>), grid, dim3(1024), 0, s, pm); break;
        case 2: hipLaunchKernelGGL((gemv_tile4_rows_kernel<FMT, XF32, 2>), grid, dim3(1024), 0, s, pm); break;
        case 3: hipLaunchKernelGGL((gemv_tile4_rows_kernel<FMT, XF32, 3>), grid, dim3(1024), 0, s, pm); break;
        default: return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no tile kernel for this IN");
    }
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// The K split of the M-tile kernel, from IN alone: JPW steps per wavefront, KW wavefronts per group (at least 4, so
// that a group has the 256 threads that finish its tile), 16 / KW groups; the choice that keeps most of the 16
// wavefronts busy.
inline void mt_split(int nj, bool xf32, int& jpw, int& kw) {
    double best = -1.0;
    jpw = 0, kw = 0;
    for (int j = 1; j <= (xf32 ? 1 : 3); j++) {
        const int w = std::max(4, (nj + j - 1) / j);
        if (w > 16) continue;
        const double util = (double)nj / (w * j) * ((16 / w) * w) / 16.0;
        if (util > best + 1e-9) best = util, jpw = j, kw = w;
    }
}

template <int FMT, bool XF32>
int32_t launch4_mt(const TileMrParams& pm, hipStream_t s) {
    int jpw, kw;
    mt_split(pm.t.NJ, XF32, jpw, kw);
    if (!jpw) return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no M-tile kernel for this IN");
    int dev = 0, cus = 0;
    NQ_HIP(hipGetDevice(&dev));
    NQ_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int ng = 16 / kw, ntiles = (pm.t.N + 15) / 16, mt = (pm.M + 15) / 16;
    const int gx = std::max(1, std::min((ntiles + ng - 1) / ng, std::max(cus, 1) / mt));
    const dim3 grid((unsigned)gx, (unsigned)mt);
#define NQ_MT(XF, J)                                                                                             \
    if (pm.la2) hipLaunchKernelGGL((gemm_tile4_mt_kernel<FMT, XF, J, 1, 2>), grid, dim3(1024), 0, s, pm, kw);        \
    else if (pm.la) hipLaunchKernelGGL((gemm_tile4_mt_kernel<FMT, XF, J, 1, 1>), grid, dim3(1024), 0, s, pm, kw);    \
    else hipLaunchKernelGGL((gemm_tile4_mt_kernel<FMT, XF, J, 1, 0>), grid, dim3(1024), 0, s, pm, kw);
    if constexpr (XF32) {
        NQ_MT(true, 1)
    } else {
        switch (jpw) {
            case 1: NQ_MT(false, 1) break;
            case 2: NQ_MT(false, 2) break;
            default:  // (three steps per wavefront leave no registers for an adapter's operands: lora_foldable says no)
                hipLaunchKernelGGL((gemm_tile4_mt_kernel<FMT, false, 3, 1, 0>), grid, dim3(1024), 0, s, pm, kw);
                break;
        }
    }
#undef NQ_MT
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace

// Which layers get the tile-ordered copy (a second copy of the codes: 0.5 or 1 byte per weight on top): those whose
// default dispatch has a kernel that reads it.
//   - weights of 4 M codes and more, whose single-row calls are bound by the weight stream.  4-bit: Q4_0 or groups of
//     exactly 128, IN a multiple of 128 in 2048 .. 16384; int8: IN a multiple of 64, at least 1024;
//   - 4-bit layers whose rows are at most 6144 codes long and which are (or, row-fused, hold a part) at least MT_WIDE
//     columns wide: the kernel for tens to hundreds of activation rows takes those parts.  A narrower layer's calls
//     all run on the row-ordered codes, and a copy nobody reads would double its device memory for nothing
//     (960 -> 960 or 2560 -> 960: 0.5625 bytes per weight, not 1.06);
//   - any 4-bit layer of such rows made with NQ_FLAG_PREFER_TILE.
constexpr int MT_WIDE = 2048;
bool tile_copy_wanted(const nq_layer* L) {
    if (L->no_tile_copy) return false;
    if ((int64_t)((L->in + 127) / 128 * 128) * ((L->out + 15) / 16 * 16) >= ((int64_t)1 << 32)) return false;  // (32-bit offsets in a tile copy)
    const bool four = L->format == NQ_FMT_Q4_0 || (L->format == NQ_FMT_W4_GROUP && L->group == 128);
    if (four && L->in % 32 == 0 && L->in >= 512 && L->in <= 6144) {
        int widest = L->seg_end.empty() ? L->out : 0;
        for (size_t i = 0, prev = 0; i < L->seg_end.size(); prev = (size_t)L->seg_end[i], i++)
            widest = std::max(widest, (int)(L->seg_end[i] - (int32_t)prev));
        if (L->prefer_tile || widest >= MT_WIDE) return true;
    }
    if ((int64_t)L->in * L->out < ((int64_t)4 << 20)) return false;
    if (four) return L->in % 128 == 0 && L->in >= 2048 && L->in <= 16384;
    if (L->format == NQ_FMT_W8_CHANNEL) return L->in % 64 == 0 && L->in >= 1024;
    return false;
}

// the layers whose single-row (and 2 .. 16 row) calls are bound by the weight stream: 4 M codes and more
static bool stream_bound_layer(const nq_layer* L) {
    if ((int64_t)L->in * L->out < ((int64_t)4 << 20)) return false;
    if (L->format == NQ_FMT_W8_CHANNEL) return true;
    return L->in % 128 == 0 && L->in >= 2048;
}

// builds (or drops) the tile-ordered copy from the row-ordered device arrays of a loaded layer
int32_t build_tile_copy(nq_layer* L, hipStream_t s) {
    if (L->d_tile16) (void)hipFree(L->d_tile16);
    if (L->d_tile16_scales) (void)hipFree(L->d_tile16_scales);
    L->d_tile16 = nullptr, L->d_tile16_scales = nullptr, L->tile_nj = 0;
    if (!tile_copy_wanted(L)) return NQ_OK;
    const int64_t N = L->out, R = (N + 15) / 16;
    const bool w8 = L->format == NQ_FMT_W8_CHANNEL;
    const int64_t NJ = w8 ? L->in / 64 : (L->in + 127) / 128;
    const int64_t slots = R * NJ * 64;
    NQ_HIP(hipMalloc((void**)&L->d_tile16, (size_t)slots * 16));
    if (w8) {
        hipLaunchKernelGGL(tile8_repack_kernel, dim3((unsigned)((slots + 255) / 256)), dim3(256), 0, s, L->d_codes,
                           reinterpret_cast<u32x4*>(L->d_tile16), N, (int64_t)L->in, NJ, slots);
    } else {
        const bool g128 = L->format == NQ_FMT_W4_GROUP;
        const int64_t count = R * NJ * 16;
        NQ_HIP(hipMalloc(&L->d_tile16_scales, (size_t)count * (g128 ? 4 : 8)));
        hipLaunchKernelGGL(tile4_repack_kernel, dim3((unsigned)((slots + 255) / 256)), dim3(256), 0, s,
                           reinterpret_cast<const uint32_t*>(L->d_codes), reinterpret_cast<u32x4*>(L->d_tile16), N, NJ,
                           (int64_t)L->in / 32, slots);
        hipLaunchKernelGGL(tile4_scales_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, s,
                           reinterpret_cast<const uint16_t*>(L->d_scales), L->d_zps,
                           reinterpret_cast<uint32_t*>(L->d_tile16_scales), N, NJ, (int64_t)L->in / 32, count, (int)g128);
    }
    NQ_HIP(hipGetLastError());
    L->tile_nj = (int32_t)NJ;
    return NQ_OK;
}

bool gemv_tile_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (a.M != 1 || !L->d_tile16 || L->glu || !stream_bound_layer(L)) return false;
    if (a.x_dtype != NQ_DT_BF16 && a.x_dtype != NQ_DT_F32) return false;
    return a.y_dtype == NQ_DT_F32 || a.y_dtype == NQ_DT_BF16;
}

// 2 .. 16 rows of bf16 activations, 2 .. 5 of fp32, over a 4-bit layer that keeps its tile copy, K <= 6144 (a
// wavefront's A operands for up to three steps of K fit its registers beside the codes of two tiles; with four
// the kernel spills)
bool gemv_tile_rows_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (!L->d_tile16 || L->format == NQ_FMT_W8_CHANNEL || L->tile_nj > 48 || L->glu || !stream_bound_layer(L)) return false;
    if (a.y_dtype != NQ_DT_F32 && a.y_dtype != NQ_DT_BF16) return false;
    if (a.x_dtype == NQ_DT_BF16) return a.M >= 2 && a.M <= 16;
    if (a.x_dtype == NQ_DT_F32) return a.M >= 2 && a.M <= 5;
    return false;
}

// 2 .. 16 rows of bf16 activations, 2 .. 5 of fp32 ones, over an int8 layer that keeps its tile copy, K <= 4096 (four
// steps of K per wavefront: its A operands and two tiles' codes stay in registers).  Taken where it measured faster
// than the kernels over the row-ordered codes: rows of 2048 codes and more; up to 4 activation rows always, up to 8
// from 8 M codes, more from rows of 4096 codes and 8192 of them (every workgroup reads all the activations: with
// 16 rows and one tile per workgroup that is twice its share of the weights).
bool gemv_tile8_rows_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (!L->d_tile16 || L->format != NQ_FMT_W8_CHANNEL || L->tile_nj > 64 || L->glu) return false;
    if (a.y_dtype != NQ_DT_F32 && a.y_dtype != NQ_DT_BF16) return false;
    if (a.x_dtype != NQ_DT_BF16 && a.x_dtype != NQ_DT_F32) return false;
    if (a.M < 2 || a.M > (a.x_dtype == NQ_DT_F32 ? 5 : 16)) return false;
    if (L->prefer_tile) return true;
    if (L->tile_nj < 32) return false;
    if (a.M <= 4) return true;
    if (a.M <= 8) return (int64_t)L->in * L->out >= ((int64_t)8 << 20);
    return L->tile_nj == 64 && L->out >= 8192;
}

int32_t launch_gemv_tile8_rows(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    TileMrParams pm{};
    TileParams& p = pm.t;
    p.tile = reinterpret_cast<const u32x4*>(L->d_tile16), p.tscales = nullptr;
    p.col_scale = reinterpret_cast<const float*>(L->d_scales);
    p.x = a.x, p.bias = a.bias, p.seg = a.seg;
    p.N = L->out, p.K = L->in, p.NJ = L->tile_nj;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    pm.M = a.M;
    int dev = 0, cus = 0;
    NQ_HIP(hipGetDevice(&dev));
    NQ_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int ntiles = (p.N + 15) / 16;
    const dim3 grid((unsigned)std::min(ntiles, std::max(std::max(cus, 1), (ntiles + TR_MAXT - 1) / TR_MAXT)));
    const int jpw = (p.NJ + 15) / 16;
    const bool xf32 = a.x_dtype == NQ_DT_F32;
#define NQ_T8R(J_)                                                                                                      \
    case J_:                                                                                                           \
        if (xf32) hipLaunchKernelGGL((gemv_tile8_rows_kernel<true, J_>), grid, dim3(1024), 0, a.stream, pm);            \
        else hipLaunchKernelGGL((gemv_tile8_rows_kernel<false, J_>), grid, dim3(1024), 0, a.stream, pm);                \
        break;
    switch (jpw) {
        NQ_T8R(1) NQ_T8R(2) NQ_T8R(3) NQ_T8R(4)
        default: return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no int8 rows kernel for this IN");
    }
#undef NQ_T8R
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// 17 .. 511 rows of bf16 activations, or of fp32 ones where IN <= 2048, over a wide 4-bit layer with a tile copy.
// Everything but the width:
static bool mt_shape_ok(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (!L->d_tile16 || L->format == NQ_FMT_W8_CHANNEL || L->tile_nj > 48) return false;
    if (a.y_dtype != NQ_DT_F32 && a.y_dtype != NQ_DT_BF16) return false;
    if ((int64_t)a.M * L->in >= ((int64_t)1 << 31)) return false;
    if (a.M < 2 || a.M > 512) return false;
    if (!L->prefer_tile && (a.M < 17 || a.M > 511)) return false;  // (from 512 rows on: the many-rows kernel)
    if (a.x_dtype == NQ_DT_BF16) return true;
    return a.x_dtype == NQ_DT_F32 && L->tile_nj <= 16;
}
// What a call of this kernel takes, in microseconds.  Its workgroups (M tiles x column groups, at most one per CU)
// run in one round and each walks `iters` sets of weight tiles; over IN = 512 .. 6144, OUT = 960 .. 11008 and
// M = 17 .. 384 (2000 calls) a call took F + iters * q within 4 - 5 % on average, F and q by format, activation type
// and the steps of K per wavefront.
static float mt_estimate_us(const ForwardArgs& a, int width) {
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    int jpw, kw;
    mt_split(a.L->tile_nj, xf32, jpw, kw);
    if (jpw < 1 || jpw > 3) return 0.0f;
    static const float fq[2][4][2] = {
        // Q4_0: bf16 activations with 1, 2, 3 steps per wavefront; fp32 activations
        {{4.15f, 0.938f}, {5.51f, 1.660f}, {6.84f, 2.559f}, {6.19f, 0.905f}},
        // groups of 128 with zero points
        {{4.15f, 0.860f}, {5.46f, 1.454f}, {7.18f, 1.835f}, {6.11f, 0.846f}},
    };
    const float* c = fq[a.L->format == NQ_FMT_Q4_0 ? 0 : 1][xf32 ? 3 : jpw - 1];
    const int ng = 16 / kw, sets = ((width + 15) / 16 + ng - 1) / ng, mt = (a.M + 15) / 16;
    const int gx = std::max(1, std::min(sets, 256 / mt));
    return c[0] + (float)((sets + gx - 1) / gx) * c[1];
}

// ... and the width, which is each part's own: 2048 columns and more (a narrower layer gives a workgroup one or two
// weight tiles to amortise its start over), and wherever this kernel's estimate is below the medium-M kernel's for the
// same part.  Measured side by side over the calls above, the pair of estimates picks the slower kernel by more than
// a tenth in 70 of 2000 calls and costs 0.3 - 1.3 % in total against always picking the faster one (the rules
// it replaces - row counts from 96, a round of the other kernel's widest tile, three steps of K only over groups of
// 128 - cost 0.5 - 3.1 %, and up to 50 % where they did not look: fp32 activations below 96 rows over the widest
// layers, 2048 -> 11008 at M = 33 24 -> 15 us, groups of 128 at IN = 2560 .. 3072 and a hundred rows, 2560 -> 4096
// 13.7 -> 8.9 us).
static bool mt_part_ok(const ForwardArgs& a, int width) {
    if (width < MT_WIDE) return false;
    const float mine = mt_estimate_us(a, width);
    if (mine == 0.0f) return false;
    // (estimates within a tenth of each other go to this kernel: it is the one that can carry an adapter in the same
    // launch, and over the measured calls that margin costs 0.1 - 0.2 % more)
    return mine < 1.10f * gemm_a16_best_estimate_us(a.L->format, a.x_dtype == NQ_DT_F32, a.M, width, a.L->in);
}

// A row-fused layer runs on this kernel in one launch when all its parts pass, on the other kernel when none does,
// and part by part when they differ (gemm_tile_mt_splits_parts), so that a part gets the kernel - and the bits - of
// its own layer's forward.
bool gemm_tile_mt_applicable(const ForwardArgs& a) {
    if (!mt_shape_ok(a)) return false;
    if (a.L->prefer_tile) return true;
    if (a.L->glu) return mt_part_ok(a, a.L->out);
    for (int i = 0, prev = 0; i < a.seg.nseg; prev = a.seg.end[i], i++)
        if (!mt_part_ok(a, a.seg.end[i] - prev)) return false;
    return true;
}

// whether the kernel can run the call at all (its shapes), whatever the estimates say about other kernels
bool gemm_tile_mt_takes_shape(const ForwardArgs& a) { return mt_shape_ok(a); }

// an adapter can ride along where a wavefront holds at most two steps of K (IN <= 4096; measured there at
// 4096 -> 4096, T = 135, bf16 x: 36.3 us folded against 38.2 us as two launches)
bool gemm_tile_mt_lora_foldable(const ForwardArgs& a) {
    int jpw, kw;
    mt_split(a.L->tile_nj, a.x_dtype == NQ_DT_F32, jpw, kw);
    return jpw >= 1 && jpw <= 2;
}

bool gemm_tile_mt_splits_parts(const ForwardArgs& a) {
    if (a.seg.nseg < 2 || a.L->prefer_tile || !mt_shape_ok(a)) return false;
    int wide = 0;
    for (int i = 0, prev = 0; i < a.seg.nseg; prev = a.seg.end[i], i++) wide += mt_part_ok(a, a.seg.end[i] - prev);
    return wide > 0 && wide < a.seg.nseg;
}

int32_t launch_gemm_tile_mt(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    TileMrParams pm{};
    TileParams& p = pm.t;
    p.tile = reinterpret_cast<const u32x4*>(L->d_tile16), p.tscales = L->d_tile16_scales, p.col_scale = nullptr;
    p.x = a.x, p.bias = a.bias, p.seg = a.seg;
    p.N = L->out, p.K = L->in, p.NJ = L->tile_nj;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    pm.M = a.M;
    pm.la = a.lora_a, pm.lb = a.lora_b, pm.lr = a.lora_r, pm.ls = a.lora_s;
    pm.la2 = a.lora_a2, pm.lb2 = a.lora_b2, pm.ls2 = a.lora_s2;
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    if (L->format == NQ_FMT_Q4_0)
        return xf32 ? launch4_mt<NQ_FMT_Q4_0, true>(pm, a.stream) : launch4_mt<NQ_FMT_Q4_0, false>(pm, a.stream);
    return xf32 ? launch4_mt<NQ_FMT_W4_GROUP, true>(pm, a.stream) : launch4_mt<NQ_FMT_W4_GROUP, false>(pm, a.stream);
}

int32_t launch_gemv_tile_rows(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    TileMrParams pm{};
    TileParams& p = pm.t;
    p.tile = reinterpret_cast<const u32x4*>(L->d_tile16), p.tscales = L->d_tile16_scales, p.col_scale = nullptr;
    p.x = a.x, p.bias = a.bias, p.seg = a.seg;
    p.N = L->out, p.K = L->in, p.NJ = L->tile_nj;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    pm.M = a.M;
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    if (L->format == NQ_FMT_Q4_0)
        return xf32 ? launch4_rows<NQ_FMT_Q4_0, true>(pm, a.stream) : launch4_rows<NQ_FMT_Q4_0, false>(pm, a.stream);
    return xf32 ? launch4_rows<NQ_FMT_W4_GROUP, true>(pm, a.stream) : launch4_rows<NQ_FMT_W4_GROUP, false>(pm, a.stream);
}

int32_t launch_gemv_tile(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    TileParams p{};
    p.tile = reinterpret_cast<const u32x4*>(L->d_tile16), p.tscales = L->d_tile16_scales;
    p.col_scale = L->format == NQ_FMT_W8_CHANNEL ? reinterpret_cast<const float*>(L->d_scales) : nullptr;
    p.x = a.x, p.bias = a.bias, p.seg = a.seg;
    p.N = L->out, p.K = L->in, p.NJ = L->tile_nj;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    p.prefer = L->prefer_tile;
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    switch (L->format) {
        case NQ_FMT_Q4_0:
            return xf32 ? launch4<NQ_FMT_Q4_0, true>(p, a.stream) : launch4<NQ_FMT_Q4_0, false>(p, a.stream);
        case NQ_FMT_W4_GROUP:
            return xf32 ? launch4<NQ_FMT_W4_GROUP, true>(p, a.stream) : launch4<NQ_FMT_W4_GROUP, false>(p, a.stream);
        case NQ_FMT_W8_CHANNEL: return xf32 ? launch8<true>(p, a.stream) : launch8<false>(p, a.stream);
    }
    return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no tile GEMV for this format");
}

}  // namespace nq
