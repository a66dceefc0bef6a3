// 8-bit x 8-bit products for few activation rows on the matrix cores:
//     fp8 e4m3 x fp8 e4m3:  y[M, N] = epi( (x[M, K] @ W[N, K]^T) * s_w * s_x + bias )
//     int8 x int8:          y[M, N] = epi( (x . W^T)_int32 * s_x[m] * s_w[n] + bias ), or the raw int32 sums
//
// The call is bound by the weight stream (K = 4096, N = 11008 is 45 MB), and what a
// streaming kernel can lose is issue slots: converting an 8-bit code and multiplying it on the
// vector ALU costs about two instructions per weight per wavefront, which at one row per
// wavefront is more instruction issue than the loads leave room for.  One
// v_mfma_f32_16x16x128_f8f6f4 (or two v_mfma_i32_16x16x64_i8) multiplies a 16-row x 128-k slab
// of weights (2 KB) by 16 activation rows, so the kernel is loads plus a handful of MFMAs:
//   - a workgroup owns 16 weight rows and up to 64 activation rows (MT tiles of 16; more rows
//     take more workgroups along grid.y, re-reading the weights from L2); its KW wavefronts
//     split K, SPW steps of 128 k each.  With 64 rows and more, and enough weight rows that
//     160 workgroups remain, a workgroup takes NT = 2 or 4 weight tiles: an activation
//     fragment then serves NT MFMAs, and the activations (the larger operand at 64 rows
//     against 16) are fetched once per 16 NT weight rows;
//   - loads are row-contiguous: 8 rows x 128 bytes per instruction, eight adjacent lanes per row
//     (a load instruction is priced by the pieces of cache line its lanes touch), and reach the
//     MFMA operand layout through a private 4 KiB of LDS per wavefront: one 128-bit store and
//     one 128-bit read per register quad, the 16-byte slot XORed with a function of the row so
//     that neither side has bank conflicts; no barrier, LDS executes one wavefront's accesses in
//     order;
//   - all of a wavefront's loads of a round are issued before its first MFMA (up to 16 KB of
//     weights per wavefront in flight);
//   - the KW partial 16 x 16 tiles are summed through LDS in wave order (fixed, so a repeated
//     call returns the same bits; the int32 sums are exact in any order) and thread (m, n)
//     applies scales, bias and epilogue.
// The same kernel serves up to several hundred rows where the 256 x 256-tile GEMM would leave most
// of the chip idle (M = 64 .. 768 over a 4096 x 4096 weight is 16 .. 48 tiles on 256 CUs):
// tile8_wins holds the measured crossover.
//
// A single activation row (M = 1) takes a second kernel whose loads are fully coalesced: one
// wavefront owns ONE weight row and reads it as 1 KB contiguous per load instruction (lane l
// takes the 16-byte chunks l, l + 64, ...).  The MFMA is then used "diagonally": the 16 B
// columns are 16 different 128-byte segments of that row and the 16 A rows are the matching
// segments of x (lane l of A holds x at the very offsets lane l of B holds W), so
// D[c][c] = <x segment c, W segment c> and the row's dot product is the trace of D.  15/16 of
// the MFMA is wasted, which costs nothing here: the instruction replaces ~250 VALU
// instructions per KB-row and the kernel issues little besides its loads.
#include <algorithm>
#include <type_traits>

#include "nq_common.h"


namespace nq {

namespace {

typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

struct Fp8GemvParams {
    const uint8_t* w;
    const uint8_t* x;
    const float* x_scale;    // fp8: [1]; int8: per activation row [M] (null with raw int32 output)
    const float* col_scale;  // int8: per output channel [N]
    void* y;
    const void* bias;
    int32_t M, N, K;
    int32_t nsteps;  // steps of 128 k, the last one possibly cut short by K
    float tscale;
    int32_t y_dtype, bias_dtype, epilogue;
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

template <bool I8, int SPW, int KW, int MT, int NT>
__global__ __launch_bounds__(64 * KW) void tile8_kernel(const Fp8GemvParams p) {
    typedef typename std::conditional<I8, i32x4, f32x4>::type acc_t;
    __shared__ uint32_t red[KW][NT * 256];
    __shared__ __attribute__((aligned(16))) uint8_t stage[KW][4096];  // [weights 16 x 128 | activations 16 x 128]
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ln = lane & 15, kb = lane >> 4;
    const int n_base = blockIdx.x * (16 * NT);
    const int m_base = blockIdx.y * (16 * MT);

    // a load: lane -> row 8 t + lane / 8 of the tile, 16-byte piece lane % 8 of the step's 128 bytes
    const int trow = lane >> 3, tpc = lane & 7;
    int64_t wsrc[NT][2], xsrc[MT][2];
    uint32_t st[2], rd[2];
    // slot swizzle of a 128-byte row.  A 128-bit LDS read is served in passes of 16 lanes that are not
    // consecutive: within each half of the wavefront first the quads of lanes with an even-parity index
    // (lanes 0-3, 12-15, 20-23, 24-27), then the others.  Rows two apart differ by row / 2; the quads a pass
    // takes from the next kb (rows 4 .. 11) sit D slots further, D = the slot distance between kb and kb + 1.
    constexpr int D = I8 ? 1 : 2;
    auto swz = [](int row) { return ((row >> 1) ^ ((((row >> 2) ^ (row >> 3)) & 1) * D)) & 7; };
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const int row = 8 * t + trow;
#pragma unroll
        for (int j = 0; j < NT; j++) wsrc[j][t] = (int64_t)min(n_base + 16 * j + row, p.N - 1) * p.K + tpc * 16;
#pragma unroll
        for (int i = 0; i < MT; i++) xsrc[i][t] = (int64_t)min(m_base + 16 * i + row, p.M - 1) * p.K + tpc * 16;
        st[t] = row * 128 + ((tpc ^ swz(row)) & 7) * 16;
        // the fragment of this lane.  fp8: one MFMA of 128 k, k = 32 kb .. 32 kb + 31 (pieces 2 kb, 2 kb + 1);
        // int8: two MFMAs of 64 k, the t-th takes k = 64 t + 16 kb .. + 15 (piece 4 t + kb)
        const int piece = I8 ? 4 * t + kb : 2 * kb + t;
        rd[t] = ln * 128 + ((piece ^ swz(ln)) & 7) * 16;
    }
    uint8_t* scr = stage[wave];
    auto lds16 = [&](uint32_t off) -> u32x4& { return *reinterpret_cast<u32x4*>(scr + off); };

    // What the finishing threads need besides the sums - channel scale, bias, the rows' activation scales - is
    // requested here, ahead of the K loop: asked for where it is used, after the barrier, it was one more trip to
    // memory at the end of every call.  Thread t finishes outputs t, t + 64 KW, ... of a [16 x 16 NT] tile.
    constexpr int FIT = (NT * 256 + 64 * KW - 1) / (64 * KW);
    // (loads in inline assembly: the compiler would move its own down to their use.  Unconditional and in straight
    // code - an operand the call does not have is read from the weights' first bytes and ignored - because a load
    // under a branch gets its register copied at the join, before the data has landed.  They are the oldest loads of
    // the wavefront and the wait for them stands after the K loop, before the first barrier.)
    // From two activation tiles per workgroup on, where every tile's finish paid that trip (4096 x 4096 int8 at 63
    // rows: 10.6 -> 10.0 us, 1024 x 1024: 4.8 -> 4.2); with one tile the registers these operands hold through the
    // K loop cost a streaming call more than the trip (4096 -> 11008 at 2 .. 16 rows: 9.4 -> 10.6 us).  And not
    // where 16 wavefronts hold four activation tiles each: there the registers run out, and a register spilled while
    // its load is under way is saved before the data has landed.  The build refuses spills in these kernels.
    constexpr bool PF = MT >= 2 && !(KW == 16 && MT == 4);
    uint32_t f_cs[FIT], f_xs[MT][FIT], f_b32[FIT], f_b16[FIT];
    const bool scaled = I8 && p.y_dtype != NQ_DT_I32;
    const bool b32 = p.bias && p.bias_dtype == NQ_DT_F32, b16 = p.bias && p.bias_dtype != NQ_DT_F32;
#pragma unroll
    for (int it = 0; PF && it < FIT; it++) {
        const int t = min((int)threadIdx.x + it * 64 * KW, NT * 256 - 1);
        const int n = min(n_base + 16 * (t >> 8) + (t & 15), p.N - 1);
        const void* const a_cs = scaled ? (const void*)(p.col_scale + n) : (const void*)p.w;
        const void* const a_b32 = b32 ? (const void*)(reinterpret_cast<const uint32_t*>(p.bias) + n) : (const void*)p.w;
        const void* const a_b16 = b16 ? (const void*)(reinterpret_cast<const uint16_t*>(p.bias) + n) : (const void*)p.w;
        if constexpr (I8) asm volatile("global_load_dword %0, %1, off ; pf" : "=v"(f_cs[it]) : "v"(a_cs));
        else f_cs[it] = 0;  // (fp8: one scale per tensor, below)
        asm volatile("global_load_dword %0, %1, off ; pf" : "=v"(f_b32[it]) : "v"(a_b32));
        asm volatile("global_load_ushort %0, %1, off ; pf" : "=v"(f_b16[it]) : "v"(a_b16));
#pragma unroll
        for (int i = 0; i < MT; i++) {
            const void* const a_xs = scaled ? (const void*)(p.x_scale + min(m_base + 16 * i + ((t & 255) >> 4), p.M - 1))
                                            : (!I8 ? (const void*)p.x_scale : (const void*)p.w);  // (fp8: per tensor)
            // (a condition on unrolled indices: decided at compile time, no branch)
            if (I8 || (i == 0 && it == 0)) asm volatile("global_load_dword %0, %1, off ; pf" : "=v"(f_xs[i][it]) : "v"(a_xs));
            else f_xs[i][it] = 0;
        }
    }

    acc_t acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; i++)
#pragma unroll
        for (int j = 0; j < NT; j++) acc[i][j] = (acc_t){0, 0, 0, 0};
    // K need not be a multiple of the step: a lane's 16-byte piece of the last step may lie past the row.
    // Its address is then moved to the start of the step (inside the row) and, when the step is
    // staged, both operands' pieces are replaced by zeros (an fp8 NaN times zero would not be zero).
    const int klast = (p.K - 1) / 128 * 128;           // first k of the last step
    const bool in_last = klast + tpc * 16 < p.K;       // this lane's piece of the last step lies inside K
    const int64_t poff = in_last ? 0 : -(int64_t)tpc * 16;
    for (int s0 = wave * SPW; s0 < p.nsteps; s0 += KW * SPW) {
        u32x4 wv[NT][SPW][2], xv[MT][SPW][2];
        // unconditional loads from clamped step indices; a step past K meets zero activations
#pragma unroll
        for (int s = 0; s < SPW; s++) {
            const int ks = min(s0 + s, p.nsteps - 1);
            const int64_t k0 = (int64_t)ks * 128 + (ks == p.nsteps - 1 ? poff : 0);
#pragma unroll
            for (int j = 0; j < NT; j++) {
                wv[j][s][0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.w + wsrc[j][0] + k0));
                wv[j][s][1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p.w + wsrc[j][1] + k0));
            }
        }
#pragma unroll
        for (int i = 0; i < MT; i++)
#pragma unroll
            for (int s = 0; s < SPW; s++) {
                const int ks = min(s0 + s, p.nsteps - 1);
                const int64_t k0 = (int64_t)ks * 128 + (ks == p.nsteps - 1 ? poff : 0);
                xv[i][s][0] = *reinterpret_cast<const u32x4*>(p.x + xsrc[i][0] + k0);
                xv[i][s][1] = *reinterpret_cast<const u32x4*>(p.x + xsrc[i][1] + k0);
            }
#pragma unroll
        for (int s = 0; s < SPW; s++) {
            if (s0 + s == p.nsteps - 1 && (p.K & 127)) {  // uniform over the wavefront: the step K cuts short
                const uint32_t keep = in_last ? ~0u : 0u;
#pragma unroll
                for (int t = 0; t < 2; t++) {
#pragma unroll
                    for (int j = 0; j < NT; j++)
#pragma unroll
                        for (int e = 0; e < 4; e++) wv[j][s][t][e] &= keep;
#pragma unroll
                    for (int i = 0; i < MT; i++)
#pragma unroll
                        for (int e = 0; e < 4; e++) xv[i][s][t][e] &= keep;
                }
            }
            // (a wavefront's LDS accesses execute in order: tile j + 1 may overwrite tile j once its reads are issued)
            u32x4 b0[NT], b1[NT];
#pragma unroll
            for (int j = 0; j < NT; j++) {
                lds16(st[0]) = wv[j][s][0], lds16(st[1]) = wv[j][s][1];
                b0[j] = lds16(rd[0]), b1[j] = lds16(rd[1]);
            }
#pragma unroll
            for (int i = 0; i < MT; i++) {
                lds16(2048 + st[0]) = xv[i][s][0], lds16(2048 + st[1]) = xv[i][s][1];
                u32x4 a0 = lds16(2048 + rd[0]), a1 = lds16(2048 + rd[1]);
                if (s0 + s >= p.nsteps) a0 = a1 = (u32x4){0, 0, 0, 0};  // uniform over the wavefront
#pragma unroll
                for (int j = 0; j < NT; j++) {
                    if constexpr (I8) {
                        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a0),
                                                                          __builtin_bit_cast(i32x4, b0[j]), acc[i][j], 0, 0, 0);
                        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a1),
                                                                          __builtin_bit_cast(i32x4, b1[j]), acc[i][j], 0, 0, 0);
                    } else {
                        const i32x8 a = {(int)a0[0], (int)a0[1], (int)a0[2], (int)a0[3],
                                         (int)a1[0], (int)a1[1], (int)a1[2], (int)a1[3]};
                        const i32x8 b = {(int)b0[j][0], (int)b0[j][1], (int)b0[j][2], (int)b0[j][3],
                                         (int)b1[j][0], (int)b1[j][1], (int)b1[j][2], (int)b1[j][3]};
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[i][j], 0, 0, 0, 0, 0, 0);
                    }
                }
            }
        }
    }

    if constexpr (PF) asm volatile("s_waitcnt vmcnt(0) ; pfw");  // the finishing operands requested at the top (nothing else is under way here)
#pragma unroll
    for (int it = 0; PF && it < FIT; it++) {
        asm volatile("" : "+v"(f_cs[it]), "+v"(f_b32[it]), "+v"(f_b16[it]));
#pragma unroll
        for (int i = 0; i < MT; i++) asm volatile("" : "+v"(f_xs[i][it]));
    }
    // D layout: lane holds column n = lane % 16, rows m = 4 (lane / 16) + r.  The K-slices of one
    // activation tile (all its NT weight tiles) at a time are summed in wave order (fixed, so results
    // repeat bit for bit).
#pragma unroll
    for (int i = 0; i < MT; i++) {
        if (i) __syncthreads();
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                red[wave][j * 256 + (4 * kb + r) * 16 + ln] =
                    I8 ? (uint32_t)acc[i][j][r] : __float_as_uint((float)acc[i][j][r]);
        __syncthreads();
#pragma unroll
        for (int it = 0; it < FIT; it++) {
            const int t = (int)threadIdx.x + it * 64 * KW;
            if (t >= NT * 256) break;
            const int m = m_base + 16 * i + ((t & 255) >> 4), n = n_base + 16 * (t >> 8) + (t & 15);
            if (m < p.M && n < p.N) {
                const int64_t o = (int64_t)m * p.N + n;
                float z;
                if constexpr (I8) {
                    int32_t sum = (int32_t)red[0][t];
#pragma unroll
                    for (int w = 1; w < KW; w++) sum += (int32_t)red[w][t];
                    if (p.y_dtype == NQ_DT_I32) {
                        reinterpret_cast<int32_t*>(p.y)[o] = sum;
                        continue;
                    }
                    z = PF ? (float)sum * (__uint_as_float(f_xs[i][it]) * __uint_as_float(f_cs[it]))
                           : (float)sum * (p.x_scale[m] * p.col_scale[n]);
                } else {
                    z = __uint_as_float(red[0][t]);
#pragma unroll
                    for (int w = 1; w < KW; w++) z += __uint_as_float(red[w][t]);
                    z *= p.tscale * (PF ? __uint_as_float(f_xs[0][0]) : p.x_scale[0]);
                }
                if constexpr (PF) {
                    if (p.bias) z += __uint_as_float(b32 ? f_b32[it] : f_b16[it] << 16);
                } else if (p.bias) {
                    z += b32 ? reinterpret_cast<const float*>(p.bias)[n]
                             : __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n] << 16);
                }
                if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
                if (p.y_dtype == NQ_DT_F32)
                    reinterpret_cast<float*>(p.y)[o] = z;
                else
                    reinterpret_cast<uint16_t*>(p.y)[o] = f32_to_bf16_rne(z);
            }
        }
    }
}


// ---- M = 1: one wavefront per weight row (or SPLIT wavefronts, each on a 1 / SPLIT share of it), coalesced loads,
// trace of the MFMA tile.  CPL: 16-byte chunks of the row per lane of ONE wavefront (CPL * SPLIT * 64 chunks cover K).
template <bool I8, int CPL, int WAVES, int SPLIT>
__global__ __launch_bounds__(64 * WAVES) void gemv8_row_kernel(const Fp8GemvParams p) {
    constexpr int ROWS = WAVES / SPLIT;   // rows per workgroup
    constexpr int XCH = CPL * SPLIT * 64; // chunks of x staged
    __shared__ u32x4 xs[XCH];  // the activation row, shared by the workgroup's rows
    __shared__ uint32_t part[ROWS][SPLIT];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wrow = wave / SPLIT, share = wave % SPLIT;
    const int64_t row = (int64_t)blockIdx.x * ROWS + wrow;
    const int64_t rowc = min(row, (int64_t)p.N - 1);
    const int nch = p.K >> 4;  // 16-byte chunks per row
    const u32x4* wr = reinterpret_cast<const u32x4*>(p.w + rowc * p.K);
    const u32x4* xr = reinterpret_cast<const u32x4*>(p.x);
    const int c0 = share * CPL * 64;  // this wavefront's first chunk of the row

    // x goes first so that waiting for it leaves the weight loads in flight; every load is
    // unconditional from a clamped chunk index, and a chunk past K meets x = 0
    constexpr int XPT = (XCH + 64 * WAVES - 1) / (64 * WAVES);  // chunks of x per thread
    u32x4 xg[XPT];
    u32x4 wv[CPL], xv[CPL];
#pragma unroll
    for (int i = 0; i < XPT; i++) xg[i] = xr[min((int)threadIdx.x + i * 64 * WAVES, nch - 1)];
#pragma unroll
    for (int j = 0; j < CPL; j++) wv[j] = __builtin_nontemporal_load(wr + min(c0 + j * 64 + lane, nch - 1));
    // the epilogue's operands travel with the codes, raw: nothing is computed from them before the end
    const bool raw_out = I8 && p.y_dtype == NQ_DT_I32;
    float xsraw = 1.0f, csraw = 1.0f;
    if (!raw_out) xsraw = p.x_scale[0];
    if (I8 && !raw_out) csraw = p.col_scale[rowc];
    uint32_t braw = 0;
    if (p.bias)
        braw = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[rowc]
                                           : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[rowc];
#pragma unroll
    for (int i = 0; i < XPT; i++) {
        const int c = (int)threadIdx.x + i * 64 * WAVES;
        if (c < XCH) xs[c] = (c < nch) ? xg[i] : (u32x4){0, 0, 0, 0};
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < CPL; j++) xv[j] = xs[c0 + j * 64 + lane];

    // lane holds D[4 (lane / 16) + r][lane % 16]: its diagonal entry, if any, is r = c % 4 where
    // c = lane % 16 and c / 4 == lane / 16
    const int c = lane & 15, r = c & 3;
    const bool holder = (c >> 2) == (lane >> 4);
    uint32_t vbits;  // the lane's share of the trace: fp32 bits, or an int32
    if constexpr (I8) {
        i32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < CPL; j++)
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, xv[j]),
                                                        __builtin_bit_cast(i32x4, wv[j]), acc, 0, 0, 0);
        const int d = r == 0 ? acc[0] : r == 1 ? acc[1] : r == 2 ? acc[2] : acc[3];
        vbits = holder ? (uint32_t)d : 0u;
    } else {
        f32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < CPL; j += 2) {
            const u32x4 x1 = (j + 1 < CPL) ? xv[j + 1] : (u32x4){0, 0, 0, 0};
            const u32x4 w1 = (j + 1 < CPL) ? wv[j + 1] : (u32x4){0, 0, 0, 0};
            const i32x8 a = {(int)xv[j][0], (int)xv[j][1], (int)xv[j][2], (int)xv[j][3],
                             (int)x1[0],    (int)x1[1],    (int)x1[2],    (int)x1[3]};
            const i32x8 b = {(int)wv[j][0], (int)wv[j][1], (int)wv[j][2], (int)wv[j][3],
                             (int)w1[0],    (int)w1[1],    (int)w1[2],    (int)w1[3]};
            acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc, 0, 0, 0, 0, 0, 0);
        }
        const float d = r == 0 ? acc[0] : r == 1 ? acc[1] : r == 2 ? acc[2] : acc[3];
        vbits = holder ? __float_as_uint(d) : 0u;
    }
    // fixed butterfly over the 64 lanes (so a repeated call returns the same bits; the int32 sum is exact)
    auto add = [](uint32_t a, uint32_t b) -> uint32_t {
        if constexpr (I8) return (uint32_t)((int32_t)a + (int32_t)b);
        else return __float_as_uint(__uint_as_float(a) + __uint_as_float(b));
    };
    vbits = add(vbits, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)vbits, 0xB1, 0xF, 0xF, false));
    vbits = add(vbits, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)vbits, 0x4E, 0xF, 0xF, false));
    vbits = add(vbits, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)vbits, 0x141, 0xF, 0xF, false));
    vbits = add(vbits, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)vbits, 0x140, 0xF, 0xF, false));
    {
        const auto sw = __builtin_amdgcn_permlane16_swap(vbits, vbits, false, false);
        vbits = add(sw[0], sw[1]);
    }
    {
        const auto sw = __builtin_amdgcn_permlane32_swap(vbits, vbits, false, false);
        vbits = add(sw[0], sw[1]);
    }
    if constexpr (SPLIT > 1) {
        // the shares of a row meet in LDS, in their order (fixed: the same bits on every call)
        if (lane == 0) part[wrow][share] = vbits;
        __syncthreads();
        if (share != 0) return;
        vbits = part[wrow][0];
#pragma unroll
        for (int k = 1; k < SPLIT; k++) vbits = add(vbits, part[wrow][k]);
    }
    if (lane == 0 && row < p.N) {
        if (raw_out) {
            reinterpret_cast<int32_t*>(p.y)[row] = (int32_t)vbits;
            return;
        }
        const float bias = p.bias_dtype == NQ_DT_F32 ? __uint_as_float(braw) : __uint_as_float(braw << 16);
        float z = I8 ? (float)(int32_t)vbits * (xsraw * csraw) + bias : __uint_as_float(vbits) * (p.tscale * xsraw) + bias;
        if (p.epilogue == NQ_EPI_RELU) z = z > 0.0f ? z : 0.0f;
        if (p.y_dtype == NQ_DT_F32)
            reinterpret_cast<float*>(p.y)[row] = z;
        else
            reinterpret_cast<uint16_t*>(p.y)[row] = f32_to_bf16_rne(z);
    }
}

// How many wavefronts a workgroup has and how many share a row, by the bytes of the weight (measured on e4m3 and int8
// weights of K = 4096 and 8192, cold, medians of replays of a graph of 60 calls):
//   16.8 MB (4096 x 4096):    8 x 1: 4.49 us; 4 x 1: 4.62; 8 wavefronts, two per row: 4.71
//   45 MB   (4096 -> 11008):  8 x 1: 8.62;    4 x 1: 8.40; 4 wavefronts, two per row: 8.45; 8, two per row: 8.51; 2 x 1: 8.50;
//                             16 wavefronts, two per row: 9.68; x fetched per lane instead of staged in LDS: 8.44
//   235 MB  (8192 -> 28672):  8 x 1: 36.05;   4 x 1: 34.58; 4, two per row: 33.06; 8, four per row: 32.90 (89 % of 8 TB/s)
// On the largest layers smaller workgroups with less of a row per wavefront are worth 8 %.  At 45 MB the differences
// are within what two timing protocols disagree on: under replays of a graph of 200 steps, on one box in turn, 8 x 1
// took 8.178 / 8.180 / 8.163 us and 4 x 1 8.202 / 8.239 / 8.157, so it stays as it was.  (A kernel that only reads shows
// the same taste for small pieces - 1 or 2 KiB per wavefront: 7.7 us for 45 MB, 4 KiB: 8.0, 8 KiB: 8.6 - and gains
// from fewer resident workgroups, 7.75 with two or three per CU; a kernel with a chain behind its loads loses with
// fewer: 8.9 / 9.6 us.)
template <bool I8, int CPL>
int32_t launch_row(const Fp8GemvParams& p, hipStream_t s) {
    // (CPL counts the row's 16-byte chunks per lane of one wavefront that holds the whole row)
    const int64_t bytes = (int64_t)p.N * p.K;
    // fp8: a wavefront's chunks go to the MFMA in pairs
    constexpr bool HALVES_OK = CPL % 2 == 0 && (I8 || (CPL / 2) % 2 == 0 || CPL / 2 == 1);
    if (HALVES_OK && bytes >= ((int64_t)100 << 20)) {
        if constexpr (HALVES_OK)
            hipLaunchKernelGGL((gemv8_row_kernel<I8, CPL / 2, 4, 2>), dim3((unsigned)((p.N + 1) / 2)), dim3(256), 0, s, p);
    } else {
        hipLaunchKernelGGL((gemv8_row_kernel<I8, CPL, 8, 1>), dim3((unsigned)((p.N + 7) / 8)), dim3(512), 0, s, p);
    }
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

template <bool I8>
int32_t launch_row_cpl(const Fp8GemvParams& p, hipStream_t s) {
    // a wavefront per weight row: CPL chunks of 16 bytes per lane
    switch ((p.K / 16 + 63) / 64) {
        case 1: return launch_row<I8, 1>(p, s);
        case 2: return launch_row<I8, 2>(p, s);
        case 3: return launch_row<I8, 3>(p, s);
        case 4: return launch_row<I8, 4>(p, s);
        case 5: return launch_row<I8, 5>(p, s);
        case 6: return launch_row<I8, 6>(p, s);
        case 7: return launch_row<I8, 7>(p, s);
        default: return launch_row<I8, 8>(p, s);
    }
}

template <bool I8, int SPW, int MT, int NT>
int32_t launch_kw(const Fp8GemvParams& p, int kw, dim3 grid, hipStream_t s) {
    if (kw == 4)
        hipLaunchKernelGGL((tile8_kernel<I8, SPW, 4, MT, NT>), grid, dim3(256), 0, s, p);
    else if (kw == 8)
        hipLaunchKernelGGL((tile8_kernel<I8, SPW, 8, MT, NT>), grid, dim3(512), 0, s, p);
    else if constexpr (SPW * MT <= 4 && NT == 1)
        hipLaunchKernelGGL((tile8_kernel<I8, SPW, 16, MT, 1>), grid, dim3(1024), 0, s, p);
    else
        return fail(NQ_ERR_INVALID, "nq_forward: no 8-bit tile kernel of that shape");
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// weight tiles (of 16 rows) per workgroup: with 64 activation rows per workgroup, the most that still
// leaves 160 workgroups (measured: 4096 x 4096 at 64 / 128 / 256 rows is best with 1 / 2 / 4); one for
// K < 1024, where a wavefront has a single step and more, smaller workgroups hide its latency better
int tile8_weight_tiles(int M, int64_t out, int K) {
    const int mt_all = (M + 15) / 16;
    if (mt_all < 4 || K < 1024) return 1;
    for (int c = 4; c >= 2; c /= 2)
        if (((out + 16 * c - 1) / (16 * c)) * ((mt_all + 3) / 4) >= 160) return c;
    return 1;
}

template <bool I8>
int32_t launch_tile8(const Fp8GemvParams& p, int64_t out, hipStream_t stream) {
    // Up to four tiles of activation rows per workgroup (the weights are then read once for up to 64
    // rows; more rows go to grid.y).  K split: up to 8 steps (16 KB) of weights per wavefront and
    // round, fewer with more activation tiles (registers), and enough wavefronts per workgroup that
    // a small N still fills the chip.
    const int mt_all = (p.M + 15) / 16;
    const int mt = mt_all <= 4 ? mt_all : 4;
    int kw = 4, spw = mt == 1 ? 8 : mt == 2 ? 4 : 2;
    const int64_t wgs = (out + 15) / 16;
    const int64_t all = wgs * ((mt_all + mt - 1) / mt);  // workgroups of the launch
    if (all < 512 && p.nsteps > 4) kw = 8;
    if (all < 128 && p.nsteps > 8) kw = 16;
    while (spw > 1 && kw * (spw / 2) >= p.nsteps) spw /= 2;
    if (kw == 16 && spw * mt > 4) {
        if (mt <= 2) spw = 4 / mt;
        else kw = 8;
    }
    // Several weight tiles per workgroup (an activation fragment then serves NT MFMAs and is fetched once
    // per 16 NT weight rows) wherever that still leaves workgroups for every CU
    const int nt = tile8_weight_tiles(p.M, out, p.K);
    if (nt > 1) {
        const int64_t wgn = (out + 16 * nt - 1) / (16 * nt);
        const dim3 gridn((unsigned)wgn, (unsigned)((mt_all + 3) / 4));
        const int kwn = p.nsteps > 4 ? 8 : 4;
        if (nt == 4) return launch_kw<I8, 1, 4, 4>(p, kwn, gridn, stream);
        return launch_kw<I8, 1, 4, 2>(p, kwn, gridn, stream);
    }
    const dim3 grid((unsigned)wgs, (unsigned)((mt_all + mt - 1) / mt));
#define NQ_T8_CASE(SPW_, MT_) \
    if (spw == SPW_ && mt == MT_) return launch_kw<I8, SPW_, MT_, 1>(p, kw, grid, stream);
    NQ_T8_CASE(1, 1) NQ_T8_CASE(2, 1) NQ_T8_CASE(4, 1) NQ_T8_CASE(8, 1)
    NQ_T8_CASE(1, 2) NQ_T8_CASE(2, 2) NQ_T8_CASE(4, 2)
    NQ_T8_CASE(1, 3) NQ_T8_CASE(2, 3)
    NQ_T8_CASE(1, 4) NQ_T8_CASE(2, 4)
#undef NQ_T8_CASE
    return fail(NQ_ERR_INVALID, "nq_forward: no 8-bit tile kernel of that shape");
}

}  // namespace

// a row of 768..8192 codes takes the one-row kernel (M = 1, K a multiple of 16); otherwise the
// 16-row tile kernel (K a multiple of 16: a last step that K cuts short is padded with zeros)
static bool row_kernel_fits(const ForwardArgs& a) {
    return a.M == 1 && a.L->in % 16 == 0 && a.L->in >= 768 && a.L->in <= 8192;
}

// The tile kernel against the 256 x 256-tile GEMM (nq_gemm8.hip), both measured over K = 512 .. 8192,
// N = 1024 .. 11008, M = 64 .. 2048.  What the GEMM takes on the tile form it picks: gemm8_estimate_us.
// The tile kernel with 2 or 4 weight tiles per workgroup takes, per round of 256 workgroups, a fixed 5.5 us
// (3.75 with four wavefronts) + 0.25 / 0.31 us per 128 k, half as much again when 64 rows at a time stream a
// weight larger than the caches hold; with one weight tile (small launches, short K) about 4 us + 5.6 us per
// 10^9 multiply-adds, more with few steps of K.  Below 64 rows the GEMM does not apply.
static bool tile8_wins(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (L->in % 16 != 0) return false;
    if (a.M < 64 || L->in % 128 != 0) return true;  // (the GEMM needs 64 rows and whole 128-byte steps)
    const double steps = (double)L->in / 128.0;
    const bool i8 = a.x_dtype == NQ_DT_I8;
    const double gemm_us = gemm8_estimate_us(a.M, L->out, L->in, i8);
    const int nt = tile8_weight_tiles(a.M, L->out, L->in);
    double tile_us;
    if (nt == 1) {
        tile_us = 4.0 + (5.6 + 9.6 / steps) * ((double)a.M * (double)L->in * (double)L->out * 1e-9);
    } else {
        const double wgs = (double)((L->out + 16 * nt - 1) / (16 * nt)) * (double)((a.M + 63) / 64);
        tile_us = std::max(1.0, wgs / 256.0) * ((steps > 4 ? 5.5 : 3.75) + (nt == 4 ? 0.31 : 0.25) * steps);
        if (a.M >= 128 && (int64_t)L->in * L->out > ((int64_t)32 << 20)) tile_us *= 1.5;
    }
    return tile_us < gemm_us;
}

bool gemv_fp8_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (L->format != NQ_FMT_FP8_E4M3 || a.x_dtype != NQ_DT_FP8_E4M3 || a.x_scale == nullptr) return false;
    return row_kernel_fits(a) || tile8_wins(a);
}

bool tile8_i8_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (L->format != NQ_FMT_W8_CHANNEL || a.x_dtype != NQ_DT_I8) return false;
    return row_kernel_fits(a) || tile8_wins(a);
}

static Fp8GemvParams tile8_params(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    Fp8GemvParams p{};
    p.w = L->d_codes, p.x = reinterpret_cast<const uint8_t*>(a.x), p.x_scale = a.x_scale;
    p.col_scale = reinterpret_cast<const float*>(L->d_scales);
    p.y = a.y, p.bias = a.bias;
    p.M = a.M, p.N = L->out, p.K = L->in, p.nsteps = (L->in + 127) / 128;
    p.tscale = L->scale;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    return p;
}

int32_t launch_tile8_i8(const ForwardArgs& a) {
    const Fp8GemvParams p = tile8_params(a);
    if (row_kernel_fits(a)) return launch_row_cpl<true>(p, a.stream);
    return launch_tile8<true>(p, a.L->out, a.stream);
}

int32_t launch_gemv_fp8(const ForwardArgs& a) {
    const Fp8GemvParams p = tile8_params(a);
    // one row: a wavefront per weight row once a row fills most of its 64 lanes (K >= 768)
    if (row_kernel_fits(a)) return launch_row_cpl<false>(p, a.stream);
    return launch_tile8<false>(p, a.L->out, a.stream);
}

}  // namespace nq
