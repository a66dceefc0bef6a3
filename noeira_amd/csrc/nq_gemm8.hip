// Large-M GEMM over 8-bit operands on the CDNA4 matrix cores:
//     fp8 e4m3 x fp8 e4m3 -> fp32   (v_mfma_f32_32x32x64_f8f6f4)
//     int8     x int8     -> int32  (v_mfma_i32_32x32x32_i8)
//   y[M, N] = epi( (x[M, K] . w[N, K]^T) * scale + bias[N] )
// Both operands are K-contiguous, which is the layout the MFMA wants: a lane
// supplies 32 consecutive bytes of one row.
//
// Tiling.  One workgroup of 4 wavefronts (2 x 2) owns a 256 x 256 tile of y;
// each wavefront owns 128 x 128 of it as 4 x 4 MFMA tiles of 32 x 32, i.e. 256
// fp32/int32 accumulators per lane (the AGPR half of the unified register
// file), one workgroup per CU.  A wavefront tile this large is what keeps the
// kernel MFMA-bound: per 64-byte k-step a wavefront issues 16 MFMAs (1024
// cycles) for 16 KiB of LDS reads, half the LDS bandwidth; at 64 x 64 the LDS
// would be the limit.
//
// K loop.  Stages of BK = 128 bytes: x tile 256 x 128 B and w tile 256 x 128 B
// (64 KiB), double-buffered in LDS (128 of the CU's 160 KiB).  While a stage is
// being multiplied, the next stage streams from global memory straight into the
// other LDS buffer (global_load_lds_dwordx4, 16 per lane per stage): no
// registers, no ds_write, one wait + one barrier per stage.
//
// LDS layout.  Row-major [256][128 B] with the eight 16-byte slots of a row
// permuted by slot ^= (row >> 1) & 7.  Rows r and r + 1 then sit 128 B apart in
// different bank halves and rows two apart in different slots, so both the
// 128-bit fragment reads (32 rows x 2 slots per wavefront instruction) and the
// staging writes are conflict free.
//
// Epilogue.  The MFMA takes the weight tile as its first operand, so a lane
// ends up with one token and runs of four consecutive channels; results are
// staged per wavefront through LDS and leave as 128-bit stores covering whole
// 256/512-byte row segments of y (2-byte scattered stores cost 37 % of the
// kernel before).
//
// Workgroup order.  Hardware deals consecutive workgroup ids round-robin to
// the 8 XCDs, each with its own L2.  Ids are first regrouped so that each XCD
// gets one contiguous run of tiles, and runs walk the tile grid in bands of 8
// row tiles, so the ~32 tiles resident on an XCD share 8 x-tiles and 4 w-tiles
// in that XCD's L2 instead of 32 + 32.
#include <type_traits>

#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int STAGE_BYTES = (BM + BN) * BK;  // 64 KiB

struct Gemm8Params {
    const uint8_t* a;  // x [M][K]
    const uint8_t* b;  // w [N][K]
    void* y;
    const void* bias;
    const float* row_scale;  // int8: per-row activation scales [M]; fp8: [1]
    const float* col_scale;  // int8: per-channel weight scales [N]
    float tscale;            // fp8: the weight's per-tensor scale
    int32_t M, N, K;
    int32_t tiles_m, tiles_n;
    int32_t y_dtype, bias_dtype, epilogue;
};

__device__ __forceinline__ uint16_t f32_to_bf16(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ int lds_off(int row, int slot) {
    return row * BK + ((slot ^ ((row >> 1) & 7)) << 4);
}

template <bool FP8>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm8_kernel(const Gemm8Params p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- XCD-aware tile assignment
    const int nb = gridDim.x;
    const int bid = blockIdx.x;
    const int per = nb / 8, rem = nb % 8;
    const int xcd = bid % 8, local = bid / 8;
    const int lid = xcd * per + min(xcd, rem) + local;
    constexpr int GM = 8;
    const int band = lid / (GM * p.tiles_n);
    const int first_m = band * GM;
    const int band_rows = min(GM, p.tiles_m - first_m);
    const int in_band = lid - band * GM * p.tiles_n;
    const int tm = first_m + in_band % band_rows;
    const int tn = in_band / band_rows;
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- global -> LDS, direct (global_load_lds_dwordx4): no register round trip.  One
    // instruction fills 1 KiB of LDS, lane l at byte 16 l, i.e. 8 rows of 128 B; wavefront w owns
    // rows [64 w, 64 w + 64) of both tiles.  The slot swizzle is applied on the global side: the
    // lane that lands in physical slot l % 8 of its row fetches logical slot (l % 8) ^ swz(row).
    typedef __attribute__((address_space(1))) const void gptr_t;
    typedef __attribute__((address_space(3))) void lptr_t;
    const uint8_t* da[8];
    const uint8_t* db[8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
        const int row = wave * 64 + t * 8 + (lane >> 3);
        const int slot = (lane & 7) ^ ((row >> 1) & 7);
        da[t] = p.a + (int64_t)min(m0 + row, p.M - 1) * p.K + slot * 16;
        db[t] = p.b + (int64_t)min(n0 + row, p.N - 1) * p.K + slot * 16;
    }
    auto dma = [&](int k0, int buf) {
        uint8_t* base = lds + buf * STAGE_BYTES + wave * 64 * BK;
#pragma unroll
        for (int t = 0; t < 8; t++) {
            __builtin_amdgcn_global_load_lds((gptr_t*)(da[t] + k0), (lptr_t*)(base + t * 1024), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t*)(db[t] + k0), (lptr_t*)(base + BM * BK + t * 1024), 16, 0, 0);
        }
    };
    const float fp8_scale = FP8 ? p.tscale * p.row_scale[0] : 0.0f;  // requested now, used in the epilogue

    typedef typename std::conditional<FP8, f32x16, i32x16>::type acc_t;
    acc_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    // Fragment addressing.  fp8: a 64-byte k-step, this lane supplies bytes [32 h, 32 h + 32) of
    // its row (h = lane / 32), i.e. slots 4 s + 2 h and 4 s + 2 h + 1.  int8: a 32-byte k-step,
    // bytes [16 h, 16 h + 16), slot 2 s + h.  Tile bases are multiples of 32 rows, so the swizzle
    // term depends on the row within the tile only.
    const int frow = lane & 31;
    const int fh = lane >> 5;
    const int fsw = (frow >> 1) & 7;

    // ---- main loop, software-pipelined by hand.  A wavefront has its SIMD to itself (the
    // 128 x 128 accumulator leaves room for one), so nothing hides an LDS round trip unless
    // the program order does: every fragment is read one MFMA group (4 MFMAs, ~256 cycles)
    // before the group that consumes it, the next sub-step's weight fragments are spread over
    // the four groups of the current one, and the one barrier of a K step sits before its LAST
    // group, followed at once by the first reads of the next stage, so that barrier skew and
    // read latency are both covered by matrix-core work already queued.
    // __builtin_amdgcn_sched_barrier(0) pins that order against the instruction scheduler.
    constexpr int NS = FP8 ? 2 : 4;  // sub-steps (one MFMA k-extent each) per K step
    typedef typename std::conditional<FP8, i32x8, i32x4>::type frag_t;
    auto read_frag = [&](const uint8_t* base, int sub, int t) -> frag_t {
        if constexpr (FP8) {
            const int o0 = ((4 * sub + 2 * fh) ^ fsw) << 4, o1 = ((4 * sub + 2 * fh + 1) ^ fsw) << 4;
            const i32x4 lo = *reinterpret_cast<const i32x4*>(base + t * 32 * BK + o0);
            const i32x4 hi = *reinterpret_cast<const i32x4*>(base + t * 32 * BK + o1);
            return (i32x8){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        } else {
            const int o0 = ((2 * sub + fh) ^ fsw) << 4;
            return *reinterpret_cast<const i32x4*>(base + t * 32 * BK + o0);
        }
    };
    auto stage_a = [&](int kt) { return lds + (kt & 1) * STAGE_BYTES + (wm * 128 + frow) * BK; };
    auto stage_b = [&](int kt) { return lds + (kt & 1) * STAGE_BYTES + BM * BK + (wn * 128 + frow) * BK; };

    const int KT = p.K / BK;
    dma(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    // Fragment registers are two named sets used in turn (groups alternate between af[0] and
    // af[1], sub-steps between bf[0] and bf[1]); a K step has an even number of both, so the
    // sets line up again at the loop's back edge and nothing is copied.
    frag_t af[2], bf[2][4];
#pragma unroll
    for (int j = 0; j < 4; j++) bf[0][j] = read_frag(stage_b(0), 0, j);
    af[0] = read_frag(stage_a(0), 0, 0);
    for (int kt = 0; kt < KT; kt++) {
        // stage kt+1 streams into the other buffer while stage kt is multiplied; the barrier
        // inside the previous iteration guarantees nobody still reads that buffer
        if (kt + 1 < KT) dma((kt + 1) * BK, (kt + 1) & 1);
        const uint8_t* sa = stage_a(kt);
        const uint8_t* sb = stage_b(kt);
#pragma unroll
        for (int sub = 0; sub < NS; sub++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int g = sub * 4 + i;  // group index within the K step
                const bool last = (sub == NS - 1 && i == 3);
                frag_t& acur = af[g & 1];
                frag_t& anext = af[(g + 1) & 1];
                frag_t(&bcur)[4] = bf[sub & 1];
                frag_t(&bnext)[4] = bf[(sub + 1) & 1];
                if (last) {
                    // every read of stage kt has been issued and waited for; once all wavefronts
                    // are here stage kt+1 is complete and stage kt's buffer may be overwritten
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    __syncthreads();
                }
                __builtin_amdgcn_sched_barrier(0);
                // the first MFMA of the group goes ahead of the prefetch so that the reads are
                // issued while the matrix core is busy and have the rest of the group to land
                if constexpr (FP8)
                    acc[i][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bcur[0], acur, acc[i][0], 0, 0, 0, 0,
                                                                                 0, 0);
                else
                    acc[i][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bcur[0], acur, acc[i][0], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (!last) {
                    anext = (i < 3) ? read_frag(sa, sub, i + 1) : read_frag(sa, sub + 1, 0);
                    if (sub + 1 < NS) bnext[i] = read_frag(sb, sub + 1, i);
                } else if (kt + 1 < KT) {
                    anext = read_frag(stage_a(kt + 1), 0, 0);
#pragma unroll
                    for (int j = 0; j < 4; j++) bnext[j] = read_frag(stage_b(kt + 1), 0, j);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 1; j < 4; j++) {
                    if constexpr (FP8)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bcur[j], acur, acc[i][j], 0, 0, 0,
                                                                                     0, 0, 0);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bcur[j], acur, acc[i][j], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    // ---- epilogue.  The MFMA was issued with the weight tile as its first operand, so in
    // acc[i][j] a lane holds ONE token m = 32 i + lane % 32 (MFMA column) and, for g = 0..3, the
    // four consecutive channels n = 32 j + 8 g + 4 (lane / 32) + 0..3 (MFMA rows, registers 4g..4g+3).
    // Per-token work is lane-local and four outputs of a row of y are adjacent.  Each wavefront
    // stages its results through its own LDS region (free now: the loop ended on a barrier) as
    // [token][channel] rows, and writes them out as 128-bit stores, 256 B (bf16) or 512 B (fp32 /
    // int32) contiguous per row of y.
    const int wm0 = m0 + wm * 128, wn0 = n0 + wn * 128;
    const int lm = lane & 31, lh = lane >> 5;
    const bool full_tile = (m0 + BM <= p.M) && (n0 + BN <= p.N) && (p.N % 8 == 0);

    // channel scale and bias for the lane's channels of tile j, group g (needs n < N: clamped)
    auto chan = [&](int j, int g, float (&cs)[4], float (&cb)[4], bool need_scale) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int n = min(wn0 + 32 * j + 8 * g + 4 * lh + r, p.N - 1);
            cs[r] = need_scale ? p.col_scale[n] : 1.0f;
            cb[r] = 0.0f;
            if (p.bias)
                cb[r] = (p.bias_dtype == NQ_DT_F32)
                            ? reinterpret_cast<const float*>(p.bias)[n]
                            : __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n] << 16);
        }
    };

    auto emit = [&](auto kind) {
        constexpr int KIND = decltype(kind)::value;  // 0: fp32, 1: bf16, 2: raw int32
        constexpr int ES = (KIND == 1) ? 2 : 4;      // bytes per output element
        constexpr int IP = (KIND == 1) ? 2 : 1;      // token tiles (of 32) staged per pass
        constexpr int ROWB = 128 * ES + 16;          // staged row: 128 channels + pad (bank spread)
        uint8_t* stage = lds + wave * (32 * IP * ROWB);
#pragma unroll
        for (int ip = 0; ip < 4; ip += IP) {
            // ---- registers -> LDS (this wavefront's region only).  Channel scales and biases are
            // fetched per channel tile j; the compiler barrier keeps it from hoisting all 16 (j, g)
            // sets above the loop, which would spill.
            float rscale[IP];
#pragma unroll
            for (int ii = 0; ii < IP; ii++) {
                rscale[ii] = 1.0f;
                if constexpr (!FP8 && KIND != 2) rscale[ii] = p.row_scale[min(wm0 + 32 * (ip + ii) + lm, p.M - 1)];
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float cs[4][4], cb[4][4];
                if constexpr (KIND != 2) {
#pragma unroll
                    for (int g = 0; g < 4; g++) chan(j, g, cs[g], cb[g], !FP8);
                }
                if constexpr (KIND == 2) {
#pragma unroll
                    for (int ii = 0; ii < IP; ii++) {
                        const int i = ip + ii;
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            uint8_t* dst = stage + (32 * ii + lm) * ROWB + (32 * j + 8 * g + 4 * lh) * ES;
                            *reinterpret_cast<i32x4*>(dst) = (i32x4){(int)acc[i][j][4 * g], (int)acc[i][j][4 * g + 1],
                                                                      (int)acc[i][j][4 * g + 2], (int)acc[i][j][4 * g + 3]};
                        }
                    }
                } else {
                    float z[IP][4][4];
#pragma unroll
                    for (int ii = 0; ii < IP; ii++)
#pragma unroll
                        for (int g = 0; g < 4; g++)
#pragma unroll
                            for (int r = 0; r < 4; r++) {
                                if constexpr (FP8)
                                    z[ii][g][r] = acc[ip + ii][j][4 * g + r] * fp8_scale + cb[g][r];
                                else
                                    z[ii][g][r] = (float)acc[ip + ii][j][4 * g + r] * (rscale[ii] * cs[g][r]) + cb[g][r];
                            }
                    if (p.epilogue == NQ_EPI_RELU) {
                        // a real (uniform) branch: one v_max per value when asked for, nothing otherwise
                        asm volatile("" ::: "memory");
#pragma unroll
                        for (int ii = 0; ii < IP; ii++)
#pragma unroll
                            for (int g = 0; g < 4; g++)
#pragma unroll
                                for (int r = 0; r < 4; r++) z[ii][g][r] = z[ii][g][r] > 0.0f ? z[ii][g][r] : 0.0f;
                    }
#pragma unroll
                    for (int ii = 0; ii < IP; ii++)
#pragma unroll
                        for (int g = 0; g < 4; g++) {
                            uint8_t* dst = stage + (32 * ii + lm) * ROWB + (32 * j + 8 * g + 4 * lh) * ES;
                            if constexpr (KIND == 0) {
                                *reinterpret_cast<float4*>(dst) =
                                    make_float4(z[ii][g][0], z[ii][g][1], z[ii][g][2], z[ii][g][3]);
                            } else {
                                // v_cvt_pk_bf16_f32: round to nearest even in hardware
                                const bf16x4 pk = __builtin_convertvector(
                                    (f32x4){z[ii][g][0], z[ii][g][1], z[ii][g][2], z[ii][g][3]}, bf16x4);
                                *reinterpret_cast<bf16x4*>(dst) = pk;
                            }
                        }
                }
                asm volatile("" ::: "memory");
            }
            // the region is this wavefront's own and DS operations of a wavefront execute in order:
            // no block barrier, only a fence against compiler reordering
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // ---- LDS -> global: 16 bytes per lane, rows of y contiguous
            constexpr int LPRW = 128 * ES / 16;          // lanes per staged row (16 or 32)
            constexpr int RPI = 64 / LPRW;               // rows per wavefront instruction
#pragma unroll
            for (int t = 0; t < 32 * IP / RPI; t++) {
                const int row = t * RPI + lane / LPRW, c16 = lane % LPRW;
                const i32x4 v = *reinterpret_cast<const i32x4*>(stage + row * ROWB + c16 * 16);
                const int m = wm0 + 32 * ip + row;
                const int n = wn0 + c16 * (16 / ES);
                if (full_tile) {
                    *reinterpret_cast<i32x4*>(reinterpret_cast<uint8_t*>(p.y) + ((int64_t)m * p.N + n) * ES) = v;
                } else if (m < p.M) {
                    // ragged edge: element by element
#pragma unroll
                    for (int e = 0; e < 16 / ES; e++) {
                        if (n + e >= p.N) break;
                        if constexpr (ES == 2) {
                            const uint32_t wv = (uint32_t)v[e >> 1];
                            reinterpret_cast<uint16_t*>(p.y)[(int64_t)m * p.N + n + e] = (uint16_t)(wv >> (16 * (e & 1)));
                        } else {
                            reinterpret_cast<int32_t*>(p.y)[(int64_t)m * p.N + n + e] = v[e];
                        }
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    };
    if (p.y_dtype == NQ_DT_F32)
        emit(std::integral_constant<int, 0>{});
    else if (p.y_dtype == NQ_DT_BF16)
        emit(std::integral_constant<int, 1>{});
    else if constexpr (!FP8)
        emit(std::integral_constant<int, 2>{});
}

}  // namespace

bool gemm8_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    const bool fp8 = (a.x_dtype == NQ_DT_FP8_E4M3 && L->format == NQ_FMT_FP8_E4M3);
    const bool i8 = (a.x_dtype == NQ_DT_I8 && L->format == NQ_FMT_W8_CHANNEL);
    return (fp8 || i8) && (L->in % BK == 0) && a.M >= 64;
}

int32_t launch_gemm8(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    Gemm8Params p{};
    p.a = reinterpret_cast<const uint8_t*>(a.x);
    p.b = L->d_codes;
    p.y = a.y, p.bias = a.bias;
    p.row_scale = a.x_scale;
    p.col_scale = reinterpret_cast<const float*>(L->d_scales);
    p.tscale = L->scale;
    p.M = a.M, p.N = L->out, p.K = L->in;
    p.tiles_m = (a.M + BM - 1) / BM, p.tiles_n = (L->out + BN - 1) / BN;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    const dim3 grid(p.tiles_m * p.tiles_n);
    const size_t lds = 2 * STAGE_BYTES;
    static bool attr_set[2] = {false, false};
    if (a.x_dtype == NQ_DT_FP8_E4M3) {
        if (!attr_set[0]) {
            NQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_kernel<true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            attr_set[0] = true;
        }
        hipLaunchKernelGGL(gemm8_kernel<true>, grid, dim3(256), lds, a.stream, p);
    } else {
        if (!attr_set[1]) {
            NQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(gemm8_kernel<false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            attr_set[1] = true;
        }
        hipLaunchKernelGGL(gemm8_kernel<false>, grid, dim3(256), lds, a.stream, p);
    }
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace nq
