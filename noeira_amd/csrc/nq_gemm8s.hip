// The 8-bit GEMM (fp8 x fp8 -> fp32, int8 x int8 -> int32; nq_gemm8.hip) for a few hundred to a few thousand rows:
// the same arithmetic on 128 x 128 tiles.
//
// Why a second tile size.  A 256 x 256 tile takes its 41 - 46 us (fp8, K = 4096) however few of them a call has:
// 41.6 us at M = 1024 (64 tiles on 256 CUs), 45.8 at 2048.  With 128 x 128 tiles the same call has four times as
// many workgroups of a quarter of the arithmetic each.  A stage of such a tile has 16 MFMAs per wavefront (0.22 us)
// behind a barrier and sixteen fragment reads that nothing overlaps, and takes about 0.6 us; a round of 128 x 128
// tiles then takes 21 - 25 us at K = 4096 where a round of the large ones takes 42 - 46 for four times the work.  The
// small tile wins while its tiles fit one round (M = 1024 over 4096 x 4096: 24.8 us against 41.6, int8 31.2 against
// 48.6; M = 512: 21.1 against the 16-row tile kernel's 25.7) and loses from two rounds on (M = 2048: 49 against 45.8).
// No split of K, hence no partial sums, no workspace and no second pass: every output is one accumulator's sum over
// K in ascending order, the order of the large kernel.
//
// The kernel is the plain form of the large one: 4 wavefronts (2 x 2), each 64 x 64 as 4 x 4 MFMA tiles of 16 x 16;
// stages of 128 bytes of K, x tile and w tile 16 KiB each, four stages in LDS (128 KiB: one multiplied, three on
// their way), filled straight from global memory (global_load_lds_dwordx4, 8 per wavefront and stage, issued one at a
// time between the MFMAs) with the large kernel's slot permutation applied on the global side, so that the 128-bit
// fragment reads are conflict-free.  One barrier per stage: it proves the stage landed and that the buffer of the
// stage before has been read out.  Scheduling inside a stage is otherwise the compiler's.
// Epilogue: per-token scale x per-channel scale (int8) or the tensor scales (fp8), bias, ReLU, fp32 / bf16 / raw int32
// out, staged through LDS per wavefront and stored 16 bytes per lane - the large kernel's formulas, so a value is
// the same bits whichever of the two kernels produced it.
#include <type_traits>

#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(8))) int i32x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

constexpr int SM = 128, SN = 128, SK = 128;  // tile of y, bytes of K per stage
constexpr int S_STAGE = (SM + SN) * SK;      // 32 KiB
constexpr int S_NS = 4;                      // stages in LDS: one being multiplied, up to three on their way
constexpr int S_LDS = S_NS * S_STAGE;

struct Gemm8sParams {
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

// KIND: 0 fp32, 1 bf16, 2 raw int32 accumulators
template <bool FP8, int KIND>
__global__ __launch_bounds__(256) void gemm8s_kernel(const Gemm8sParams p) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int TI = 4, TJ = 4;
    constexpr int SLOTS = SK / 16;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    // ---- tile assignment: consecutive workgroup ids go round-robin to the 8 XCDs; regrouped so that each XCD gets a
    // contiguous run of tiles, runs walking the grid in bands of 8 row tiles (its L2 then serves 8 x tiles and a few
    // w tiles instead of one of each per workgroup)
    const int nb = gridDim.x, bid = blockIdx.x;
    const int per = nb / 8, rem = nb % 8;
    const int xcd = bid % 8, local = bid / 8;
    const int lid = xcd * per + min(xcd, rem) + local;
    constexpr int GM = 8;
    const int band = lid / (GM * p.tiles_n);
    const int first_m = band * GM;
    const int band_rows = min(GM, p.tiles_m - first_m);
    const int in_band = lid - band * GM * p.tiles_n;
    const int tm = first_m + in_band % band_rows, tn = in_band / band_rows;
    const int m0 = tm * SM, n0 = tn * SN;

    auto swz = [](int row) { return (((row >> 1) & 7) + 6) & 7; };

    // ---- global -> LDS: one instruction fills 1 KiB (8 rows of 128 B), lane l at byte 16 l; wavefront w owns rows
    // 32 w .. 32 w + 31 of both tiles (4 + 4 instructions per stage).  The lane that lands in physical slot s of its
    // row fetches logical slot s ^ swz(row).  Rows past M / N are read from the last valid row (never stored).
    typedef __attribute__((address_space(3))) void lptr_t;
    const uint8_t* const abase = p.a + (int64_t)m0 * p.K;
    const uint8_t* const bbase = p.b + (int64_t)n0 * p.K;
    uint32_t doff[8];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const int row = wave * 32 + t * 8 + lane / SLOTS;
        const int slot = (lane % SLOTS) ^ swz(row);
        doff[t] = (uint32_t)(min(m0 + row, p.M - 1) - m0) * (uint32_t)p.K + slot * 16;
        doff[4 + t] = (uint32_t)(min(n0 + row, p.N - 1) - n0) * (uint32_t)p.K + slot * 16;
    }
    const uint32_t lds_addr0 = (uint32_t)(uintptr_t)(lptr_t*)lds;
    // (M0 holds the LDS destination of the instruction that follows; the compiler sets M0 itself before each of its
    // own uses, so writing it here needs no clobber; SCC does)
#define NQ_S_DMA(t, dst, off, src)                                                          \
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"    \
                 :                                                                      \
                 : "s"(dst), "v"(off), "s"(src), "n"(((t) & 3) * 1024)                  \
                 : "memory", "scc")
    // transfer t (0 .. 7) of stage st into buffer buf
    auto fill1 = [&](auto tc, int buf, int st) {
        constexpr int t = decltype(tc)::value;
        const uint8_t* const src = (t < 4 ? abase : bbase) + (int64_t)st * SK;
        // (named outside the asm statement so that the lambda captures them)
        const uint32_t dst = lds_addr0 + buf * S_STAGE + (t < 4 ? 0 : SM * SK) + wave * 32 * SK;
        const uint32_t off = doff[t];
        NQ_S_DMA(t, dst, off, src);
    };
    auto fill = [&](int buf, int st) {
        static_for<8>([&](auto tc) { fill1(tc, buf, st); });
    };
    const float fp8_scale = FP8 ? p.tscale * p.row_scale[0] : 0.0f;  // requested now, used in the epilogue

    typedef typename std::conditional<FP8, f32x4, i32x4>::type acc_t;
    acc_t acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++) acc[i][j] = acc_t{};

    // a fragment: 16 rows; lane l is on row l % 16.  fp8: bytes [32 c, 32 c + 32) of the stage's 128, c = l / 16 (slots
    // 2 c, 2 c + 1); int8: two k-halves of 64 bytes, bytes [16 c, 16 c + 16) of the half u (slot 4 u + c)
    const int frow = lane & 15, fc = lane >> 4, fsw = swz(frow);
    const uint8_t* const xrow = lds + (wm * 64 + frow) * SK;
    const uint8_t* const wrow = lds + SM * SK + (wn * 64 + frow) * SK;
    const int so0 = ((FP8 ? 2 * fc : fc) ^ fsw) << 4, so1 = ((FP8 ? 2 * fc + 1 : 4 + fc) ^ fsw) << 4;

    const int KT = p.K / SK;
    // Stage st lives in buffer st % 4.  A trip from L2 takes longer than a stage's MFMAs, so three stages are under way
    // while one is multiplied, and the transfers of the stage three ahead are issued one at a time between this
    // stage's MFMAs: a wavefront issues in order and a transfer holds its issue for some seventy cycles, which the
    // matrix core spends on the MFMA before it.  (Measured at M = 64 .. 1024 over 4096 x 4096, microseconds per stage:
    // one stage under way and the transfers in a batch behind the barrier 0.68 - of which the transfers alone 0.28,
    // the fragment reads and MFMAs alone 0.42; three under way, still in a batch, the same 0.68; spread between the
    // MFMAs 0.6.  The MFMAs take 0.22: what remains is the barrier and the fragment reads at the head of every
    // stage.  Reading a stage's fragments during the MFMAs of the stage before, into a second register set, made the
    // compiler rotate the sets through copies - four moves per MFMA - and measured slower, 0.8.)
    // The transfers are the loop's only vector-memory instructions, 8 per wavefront and stage, landing in order:
    // "all but the youngest 16" is everything up to stage st.
    fill(0, 0);
    if (KT > 1) fill(1, 1);
    if (KT > 2) fill(2, 2);
    for (int st = 0; st < KT; st++) {
        const int buf = st & (S_NS - 1);
        if (st + 2 < KT) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else if (st + 1 < KT) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // stage st has landed everywhere; everyone is done reading the buffer of stage st - 1
        const bool more = st + 3 < KT;
        const int nbuf = (st + 3) & (S_NS - 1);
        const uint8_t* const xb = xrow + buf * S_STAGE;
        const uint8_t* const wb = wrow + buf * S_STAGE;
        i32x4 xf[TI][2], wf[TJ][2];
#pragma unroll
        for (int i = 0; i < TI; i++) {
            xf[i][0] = *reinterpret_cast<const i32x4*>(xb + i * 16 * SK + so0);
            xf[i][1] = *reinterpret_cast<const i32x4*>(xb + i * 16 * SK + so1);
        }
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            wf[j][0] = *reinterpret_cast<const i32x4*>(wb + j * 16 * SK + so0);
            wf[j][1] = *reinterpret_cast<const i32x4*>(wb + j * 16 * SK + so1);
        }
        static_for<TI * TJ>([&](auto ijc) {
            constexpr int ij = decltype(ijc)::value, i = ij / TJ, j = ij % TJ;
            // (the weight fragment first: a lane then holds one token and four consecutive channels)
            if constexpr (FP8) {
                const i32x8 av = {xf[i][0][0], xf[i][0][1], xf[i][0][2], xf[i][0][3], xf[i][1][0], xf[i][1][1], xf[i][1][2], xf[i][1][3]};
                const i32x8 bv = {wf[j][0][0], wf[j][0][1], wf[j][0][2], wf[j][0][3], wf[j][1][0], wf[j][1][1], wf[j][1][2], wf[j][1][3]};
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bv, av, acc[i][j], 0, 0, 0, 0, 0, 0);
            } else {
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[j][0], xf[i][0], acc[i][j], 0, 0, 0);
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[j][1], xf[i][1], acc[i][j], 0, 0, 0);
            }
            if constexpr (ij % 2 == 1) {
                if (more) fill1(std::integral_constant<int, ij / 2>{}, nbuf, st + 3);
            }
        });
    }
#undef NQ_S_DMA
    __syncthreads();  // every wavefront is done with the stage buffers: the epilogue stages through them

    // ---- epilogue.  In acc[i][j] a lane holds token m = 16 i + lane % 16 and channels n = 16 j + 4 (lane / 16) + 0..3.
    // A wavefront stages its 64 x 64 results in its own LDS region as [token][channel] rows (+ 16 bytes of pad) and
    // writes them out 16 bytes per lane, rows of y contiguous.
    constexpr int ES = (KIND == 1) ? 2 : 4;
    constexpr int ROWB = 64 * ES + 16;
    const int wm0 = m0 + wm * 64, wn0 = n0 + wn * 64;
    const int lm = lane & 15, lq = lane >> 4;
    const bool full_cols = (n0 + SN <= p.N) && (p.N % 8 == 0) && (((uintptr_t)p.y & 15) == 0);
    uint8_t* const stg = lds + wave * (32 * ROWB);
    constexpr int LPRW = 64 * ES / 16;  // lanes per staged row (8 or 16)
    constexpr int RPI = 64 / LPRW;      // rows per wavefront instruction
#pragma unroll
    for (int ip = 0; ip < TI; ip += 2) {  // two token fragments (32 rows) per pass
#pragma unroll
        for (int ii = 0; ii < 2; ii++) {
            const int i = ip + ii;
            float rscale = 1.0f;
            if constexpr (!FP8 && KIND != 2) rscale = p.row_scale[min(wm0 + 16 * i + lm, p.M - 1)];
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                uint8_t* const dst = stg + (16 * ii + lm) * ROWB + (16 * j + 4 * lq) * ES;
                if constexpr (KIND == 2) {
                    *reinterpret_cast<i32x4*>(dst) = (i32x4){(int)acc[i][j][0], (int)acc[i][j][1], (int)acc[i][j][2], (int)acc[i][j][3]};
                } else {
                    float z[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int n = min(wn0 + 16 * j + 4 * lq + r, p.N - 1);
                        float cb = 0.0f;
                        if (p.bias)
                            cb = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const float*>(p.bias)[n]
                                                             : __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[n] << 16);
                        if constexpr (FP8) z[r] = acc[i][j][r] * fp8_scale + cb;
                        else z[r] = (float)acc[i][j][r] * (rscale * p.col_scale[n]) + cb;
                        if (p.epilogue == NQ_EPI_RELU) z[r] = z[r] > 0.0f ? z[r] : 0.0f;
                    }
                    if constexpr (KIND == 0) {
                        *reinterpret_cast<float4*>(dst) = make_float4(z[0], z[1], z[2], z[3]);
                    } else {
                        const bf16x4 pk = __builtin_convertvector((f32x4){z[0], z[1], z[2], z[3]}, bf16x4);  // round to nearest even
                        *reinterpret_cast<bf16x4*>(dst) = pk;
                    }
                }
            }
        }
        // (the region is this wavefront's own and a wavefront's LDS accesses execute in order)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int t = 0; t < 32 / RPI; t++) {
            const int row = t * RPI + lane / LPRW, c16 = lane % LPRW;
            const i32x4 v = *reinterpret_cast<const i32x4*>(stg + row * ROWB + c16 * 16);
            const int m = wm0 + 16 * ip + row, n = wn0 + c16 * (16 / ES);
            if (m >= p.M) continue;
            if (full_cols) {
                *reinterpret_cast<i32x4*>(reinterpret_cast<uint8_t*>(p.y) + ((int64_t)m * p.N + n) * ES) = v;
            } else {
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
}

template <typename K>
int32_t launch_s(K kernel, LdsAttrOnce* attr, const Gemm8sParams& p, hipStream_t s) {
    NQ_HIP(set_max_lds_once(*attr, reinterpret_cast<const void*>(kernel), S_LDS));
    hipLaunchKernelGGL(kernel, dim3(p.tiles_m * p.tiles_n), dim3(256), S_LDS, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace

// What a call takes on either tile size, from the measurements above (rounds of 256 workgroups; a fixed part and a part
// per stage of 128 bytes of K): the dispatch takes the smaller, and the 16-row tile kernels are weighed against it.
double gemm8_estimate_us(int M, int N, int K, bool i8, bool small_tile) {
    const double steps = (double)K / 128.0;
    if (small_tile) {
        const int64_t tiles = (int64_t)((M + SM - 1) / SM) * ((N + SN - 1) / SN);
        return (double)((tiles + 255) / 256) * (i8 ? 3.0 + 0.74 * steps : 2.5 + 0.6 * steps);
    }
    const int64_t tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    if (tiles <= 128) {
        // the 128 x 256 tile form (what launch_gemm8 takes for at most half a round of 256 x 256 tiles): a stage
        // lengthens as more than half the CUs draw on L2 at once (fp8, K = 4096: 24.7 us on 128 workgroups, 26.9 on
        // 192, 31.3 on 256; int8 28.8 / 30.8 / 35.2)
        const int64_t wgs = (int64_t)((M + 127) / 128) * ((N + 255) / 256);
        const double crowd = wgs > 128 ? (double)(wgs - 128) / 128.0 : 0.0;
        return i8 ? 7.0 + steps * (0.68 + 0.2 * crowd) : 6.5 + steps * (0.58 + 0.21 * crowd);
    }
    return (double)((tiles + 255) / 256) * (i8 ? 9.5 + 1.03 * steps : 10.0 + 1.1 * steps);
}

bool gemm8s_applicable(const ForwardArgs& a) {
    if (!gemm8_applicable(a)) return false;
    const nq_layer* L = a.L;
    const bool i8 = a.x_dtype == NQ_DT_I8;
    return gemm8_estimate_us(a.M, L->out, L->in, i8, true) < gemm8_estimate_us(a.M, L->out, L->in, i8, false);
}

int32_t launch_gemm8s(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    Gemm8sParams p{};
    p.a = reinterpret_cast<const uint8_t*>(a.x);
    p.b = L->d_codes;
    p.y = a.y, p.bias = a.bias;
    p.row_scale = a.x_scale;
    p.col_scale = reinterpret_cast<const float*>(L->d_scales);
    p.tscale = L->scale;
    p.M = a.M, p.N = L->out, p.K = L->in;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    p.tiles_m = (a.M + SM - 1) / SM, p.tiles_n = (L->out + SN - 1) / SN;
    static LdsAttrOnce attr_set[5];
    const bool f32 = a.y_dtype == NQ_DT_F32;
    if (a.x_dtype == NQ_DT_FP8_E4M3)
        return f32 ? launch_s(gemm8s_kernel<true, 0>, &attr_set[0], p, a.stream) : launch_s(gemm8s_kernel<true, 1>, &attr_set[1], p, a.stream);
    if (a.y_dtype == NQ_DT_I32) return launch_s(gemm8s_kernel<false, 2>, &attr_set[4], p, a.stream);
    return f32 ? launch_s(gemm8s_kernel<false, 0>, &attr_set[2], p, a.stream) : launch_s(gemm8s_kernel<false, 1>, &attr_set[3], p, a.stream);
}

}  // namespace nq
