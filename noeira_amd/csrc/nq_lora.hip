// A frozen LoRA adapter's share of a linear's output, added in place:
//     y[T, OUT] += s * (x[T, IN] @ A[IN, R]) @ B[R, OUT]
// `LoRAAdapter.forward_add` (noeira/nn/peft/lora.mojo:292-349), called right after the base
// layer's forward with the same x and y.  The reference runs two GEMMs (and, off NVIDIA, a
// third kernel for the accumulation) through a [T, R] scratch; here it is one launch and no
// scratch: a workgroup owns 16 tokens x 256 output columns, forms h = x A for its 16 tokens
// itself (the general kernel: on the fp32 matrix cores; R = 16 as stored has its own further down, on the bf16 ones
// with exact three-term splits; either way k split eight ways over the wavefronts and reduced through
// LDS; recomputed by each column tile, which costs less than a launch) and then adds s * h B
// to its tile of y with coalesced read-modify-writes.  fp32 throughout; x may be bf16.
//
// The kernel is a chain of memory round trips, so it is written to pay few of them: the tile
// of y and the columns of B a thread needs are requested before anything else, and the loads
// of x and A go out in batches of eight 16-k runs per wavefront before the first MFMA that
// uses them.
#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {  // round to nearest even, NaN stays NaN
    const uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

constexpr int LR_ROWS = 16;   // tokens per workgroup
constexpr int LR_COLS = 256;  // output columns per workgroup
constexpr int LR_R = 16;      // adapter columns handled per pass
constexpr int LR_BATCH = 8;   // 16-k runs whose loads are in flight together
constexpr int LR_WAVES = 8;   // wavefronts per workgroup: k is split this many ways
constexpr int LR_RG = LR_WAVES * 64 / LR_COLS;  // row groups in the second phase
constexpr int LR_RPT = LR_ROWS / LR_RG;         // rows of y per thread

// VEC: IN % 4 == 0, so a lane's four consecutive k are one aligned 16-byte (fp32) or 8-byte (bf16) load
template <bool XBF16, bool VEC>
__global__ __launch_bounds__(64 * LR_WAVES) void lora_add_kernel(const void* __restrict__ xv, const float* __restrict__ A,
                                                       const float* __restrict__ B, float* __restrict__ y, int T,
                                                       int IN, int OUT, int R, float s) {
    __shared__ float part[LR_WAVES][LR_ROWS][LR_R + 1];
    __shared__ float h[LR_ROWS][LR_R + 1];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * LR_ROWS, n0 = blockIdx.x * LR_COLS;
    const int n = n0 + (tid % LR_COLS), nc = min(n, OUT - 1);
    const int rg0 = (tid / LR_COLS) * LR_RPT;  // this thread's rows of the tile: rg0 .. rg0 + LR_RPT - 1
    // requested first, used last
    float yv[LR_RPT], b[LR_R];
#pragma unroll
    for (int i = 0; i < LR_RPT; i++) yv[i] = y[(int64_t)min(m0 + rg0 + i, T - 1) * OUT + nc];
#pragma unroll
    for (int rr = 0; rr < LR_R; rr++) b[rr] = B[(int64_t)min(rr, R - 1) * OUT + nc];
    float out[LR_RPT];
#pragma unroll
    for (int i = 0; i < LR_RPT; i++) out[i] = 0.0f;

    // four consecutive k of row m starting at kb (a multiple of 4), from clamped addresses (always valid);
    // what lies past IN is masked off by the caller after ALL of a batch's loads are on their way
    auto ldx4 = [&](int m, int kb, float (&v)[4]) {
        if (VEC) {
            const uint32_t at = (uint32_t)m * (uint32_t)IN + (uint32_t)min(kb, IN - 4);
            if (XBF16) {
                const uint2 w = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(xv) + at);
                v[0] = __uint_as_float(w.x << 16), v[1] = __uint_as_float(w.x & 0xFFFF0000u);
                v[2] = __uint_as_float(w.y << 16), v[3] = __uint_as_float(w.y & 0xFFFF0000u);
            } else {
                const float4 w = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(xv) + at);
                v[0] = w.x, v[1] = w.y, v[2] = w.z, v[3] = w.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t at = (uint32_t)m * (uint32_t)IN + (uint32_t)min(kb + j, IN - 1);
                v[j] = XBF16 ? __uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(xv)[at] << 16)
                             : reinterpret_cast<const float*>(xv)[at];
            }
        }
    };

    for (int r0 = 0; r0 < R; r0 += LR_R) {
        // ---- h[m][r] = sum_k x[m][k] A[k][r0 + r] on the fp32 matrix cores (v_mfma_f32_16x16x4_f32: the
        // products and sums are fp32, nothing is rounded to a narrower type).  Wavefront w takes the runs of
        // 16 k with index = w mod LR_WAVES; in a run, lane (i = lane % 16, q = lane / 16) holds x[m0 + i][k0 + 4q ..
        // 4q + 3], and MFMA j of the run multiplies the k = k0 + 4q + j of every q, so its second operand is
        // A[k0 + 4q + j][r].
        const int i16 = lane & 15, q4 = lane >> 4;
        const bool rlive = r0 + i16 < R;
        const int rcol = min(r0 + i16, R - 1);
        const int mrow = min(m0 + i16, T - 1);
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int kk = wave * 16; kk < IN; kk += 16 * LR_WAVES * LR_BATCH) {
            float xa[LR_BATCH][4], ab[LR_BATCH][4];
#pragma unroll
            for (int t = 0; t < LR_BATCH; t++) {
                const int kb = kk + 16 * LR_WAVES * t + 4 * q4;
                ldx4(mrow, kb, xa[t]);
#pragma unroll
                for (int j = 0; j < 4; j++) ab[t][j] = A[(uint32_t)(min(kb + j, IN - 1) * R + rcol)];
            }
            // every load of the batch is issued before the first use: left to itself the scheduler
            // interleaves them with the MFMAs three deep, and the batch then costs ten latencies, not one
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < LR_BATCH; t++) {
                const int kb = kk + 16 * LR_WAVES * t + 4 * q4;
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t keep = (kb + j < IN) ? ~0u : 0u;
                    const float xv_ = __uint_as_float(__float_as_uint(xa[t][j]) & keep);
                    const float av_ = __uint_as_float(__float_as_uint(ab[t][j]) & (rlive ? keep : 0u));
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(xv_, av_, acc, 0, 0, 0);
                }
            }
        }
        __syncthreads();  // the previous pass no longer reads h
#pragma unroll
        for (int v = 0; v < 4; v++) part[wave][4 * q4 + v][i16] = acc[v];  // D[row 4 (lane / 16) + v][col lane % 16]
        __syncthreads();
        if (tid < LR_ROWS * LR_R) {
            const int m = tid >> 4, rr = tid & 15;
            float t = 0.0f;
#pragma unroll
            for (int w = 0; w < LR_WAVES; w++) t += part[w][m][rr];
            h[m][rr] = t;
        }
        __syncthreads();
        // ---- out[m] += sum_r h[m][r] B[r0 + r][n]
        if (r0 > 0) {
#pragma unroll
            for (int rr = 0; rr < LR_R; rr++) b[rr] = B[(int64_t)min(r0 + rr, R - 1) * OUT + nc];
        }
#pragma unroll
        for (int rr = 0; rr < LR_R; rr++)
            if (r0 + rr >= R) b[rr] = 0.0f;
#pragma unroll
        for (int i = 0; i < LR_RPT; i++)
#pragma unroll
            for (int rr = 0; rr < LR_R; rr++) out[i] = fmaf(h[rg0 + i][rr], b[rr], out[i]);
    }
    if (n < OUT) {
#pragma unroll
        for (int i = 0; i < LR_RPT; i++)
            if (m0 + rg0 + i < T) y[(int64_t)(m0 + rg0 + i) * OUT + n] = fmaf(s, out[i], yv[i]);
    }
}

// ---- the usual case: R = 16 as stored, IN a multiple of 32, OUT a multiple of 4, 16-byte aligned operands --------
// The kernel above is bound by its load instructions (a dword per lane and k of A: IN / 4 of them per wavefront, and
// an instruction costs the CU's address unit the same whatever it fetches) and by the fp32 matrix cores (a sixteenth
// of the bf16 rate): 5.8 us at 960 -> 2560 for one token, 12.8 us at IN = 2560, 16.4 at 4096.  Here A's rows (16
// ranks = 64 bytes, so a chunk of 32 k is 2 KiB in one piece) are fetched 16 bytes per lane and turned into the
// MFMA's operand through the wavefront's own 2 KiB of LDS (the 16-byte quarter of row k sits at quarter ^ (k / 8) % 4:
// the four k-pieces of a rank then read different banks); h = x A runs on the bf16 matrix cores with A as three exact
// bf16 terms against the one (bf16 x) or three (fp32 x) terms of the activations, products below 2^-24 of the largest
// left out - the arithmetic of the adapter folded into the base call (nq_gemv_tile.hip); the tiles of B and y are
// fetched 16 bytes per lane as well, B through LDS.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
constexpr int L16_NB = 4;  // chunks of 32 k whose loads are in flight together, per wavefront

// The LDS one adapter's tile needs (eight wavefronts): where it lies is the caller's business.
struct Lora16Lds {
    float (*part)[LR_ROWS][LR_R + 1];  // [LR_WAVES]: the wavefronts' shares of h
    float (*h)[LR_R];                  // [LR_ROWS]
    float (*sta)[2][256];              // [LR_WAVES]: a chunk of A per wavefront, turned
    float (*bt)[LR_COLS];              // [LR_R]: the tile of B
};
constexpr int L16_LDS_FLOATS = LR_WAVES * LR_ROWS * (LR_R + 1) + LR_ROWS * LR_R + LR_WAVES * 2 * 256 + LR_R * LR_COLS;
__device__ __forceinline__ Lora16Lds lora16_lds_at(float* base) {  // (every piece a multiple of 16 bytes)
    Lora16Lds L;
    L.part = reinterpret_cast<float (*)[LR_ROWS][LR_R + 1]>(base);
    L.h = reinterpret_cast<float (*)[LR_R]>(base + LR_WAVES * LR_ROWS * (LR_R + 1));
    L.sta = reinterpret_cast<float (*)[2][256]>(base + LR_WAVES * LR_ROWS * (LR_R + 1) + LR_ROWS * LR_R);
    L.bt = reinterpret_cast<float (*)[LR_COLS]>(base + LR_WAVES * LR_ROWS * (LR_R + 1) + LR_ROWS * LR_R + LR_WAVES * 2 * 256);
    return L;
}

// The adapter's share of one tile: out[i][e] = sum_r (x A)[m0 + 2 rp + i][r] B[r][ncl + e] for thread tid = (cq, rp) of
// the eight wavefronts that share `lds` (unscaled; the caller adds s * out into what it loaded of y).  Its barriers are
// the workgroup's: every wavefront of the workgroup runs it, on its group's adapter, the same number of times; a caller
// that runs it twice on the same LDS puts a barrier between the runs.
template <bool XBF16>
__device__ __forceinline__ void lora16_tile(const Lora16Lds& lds, const int tid, const void* __restrict__ xv, const float* __restrict__ A,
                                            const float* __restrict__ B, int T, int IN, int OUT, int m0, int ncl, f32x4 (&out)[2]) {
    constexpr int NT = XBF16 ? 1 : 3;
    float (*const part)[LR_ROWS][LR_R + 1] = lds.part;
    float (*const h)[LR_R] = lds.h;
    float (*const sta)[2][256] = lds.sta;
    float (*const bt)[LR_COLS] = lds.bt;
    const int lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, q = lane >> 4;
    const int cq = tid & 63, rp = tid >> 6;
    // requested first, used last: the tile of B (rows 2 rp, 2 rp + 1 of it per thread)
    f32x4 bv[2];
#pragma unroll
    for (int i = 0; i < 2; i++) bv[i] = *reinterpret_cast<const f32x4*>(B + (int64_t)(2 * rp + i) * OUT + ncl);

    // ---- h = x A: wavefront w takes the chunks w, w + 8, ... of 32 k, L16_NB of them under way at a time
    const int nch = IN >> 5;
    const int mrow = min(m0 + c, T - 1);
    f32x4 hacc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c0 = wave; c0 < nch; c0 += LR_WAVES * L16_NB) {
        u32x4 ar[L16_NB][2], xr[L16_NB][XBF16 ? 1 : 2];
#pragma unroll
        for (int b = 0; b < L16_NB; b++) {
            const int k0 = min(c0 + b * LR_WAVES, nch - 1) << 5;  // (a chunk past K: read again, not used)
            if constexpr (XBF16) {
                xr[b][0] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(xv) + (int64_t)mrow * IN + k0 + 8 * q);
            } else {
                const float* xf = reinterpret_cast<const float*>(xv) + (int64_t)mrow * IN + k0 + 8 * q;
                xr[b][0] = *reinterpret_cast<const u32x4*>(xf), xr[b][XBF16 ? 0 : 1] = *reinterpret_cast<const u32x4*>(xf + 4);
            }
#pragma unroll
            for (int t = 0; t < 2; t++)
                ar[b][t] = *reinterpret_cast<const u32x4*>(A + (int64_t)(k0 + 16 * t + (lane >> 2)) * LR_R + 4 * (lane & 3));
        }
        __builtin_amdgcn_sched_barrier(0);  // every load of the batch ahead of the first wait
#pragma unroll
        for (int b = 0; b < L16_NB; b++) {
            if (c0 + b * LR_WAVES >= nch) break;  // (uniform over the wavefront)
            // A's chunk [32 k][16 ranks] -> 8 consecutive k of rank c per lane
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const int row = lane >> 2, kq = (2 * t + (row >> 3)) & 3;  // k / 8 of row 16 t + row
                *reinterpret_cast<u32x4*>(&sta[wave][t][row * 16 + 4 * ((lane & 3) ^ kq)]) = ar[b][t];
            }
            uint32_t av[8];
#pragma unroll
            for (int i = 0; i < 8; i++)
                av[i] = __float_as_uint(sta[wave][q >> 1][(8 * (q & 1) + i) * 16 + 4 * ((c >> 2) ^ q) + (c & 3)]);
            // hi + mid + lo = the fp32 value (each split truncates: every residual is exact)
            u32x4 pl[3], xt[NT];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t a0 = av[2 * i], b0 = av[2 * i + 1];
                const float ra = __uint_as_float(a0) - __uint_as_float(a0 & 0xFFFF0000u);
                const float rb = __uint_as_float(b0) - __uint_as_float(b0 & 0xFFFF0000u);
                const float sa = ra - __uint_as_float(__float_as_uint(ra) & 0xFFFF0000u);
                const float sb = rb - __uint_as_float(__float_as_uint(rb) & 0xFFFF0000u);
                pl[0][i] = __builtin_amdgcn_perm(b0, a0, 0x07060302u);
                pl[1][i] = __builtin_amdgcn_perm(__float_as_uint(rb), __float_as_uint(ra), 0x07060302u);
                pl[2][i] = __builtin_amdgcn_perm(__float_as_uint(sb), __float_as_uint(sa), 0x07060302u);
            }
            if constexpr (XBF16) {
                xt[0] = xr[b][0];
            } else {
                uint32_t v[8];
#pragma unroll
                for (int i = 0; i < 4; i++) v[i] = xr[b][0][i], v[4 + i] = xr[b][XBF16 ? 0 : 1][i];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t a0 = v[2 * i], b0 = v[2 * i + 1];
                    const float ra = __uint_as_float(a0) - __uint_as_float(a0 & 0xFFFF0000u);
                    const float rb = __uint_as_float(b0) - __uint_as_float(b0 & 0xFFFF0000u);
                    const float sa = ra - __uint_as_float(__float_as_uint(ra) & 0xFFFF0000u);
                    const float sb = rb - __uint_as_float(__float_as_uint(rb) & 0xFFFF0000u);
                    xt[0][i] = __builtin_amdgcn_perm(b0, a0, 0x07060302u);
                    xt[NT / 2][i] = __builtin_amdgcn_perm(__float_as_uint(rb), __float_as_uint(ra), 0x07060302u);
                    xt[NT - 1][i] = __builtin_amdgcn_perm(__float_as_uint(sb), __float_as_uint(sa), 0x07060302u);
                }
            }
            auto mm = [&](int xi, int ai) {
                hacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xt[xi]), __builtin_bit_cast(bf16x8, pl[ai]),
                                                               hacc, 0, 0, 0);
            };
            if constexpr (XBF16) {  // smallest products first
                mm(0, 2), mm(0, 1), mm(0, 0);
            } else {
                mm(NT / 2, 1), mm(NT - 1, 0), mm(0, 2), mm(NT / 2, 0), mm(0, 1), mm(0, 0);  // (x term, A term): 1 1, 2 0, 0 2, ...
            }
        }
    }
    // D[token 4 (lane / 16) + v][rank lane % 16]: the wavefronts' shares, summed in wave order
#pragma unroll
    for (int v = 0; v < 4; v++) part[wave][4 * q + v][c] = hacc[v];
#pragma unroll
    for (int i = 0; i < 2; i++) *reinterpret_cast<f32x4*>(&bt[2 * rp + i][4 * cq]) = bv[i];
    __syncthreads();
    if (tid < LR_ROWS * LR_R) {
        const int m = tid >> 4, rr = tid & 15;
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < LR_WAVES; w++) t += part[w][m][rr];
        h[m][rr] = t;
    }
    __syncthreads();
    // ---- sum_r h[m][r] B[r][n], r ascending
    out[0] = out[1] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int r4 = 0; r4 < LR_R; r4 += 4) {
        const f32x4 h0 = *reinterpret_cast<const f32x4*>(&h[2 * rp][r4]), h1 = *reinterpret_cast<const f32x4*>(&h[2 * rp + 1][r4]);
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const f32x4 bq = *reinterpret_cast<const f32x4*>(&bt[r4 + rr][4 * cq]);
#pragma unroll
            for (int e = 0; e < 4; e++) out[0][e] = fmaf(h0[rr], bq[e], out[0][e]), out[1][e] = fmaf(h1[rr], bq[e], out[1][e]);
        }
    }
}

template <bool XBF16>
__global__ __launch_bounds__(64 * LR_WAVES) void lora_add16_kernel(const void* __restrict__ xv, const float* __restrict__ A,
                                                                   const float* __restrict__ B, float* __restrict__ y, int T,
                                                                   int IN, int OUT, float s) {
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * LR_ROWS, n0 = blockIdx.x * LR_COLS;
    // second phase: thread (column quad cq, row pair rp) owns y[m0 + 2 rp .. + 1][n0 + 4 cq .. + 3]
    const int cq = tid & 63, rp = tid >> 6;
    const bool cols_in = n0 + 4 * cq < OUT;  // (OUT is a multiple of 4: a quad is inside or outside)
    const int ncl = min(n0 + 4 * cq, OUT - 4);
    // requested first, used last: the tile of y
    f32x4 yv[2];
#pragma unroll
    for (int i = 0; i < 2; i++) yv[i] = *reinterpret_cast<const f32x4*>(y + (int64_t)min(m0 + 2 * rp + i, T - 1) * OUT + ncl);
    f32x4 out[2];
    __shared__ __attribute__((aligned(16))) float lds_raw[L16_LDS_FLOATS];
    lora16_tile<XBF16>(lora16_lds_at(lds_raw), tid, xv, A, B, T, IN, OUT, m0, ncl, out);
    if (cols_in) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (m0 + 2 * rp + i >= T) break;
            f32x4 z;
#pragma unroll
            for (int e = 0; e < 4; e++) z[e] = fmaf(s, out[i][e], yv[i][e]);
            *reinterpret_cast<f32x4*>(y + (int64_t)(m0 + 2 * rp + i) * OUT + ncl) = z;
        }
    }
}

// ---- the adapters of a row-fused layer's parts in one launch ------------------------------------------------------
// (the caller's q | k | v and gate | up: `DecoderLayerWeights` keeps one adapter per projection, layer_weights.mojo:713-739.)
// A workgroup looks its part up by its column-tile index and does what lora_add16_kernel does for that part.  GLU: the
// layer's two parts are gate and up of one MLP; a workgroup takes the same column tile of both, adds each adapter's
// share to the base projections it reads from ys[0] and ys[1] (which stay as they are) and writes
// up * silu(gate) (`SwiGLU.forward`, swiglu.mojo:41-60): the adapters act before the activation, so this is where a
// trailing launch can still apply it.
struct LoraPartDev {
    const float* a;
    const float* b;   // null: the part has no adapter (its tiles return at once; GLU: its share is zero)
    float* y;
    int32_t out;
    int32_t tile0;    // the part's first column tile in the grid
    float s;
};
struct LoraMultiDev {
    LoraPartDev p[4];
    int32_t n;
};

template <bool XBF16, bool GLU>
__global__ __launch_bounds__(64 * LR_WAVES) void lora_multi16_kernel(const void* __restrict__ xv, const LoraMultiDev mp, int T, int IN,
                                                                     void* __restrict__ glu_out, int glu_dtype) {
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * LR_ROWS;
    const int cq = tid & 63, rp = tid >> 6;
    __shared__ __attribute__((aligned(16))) float lds_raw[L16_LDS_FLOATS];
    const Lora16Lds lds = lora16_lds_at(lds_raw);
    if constexpr (!GLU) {
        // (constant indices: the table stays in scalar registers)
        LoraPartDev me = mp.p[0];
        if (mp.n > 1 && (int)blockIdx.x >= mp.p[1].tile0) me = mp.p[1];
        if (mp.n > 2 && (int)blockIdx.x >= mp.p[2].tile0) me = mp.p[2];
        if (mp.n > 3 && (int)blockIdx.x >= mp.p[3].tile0) me = mp.p[3];
        if (!me.b) return;
        const int n0 = ((int)blockIdx.x - me.tile0) * LR_COLS;
        const bool cols_in = n0 + 4 * cq < me.out;
        const int ncl = min(n0 + 4 * cq, me.out - 4);
        f32x4 yv[2];
#pragma unroll
        for (int i = 0; i < 2; i++) yv[i] = *reinterpret_cast<const f32x4*>(me.y + (int64_t)min(m0 + 2 * rp + i, T - 1) * me.out + ncl);
        f32x4 out[2];
        lora16_tile<XBF16>(lds, tid, xv, me.a, me.b, T, IN, me.out, m0, ncl, out);
        if (cols_in) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                if (m0 + 2 * rp + i >= T) break;
                f32x4 z;
#pragma unroll
                for (int e = 0; e < 4; e++) z[e] = fmaf(me.s, out[i][e], yv[i][e]);
                *reinterpret_cast<f32x4*>(me.y + (int64_t)(m0 + 2 * rp + i) * me.out + ncl) = z;
            }
        }
    } else {
        const int OUT = mp.p[0].out;
        const int n0 = (int)blockIdx.x * LR_COLS;
        const bool cols_in = n0 + 4 * cq < OUT;
        const int ncl = min(n0 + 4 * cq, OUT - 4);
        f32x4 g[2], u[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int64_t at = (int64_t)min(m0 + 2 * rp + i, T - 1) * OUT + ncl;
            g[i] = *reinterpret_cast<const f32x4*>(mp.p[0].y + at), u[i] = *reinterpret_cast<const f32x4*>(mp.p[1].y + at);
        }
        f32x4 out[2];
        if (mp.p[0].b) {  // (uniform)
            lora16_tile<XBF16>(lds, tid, xv, mp.p[0].a, mp.p[0].b, T, IN, OUT, m0, ncl, out);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) g[i][e] = fmaf(mp.p[0].s, out[i][e], g[i][e]);
            __syncthreads();
        }
        if (mp.p[1].b) {
            lora16_tile<XBF16>(lds, tid, xv, mp.p[1].a, mp.p[1].b, T, IN, OUT, m0, ncl, out);
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) u[i][e] = fmaf(mp.p[1].s, out[i][e], u[i][e]);
        }
        if (cols_in) {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                if (m0 + 2 * rp + i >= T) break;
                f32x4 z;
#pragma unroll
                for (int e = 0; e < 4; e++) z[e] = swiglu_f32(u[i][e], g[i][e]);
                const int64_t at = (int64_t)(m0 + 2 * rp + i) * OUT + ncl;
                if (glu_dtype == NQ_DT_F32) {
                    *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(glu_out) + at) = z;
                } else {
                    uint2 pk;
                    pk.x = (uint32_t)f32_to_bf16_bits(z[0]) | ((uint32_t)f32_to_bf16_bits(z[1]) << 16);
                    pk.y = (uint32_t)f32_to_bf16_bits(z[2]) | ((uint32_t)f32_to_bf16_bits(z[3]) << 16);
                    *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(glu_out) + at) = pk;
                }
            }
        }
    }
}

// gate and up both with an adapter: sixteen wavefronts, the first eight on gate's adapter, the other eight on up's, at
// the same time (run one after the other in one workgroup of eight the call took 10.7 us at 960 -> 2560 and 135
// rows); up's sums then cross over through LDS to the threads that hold gate's.
constexpr int LGLU_LDS_BYTES = (2 * L16_LDS_FLOATS + LR_ROWS * LR_COLS) * 4;
template <bool XBF16>
__global__ __launch_bounds__(128 * LR_WAVES) void lora_glu16_kernel(const void* __restrict__ xv, const LoraMultiDev mp, int T, int IN,
                                                                    void* __restrict__ glu_out, int glu_dtype) {
    extern __shared__ __attribute__((aligned(16))) float lglu_raw[];
    const int ga = __builtin_amdgcn_readfirstlane(threadIdx.x >> 9), tid = threadIdx.x & 511;
    const Lora16Lds lds = lora16_lds_at(lglu_raw + ga * L16_LDS_FLOATS);
    float (*const ex)[LR_COLS] = reinterpret_cast<float (*)[LR_COLS]>(lglu_raw + 2 * L16_LDS_FLOATS);
    const LoraPartDev me = ga ? mp.p[1] : mp.p[0];
    const int m0 = blockIdx.y * LR_ROWS, n0 = (int)blockIdx.x * LR_COLS, OUT = me.out;
    const int cq = tid & 63, rp = tid >> 6;
    const bool cols_in = n0 + 4 * cq < OUT;
    const int ncl = min(n0 + 4 * cq, OUT - 4);
    f32x4 z[2];
#pragma unroll
    for (int i = 0; i < 2; i++) z[i] = *reinterpret_cast<const f32x4*>(me.y + (int64_t)min(m0 + 2 * rp + i, T - 1) * OUT + ncl);
    f32x4 out[2];
    lora16_tile<XBF16>(lds, tid, xv, me.a, me.b, T, IN, OUT, m0, ncl, out);
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int e = 0; e < 4; e++) z[i][e] = fmaf(me.s, out[i][e], z[i][e]);
    if (ga == 1) {
#pragma unroll
        for (int i = 0; i < 2; i++) *reinterpret_cast<f32x4*>(&ex[2 * rp + i][4 * cq]) = z[i];
    }
    __syncthreads();
    if (ga == 0 && cols_in) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (m0 + 2 * rp + i >= T) break;
            const f32x4 u = *reinterpret_cast<const f32x4*>(&ex[2 * rp + i][4 * cq]);
            f32x4 g;
#pragma unroll
            for (int e = 0; e < 4; e++) g[e] = swiglu_f32(u[e], z[i][e]);
            const int64_t at = (int64_t)(m0 + 2 * rp + i) * OUT + ncl;
            if (glu_dtype == NQ_DT_F32) {
                *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(glu_out) + at) = g;
            } else {
                uint2 pk;
                pk.x = (uint32_t)f32_to_bf16_bits(g[0]) | ((uint32_t)f32_to_bf16_bits(g[1]) << 16);
                pk.y = (uint32_t)f32_to_bf16_bits(g[2]) | ((uint32_t)f32_to_bf16_bits(g[3]) << 16);
                *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(glu_out) + at) = pk;
            }
        }
    }
}

// up * silu(gate) over n values (the path of last resort: adapters the fast kernel does not take, then this)
__global__ __launch_bounds__(256) void swiglu_kernel(const float* __restrict__ g, const float* __restrict__ u, void* __restrict__ out,
                                                     int64_t n, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float z = swiglu_f32(u[i], g[i]);
    if (dtype == NQ_DT_F32) reinterpret_cast<float*>(out)[i] = z;
    else reinterpret_cast<uint16_t*>(out)[i] = f32_to_bf16_bits(z);
}

}  // namespace

int32_t launch_lora_add(const void* x, int32_t x_dtype, const float* A, const float* B, float* y, int32_t T, int32_t IN,
                        int32_t OUT, int32_t R, float s, hipStream_t stream) {
    dim3 grid((OUT + LR_COLS - 1) / LR_COLS, (T + LR_ROWS - 1) / LR_ROWS);
    const bool bf = x_dtype == NQ_DT_BF16;
    const auto al16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    if (R == LR_R && IN % 32 == 0 && OUT % 4 == 0 && al16(x) && al16(A) && al16(B) && al16(y)) {
        if (bf) hipLaunchKernelGGL((lora_add16_kernel<true>), grid, dim3(64 * LR_WAVES), 0, stream, x, A, B, y, T, IN, OUT, s);
        else hipLaunchKernelGGL((lora_add16_kernel<false>), grid, dim3(64 * LR_WAVES), 0, stream, x, A, B, y, T, IN, OUT, s);
        NQ_HIP(hipGetLastError());
        return NQ_OK;
    }
    const bool vec = IN % 4 == 0 && ((uintptr_t)x & 15) == 0;
#define NQ_LORA(BF, VEC) \
    hipLaunchKernelGGL((lora_add_kernel<BF, VEC>), grid, dim3(64 * LR_WAVES), 0, stream, x, A, B, y, T, IN, OUT, R, s)
    if (bf) {
        if (vec) NQ_LORA(true, true); else NQ_LORA(true, false);
    } else {
        if (vec) NQ_LORA(false, true); else NQ_LORA(false, false);
    }
#undef NQ_LORA
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

int32_t launch_lora_multi(const void* x, int32_t x_dtype, int32_t T, int32_t IN, int32_t n, const LoraPartArgs* parts, void* glu_out,
                          int32_t glu_dtype, hipStream_t stream) {
    const auto al16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    const bool bf = x_dtype == NQ_DT_BF16;
    bool fast = IN % 32 == 0 && al16(x) && (!glu_out || al16(glu_out));
    for (int t = 0; t < n; t++)
        fast = fast && parts[t].out % 4 == 0 && al16(parts[t].y) && (!parts[t].b || (parts[t].r == LR_R && al16(parts[t].a) && al16(parts[t].b)));
    if (fast) {
        LoraMultiDev mp{};
        mp.n = n;
        int tiles = 0;
        for (int t = 0; t < n; t++) {
            mp.p[t] = LoraPartDev{parts[t].a, parts[t].b, parts[t].y, parts[t].out, tiles, parts[t].s};
            tiles += (parts[t].out + LR_COLS - 1) / LR_COLS;
        }
        const dim3 grid(glu_out ? (parts[0].out + LR_COLS - 1) / LR_COLS : tiles, (T + LR_ROWS - 1) / LR_ROWS);
        if (glu_out && parts[0].b && parts[1].b) {  // both halves carry an adapter: side by side
            static LdsAttrOnce attr[2];
            if (bf) {
                NQ_HIP(set_max_lds_once(attr[0], reinterpret_cast<const void*>(lora_glu16_kernel<true>), LGLU_LDS_BYTES));
                hipLaunchKernelGGL((lora_glu16_kernel<true>), grid, dim3(128 * LR_WAVES), LGLU_LDS_BYTES, stream, x, mp, T, IN, glu_out, glu_dtype);
            } else {
                NQ_HIP(set_max_lds_once(attr[1], reinterpret_cast<const void*>(lora_glu16_kernel<false>), LGLU_LDS_BYTES));
                hipLaunchKernelGGL((lora_glu16_kernel<false>), grid, dim3(128 * LR_WAVES), LGLU_LDS_BYTES, stream, x, mp, T, IN, glu_out, glu_dtype);
            }
            NQ_HIP(hipGetLastError());
            return NQ_OK;
        }
#define NQ_LM(BF, GLU) \
    hipLaunchKernelGGL((lora_multi16_kernel<BF, GLU>), grid, dim3(64 * LR_WAVES), 0, stream, x, mp, T, IN, glu_out, glu_dtype)
        if (glu_out) {
            if (bf) NQ_LM(true, true); else NQ_LM(false, true);
        } else {
            if (bf) NQ_LM(true, false); else NQ_LM(false, false);
        }
#undef NQ_LM
        NQ_HIP(hipGetLastError());
        return NQ_OK;
    }
    for (int t = 0; t < n; t++) {
        if (!parts[t].b) continue;
        const int32_t rc = launch_lora_add(x, x_dtype, parts[t].a, parts[t].b, parts[t].y, T, IN, parts[t].out, parts[t].r, parts[t].s, stream);
        if (rc) return rc;
    }
    if (glu_out) {
        const int64_t cnt = (int64_t)T * parts[0].out;
        hipLaunchKernelGGL(swiglu_kernel, dim3((unsigned)((cnt + 255) / 256)), dim3(256), 0, stream, parts[0].y, parts[1].y, glu_out, cnt, glu_dtype);
        NQ_HIP(hipGetLastError());
    }
    return NQ_OK;
}

}  // namespace nq
