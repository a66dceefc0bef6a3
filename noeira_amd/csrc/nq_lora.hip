// A frozen LoRA adapter's share of a linear's output, added in place:
//     y[T, OUT] += s * (x[T, IN] @ A[IN, R]) @ B[R, OUT]
// `LoRAAdapter.forward_add` (noeira/nn/peft/lora.mojo:292-349), called right after the base
// layer's forward with the same x and y.  The reference runs two GEMMs (and, off NVIDIA, a
// third kernel for the accumulation) through a [T, R] scratch; here it is one launch and no
// scratch: a workgroup owns 16 tokens x 256 output columns, forms h = x A for its 16 tokens
// itself (on the fp32 matrix cores, k split eight ways over the wavefronts and reduced through
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

}  // namespace

int32_t launch_lora_add(const void* x, int32_t x_dtype, const float* A, const float* B, float* y, int32_t T, int32_t IN,
                        int32_t OUT, int32_t R, float s, hipStream_t stream) {
    dim3 grid((OUT + LR_COLS - 1) / LR_COLS, (T + LR_ROWS - 1) / LR_ROWS);
    const bool bf = x_dtype == NQ_DT_BF16;
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

}  // namespace nq
