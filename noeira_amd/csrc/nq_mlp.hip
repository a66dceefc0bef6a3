// Three W8A8 linears as ONE launch: the batched-env actor MLP
//     h1 = relu(L1(q8(x))),  h2 = relu(L2(q8(h1))),  y = L3(q8(h2))
// (SAC / PPO actors over M parallel envs; shapes such as 64 -> 256 -> 256 -> 8,
// noeira/deep_agents/sac/config.mojo:58-67).  At M = 4096 the three GEMMs are
// 0.69 GOP, a fraction of a microsecond of matrix-core time, so the cost of the
// unfused chain is its six launches and the activations it writes and re-reads.
// Here one wavefront carries 16 tokens through all three layers without ever
// leaving registers.
//
// Orientation.  The MFMA (v_mfma_i32_16x16x64_i8) is issued "transposed":
// the weight tile is the A operand (16 output channels x 64 k) and the tokens
// are the B operand (64 k x 16 tokens), so in the result a lane holds one token
// (column = lane % 16) and four consecutive output channels per tile (rows
// 4 * (lane / 16) + r).  That makes the per-token work lane-local:
//   - the absmax of a token's activations is a max over the lane's own values
//     and the three other lanes of its column (two shuffles);
//   - four consecutive int8 codes pack into one dword;
//   - the next layer's B operand (16 consecutive k per lane) is those dwords
//     gathered from the four lanes of the column: a 4 x 4 dword transpose done
//     with v_permlane32_swap / v_permlane16_swap, no LDS.
// Weights stay in L2 (84 KB for the actor); each wavefront reads its fragments
// with 128-bit loads.
//
// Arithmetic is the unfused path's: per-token scale s = absmax / 127 (1 where
// 0), q = clip(rint(v / s), -127, 127) with a true division, exact int32
// accumulation, z = float(acc) * (s * sw[n]) + b[n], ReLU as z > 0 ? z : 0.
#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) int i32x4;

constexpr int MAXT = 16;  // 16-channel tiles per layer (OUT <= 256)
constexpr int MAXS = 4;   // 64-wide k-steps per layer (IN <= 256)

struct MlpLayer {
    const int8_t* w;      // [N][K]
    const float* sw;      // [N]
    const float* bias;    // [N] or null
    int32_t N, K;
};

struct MlpParams {
    MlpLayer l[3];
    const float* x;  // [M][K0]
    float* y;        // [M][N2]
    int32_t M;
    int32_t final_relu;
};

__device__ __forceinline__ int q8(float v, float s) {
    float t = rintf(__fdiv_rn(v, s));
    t = t > -127.0f ? t : -127.0f;
    t = t < 127.0f ? t : 127.0f;
    return (int)t;
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return ((uint32_t)a & 0xFFu) | (((uint32_t)b & 0xFFu) << 8) | (((uint32_t)c & 0xFFu) << 16) |
           (((uint32_t)d & 0xFFu) << 24);
}

// One layer for this wavefront's 16 tokens.  `bop[s]` is the B operand of k-step s (16 int8 of
// the lane's token), `sx` the token's activation scale.  Returns z[j][r] = the layer's fp32
// output for channel 16 j + 4 kb + r of the lane's token (zero for channels >= N).
__device__ __forceinline__ void layer_forward(const MlpLayer& L, const i32x4 (&bop)[MAXS], float sx, bool relu,
                                              int ln, int kb, float (&z)[MAXT][4]) {
    const int tiles = (L.N + 15) >> 4;
    const int steps = (L.K + 63) >> 6;
#pragma unroll
    for (int j = 0; j < MAXT; j++) {
        if (j >= tiles) {
#pragma unroll
            for (int r = 0; r < 4; r++) z[j][r] = 0.0f;
            continue;
        }
        i32x4 acc = {0, 0, 0, 0};
        const int n_a = 16 * j + ln;  // the weight row this lane supplies to the A operand
#pragma unroll
        for (int s = 0; s < MAXS; s++) {
            if (s >= steps) break;
            const int k0 = 64 * s + 16 * kb;
            i32x4 a = {0, 0, 0, 0};
            if (n_a < L.N && k0 < L.K) a = *reinterpret_cast<const i32x4*>(L.w + (int64_t)n_a * L.K + k0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, bop[s], acc, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int n = 16 * j + 4 * kb + r;
            float v = 0.0f;
            if (n < L.N) {
                v = (float)acc[r] * (sx * L.sw[n]);
                if (L.bias) v += L.bias[n];
                if (relu) v = v > 0.0f ? v : 0.0f;
            }
            z[j][r] = v;
        }
    }
}

// Per-token int8 requantisation of z (channels 0 .. N-1) into the next layer's B operands.
__device__ __forceinline__ void requantize(const float (&z)[MAXT][4], int N, i32x4 (&bop)[MAXS], float& sx) {
    const int tiles = (N + 15) >> 4;
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < MAXT; j++) {
        if (j >= tiles) break;
#pragma unroll
        for (int r = 0; r < 4; r++) amax = fmaxf(amax, fabsf(z[j][r]));
    }
    amax = fmaxf(amax, __shfl_xor(amax, 16));
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    float s = amax / 127.0f;
    if (s == 0.0f) s = 1.0f;
    sx = s;
    // tile j of this lane = channels 16 j + 4 kb .. + 3: one dword.  k-step t needs, in lane kb',
    // the dwords of tile 4 t + kb' from the four lanes of the column, in lane order.
#pragma unroll
    for (int t = 0; t < MAXS; t++) {
        uint32_t d[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int j = 4 * t + u;
            d[u] = (j < tiles) ? pack4(q8(z[j][0], s), q8(z[j][1], s), q8(z[j][2], s), q8(z[j][3], s)) : 0u;
        }
        auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
        auto s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
        d[0] = s02[0], d[2] = s02[1], d[1] = s13[0], d[3] = s13[1];
        auto t01 = __builtin_amdgcn_permlane16_swap(d[0], d[1], false, false);
        auto t23 = __builtin_amdgcn_permlane16_swap(d[2], d[3], false, false);
        bop[t] = (i32x4){(int)t01[0], (int)t01[1], (int)t23[0], (int)t23[1]};
    }
}

__global__ __launch_bounds__(64) void mlp3_w8a8_kernel(const MlpParams p) {
    const int lane = threadIdx.x;
    const int ln = lane & 15, kb = lane >> 4;
    const int m = blockIdx.x * 16 + ln;          // this lane's token
    const int mc = min(m, p.M - 1);

    // ---- layer 1 input: fp32 x, 16 consecutive k per lane per k-step, quantised in registers
    const int K0 = p.l[0].K;
    const int steps0 = (K0 + 63) >> 6;
    float xv[MAXS][16];
    float amax = 0.0f;
#pragma unroll
    for (int s = 0; s < MAXS; s++) {
        if (s >= steps0) break;
        const int k0 = 64 * s + 16 * kb;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (k0 + 4 * q < K0) v = *reinterpret_cast<const float4*>(p.x + (int64_t)mc * K0 + k0 + 4 * q);
            xv[s][4 * q] = v.x, xv[s][4 * q + 1] = v.y, xv[s][4 * q + 2] = v.z, xv[s][4 * q + 3] = v.w;
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
    }
    amax = fmaxf(amax, __shfl_xor(amax, 16));
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    float sx = amax / 127.0f;
    if (sx == 0.0f) sx = 1.0f;
    i32x4 bop[MAXS];
#pragma unroll
    for (int s = 0; s < MAXS; s++) {
        bop[s] = (i32x4){0, 0, 0, 0};
        if (s >= steps0) continue;
#pragma unroll
        for (int q = 0; q < 4; q++)
            bop[s][q] = (int)pack4(q8(xv[s][4 * q], sx), q8(xv[s][4 * q + 1], sx), q8(xv[s][4 * q + 2], sx),
                                   q8(xv[s][4 * q + 3], sx));
    }

    float z[MAXT][4];
    layer_forward(p.l[0], bop, sx, true, ln, kb, z);
    requantize(z, p.l[0].N, bop, sx);
    layer_forward(p.l[1], bop, sx, true, ln, kb, z);
    requantize(z, p.l[1].N, bop, sx);
    layer_forward(p.l[2], bop, sx, p.final_relu != 0, ln, kb, z);

    if (m >= p.M) return;
    const int N2 = p.l[2].N;
    const int tiles2 = (N2 + 15) >> 4;
#pragma unroll
    for (int j = 0; j < MAXT; j++) {
        if (j >= tiles2) break;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int n = 16 * j + 4 * kb + r;
            if (n < N2) p.y[(int64_t)m * N2 + n] = z[j][r];
        }
    }
}

}  // namespace

int32_t launch_mlp3_w8a8(const nq_layer* l1, const nq_layer* l2, const nq_layer* l3, const float* x, float* y,
                         int32_t M, const float* b1, const float* b2, const float* b3, int32_t final_relu,
                         hipStream_t s) {
    MlpParams p{};
    const nq_layer* ls[3] = {l1, l2, l3};
    const float* bs[3] = {b1, b2, b3};
    for (int i = 0; i < 3; i++) {
        p.l[i].w = reinterpret_cast<const int8_t*>(ls[i]->d_codes);
        p.l[i].sw = reinterpret_cast<const float*>(ls[i]->d_scales);
        p.l[i].bias = bs[i];
        p.l[i].N = ls[i]->out, p.l[i].K = ls[i]->in;
    }
    p.x = x, p.y = y, p.M = M, p.final_relu = final_relu;
    hipLaunchKernelGGL(mlp3_w8a8_kernel, dim3((M + 15) / 16), dim3(64), 0, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace nq
