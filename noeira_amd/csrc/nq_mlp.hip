// Three W8A8 linears as ONE launch: the batched-env actor MLP
//     h1 = relu(L1(q8(x))),  h2 = relu(L2(q8(h1))),  y = L3(q8(h2))
// (SAC / PPO actors over M parallel envs; shapes such as 64 -> 256 -> 256 -> 8,
// noeira/deep_agents/sac/config.mojo:58-67).  At M = 4096 the three GEMMs are
// 0.69 GOP, a fraction of a microsecond of matrix-core time, so the cost of the
// unfused chain is its six launches and the activations it writes and re-reads.
// Here one workgroup of eight wavefronts carries 16 tokens through all three
// layers; activations never leave the CU (registers, plus 4 KB of LDS to hand a
// layer's int8 codes to the next one).
//
// Orientation.  The MFMA (v_mfma_i32_16x16x64_i8) is issued "transposed":
// the weight tile is the A operand (16 output channels x 64 k) and the tokens
// are the B operand (64 k x 16 tokens), so in the result a lane holds one token
// (column = lane % 16) and four consecutive output channels per tile (rows
// 4 * (lane / 16) + r).  That makes the per-token work lane-local: the absmax
// of a token's activations is a max over the lane's own values, the three
// other lanes of its column (two shuffles) and the other wavefronts (16 floats
// each through LDS); four consecutive int8 codes pack into one dword, stored to
// LDS row `token`; the next layer's B operand is one 128-bit LDS read.
// The output channels of a layer are split over the eight wavefronts (each owns
// an eighth of the 16-channel tiles), because the call is bound by the serial
// instruction stream of a wavefront, not by the matrix cores.
// Weights stay in L2 (84 KB for the actor); each wavefront requests the fragments
// of all three layers with 128-bit loads when the kernel starts, so that memory is
// waited for once and not once per layer (9.6 -> 8.7 us at M = 4096).  The fragments
// come from a copy of the codes kept as operand tiles (built when the weights are set:
// one contiguous KiB per instruction instead of 16 rows x 64 bytes, and every CU reads
// all 84 KB through its L1: 8.7 -> 7.8 us), scales and biases four channels per load
// (7.8 -> 7.4 us).
//
// Arithmetic is the unfused path's: per-token scale s = absmax / 127 (1 where
// 0), q = clip(rint(v / s), -127, 127) with a true division, exact int32
// accumulation, z = float(acc) * (s * sw[n]) + b[n], ReLU as z > 0 ? z : 0.
#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int MAXT = 16;  // 16-channel tiles per layer (OUT <= 256)
constexpr int MAXS = 4;   // 64-wide k-steps per layer (IN <= 256)

struct MlpLayer {
    const int8_t* w;      // operand tiles: (tile j, step s) at ((j * steps + s) * 1024), lane l's 16 bytes at 16 l
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
    // (v_med3_f32 clamps in one instruction; a NaN comes out as -127, as from the two compares it replaces)
    return (int)__builtin_amdgcn_fmed3f(rintf(__fdiv_rn(v, s)), -127.0f, 127.0f);
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d) {
    return ((uint32_t)a & 0xFFu) | (((uint32_t)b & 0xFFu) << 8) | (((uint32_t)c & 0xFFu) << 16) |
           (((uint32_t)d & 0xFFu) << 24);
}

constexpr int HROW = 256 + 16;     // LDS row stride of the int8 hand-over buffer (bytes)

// This wavefront's share of one layer: the 16-channel tiles TPW w .. TPW w + TPW - 1 for the 16 tokens of the
// workgroup.  The operands of ALL three layers (weight fragments, channel scales, biases) are requested at the
// start of the kernel, clamped rather than branched around and masked at use: the call then waits for memory
// once, not once per layer.
template <int TPW>
struct LayerRegs {
    i32x4 a[TPW][MAXS];
};

template <int TPW>
__device__ __forceinline__ void layer_load(const MlpLayer& L, int wave, int ln, int kb, LayerRegs<TPW>& R) {
    const int steps = (L.K + 63) >> 6;
#pragma unroll
    for (int u = 0; u < TPW; u++) {
        const int j = TPW * wave + u;
#pragma unroll
        for (int s = 0; s < MAXS; s++) {
            R.a[u][s] = (i32x4){0, 0, 0, 0};
            if (s < steps && 16 * j < L.N)  // uniform over the wavefront; one contiguous KiB per instruction
                R.a[u][s] = *reinterpret_cast<const i32x4*>(L.w + ((j * steps + s) * 1024 + 16 * (16 * kb + ln)));
        }
    }
}

// `bop[s]` is the B operand of k-step s (16 int8 of the lane's token), `sx` the token's scale.
// z[u][r] = fp32 output for channel 16 (TPW w + u) + 4 kb + r of the lane's token (0 beyond N).
// `sb` = the layer's [scales | biases] in LDS, 256 floats each (zeros beyond N and for a missing bias).
template <int TPW>
__device__ __forceinline__ void layer_forward(const MlpLayer& L, const LayerRegs<TPW>& R, const float* sb,
                                              const i32x4 (&bop)[MAXS], float sx, bool relu, int wave, int ln, int kb,
                                              float (&z)[TPW][4]) {
    const int steps = (L.K + 63) >> 6;
#pragma unroll
    for (int u = 0; u < TPW; u++) {
        const int j = TPW * wave + u;
        i32x4 acc = {0, 0, 0, 0};
        if (16 * j < L.N) {  // uniform over the wavefront (rows and k beyond the layer are zeros in the tiles)
#pragma unroll
            for (int s = 0; s < MAXS; s++) {
                if (s >= steps) break;
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(R.a[u][s], bop[s], acc, 0, 0, 0);
            }
        }
        const f32x4 sv = *reinterpret_cast<const f32x4*>(sb + 16 * j + 4 * kb);
        const f32x4 bv = *reinterpret_cast<const f32x4*>(sb + 256 + 16 * j + 4 * kb);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int n = 16 * j + 4 * kb + r;
            float v = (float)acc[r] * (sx * sv[r]) + bv[r];
            if (relu) v = v > 0.0f ? v : 0.0f;
            z[u][r] = (n < L.N) ? v : 0.0f;
        }
    }
}

// Per-token int8 requantisation of a layer's output (channels 0 .. N-1, spread over the
// wavefronts) into the next layer's B operands, through LDS.
template <int TPW>
__device__ __forceinline__ void requantize(const float (&z)[TPW][4], uint8_t* hq, float* amax_part, int wave, int ln,
                                           int kb, i32x4 (&bop)[MAXS], float& sx) {
    float amax = 0.0f;
#pragma unroll
    for (int u = 0; u < TPW; u++)
#pragma unroll
        for (int r = 0; r < 4; r++) amax = fmaxf(amax, fabsf(z[u][r]));  // channels beyond N hold 0
    amax = fmaxf(amax, __shfl_xor(amax, 16));
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    if (kb == 0) amax_part[wave * 16 + ln] = amax;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < MAXT / TPW; w++) amax = fmaxf(amax, amax_part[w * 16 + ln]);
    float s = amax / 127.0f;
    if (s == 0.0f) s = 1.0f;
    sx = s;
#pragma unroll
    for (int u = 0; u < TPW; u++) {
        const int j = TPW * wave + u;
        const uint32_t d = pack4(q8(z[u][0], s), q8(z[u][1], s), q8(z[u][2], s), q8(z[u][3], s));
        *reinterpret_cast<uint32_t*>(hq + ln * HROW + 16 * j + 4 * kb) = d;
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < MAXS; t++) bop[t] = *reinterpret_cast<const i32x4*>(hq + ln * HROW + 64 * t + 16 * kb);
}

template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void mlp3_w8a8_kernel(const MlpParams p) {
    constexpr int TPW = MAXT / WAVES;  // 16-channel tiles per wavefront and layer
    __shared__ __attribute__((aligned(16))) uint8_t hq[2][16 * HROW];
    __shared__ float amax_part[2][16 * WAVES];
    __shared__ __attribute__((aligned(16))) float xsh[16][256 + 4];
    __shared__ __attribute__((aligned(16))) float sbs[3][2 * 256];  // per layer [scales | biases]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ln = lane & 15, kb = lane >> 4;
    const int m = blockIdx.x * 16 + ln;          // this lane's token
    LayerRegs<TPW> R0, R1, R2;

    // ---- layer 1 input: the workgroup's 16 tokens of fp32 x are one contiguous piece of memory; it is fetched
    // once, a KiB per load instruction, into LDS (rows padded by 16 bytes against bank conflicts).  Each lane then
    // takes its token's 16 consecutive k per k-step from there and quantises them in registers (every wavefront
    // for the same 16 tokens: cheaper than a hand-over of the codes).  Read straight from memory in that shape,
    // a load instruction touched 64 separate 16-byte pieces, in each of the eight wavefronts.
    const int K0 = p.l[0].K;
    const int steps0 = (K0 + 63) >> 6;
    constexpr int XU = (4 * 256 + 64 * WAVES - 1) / (64 * WAVES);  // float4 units of the 16 x K0 tile per thread
    const int units = 4 * K0;                                      // (K0 is a multiple of 16)
    float4 xr[XU];
#pragma unroll
    for (int n = 0; n < XU; n++) {
        const int i = min((int)threadIdx.x + n * 64 * WAVES, units - 1);
        const int row = (4 * i) / K0, col = (4 * i) % K0;
        const int64_t mrow = min((int64_t)blockIdx.x * 16 + row, (int64_t)p.M - 1);
        xr[n] = *reinterpret_cast<const float4*>(p.x + mrow * K0 + col);
    }
    // (x is requested first and the weights right behind it: the store to LDS below waits for x alone)
    layer_load<TPW>(p.l[0], wave, ln, kb, R0);
    layer_load<TPW>(p.l[1], wave, ln, kb, R1);
    layer_load<TPW>(p.l[2], wave, ln, kb, R2);
    // Channel scales and biases: one element per thread and layer (thread t: array t / 256, channel t % 256, clamped
    // loads, zero beyond N and for a missing bias), handed round through LDS under the barrier that x needs anyway.
    // As two 16-byte loads per 16-channel tile and wavefront they were 96 of a workgroup's ~176 load instructions,
    // and an instruction costs the CU's address unit the same whatever it fetches.
    static_assert(WAVES == 8, "one scale or bias element per thread");
    float sbr[3];
#pragma unroll
    for (int l = 0; l < 3; l++) {
        const int ch = threadIdx.x & 255;
        const float* const src = (threadIdx.x >> 8) ? p.l[l].bias : p.l[l].sw;
        const float v = (src ? src : p.l[l].sw)[min(ch, p.l[l].N - 1)];
        sbr[l] = (src && ch < p.l[l].N) ? v : 0.0f;
    }
#pragma unroll
    for (int n = 0; n < XU; n++) {
        const int i = (int)threadIdx.x + n * 64 * WAVES;
        if (i < units) *reinterpret_cast<float4*>(&xsh[(4 * i) / K0][(4 * i) % K0]) = xr[n];
    }
#pragma unroll
    for (int l = 0; l < 3; l++) sbs[l][threadIdx.x] = sbr[l];
    __syncthreads();
    float xv[MAXS][16];
    float amax = 0.0f;
#pragma unroll
    for (int s = 0; s < MAXS; s++) {
        if (s >= steps0) break;
        const int k0 = 64 * s + 16 * kb;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (k0 + 4 * q < K0) v = *reinterpret_cast<const float4*>(&xsh[ln][k0 + 4 * q]);
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

    // (the hand-over rows need no clearing: every requantisation writes all 256 bytes of a token's row, zeros for the
    // channels its layer does not produce, because z is 0 there)

    float z[TPW][4];
    layer_forward<TPW>(p.l[0], R0, sbs[0], bop, sx, true, wave, ln, kb, z);
    requantize<TPW>(z, hq[0], amax_part[0], wave, ln, kb, bop, sx);
    layer_forward<TPW>(p.l[1], R1, sbs[1], bop, sx, true, wave, ln, kb, z);
    requantize<TPW>(z, hq[1], amax_part[1], wave, ln, kb, bop, sx);
    layer_forward<TPW>(p.l[2], R2, sbs[2], bop, sx, p.final_relu != 0, wave, ln, kb, z);

    if (m >= p.M) return;
    const int N2 = p.l[2].N;
#pragma unroll
    for (int u = 0; u < TPW; u++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int n = 16 * (TPW * wave + u) + 4 * kb + r;
            if (n < N2) p.y[(int64_t)m * N2 + n] = z[u][r];
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
        p.l[i].w = reinterpret_cast<const int8_t*>(ls[i]->d_tiled);
        p.l[i].sw = reinterpret_cast<const float*>(ls[i]->d_scales);
        p.l[i].bias = bs[i];
        p.l[i].N = ls[i]->out, p.l[i].K = ls[i]->in;
    }
    p.x = x, p.y = y, p.M = M, p.final_relu = final_relu;
    // eight wavefronts: with four the three layers' operands do not fit the registers (10.3 us against 8.7), with
    // sixteen the 1024-thread workgroup halves the register budget again (18.8 us)
    hipLaunchKernelGGL(mlp3_w8a8_kernel<8>, dim3((M + 15) / 16), dim3(512), 0, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

}  // namespace nq
