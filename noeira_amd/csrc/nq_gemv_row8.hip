// 8-bit dequant-GEMV for one activation row over a LARGE weight (M = 1, megabytes of codes):
//     y[N] = epi( (W[N, K] x) * scale + bias ),  W int8 with per-channel scales or fp8 e4m3 with one
//     scale, x bf16 or fp32 (fp8 x fp8 has its own kernel on the fp8 matrix cores, nq_gemv_fp8.hip).
//
// The register-resident kernel (nq_gemv_m1.hip) gives every wavefront its own copy of x, which for
// rows of 4 KiB and more is as many bytes again through the CU's load path as the row itself, and as
// many registers as leave room for few wavefronts.  Here x is staged once per workgroup into LDS as
// fp32 and the wavefronts stream rows against it:
//   - one wavefront owns one weight row and reads it as 1 KiB contiguous per load instruction
//     (lane l takes the 16-byte chunks l, l + 64, ...: CPL of them, all requested before x is staged);
//   - x sits in LDS so that the four 16-byte reads a lane needs under a chunk are each one contiguous
//     KiB across the wavefront: quarter t of chunk 64 j + l at ((4 j + t) 64 + l) 16 (no bank
//     conflicts); values past K are zero, which also cancels the clamped re-read of a last chunk;
//   - a code costs one convert and one FMA (int8: the sign-extending byte form of v_cvt_f32_i32;
//     fp8: v_cvt_pk_f32_fp8, two codes an instruction), exact fp32 products;
//   - the 64 partial sums meet in a fixed butterfly (a repeated call returns the same bits), and
//     lane 0 applies scale, bias and epilogue and stores through the part table of a row-fused layer.
#include "nq_common.h"

namespace nq {

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;

struct Row8Params {
    const uint8_t* codes;
    const float* scales;  // int8: per output channel
    float tscale;         // fp8: the tensor's scale
    const float* x_scale; // fp8: an optional scale of the activations (device, one value)
    const void* x;
    void* y;
    const void* bias;
    int32_t N, K, nch;
    int32_t y_dtype, bias_dtype, epilogue;
    SegTable seg;
};

__device__ __forceinline__ uint16_t f32_to_bf16_rne(float v) {
    uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);
}

template <int FMT, bool XF32, int CPL, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemv_row8_kernel(const Row8Params p) {
    constexpr int KPAD = CPL * 1024;  // k covered by CPL loads of a wavefront
    constexpr int NTHR = 64 * WAVES;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // x as fp32, [KPAD / 4] units of 16 bytes

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row = (int64_t)blockIdx.x * WAVES + wave;
    const int64_t r = min(row, (int64_t)p.N - 1);
    const u32x4* wq = reinterpret_cast<const u32x4*>(p.codes) + r * p.nch;

    // Every load is issued before anything waits: x first (it is staged first, and loads return in the order of
    // issue), then the row (unconditional loads from clamped chunk indices), its scale and the bias as stored
    // (widening a bf16 bias here would wait for it).  The scheduling barrier keeps the loads above the first wait.
    constexpr int XIT = (KPAD / 4 + NTHR - 1) / NTHR;  // staging steps per thread
    u32x4 xraw[XIT];
#pragma unroll
    for (int it = 0; it < XIT; it++) {
        const int kc = min(min(tid + it * NTHR, KPAD / 4 - 1) * 4, p.K - 4);
        if constexpr (XF32) {
            xraw[it] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const float*>(p.x) + kc);
        } else {
            const uint2 h = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p.x) + kc);
            xraw[it][0] = h.x, xraw[it][1] = h.y;
        }
    }
    u32x4 wv[CPL];
#pragma unroll
    for (int j = 0; j < CPL; j++) wv[j] = __builtin_nontemporal_load(wq + min(j * 64 + lane, p.nch - 1));
    const float scale = FMT == NQ_FMT_W8_CHANNEL ? p.scales[r] : p.tscale * (p.x_scale ? p.x_scale[0] : 1.0f);
    uint32_t braw = 0;
    if (p.bias)
        braw = (p.bias_dtype == NQ_DT_F32) ? reinterpret_cast<const uint32_t*>(p.bias)[r]
                                           : (uint32_t)reinterpret_cast<const uint16_t*>(p.bias)[r];
    __builtin_amdgcn_sched_barrier(0);

    // ---- x -> LDS as fp32: unit u = 4 consecutive k; unit t of chunk ch goes to ((4 (ch / 64) + t) 64 + ch % 64)
#pragma unroll
    for (int it = 0; it < XIT; it++) {
        const int u = tid + it * NTHR;
        if (u >= KPAD / 4) break;  // (uniform over a wavefront)
        const int k0 = u * 4;
        const uint32_t keep = k0 < p.K ? ~0u : 0u;
        u32x4 v;
        if constexpr (XF32) {
            v = xraw[it];
        } else {
            const uint32_t hx = xraw[it][0], hy = xraw[it][1];
            v[0] = hx << 16, v[1] = hx & 0xFFFF0000u, v[2] = hy << 16, v[3] = hy & 0xFFFF0000u;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] &= keep;
        const int ch = u >> 2, t = u & 3;
        *reinterpret_cast<u32x4*>(lds + (((4 * (ch >> 6) + t) * 64 + (ch & 63)) << 4)) = v;
    }
    __syncthreads();

    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < CPL; j++) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const f32x4 xv = *reinterpret_cast<const f32x4*>(lds + (((4 * j + t) * 64 + lane) << 4));
            const uint32_t w = wv[j][t];
            if constexpr (FMT == NQ_FMT_W8_CHANNEL) {
                acc = fmaf(xv[0], (float)(int)(int8_t)(w & 0xFFu), acc);
                acc = fmaf(xv[1], (float)(int)(int8_t)((w >> 8) & 0xFFu), acc);
                acc = fmaf(xv[2], (float)(int)(int8_t)((w >> 16) & 0xFFu), acc);
                acc = fmaf(xv[3], (float)((int)w >> 24), acc);
            } else {
                const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
                const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
                acc = fmaf(xv[0], a[0], acc);
                acc = fmaf(xv[1], a[1], acc);
                acc = fmaf(xv[2], b[0], acc);
                acc = fmaf(xv[3], b[1], acc);
            }
        }
    }
    float v = acc;
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
        float z = v * scale + __uint_as_float(p.bias_dtype == NQ_DT_F32 ? braw : braw << 16);
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

template <int FMT, bool XF32, int CPL>
int32_t launch_one(const Row8Params& p, hipStream_t s) {
    constexpr int WAVES = 16;  // 10.6 us against 11.4 with 8 and 12.7 with 4 (4096 -> 11008): x is staged once for 16 rows
    constexpr size_t lds = (size_t)CPL * 1024 * 4;
    auto kernel = gemv_row8_kernel<FMT, XF32, CPL, WAVES>;
    static LdsAttrOnce attr;
    if (lds > 48 * 1024) NQ_HIP(set_max_lds_once(attr, reinterpret_cast<const void*>(kernel), lds));
    hipLaunchKernelGGL(kernel, dim3((unsigned)((p.N + WAVES - 1) / WAVES)), dim3(64 * WAVES), lds, s, p);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

template <int FMT, bool XF32>
int32_t launch_cpl(const Row8Params& p, int cpl, hipStream_t s) {
    switch (cpl) {
        case 5: return launch_one<FMT, XF32, 5>(p, s);
        case 6: return launch_one<FMT, XF32, 6>(p, s);
        case 7: return launch_one<FMT, XF32, 7>(p, s);
        case 8: return launch_one<FMT, XF32, 8>(p, s);
        case 9: return launch_one<FMT, XF32, 9>(p, s);
        case 10: return launch_one<FMT, XF32, 10>(p, s);
        case 11: return launch_one<FMT, XF32, 11>(p, s);
        case 12: return launch_one<FMT, XF32, 12>(p, s);
        case 13: return launch_one<FMT, XF32, 13>(p, s);
        case 14: return launch_one<FMT, XF32, 14>(p, s);
        case 15: return launch_one<FMT, XF32, 15>(p, s);
        case 16: return launch_one<FMT, XF32, 16>(p, s);
    }
    return fail(NQ_ERR_UNSUPPORTED, "nq_forward: no 8-bit row GEMV for this IN");
}

}  // namespace

// an 8-bit weight of at least 4 MB whose rows are longer than 4 KiB (up to 16 KiB) of codes, one activation
// row in bf16 or fp32.  Up to 4 KiB a row the register-resident kernel measures the same or better (5.6
// against 6.1 us at 4096 x 4096, 11.5 both at 4096 -> 11008); beyond, x no longer fits its registers
// (17.8 -> 12.6 us at 11008 -> 4096, 17.9 -> 15.9 us at 8192 x 8192).
bool gemv_row8_applicable(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    if (a.M != 1) return false;
    if (L->format != NQ_FMT_W8_CHANNEL && L->format != NQ_FMT_FP8_E4M3) return false;
    if (a.x_dtype != NQ_DT_BF16 && a.x_dtype != NQ_DT_F32) return false;
    if (L->in % 16 != 0 || L->in <= 4096 || L->in > 16384) return false;
    return (int64_t)L->in * L->out >= ((int64_t)4 << 20);
}

int32_t launch_gemv_row8(const ForwardArgs& a) {
    const nq_layer* L = a.L;
    Row8Params p{};
    p.codes = L->d_codes, p.scales = reinterpret_cast<const float*>(L->d_scales), p.tscale = L->scale;
    p.x = a.x, p.x_scale = a.x_scale, p.y = a.y, p.bias = a.bias, p.seg = a.seg;
    p.N = L->out, p.K = L->in, p.nch = L->in / 16;
    p.y_dtype = a.y_dtype, p.bias_dtype = a.bias_dtype, p.epilogue = a.epilogue;
    const int cpl = (p.nch + 63) / 64;
    const bool xf32 = a.x_dtype == NQ_DT_F32;
    if (L->format == NQ_FMT_W8_CHANNEL)
        return xf32 ? launch_cpl<NQ_FMT_W8_CHANNEL, true>(p, cpl, a.stream)
                    : launch_cpl<NQ_FMT_W8_CHANNEL, false>(p, cpl, a.stream);
    return xf32 ? launch_cpl<NQ_FMT_FP8_E4M3, true>(p, cpl, a.stream) : launch_cpl<NQ_FMT_FP8_E4M3, false>(p, cpl, a.stream);
}

}  // namespace nq
