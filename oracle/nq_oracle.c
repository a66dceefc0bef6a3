/* nq_oracle.c — CPU restatement of noeira's quantized-linear path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (the noeira_amd package,
 * the C-ABI library) may include, link, import or call this file; it is the
 * checker that the tests, the smoke run and the benchmark's cpu_baseline leg
 * compare the HIP path against.
 *
 * Part 1 follows the reference line by line (citations are paths under the
 * reference checkout):
 *     noeira/nn/quant/q4_0.mojo        the Q4_0 format, RTN grid, pack/unpack,
 *                                      host dequantize
 *     noeira/io/safetensors.mojo:578   fp32 -> bf16 bits, ties to even
 *     noeira/nn/core/cpu_gemm.mojo:88  the Linux CPU GEMM (a triple loop)
 *     noeira/nn/quant/qlinear.mojo:416 QLinear.forward["cpu"] and vjp["cpu"]
 *     noeira/nn/peft/lora.mojo:292     LoRAAdapter.forward_add["cpu"]
 *     noeira/nn/primitives/swiglu.mojo SwiGLU.forward["cpu"] (the caller's step between gate | up and down)
 *     noeira/nn/quant/gptq.mojo,       GPTQ onto the Q4_0 grid, the factor of H^-1 it
 *       dense.mojo, hessian.mojo       reads, the calibration Hessian (load time)
 * and is pinned by the reference's own golden vectors
 * (tests/fixtures/quant/q4_0_rtn.safetensors, gptq_q4_0.safetensors) and by
 * closed forms; see tests/test_oracle_*.py.
 *
 * Part 2 defines the formats BASELINE names that the reference does not
 * implement (int8 per-channel, int8 per-token activations, uint4 group-wise
 * asymmetric, fp8 e4m3fn).  There is no reference code to follow there: each
 * function states its closed form, and the tests pin it against library
 * routines (numpy integer matmul, numpy float16, torch.float8_e4m3fn) and
 * brute force.
 *
 * Plain C99, no dependencies beyond libc/libm.  Build: oracle/Makefile.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define NQO_OK 0
#define NQO_ESIZE 1
#define NQO_ENOMEM 2

#define Q4_GROUP 32 /* q4_0.mojo:49 */
#define Q4_BLOCK 18 /* q4_0.mojo:51 */

static inline uint32_t f32_bits(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float x;
    memcpy(&x, &u, 4);
    return x;
}

/* ======================================================================== */
/* Part 1 — the reference's algorithm                                        */
/* ======================================================================== */

/* q4_0.mojo:55-58 */
int64_t nqo_q4_0_row_bytes(int64_t k) { return (k / Q4_GROUP) * Q4_BLOCK; }

/* noeira/io/safetensors.mojo:578-588: NaN -> 0x7FC0, otherwise add 0x7FFF
 * plus the lowest kept bit and keep the top 16. */
uint16_t nqo_f32_to_bf16_bits(float v) {
    uint32_t bits = f32_bits(v);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
    uint32_t bias = 0x7FFFu + ((bits >> 16) & 1u);
    return (uint16_t)((bits + bias) >> 16);
}

/* q4_0.mojo:61-64 */
float nqo_bf16_round(float x) {
    return bits_f32((uint32_t)nqo_f32_to_bf16_bits(x) << 16);
}

float nqo_bf16_bits_value(uint16_t b) { return bits_f32((uint32_t)b << 16); }

/* q4_0.mojo:67-82: floor-based round half to even. */
float nqo_round_half_even(float x) {
    float f = floorf(x);
    float frac = x - f;
    if (frac > 0.5f) return f + 1.0f;
    if (frac < 0.5f) return f;
    float half = f * 0.5f;
    return (floorf(half) == half) ? f : f + 1.0f;
}

/* q4_0.mojo:92-94: the fp32 value of fp16 bits (exact). IEEE binary16
 * decoded by hand: gcc 11 has no _Float16 on x86-64. */
float nqo_f16_value(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        /* subnormal: man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* q4_0.mojo:85-89: fp32 -> fp16 bits, round to nearest even (what the
 * hardware cast does): overflow -> inf, NaN keeps a quiet payload. */
uint16_t nqo_f16_bits(float x) {
    uint32_t u = f32_bits(x);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu));
    if (a >= 0x47800000u) {
        /* >= 65536: inf; values in [65520, 65536) round up to inf below */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (a <= 0x33000000u) return sign; /* <= 2^-25: zero (2^-25 itself ties to even) */
    int32_t e = (int32_t)(a >> 23) - 127;
    uint32_t m = (a & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
    uint32_t shift;
    uint32_t hexp;
    if (e < -14) { /* subnormal half */
        shift = (uint32_t)(13 + (-14 - e));
        hexp = 0;
    } else {
        shift = 13;
        hexp = (uint32_t)(e + 15);
    }
    uint32_t kept = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (kept & 1u))) kept += 1;
    uint32_t out;
    if (hexp == 0) {
        out = kept; /* may carry into the exponent field: that is correct */
    } else {
        out = ((hexp - 1u) << 10) + kept; /* kept includes the hidden bit (0x400) */
    }
    if (out >= 0x7C00u) out = 0x7C00u;
    return (uint16_t)(sign | out);
}

/* q4_0.mojo:97-112: the FIRST element of largest magnitude over -8; 1e-8
 * where that is 0; rounded to bf16. */
float nqo_q4_0_group_scale(const float* g) {
    int best = 0;
    float best_abs = fabsf(g[0]);
    for (int j = 1; j < Q4_GROUP; j++) {
        float a = fabsf(g[j]);
        if (a > best_abs) {
            best_abs = a;
            best = j;
        }
    }
    float d = g[best] / -8.0f;
    if (d == 0.0f) d = 1e-8f;
    return nqo_bf16_round(d);
}

/* q4_0.mojo:115-121: clip(round(w / d) + 8, 0, 15), a true division. */
uint8_t nqo_q4_0_code(float w, float d) {
    volatile float quot = w / d; /* keep the division a division */
    float v = nqo_round_half_even(quot) + 8.0f;
    /* min(max(v, 0), 15) as Mojo's max/min on floats */
    v = v > 0.0f ? v : 0.0f;
    v = v < 15.0f ? v : 15.0f;
    return (uint8_t)(int)v;
}

/* q4_0.mojo:124-154 */
int nqo_quantize_rtn_q4_0(const float* w, int64_t n, int64_t k, uint8_t* q, float* d) {
    if (k % Q4_GROUP != 0) return NQO_ESIZE;
    int64_t groups = k / Q4_GROUP;
    for (int64_t r = 0; r < n; r++) {
        for (int64_t g = 0; g < groups; g++) {
            int64_t base = r * k + g * Q4_GROUP;
            float dg = nqo_q4_0_group_scale(w + base);
            d[r * groups + g] = dg;
            for (int j = 0; j < Q4_GROUP; j++) q[base + j] = nqo_q4_0_code(w[base + j], dg);
        }
    }
    return NQO_OK;
}

/* q4_0.mojo:157-178 */
int nqo_pack_q4_0(const uint8_t* q, const uint16_t* d_bits, int64_t n, int64_t k, uint8_t* out) {
    if (k % Q4_GROUP != 0) return NQO_ESIZE;
    int64_t groups = k / Q4_GROUP;
    for (int64_t r = 0; r < n; r++) {
        for (int64_t g = 0; g < groups; g++) {
            int64_t blk = (r * groups + g) * Q4_BLOCK;
            uint16_t h = d_bits[r * groups + g];
            out[blk] = (uint8_t)(h & 0xFF);
            out[blk + 1] = (uint8_t)(h >> 8);
            int64_t base = r * k + g * Q4_GROUP;
            for (int j = 0; j < Q4_GROUP / 2; j++) {
                uint8_t lo = q[base + j] & 0xF;
                uint8_t hi = q[base + j + Q4_GROUP / 2] & 0xF;
                out[blk + 2 + j] = (uint8_t)(lo | (hi << 4));
            }
        }
    }
    return NQO_OK;
}

/* q4_0.mojo:181-204 */
int nqo_unpack_q4_0(const uint8_t* blocks, int64_t n, int64_t k, uint8_t* q, uint16_t* d_bits) {
    if (k % Q4_GROUP != 0) return NQO_ESIZE;
    int64_t groups = k / Q4_GROUP;
    for (int64_t r = 0; r < n; r++) {
        for (int64_t g = 0; g < groups; g++) {
            int64_t blk = (r * groups + g) * Q4_BLOCK;
            d_bits[r * groups + g] = (uint16_t)(blocks[blk] | ((uint16_t)blocks[blk + 1] << 8));
            int64_t base = r * k + g * Q4_GROUP;
            for (int j = 0; j < Q4_GROUP / 2; j++) {
                uint8_t byte = blocks[blk + 2 + j];
                q[base + j] = byte & 0xF;
                q[base + j + Q4_GROUP / 2] = byte >> 4;
            }
        }
    }
    return NQO_OK;
}

/* q4_0.mojo:207-216 */
int nqo_rtn_q4_0_blocks(const float* w, int64_t n, int64_t k, uint8_t* out) {
    if (k % Q4_GROUP != 0) return NQO_ESIZE;
    int64_t groups = k / Q4_GROUP;
    uint8_t* q = (uint8_t*)malloc((size_t)(n * k));
    float* d = (float*)malloc(sizeof(float) * (size_t)(n * groups));
    uint16_t* bits = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(n * groups));
    if (!q || !d || !bits) {
        free(q), free(d), free(bits);
        return NQO_ENOMEM;
    }
    nqo_quantize_rtn_q4_0(w, n, k, q, d);
    for (int64_t i = 0; i < n * groups; i++) bits[i] = nqo_f16_bits(d[i]);
    nqo_pack_q4_0(q, bits, n, k, out);
    free(q), free(d), free(bits);
    return NQO_OK;
}

/* q4_0.mojo:219-239 */
int nqo_dequantize_q4_0(const uint8_t* blocks, int64_t n, int64_t k, float* out) {
    if (k % Q4_GROUP != 0) return NQO_ESIZE;
    int64_t groups = k / Q4_GROUP;
    for (int64_t r = 0; r < n; r++) {
        for (int64_t g = 0; g < groups; g++) {
            int64_t blk = (r * groups + g) * Q4_BLOCK;
            float dg = nqo_f16_value((uint16_t)(blocks[blk] | ((uint16_t)blocks[blk + 1] << 8)));
            int64_t base = r * k + g * Q4_GROUP;
            for (int j = 0; j < Q4_GROUP / 2; j++) {
                uint8_t byte = blocks[blk + 2 + j];
                out[base + j] = ((float)(int)(byte & 0xF) - 8.0f) * dg;
                out[base + j + Q4_GROUP / 2] = ((float)(int)(byte >> 4) - 8.0f) * dg;
            }
        }
    }
    return NQO_OK;
}

/* cpu_gemm.mojo:88-98: c = alpha * sum_k op(a) op(b) + beta * c, k ascending,
 * one fp32 accumulator per output, c not read when beta == 0. */
void nqo_gemm_cpu(int ta, int tb, int64_t M, int64_t N, int64_t K, float alpha, const float* a,
                  int64_t lda, const float* b, int64_t ldb, float beta, float* c, int64_t ldc) {
    for (int64_t i = 0; i < M; i++) {
        for (int64_t j = 0; j < N; j++) {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; k++) {
                float av = ta ? a[k * lda + i] : a[i * lda + k];
                float bv = tb ? b[j * ldb + k] : b[k * ldb + j];
                acc += av * bv;
            }
            float prev = 0.0f;
            if (beta != 0.0f) prev = beta * c[i * ldc + j];
            c[i * ldc + j] = alpha * acc + prev;
        }
    }
}

/* qlinear.mojo:416-426: a FRESH dequantize of the [OUT, IN] blocks, then
 * gemm_cpu[False, True](B, OUT, IN, 1, x, IN, w, IN, 0, y, OUT). */
int nqo_qlinear_forward_cpu(const uint8_t* blocks, int64_t in, int64_t out, const float* x,
                            int64_t B, float* y) {
    if (in % Q4_GROUP != 0) return NQO_ESIZE;
    float* w = (float*)malloc(sizeof(float) * (size_t)(in * out));
    if (!w) return NQO_ENOMEM;
    nqo_dequantize_q4_0(blocks, out, in, w);
    nqo_gemm_cpu(0, 1, B, out, in, 1.0f, x, in, w, in, 0.0f, y, out);
    free(w);
    return NQO_OK;
}

/* qlinear.mojo:495-503: gx[B, IN] = gy[B, OUT] @ deq(W), gemm_cpu[False, False]. */
int nqo_qlinear_vjp_cpu(const uint8_t* blocks, int64_t in, int64_t out, const float* gy, int64_t B,
                        float* gx) {
    if (in % Q4_GROUP != 0) return NQO_ESIZE;
    float* w = (float*)malloc(sizeof(float) * (size_t)(in * out));
    if (!w) return NQO_ENOMEM;
    nqo_dequantize_q4_0(blocks, out, in, w);
    nqo_gemm_cpu(0, 0, B, in, out, 1.0f, gy, out, w, in, 0.0f, gx, in);
    free(w);
    return NQO_OK;
}

/* tests/nn/quant/qlinear_common.mojo:117-124: the exact product in fp64,
 * y[t, o] = sum_i x[t, i] * w[o, i], over any fp32 [N, K] weight. */
void nqo_dense_forward_f64(const float* w, int64_t N, int64_t K, const float* x, int64_t M,
                           double* y) {
    for (int64_t t = 0; t < M; t++) {
        for (int64_t o = 0; o < N; o++) {
            double acc = 0.0;
            for (int64_t i = 0; i < K; i++) acc += (double)x[t * K + i] * (double)w[o * K + i];
            y[t * N + o] = acc;
        }
    }
}

/* tests/nn/quant/qlinear_common.mojo:39-45: max|a-b| / max|b| (0-safe). */
double nqo_rel_max(const float* a, const float* b, int64_t n) {
    double d = 0.0, m = 0.0;
    for (int64_t i = 0; i < n; i++) {
        double e = fabs((double)a[i] - (double)b[i]);
        if (e > d) d = e;
        double v = fabs((double)b[i]);
        if (v > m) m = v;
    }
    return m > 0 ? d / m : d;
}

/* qlinear.mojo:152-172: fp32 [rows, cols] -> bf16 [rows, cols_pad], zero tail. */
void nqo_cast_pad_bf16(const float* src, int64_t rows, int64_t cols, int64_t cols_pad,
                       uint16_t* dst) {
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols_pad; c++)
            dst[r * cols_pad + c] = c < cols ? nqo_f32_to_bf16_bits(src[r * cols + c]) : 0;
}

/* qlinear.mojo:175-192: bf16 [rows, cols_pad] -> fp32 [rows, cols]. */
void nqo_slice_cast_f32(const uint16_t* src, int64_t rows, int64_t cols, int64_t cols_pad,
                        float* dst) {
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++)
            dst[r * cols + c] = nqo_bf16_bits_value(src[r * cols_pad + c]);
}

/* noeira/nn/peft/lora.mojo:292-318 (the CPU branch of LoRAAdapter.forward_add):
 * h[T, R] = x[T, IN] @ A[IN, R] (gemm_cpu, beta = 0), then
 * y[T, OUT] = s * (h @ B[R, OUT]) + 1 * y (gemm_cpu with alpha = s, beta = 1).
 * R is the padded rank the parameters hold; s the adapter's scale. */
int nqo_lora_forward_add(const float* x, const float* a, const float* b, int64_t T, int64_t in, int64_t out,
                         int64_t r, float s, float* y) {
    float* h = (float*)malloc((size_t)(T * r > 0 ? T * r : 1) * sizeof(float));
    if (!h) return NQO_ESIZE;
    nqo_gemm_cpu(0, 0, T, r, in, 1.0f, x, in, a, r, 0.0f, h, r);
    nqo_gemm_cpu(0, 0, T, out, r, s, h, r, b, out, 1.0f, y, out);
    free(h);
    return NQO_OK;
}

/* swiglu.mojo:120-141 (`SwiGLU.forward["cpu"]`; the GPU kernel :41-60 is the same expression): the input row is
 * [u | v] (2 * hidden wide), s = 1 / (1 + exp(-v)), out = u * (v * s), all in fp32.  The SmolVLA caller feeds it
 * (up, gate) (fused.mojo:343-350), so out = up * silu(gate).  Here u and v come as two [rows, hidden] arrays. */
void nqo_swiglu(const float* u, const float* v, int64_t count, float* out) {
    for (int64_t i = 0; i < count; i++) {
        float s = 1.0f / (1.0f + expf(-v[i]));
        out[i] = u[i] * (v[i] * s);
    }
}

/* ------------------------------------------------------------------------ */
/* GPTQ onto the Q4_0 grid (load time, off the forward path)                 */
/* ------------------------------------------------------------------------ */

/* dense.mojo:212-289: a (n x n row-major, symmetric positive definite, lower
 * triangle read) becomes L with L L^T = a, upper triangle zeroed.  Returns 0,
 * or 1 + the index of the first non-positive pivot.  Right-looking and blocked
 * like the reference's (by CHOL_BLOCK columns: factor the diagonal block, solve
 * the panel below it, subtract the panel's outer product from the trailing
 * matrix), with every sum in one stated order: a dot product runs over the
 * block's columns ascending from 0 and is subtracted once; the trailing update
 * is c + (-1 * dot) (gemm_acc with alpha = -1, dense.mojo:54-124). */
#define CHOL_BLOCK 64
int64_t nqo_cholesky_f64(double* a, int64_t n) {
    for (int64_t k0 = 0; k0 < n; k0 += CHOL_BLOCK) {
        int64_t k1 = k0 + CHOL_BLOCK < n ? k0 + CHOL_BLOCK : n;
        for (int64_t j = k0; j < k1; j++) {
            double dot = 0;
            for (int64_t t = k0; t < j; t++) dot += a[j * n + t] * a[j * n + t];
            double s = a[j * n + j] - dot;
            if (!(s > 0)) return j + 1;
            double d = sqrt(s);
            a[j * n + j] = d;
            for (int64_t i = j + 1; i < k1; i++) {
                dot = 0;
                for (int64_t t = k0; t < j; t++) dot += a[i * n + t] * a[j * n + t];
                a[i * n + j] = (a[i * n + j] - dot) / d;
            }
        }
        for (int64_t i = k1; i < n; i++)
            for (int64_t j = k0; j < k1; j++) {
                double dot = 0;
                for (int64_t t = k0; t < j; t++) dot += a[i * n + t] * a[j * n + t];
                a[i * n + j] = (a[i * n + j] - dot) / a[j * n + j];
            }
        for (int64_t i = k1; i < n; i++)
            for (int64_t j = k1; j <= i; j++) {
                double dot = 0;
                for (int64_t t = k0; t < k1; t++) dot += a[i * n + t] * a[j * n + t];
                a[i * n + j] = a[i * n + j] + -1.0 * dot;
            }
    }
    for (int64_t i = 0; i < n; i++)
        for (int64_t j = i + 1; j < n; j++) a[i * n + j] = 0;
    return 0;
}

/* dense.mojo:291-352: X = L^-1 by blocked forward substitution of L X = I:
 * block row k is solved against L's diagonal block (each term subtracted in
 * turn, q ascending, then the division), then subtracted from every row below
 * as c + (-1 * dot over the block). */
void nqo_tri_inv_lower_f64(const double* l, int64_t n, double* x) {
    for (int64_t i = 0; i < n * n; i++) x[i] = 0;
    for (int64_t i = 0; i < n; i++) x[i * n + i] = 1.0;
    for (int64_t k0 = 0; k0 < n; k0 += CHOL_BLOCK) {
        int64_t k1 = k0 + CHOL_BLOCK < n ? k0 + CHOL_BLOCK : n;
        for (int64_t i = k0; i < k1; i++) {
            for (int64_t q = k0; q < i; q++) {
                double f = l[i * n + q];
                for (int64_t j = 0; j < k1; j++) x[i * n + j] = x[i * n + j] - f * x[q * n + j];
            }
            double d = l[i * n + i];
            for (int64_t j = 0; j < k1; j++) x[i * n + j] = x[i * n + j] / d;
        }
        for (int64_t i = k1; i < n; i++)
            for (int64_t j = 0; j < k1; j++) {
                double dot = 0;
                for (int64_t q = k0; q < k1; q++) dot += l[i * n + q] * x[q * n + j];
                x[i * n + j] = x[i * n + j] + -1.0 * dot;
            }
    }
}

static void reverse_f64(double* v, int64_t n) {
    for (int64_t i = 0; i < n / 2; i++) {
        double t = v[i];
        v[i] = v[n - 1 - i];
        v[n - 1 - i] = t;
    }
}

/* dense.mojo:355-363: U upper triangular with U^T U = h^-1, as J chol(J h J)^-1 J
 * (J reverses the indices: on a row-major n x n array, reversing the flat
 * array).  h is consumed.  Returns nqo_cholesky_f64's status. */
int64_t nqo_hinv_upper_f64(double* h, int64_t n, double* u) {
    reverse_f64(h, n * n);
    int64_t rc = nqo_cholesky_f64(h, n);
    if (rc) return rc;
    nqo_tri_inv_lower_f64(h, n, u);
    reverse_f64(u, n * n);
    return 0;
}

/* gptq.mojo:62-150.  w [n, k] fp32, h [k, k] fp64 (consumed) -> codes q [n, k],
 * scales d [n, k/32] (bf16-rounded fp32).  Dead inputs (h_ii == 0): weights
 * zeroed, diagonal 1.  Damping damp_frac * mean(diag).  U in fp64, rounded to
 * fp32; the column loop in fp32, blocks of 128 columns, each row on its own:
 *   at c % 32 == 0 the group's scale from the current weights; the code;
 *   e = (w_c - deq) / U[c,c];  w[c .. block end) -= e * U[c, c .. block end);
 *   after the block  w[block end ..) -= E @ U[block, block end ..)
 * (dense.mojo:54-124 with alpha = -1: the sum over the block's columns in
 * ascending order, then c + (-1 * sum)).  Multiplications and additions are
 * separate roundings here (the file is compiled with -ffp-contract=off), as in
 * the numpy transcription the reference's fixture was written by
 * (tools/quant/gptq_q4_0_reference.py:57-86). */
#define GPTQ_BLOCK 128
int nqo_gptq_q4_0(const float* w, int64_t n, int64_t k, double* h, uint8_t* q, float* d, double damp_frac,
                  int64_t* dead_out, double* damp_out) {
    if (k % Q4_GROUP != 0) return NQO_ESIZE;
    float* ww = (float*)malloc((size_t)(n * k) * sizeof(float));
    double* u64 = (double*)malloc((size_t)(k * k) * sizeof(double));
    float* u = (float*)malloc((size_t)(k * k) * sizeof(float));
    float* err = (float*)malloc((size_t)GPTQ_BLOCK * sizeof(float));
    if (!ww || !u64 || !u || !err) {
        free(ww), free(u64), free(u), free(err);
        return NQO_ESIZE;
    }
    for (int64_t i = 0; i < n * k; i++) ww[i] = w[i];
    int64_t dead = 0;
    double mean = 0;
    for (int64_t i = 0; i < k; i++) {
        if (h[i * k + i] == 0) {
            dead++;
            h[i * k + i] = 1.0;
            for (int64_t r = 0; r < n; r++) ww[r * k + i] = 0;
        }
        mean += h[i * k + i];
    }
    double damp = damp_frac * mean / (double)k;
    for (int64_t i = 0; i < k; i++) h[i * k + i] += damp;
    if (dead_out) *dead_out = dead;
    if (damp_out) *damp_out = damp;
    if (nqo_hinv_upper_f64(h, k, u64)) {
        free(ww), free(u64), free(u), free(err);
        return NQO_ESIZE + 1; /* not positive definite */
    }
    for (int64_t i = 0; i < k * k; i++) u[i] = (float)u64[i];
    int64_t groups = k / Q4_GROUP;
    for (int64_t r = 0; r < n; r++) {
        float* row = ww + r * k;
        for (int64_t i1 = 0; i1 < k; i1 += GPTQ_BLOCK) {
            int64_t i2 = i1 + GPTQ_BLOCK < k ? i1 + GPTQ_BLOCK : k;
            float dg = 0;
            for (int64_t c = i1; c < i2; c++) {
                if (c % Q4_GROUP == 0) {
                    dg = nqo_q4_0_group_scale(row + c);
                    d[r * groups + c / Q4_GROUP] = dg;
                }
                float x = row[c];
                uint8_t code = nqo_q4_0_code(x, dg);
                q[r * k + c] = code;
                float deq = ((float)(int)code - 8.0f) * dg;
                float e = (x - deq) / u[c * k + c];
                for (int64_t j = c; j < i2; j++) {
                    float t = e * u[c * k + j];
                    row[j] = row[j] - t;
                }
                err[c - i1] = e;
            }
            for (int64_t j = i2; j < k; j++) {
                float acc = 0;
                for (int64_t c = i1; c < i2; c++) {
                    float t = err[c - i1] * u[c * k + j];
                    acc = acc + t;
                }
                float t = -1.0f * acc;
                row[j] = row[j] + t;
            }
        }
    }
    free(ww), free(u64), free(u), free(err);
    return NQO_OK;
}

/* gptq.mojo:152-189: tr((W - What) H (W - What)^T) in fp64, What = (q - 8) d, H undamped. */
double nqo_q4_0_objective(const float* w, const uint8_t* q, const float* d, int64_t n, int64_t k, const double* h) {
    int64_t groups = k / Q4_GROUP;
    double* delta = (double*)malloc((size_t)k * sizeof(double));
    double s = 0;
    for (int64_t r = 0; r < n; r++) {
        for (int64_t c = 0; c < k; c++) {
            double deq = ((double)(int)q[r * k + c] - 8.0) * (double)d[r * groups + c / Q4_GROUP];
            delta[c] = (double)w[r * k + c] - deq;
        }
        for (int64_t j = 0; j < k; j++) {
            double acc = 0;
            for (int64_t c = 0; c < k; c++) acc += delta[c] * h[c * k + j];
            s += acc * delta[j];
        }
    }
    free(delta);
    return s;
}

/* hessian.mojo:24-77: H += X^T X in fp64 over the first `rows` rows of x [rows, n] fp32. */
void nqo_hessian_add(double* h, int64_t n, const float* x, int64_t rows) {
    for (int64_t r = 0; r < rows; r++)
        for (int64_t i = 0; i < n; i++) {
            double xi = (double)x[r * n + i];
            if (xi == 0) continue;
            for (int64_t j = 0; j < n; j++) h[i * n + j] += xi * (double)x[r * n + j];
        }
}

/* ======================================================================== */
/* Part 2 — formats the reference does not implement (closed forms)          */
/* ======================================================================== */

/* ReLU as nn/primitives/ops/relu_op.mojo:29-31: x if x > 0 else 0
 * (NaN -> 0, -0.0 -> +0.0). */
static inline float relu_ref(float z) { return z > 0.0f ? z : 0.0f; }

/* int8 weights [N, K], per-output-channel fp32 scales [N], fp32 activations
 * (bf16 inputs are widened exactly by the caller):
 *     y[m, n] = epi( (sum_k x[m,k] * float(w[n,k])) * s[n] + bias[n] )
 * fp32, k ascending — "accumulate, then scale".  bias may be NULL. */
void nqo_w8_forward_f32(const int8_t* w, const float* s, int64_t N, int64_t K, const float* x,
                        int64_t M, const float* bias, int relu, float* y) {
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; k++) acc += x[m * K + k] * (float)w[n * K + k];
            float z = acc * s[n];
            if (bias) z = z + bias[n];
            y[m * N + n] = relu ? relu_ref(z) : z;
        }
    }
}

/* the same in fp64 (the exact value the fp32 paths approximate). */
void nqo_w8_forward_f64(const int8_t* w, const float* s, int64_t N, int64_t K, const float* x,
                        int64_t M, const float* bias, int relu, double* y) {
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; k++) acc += (double)x[m * K + k] * (double)w[n * K + k];
            double z = acc * (double)s[n];
            if (bias) z += (double)bias[n];
            y[m * N + n] = (relu && !(z > 0.0)) ? 0.0 : z;
        }
    }
}

/* per-token (row) absmax int8 quantization, by analogy with the RTN grid
 * (q4_0.mojo:30-32 insists on a division and ties-to-even):
 *     s[m] = absmax(x[m, :]) / 127   (1 where that is 0)
 *     q[m, k] = clip(round_half_even(x[m,k] / s[m]), -127, 127) */
void nqo_quantize_rows_i8(const float* x, int64_t M, int64_t K, int8_t* q, float* s) {
    for (int64_t m = 0; m < M; m++) {
        float amax = 0.0f;
        for (int64_t k = 0; k < K; k++) {
            float a = fabsf(x[m * K + k]);
            if (a > amax) amax = a;
        }
        float sc = amax / 127.0f;
        if (sc == 0.0f) sc = 1.0f;
        s[m] = sc;
        for (int64_t k = 0; k < K; k++) {
            volatile float quot = x[m * K + k] / sc;
            float v = nqo_round_half_even(quot);
            v = v > -127.0f ? v : -127.0f;
            v = v < 127.0f ? v : 127.0f;
            q[m * K + k] = (int8_t)(int)v;
        }
    }
}

/* int8 x int8 -> int32 accumulators, acc[m, n] = sum_k xq[m,k] * w[n,k]
 * (exact in any order: |acc| <= K * 127^2). */
void nqo_w8a8_acc_i32(const int8_t* xq, const int8_t* w, int64_t M, int64_t N, int64_t K,
                      int32_t* acc) {
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            int32_t a = 0;
            for (int64_t k = 0; k < K; k++) a += (int32_t)xq[m * K + k] * (int32_t)w[n * K + k];
            acc[m * N + n] = a;
        }
}

/* the W8A8 epilogue:  y = epi( float(acc) * (sx[m] * sw[n]) + bias[n] ), fp32. */
void nqo_w8a8_epilogue(const int32_t* acc, const float* sx, const float* sw, const float* bias,
                       int relu, int64_t M, int64_t N, float* y) {
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            float z = (float)acc[m * N + n] * (sx[m] * sw[n]);
            if (bias) z = z + bias[n];
            y[m * N + n] = relu ? relu_ref(z) : z;
        }
}

/* uint4 group-wise asymmetric.  Layout (stated here, there is no precedent
 * in the reference beyond Q4_0's own split-half order, which is tied to
 * 32-wide groups):
 *   codes  [N, K/2] bytes, byte i of a row holds element 2i in its LOW nibble
 *          and element 2i+1 in its HIGH nibble (K even);
 *   scales [N, G] fp16 bits, G = ceil(K / group); the last group is ragged
 *          when group does not divide K (K = 960, group = 128: 64 wide);
 *   zps    [N, ceil(G/2)] bytes, byte i holds group 2i (low) and 2i+1 (high).
 *   value(n, k) = (float(q) - float(z[n, k/group])) * fp32(fp16 s[n, k/group]) */
void nqo_w4g_dequantize(const uint8_t* codes, const uint16_t* scales, const uint8_t* zps,
                        int64_t N, int64_t K, int64_t group, float* out) {
    int64_t G = (K + group - 1) / group;
    int64_t zrow = (G + 1) / 2;
    for (int64_t n = 0; n < N; n++)
        for (int64_t k = 0; k < K; k++) {
            uint8_t byte = codes[n * (K / 2) + k / 2];
            int q = (k & 1) ? (byte >> 4) : (byte & 0xF);
            int64_t g = k / group;
            uint8_t zb = zps[n * zrow + g / 2];
            int z = (g & 1) ? (zb >> 4) : (zb & 0xF);
            out[n * K + k] = ((float)q - (float)z) * nqo_f16_value(scales[n * G + g]);
        }
}

/* OCP fp8 e4m3fn (gfx950's native flavour): 1-4-3, bias 7, no infinities,
 * S.1111.111 is NaN, max finite 448. */
float nqo_e4m3_decode(uint8_t v) {
    int sign = v >> 7;
    int e = (v >> 3) & 0xF;
    int m = v & 7;
    float r;
    if (e == 15 && m == 7) return bits_f32(0x7FC00000u);
    if (e == 0)
        r = ldexpf((float)m, -9); /* subnormal: m/8 * 2^-6 */
    else
        r = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return sign ? -r : r;
}

/* fp32 -> e4m3fn, round to nearest even, SATURATING to +-448 (NaN -> 0x7F). */
uint8_t nqo_e4m3_encode(float x) {
    uint32_t u = f32_bits(x);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    float a = fabsf(x);
    if (a != a) return (uint8_t)(sign | 0x7F);
    if (a >= 448.0f) {
        /* everything above the largest finite saturates; 448 is exact */
        return (uint8_t)(sign | 0x7E);
    }
    if (a < 0.0009765625f) { /* < 2^-10: rounds to 0 (2^-10 is a tie to even = 0) */
        return sign;
    }
    int e;
    float fr = frexpf(a, &e); /* a = fr * 2^e, fr in [0.5, 1) */
    int E = e - 1;            /* a = (2 fr) * 2^E, 2fr in [1, 2) */
    float scaled;
    int ebits;
    if (E < -6) { /* subnormal: units of 2^-9 */
        scaled = ldexpf(a, 9);
        ebits = 0;
    } else {
        scaled = ldexpf(fr * 2.0f, 3); /* [8, 16) in units of 1/8 */
        ebits = E + 7;
    }
    float r = nqo_round_half_even(scaled);
    int mi = (int)r;
    int out;
    if (ebits == 0) {
        out = mi; /* 8 carries into exponent 1: correct */
    } else {
        out = ((ebits - 1) << 3) + mi; /* mi in [8, 16] includes the hidden bit */
    }
    if (out > 0x7E) out = 0x7E;
    return (uint8_t)(sign | out);
}

/* fp8 x fp8:  y[m, n] = bf16( (sum_k a[m,k] * b[n,k]) * (sa * sb) ), the sum
 * in fp64 here (each product is exact in fp32; the hardware accumulates in
 * fp32, so the fp64 sum is the value to approximate).  out_bf16 may be NULL;
 * y64 gets the unrounded value. */
void nqo_fp8_forward_f64(const uint8_t* a, const uint8_t* b, int64_t M, int64_t N, int64_t K,
                         float sa, float sb, double* y64, uint16_t* out_bf16) {
    float lut[256];
    for (int i = 0; i < 256; i++) lut[i] = nqo_e4m3_decode((uint8_t)i);
    double sc = (double)(sa * sb);
    for (int64_t m = 0; m < M; m++)
        for (int64_t n = 0; n < N; n++) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; k++)
                acc += (double)lut[a[m * K + k]] * (double)lut[b[n * K + k]];
            double v = acc * sc;
            if (y64) y64[m * N + n] = v;
            if (out_bf16) out_bf16[m * N + n] = nqo_f32_to_bf16_bits((float)v);
        }
}

/* fp8 weights, decoded to fp32 [N, K] (exact). */
void nqo_e4m3_dequantize(const uint8_t* w, int64_t n, float* out) {
    for (int64_t i = 0; i < n; i++) out[i] = nqo_e4m3_decode(w[i]);
}

/* the dequantize-then-GEMM baseline for any format already expanded to an
 * fp32 [N, K] weight: the same two steps QLinear.forward["cpu"] takes
 * (qlinear.mojo:416-426) with the expansion done by the caller. */
void nqo_dense_forward_cpu(const float* w, int64_t N, int64_t K, const float* x, int64_t M,
                           float* y) {
    nqo_gemm_cpu(0, 1, M, N, K, 1.0f, x, K, w, K, 0.0f, y, N);
}

/* array forms of the scalar routines, for the numpy front end */
void nqo_e4m3_encode_array(const float* x, int64_t n, uint8_t* out) {
    for (int64_t i = 0; i < n; i++) out[i] = nqo_e4m3_encode(x[i]);
}
void nqo_f16_bits_array(const float* x, int64_t n, uint16_t* out) {
    for (int64_t i = 0; i < n; i++) out[i] = nqo_f16_bits(x[i]);
}
void nqo_f16_value_array(const uint16_t* h, int64_t n, float* out) {
    for (int64_t i = 0; i < n; i++) out[i] = nqo_f16_value(h[i]);
}

/* The reference's CPU forward (qlinear.mojo:416-426: a FRESH dequantize to an
 * fp32 [OUT, IN] scratch, then the serial gemm_cpu) restated for an int8
 * per-channel weight: deq[n,k] = float(w[n,k]) * s[n], y = x @ deq^T (+ bias).
 * Used as the single-core CPU baseline of the W8 workloads. */
int nqo_w8_qlinear_forward_cpu(const int8_t* w, const float* s, int64_t N, int64_t K, const float* x,
                               int64_t M, const float* bias, float* y) {
    float* deq = (float*)malloc(sizeof(float) * (size_t)(N * K));
    if (!deq) return NQO_ENOMEM;
    for (int64_t n = 0; n < N; n++)
        for (int64_t k = 0; k < K; k++) deq[n * K + k] = (float)w[n * K + k] * s[n];
    nqo_gemm_cpu(0, 1, M, N, K, 1.0f, x, K, deq, K, 0.0f, y, N);
    if (bias)
        for (int64_t m = 0; m < M; m++)
            for (int64_t n = 0; n < N; n++) y[m * N + n] += bias[n];
    free(deq);
    return NQO_OK;
}

/* The reference's CPU forward (qlinear.mojo:416-426: a FRESH dequantize to an fp32 [OUT, IN] scratch, then the
 * serial gemm_cpu) restated for an e4m3 weight under e4m3 activations with per-tensor scales: deq[n,k] =
 * decode(w[n,k]) * sb, x decoded and scaled by sa, y = x @ deq^T in fp32, then rounded to bf16 (config 5's
 * output type; out_bf16 may be NULL).  Used as the single-core CPU baseline of the fp8 workloads; pinned against
 * nqo_fp8_forward_f64 and exact small-integer products in tests/test_oracle_ext.py. */
int nqo_fp8_qlinear_forward_cpu(const uint8_t* w, float sb, int64_t N, int64_t K, const uint8_t* a, float sa,
                                int64_t M, float* y, uint16_t* out_bf16) {
    float* deq = (float*)malloc(sizeof(float) * (size_t)(N * K));
    float* xs = (float*)malloc(sizeof(float) * (size_t)(M * K));
    if (!deq || !xs) {
        free(deq);
        free(xs);
        return NQO_ENOMEM;
    }
    for (int64_t i = 0; i < N * K; i++) deq[i] = nqo_e4m3_decode(w[i]) * sb;
    for (int64_t i = 0; i < M * K; i++) xs[i] = nqo_e4m3_decode(a[i]) * sa;
    nqo_gemm_cpu(0, 1, M, N, K, 1.0f, xs, K, deq, K, 0.0f, y, N);
    if (out_bf16)
        for (int64_t i = 0; i < M * N; i++) out_bf16[i] = nqo_f32_to_bf16_bits(y[i]);
    free(deq);
    free(xs);
    return NQO_OK;
}
