// GPTQ onto the Q4_0 grid, on the device (load time, off the forward path):
//   the calibration Hessian H += X^T X in fp64      (noeira/nn/quant/hessian.mojo:41-77)
//   U, upper triangular with U^T U = H^-1, in fp64  (noeira/nn/quant/dense.mojo:204-363)
//   the column loop, in fp32, one wavefront per row (noeira/nn/quant/gptq.mojo:62-150)
//   tr((W - What) H (W - What)^T) in fp64           (noeira/nn/quant/gptq.mojo:152-189)
//
// Order of operations.  GPTQ's codes depend on the last bit of U and of every
// update (a value on a rounding boundary flips a code, and the flip feeds the rest
// of the row), so every sum here runs in one stated order with multiplication and
// addition rounded separately (__dmul_rn / __dadd_rn, __fmul_rn / __fadd_rn: the
// compiler may not contract them):
//   Cholesky, blocked by 64 columns: in the diagonal block and the panel below it
//     a[i][j] = (a[i][j] - sum_{t = block start}^{j-1} a[i][t] a[j][t]) / a[j][j]
//   (the sum ascending from 0, then one subtraction), and the trailing matrix
//     a[i][j] = a[i][j] + (-1 * sum_{t in block} a[i][t] a[j][t]);
//   the inverse of the factor by forward substitution of L X = I, 64 rows at a time:
//     x[i][j] = (x[i][j] - l[i][q] x[q][j], q ascending over the block) / l[i][i], then
//     x[i][j] = x[i][j] + (-1 * sum_{q in block} l[i][q] x[q][j]) for the rows below;
//   the Hessian adds one row of X at a time in ascending order (the products of two
//     fp32 values are exact in fp64, so only the additions round);
//   the column loop as gptq.mojo writes it, and the block's lazy update as
//     w[j] = w[j] + (-1 * sum_{c in block} e[c] U[c][j]), c ascending.
// A CPU restatement that follows the same orders reproduces the codes bit for bit.
#include <hip/hip_fp16.h>

#include <mutex>

#include "nq_common.h"

namespace nq {

namespace {

constexpr int CB = 64;           // Cholesky / inverse block
constexpr int GPTQ_BLOCK = 128;  // gptq.mojo:49
constexpr int ROWS_PER_WG = 4;   // wavefronts (rows of W) per workgroup in the column loop

// ---------------------------------------------------------------------------
// C[M, N] = C + alpha * (A[M, K] @ op(B)), fp64, row-major with row strides.
// TB: B is [N, K] (C += alpha A B^T).  64 x 64 tile per workgroup, 4 x 4 per thread,
// K through LDS in chunks of 16; each output's sum runs over k ascending from 0.
// lower: tiles wholly above C's diagonal are skipped.
// ---------------------------------------------------------------------------
template <bool TB>
__global__ __launch_bounds__(256) void dgemm_kernel(int M, int N, int K, double alpha, const double* __restrict__ A,
                                                    int64_t lda, const double* __restrict__ B, int64_t ldb,
                                                    double* __restrict__ C, int64_t ldc, int lower) {
    __shared__ double As[16][64 + 1];
    __shared__ double Bs[16][64 + 1];
    const int i0 = blockIdx.y * 64, j0 = blockIdx.x * 64;
    if (lower && j0 > min(i0 + 64, M) - 1) return;
    const int tid = threadIdx.x;
    const int ti = tid / 16, tj = tid % 16;  // rows ti*4.., cols tj + 16*b (strided: conflict-free LDS reads)
    double acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = 0.0;
    for (int k0 = 0; k0 < K; k0 += 16) {
        // A tile: 64 rows x 16 k; thread loads 4 values
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int e = tid + 256 * t;       // 0..1023
            const int r = e / 16, kk = e % 16;  // consecutive threads along k (contiguous in A)
            const int gi = i0 + r, gk = k0 + kk;
            As[kk][r] = (gi < M && gk < K) ? A[(int64_t)gi * lda + gk] : 0.0;
        }
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int e = tid + 256 * t;
            if (TB) {
                const int c = e / 16, kk = e % 16;
                const int gj = j0 + c, gk = k0 + kk;
                Bs[kk][c] = (gj < N && gk < K) ? B[(int64_t)gj * ldb + gk] : 0.0;
            } else {
                const int kk = e / 64, c = e % 64;
                const int gj = j0 + c, gk = k0 + kk;
                Bs[kk][c] = (gj < N && gk < K) ? B[(int64_t)gk * ldb + gj] : 0.0;
            }
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; kk++) {
            double av[4], bv[4];
#pragma unroll
            for (int a = 0; a < 4; a++) av[a] = As[kk][ti * 4 + a];
#pragma unroll
            for (int b = 0; b < 4; b++) bv[b] = Bs[kk][tj + 16 * b];
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++) acc[a][b] = __dadd_rn(acc[a][b], __dmul_rn(av[a], bv[b]));
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int gi = i0 + ti * 4 + a, gj = j0 + tj + 16 * b;
            if (gi < M && gj < N) {
                double* c = C + (int64_t)gi * ldc + gj;
                *c = __dadd_rn(*c, __dmul_rn(alpha, acc[a][b]));
            }
        }
}

int32_t dgemm(bool tb, int M, int N, int K, double alpha, const double* A, int64_t lda, const double* B, int64_t ldb,
              double* C, int64_t ldc, bool lower, hipStream_t s) {
    if (M <= 0 || N <= 0 || K <= 0) return NQ_OK;
    dim3 grid((N + 63) / 64, (M + 63) / 64);
    if (tb)
        hipLaunchKernelGGL(dgemm_kernel<true>, grid, dim3(256), 0, s, M, N, K, alpha, A, lda, B, ldb, C, ldc, (int)lower);
    else
        hipLaunchKernelGGL(dgemm_kernel<false>, grid, dim3(256), 0, s, M, N, K, alpha, A, lda, B, ldb, C, ldc, (int)lower);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// ---------------------------------------------------------------------------
// H[n, n] += X^T X over `rows` rows of X [rows, n] (fp32 or bf16), fp64.  Each thread
// owns a 4 x 4 patch of H and adds the rows in ascending order.
// ---------------------------------------------------------------------------
template <bool BF16>
__global__ __launch_bounds__(256) void hessian_add_kernel(double* __restrict__ H, int n, const void* __restrict__ xv,
                                                          int rows) {
    __shared__ double Xi[16][64 + 1];
    __shared__ double Xj[16][64 + 1];
    const int i0 = blockIdx.y * 64, j0 = blockIdx.x * 64;
    const int tid = threadIdx.x, ti = tid / 16, tj = tid % 16;
    auto ld = [&](int r, int c) -> double {
        if (r >= rows || c >= n) return 0.0;
        if (BF16)
            return (double)__uint_as_float((uint32_t)reinterpret_cast<const uint16_t*>(xv)[(int64_t)r * n + c] << 16);
        return (double)reinterpret_cast<const float*>(xv)[(int64_t)r * n + c];
    };
    double acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int gi = i0 + ti * 4 + a, gj = j0 + tj + 16 * b;
            acc[a][b] = (gi < n && gj < n) ? H[(int64_t)gi * n + gj] : 0.0;
        }
    for (int r0 = 0; r0 < rows; r0 += 16) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int e = tid + 256 * t;
            const int rr = e / 64, c = e % 64;
            Xi[rr][c] = ld(r0 + rr, i0 + c);
            Xj[rr][c] = ld(r0 + rr, j0 + c);
        }
        __syncthreads();
#pragma unroll
        for (int rr = 0; rr < 16; rr++) {
            double av[4], bv[4];
#pragma unroll
            for (int a = 0; a < 4; a++) av[a] = Xi[rr][ti * 4 + a];
#pragma unroll
            for (int b = 0; b < 4; b++) bv[b] = Xj[rr][tj + 16 * b];
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++) acc[a][b] = __dadd_rn(acc[a][b], __dmul_rn(av[a], bv[b]));
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const int gi = i0 + ti * 4 + a, gj = j0 + tj + 16 * b;
            if (gi < n && gj < n) H[(int64_t)gi * n + gj] = acc[a][b];
        }
}

// ---------------------------------------------------------------------------
// Cholesky pieces (dense.mojo:212-289, blocked by CB)
// ---------------------------------------------------------------------------
// the diagonal block a[k0:k0+bs, k0:k0+bs], one workgroup of 64 threads, thread i = row i
__global__ __launch_bounds__(64) void chol_diag_kernel(double* __restrict__ a, int n, int k0, int bs, int* status) {
    __shared__ double L[CB][CB + 1];
    const int i = threadIdx.x;
    for (int j = 0; j < bs; j++)
        if (i < bs) L[i][j] = a[(int64_t)(k0 + i) * n + k0 + j];
    __syncthreads();
    for (int j = 0; j < bs; j++) {
        if (i == j) {
            double dot = 0.0;
            for (int t = 0; t < j; t++) dot = __dadd_rn(dot, __dmul_rn(L[j][t], L[j][t]));
            double s = __dsub_rn(L[j][j], dot);
            if (!(s > 0.0)) {
                atomicMin(status, k0 + j);  // the first non-positive pivot
                s = 1.0;
            }
            L[j][j] = sqrt(s);
        }
        __syncthreads();
        if (i > j && i < bs) {
            double dot = 0.0;
            for (int t = 0; t < j; t++) dot = __dadd_rn(dot, __dmul_rn(L[i][t], L[j][t]));
            L[i][j] = __ddiv_rn(__dsub_rn(L[i][j], dot), L[j][j]);
        }
        __syncthreads();
    }
    for (int j = 0; j < bs; j++)
        if (i < bs) a[(int64_t)(k0 + i) * n + k0 + j] = L[i][j];
}

// the panel below it: rows k1 .. n-1, one thread per row, the row's bs values in registers
__global__ __launch_bounds__(64) void chol_panel_kernel(double* __restrict__ a, int n, int k0, int bs) {
    __shared__ double L[CB][CB + 1];
    const int k1 = k0 + bs;
    for (int e = threadIdx.x; e < CB * CB; e += 64) {
        const int r = e / CB, c = e % CB;
        L[r][c] = (r < bs && c < bs) ? a[(int64_t)(k0 + r) * n + k0 + c] : (r == c ? 1.0 : 0.0);
    }
    __syncthreads();
    const int i = k1 + blockIdx.x * 64 + threadIdx.x;
    if (i >= n) return;
    double r[CB];
#pragma unroll
    for (int j = 0; j < CB; j++) r[j] = j < bs ? a[(int64_t)i * n + k0 + j] : 0.0;
#pragma unroll
    for (int j = 0; j < CB; j++) {
        double dot = 0.0;
#pragma unroll
        for (int t = 0; t < j; t++) dot = __dadd_rn(dot, __dmul_rn(r[t], L[j][t]));
        r[j] = __ddiv_rn(__dsub_rn(r[j], dot), L[j][j]);
    }
#pragma unroll
    for (int j = 0; j < CB; j++)
        if (j < bs) a[(int64_t)i * n + k0 + j] = r[j];
}

__global__ __launch_bounds__(256) void zero_upper_kernel(double* __restrict__ a, int n) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (int64_t)n * n) return;
    if (e % n > e / n) a[e] = 0.0;
}

__global__ __launch_bounds__(256) void identity_kernel(double* __restrict__ x, int n) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= (int64_t)n * n) return;
    x[e] = (e % n == e / n) ? 1.0 : 0.0;
}

// J M J on a row-major n x n array: the flat array reversed (dense.mojo:204-209)
__global__ __launch_bounds__(256) void reverse_kernel(double* __restrict__ v, int64_t count) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= count / 2) return;
    const double t = v[e];
    v[e] = v[count - 1 - e];
    v[count - 1 - e] = t;
}

// X's block row k0 .. k0+bs, columns 0 .. k1-1, solved against L's diagonal block
// (dense.mojo:309-333): one thread per column, the column's bs values in registers
__global__ __launch_bounds__(64) void triinv_diag_kernel(const double* __restrict__ l, double* __restrict__ x, int n,
                                                         int k0, int bs) {
    __shared__ double L[CB][CB + 1];
    for (int e = threadIdx.x; e < CB * CB; e += 64) {
        const int r = e / CB, c = e % CB;
        L[r][c] = (r < bs && c < bs) ? l[(int64_t)(k0 + r) * n + k0 + c] : (r == c ? 1.0 : 0.0);
    }
    __syncthreads();
    const int j = blockIdx.x * 64 + threadIdx.x;
    if (j >= k0 + bs) return;
    double v[CB];
#pragma unroll
    for (int i = 0; i < CB; i++) v[i] = i < bs ? x[(int64_t)(k0 + i) * n + j] : 0.0;
#pragma unroll
    for (int i = 0; i < CB; i++) {
        double t = v[i];
#pragma unroll
        for (int q = 0; q < i; q++) t = __dsub_rn(t, __dmul_rn(L[i][q], v[q]));
        v[i] = __ddiv_rn(t, L[i][i]);
    }
#pragma unroll
    for (int i = 0; i < CB; i++)
        if (i < bs) x[(int64_t)(k0 + i) * n + j] = v[i];
}

__global__ __launch_bounds__(256) void f64_to_f32_kernel(const double* __restrict__ src, float* __restrict__ dst,
                                                         int64_t count) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < count) dst[e] = (float)src[e];
}

inline unsigned blocks_for(int64_t count, int per = 256) { return (unsigned)((count + per - 1) / per); }

}  // namespace

// h (n x n fp64 on the device, consumed) -> u = upper Cholesky factor of h^-1 (dense.mojo:355-363).
// status_dev: an int the caller set to INT_MAX; on return the first non-positive pivot, if any.
int32_t launch_hinv_upper_f64(double* h, int n, double* u, int* status_dev, hipStream_t s) {
    const int64_t nn = (int64_t)n * n;
    hipLaunchKernelGGL(reverse_kernel, dim3(blocks_for(nn / 2 + 1)), dim3(256), 0, s, h, nn);
    for (int k0 = 0; k0 < n; k0 += CB) {
        const int bs = std::min(CB, n - k0), k1 = k0 + bs;
        hipLaunchKernelGGL(chol_diag_kernel, dim3(1), dim3(64), 0, s, h, n, k0, bs, status_dev);
        if (k1 == n) break;
        const int m = n - k1;
        hipLaunchKernelGGL(chol_panel_kernel, dim3(blocks_for(m, 64)), dim3(64), 0, s, h, n, k0, bs);
        int32_t rc = dgemm(true, m, m, bs, -1.0, h + (int64_t)k1 * n + k0, n, h + (int64_t)k1 * n + k0, n,
                           h + (int64_t)k1 * n + k1, n, true, s);
        if (rc) return rc;
    }
    hipLaunchKernelGGL(zero_upper_kernel, dim3(blocks_for(nn)), dim3(256), 0, s, h, n);
    hipLaunchKernelGGL(identity_kernel, dim3(blocks_for(nn)), dim3(256), 0, s, u, n);
    for (int k0 = 0; k0 < n; k0 += CB) {
        const int bs = std::min(CB, n - k0), k1 = k0 + bs;
        hipLaunchKernelGGL(triinv_diag_kernel, dim3(blocks_for(k1, 64)), dim3(64), 0, s, h, u, n, k0, bs);
        if (k1 < n) {
            int32_t rc = dgemm(false, n - k1, k1, bs, -1.0, h + (int64_t)k1 * n + k0, n, u + (int64_t)k0 * n, n,
                               u + (int64_t)k1 * n, n, false, s);
            if (rc) return rc;
        }
    }
    hipLaunchKernelGGL(reverse_kernel, dim3(blocks_for(nn / 2 + 1)), dim3(256), 0, s, u, nn);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

// ---------------------------------------------------------------------------
// The same factorization for callers that cannot allocate (code under HIP graph capture, serving loops,
// harnesses that forbid it): device in, device out, the working copy of h in a file-scope device array
// instead of a hipMalloc'd one.  Every call on a GPU shares that GPU's array: calls that overlap on one
// GPU race.  Nothing of the array needs to start at zero (the copy of h overwrites all n * n values used).
// ---------------------------------------------------------------------------
constexpr int HINV_DEV_MAX_N = 1024;                                               // 8 MiB of fp64
static __device__ __align__(256) double scratch[HINV_DEV_MAX_N * HINV_DEV_MAX_N];  // (host code: a stand-in, not an address)
constexpr int MAX_DEVICES = 64;
static double* g_scratch_ptr[MAX_DEVICES];  // the array's address on each device, looked up once per device
static std::mutex g_scratch_mutex;

// the device address of `scratch` on the current device
static int32_t scratch_address(double** out) {
    int dev = -1;
    NQ_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return fail(NQ_ERR_UNSUPPORTED, "hinv_upper_f64_dev: device index out of range");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        double* ptr = nullptr;
        NQ_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return NQ_OK;
}

__global__ __launch_bounds__(256) void copy_f64_kernel(const double* __restrict__ src, double* __restrict__ dst, int64_t count,
                                                       int* __restrict__ pivot) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e == 0) *pivot = 0x7FFFFFFF;  // (a fill kernel, not a memset: a caller may capture this)
    if (e < count) dst[e] = src[e];
}

int32_t run_hinv_upper_f64_dev(const double* h_dev, int n, double* u_dev, int* pivot_dev, hipStream_t s) {
    double* work = nullptr;
    int32_t rc = scratch_address(&work);
    if (rc) return rc;
    const int64_t nn = (int64_t)n * n;
    hipLaunchKernelGGL(copy_f64_kernel, dim3(blocks_for(nn)), dim3(256), 0, s, h_dev, work, nn, pivot_dev);
    NQ_HIP(hipGetLastError());
    return launch_hinv_upper_f64(work, n, u_dev, pivot_dev, s);
}

int32_t hinv_dev_max_n() { return HINV_DEV_MAX_N; }

// Set-up: looks the scratch array's address up for the current device, so that the first call of the entry point
// above - which may stand inside a stream capture - finds it known.  Called where a layer or a Hessian is created.
void hinv_dev_setup() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return;  // (the entry point reports it)
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev]) return;
    double* ptr = nullptr;
    if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) == hipSuccess) g_scratch_ptr[dev] = ptr;
}

int32_t launch_hessian_add(double* H, int n, const void* x, int32_t x_dtype, int rows, hipStream_t s) {
    if (rows <= 0) return NQ_OK;
    dim3 grid((n + 63) / 64, (n + 63) / 64);
    if (x_dtype == NQ_DT_BF16)
        hipLaunchKernelGGL(hessian_add_kernel<true>, grid, dim3(256), 0, s, H, n, x, rows);
    else
        hipLaunchKernelGGL(hessian_add_kernel<false>, grid, dim3(256), 0, s, H, n, x, rows);
    NQ_HIP(hipGetLastError());
    return NQ_OK;
}

namespace {

// ---------------------------------------------------------------------------
// gptq.mojo:88-101: dead inputs and the damping.  One thread: the mean of the diagonal is
// summed in ascending order.  stats[0] = dead count, stats[1] = damp (as a double's bits).
// ---------------------------------------------------------------------------
__global__ void gptq_prepare_kernel(double* __restrict__ h, int k, double damp_frac, uint8_t* __restrict__ dead_flags,
                                    double* __restrict__ stats) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    double mean = 0.0;
    int dead = 0;
    for (int i = 0; i < k; i++) {
        double* dptr = h + (int64_t)i * k + i;
        const bool is_dead = *dptr == 0.0;
        dead_flags[i] = is_dead;
        if (is_dead) {
            dead++;
            *dptr = 1.0;
        }
        mean = __dadd_rn(mean, *dptr);
    }
    const double damp = __ddiv_rn(__dmul_rn(damp_frac, mean), (double)k);
    for (int i = 0; i < k; i++) {
        double* dptr = h + (int64_t)i * k + i;
        *dptr = __dadd_rn(*dptr, damp);
    }
    stats[0] = (double)dead;
    stats[1] = damp;
}

__global__ __launch_bounds__(256) void gptq_zero_dead_kernel(float* __restrict__ w, int64_t n, int k,
                                                             const uint8_t* __restrict__ dead_flags) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n * k) return;
    if (dead_flags[e % k]) w[e] = 0.0f;
}

__device__ __forceinline__ float bf16_round_f(float x) {
    uint32_t bits = __float_as_uint(x);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return __uint_as_float(0x7FC00000u);
    uint32_t bias = 0x7FFFu + ((bits >> 16) & 1u);
    return __uint_as_float((bits + bias) & 0xFFFF0000u);
}

// ---------------------------------------------------------------------------
// The column loop (gptq.mojo:112-149).  One wavefront per row of W: a block's 128
// columns live in two registers per lane (columns lane and 64 + lane of the block),
// the block of U in LDS shared by the workgroup's rows.  Per column c: at a group
// start the group's scale from the current values (the first element of largest
// magnitude, found by a butterfly over the group's 32 lanes); the code; the error e;
// every lane holding a column >= c subtracts e * U[c][column].  After the block the
// rest of the row takes w[j] += -1 * sum_c e[c] U[c][j], 64 columns per pass.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(64 * ROWS_PER_WG) void gptq_rows_kernel(float* __restrict__ w, int n, int k,
                                                                      const float* __restrict__ u,
                                                                      uint8_t* __restrict__ q, float* __restrict__ d) {
    extern __shared__ float lds[];
    float* U = lds;                                 // [128][128]
    float* E = lds + GPTQ_BLOCK * GPTQ_BLOCK;       // [ROWS_PER_WG][128]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = blockIdx.x * ROWS_PER_WG + wave;
    const bool live = r < n;
    const int groups = k / Q4_GROUP;
    float* row = w + (int64_t)(live ? r : 0) * k;
    float* err = E + wave * GPTQ_BLOCK;
    for (int i1 = 0; i1 < k; i1 += GPTQ_BLOCK) {
        const int i2 = min(i1 + GPTQ_BLOCK, k), bs = i2 - i1;
        __syncthreads();  // the previous block's U is no longer read
        for (int e = threadIdx.x; e < GPTQ_BLOCK * GPTQ_BLOCK; e += 64 * ROWS_PER_WG) {
            const int rr = e / GPTQ_BLOCK, cc = e % GPTQ_BLOCK;
            U[e] = (rr < bs && cc < bs) ? u[(int64_t)(i1 + rr) * k + i1 + cc] : 0.0f;
        }
        __syncthreads();
        if (live) {
            float v0 = lane < bs ? row[i1 + lane] : 0.0f;
            float v1 = 64 + lane < bs ? row[i1 + 64 + lane] : 0.0f;
            float e0 = 0.0f, e1 = 0.0f, dg = 0.0f;
            int code0 = 8, code1 = 8;
            for (int c = 0; c < bs; c++) {
                if (c % Q4_GROUP == 0) {
                    // q4_0_group_scale (q4_0.mojo:97-112) over columns c .. c+31 = 32 consecutive lanes
                    float bv = c < 64 ? v0 : v1;
                    float ba = fabsf(bv);
                    int bi = lane;
#pragma unroll
                    for (int off = 16; off >= 1; off >>= 1) {
                        const float ov = __shfl_xor(bv, off), oa = __shfl_xor(ba, off);
                        const int oi = __shfl_xor(bi, off);
                        if (oa > ba || (oa == ba && oi < bi)) bv = ov, ba = oa, bi = oi;
                    }
                    const float best = __shfl(bv, c & 32);  // the group's half of the wavefront
                    dg = __fdiv_rn(best, -8.0f);
                    if (dg == 0.0f) dg = 1e-8f;
                    dg = bf16_round_f(dg);
                    if (lane == 0) d[(int64_t)r * groups + (i1 + c) / Q4_GROUP] = dg;
                }
                const float x = __shfl(c < 64 ? v0 : v1, c & 63);
                // q4_0_code (q4_0.mojo:115-121): a true division, ties to even, clip
                float t = rintf(__fdiv_rn(x, dg)) + 8.0f;
                t = t > 0.0f ? t : 0.0f;
                t = t < 15.0f ? t : 15.0f;
                const int code = (int)t;
                const float deq = __fmul_rn((float)code - 8.0f, dg);
                const float e = __fdiv_rn(__fsub_rn(x, deq), U[c * GPTQ_BLOCK + c]);
                if (lane >= c) v0 = __fsub_rn(v0, __fmul_rn(e, U[c * GPTQ_BLOCK + lane]));
                if (64 + lane >= c) v1 = __fsub_rn(v1, __fmul_rn(e, U[c * GPTQ_BLOCK + 64 + lane]));
                if (lane == (c & 63)) {
                    if (c < 64)
                        code0 = code, e0 = e;
                    else
                        code1 = code, e1 = e;
                }
            }
            if (lane < bs) q[(int64_t)r * k + i1 + lane] = (uint8_t)code0;
            if (64 + lane < bs) q[(int64_t)r * k + i1 + 64 + lane] = (uint8_t)code1;
            err[lane] = e0;
            err[64 + lane] = e1;
        }
        // err is this wavefront's own: LDS operations of a wavefront complete in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (live) {
            for (int j0 = i2; j0 < k; j0 += 64) {
                const int j = j0 + lane;
                if (j < k) {
                    float acc = 0.0f;
                    const float* uc = u + (int64_t)i1 * k + j;
                    for (int c = 0; c < bs; c++) acc = __fadd_rn(acc, __fmul_rn(err[c], uc[(int64_t)c * k]));
                    row[j] = __fadd_rn(row[j], __fmul_rn(-1.0f, acc));
                }
            }
        }
    }
}

// codes [n, k] + scales [n, k/32] -> Q4_0 blocks (q4_0.mojo:157-178), one thread per group
__global__ __launch_bounds__(256) void q4_0_pack_kernel(const uint8_t* __restrict__ q, const float* __restrict__ d,
                                                        uint8_t* __restrict__ blocks, int64_t ngroups) {
    const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (g >= ngroups) return;
    const uint8_t* c = q + g * Q4_GROUP;
    uint16_t* dst = reinterpret_cast<uint16_t*>(blocks + g * Q4_BLOCK);
    dst[0] = __half_as_ushort(__float2half_rn(d[g]));
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t b0 = c[2 * i] | (c[2 * i + 16] << 4);
        const uint32_t b1 = c[2 * i + 1] | (c[2 * i + 17] << 4);
        dst[1 + i] = (uint16_t)(b0 | (b1 << 8));
    }
}

__global__ __launch_bounds__(256) void delta_kernel(const float* __restrict__ w, const float* __restrict__ deq,
                                                    double* __restrict__ delta, int64_t count) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e < count) delta[e] = (double)w[e] - (double)deq[e];
}

// partial[r] = sum_j dh[r][j] * delta[r][j], a fixed-order tree per row
__global__ __launch_bounds__(256) void rowdot_kernel(const double* __restrict__ dh, const double* __restrict__ delta,
                                                     double* __restrict__ partial, int k) {
    __shared__ double red[256];
    const int64_t base = (int64_t)blockIdx.x * k;
    double s = 0.0;
    for (int j = threadIdx.x; j < k; j += 256) s += dh[base + j] * delta[base + j];
    red[threadIdx.x] = s;
    __syncthreads();
    for (int off = 128; off >= 1; off >>= 1) {
        if ((int)threadIdx.x < off) red[threadIdx.x] += red[threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x == 0) partial[blockIdx.x] = red[0];
}

}  // namespace

// w_dev [n, k] fp32 (overwritten: it is the loop's working copy), h_dev [k, k] fp64 (consumed)
// -> blocks_dev (Q4_0, n * k/32 * 18 bytes); stats_host[0] = dead inputs, [1] = damping.
// Synchronizes the stream.  Returns NQ_ERR_INVALID when the damped Hessian is not positive definite.
int32_t run_gptq_q4_0(float* w_dev, int64_t n, int k, double* h_dev, double damp_frac, uint8_t* blocks_dev,
                      double* stats_host, hipStream_t s) {
    const int64_t kk = (int64_t)k * k;
    const int64_t ngroups = n * (k / Q4_GROUP);
    double* u64 = nullptr;
    float* u = nullptr;
    uint8_t* q = nullptr;
    float* d = nullptr;
    uint8_t* dead = nullptr;
    double* stats = nullptr;
    int* status = nullptr;
    auto cleanup = [&]() {
        (void)hipFree(u64), (void)hipFree(u), (void)hipFree(q), (void)hipFree(d), (void)hipFree(dead);
        (void)hipFree(stats), (void)hipFree(status);
    };
    hipError_t e = hipMalloc((void**)&u64, (size_t)kk * 8);
    if (e == hipSuccess) e = hipMalloc((void**)&u, (size_t)kk * 4);
    if (e == hipSuccess) e = hipMalloc((void**)&q, (size_t)(n * k) + 16);
    if (e == hipSuccess) e = hipMalloc((void**)&d, (size_t)ngroups * 4 + 16);
    if (e == hipSuccess) e = hipMalloc((void**)&dead, (size_t)k + 16);
    if (e == hipSuccess) e = hipMalloc((void**)&stats, 16);
    if (e == hipSuccess) e = hipMalloc((void**)&status, 4);
    if (e != hipSuccess) {
        cleanup();
        return fail_hip(e, "gptq_q4_0 alloc");
    }
    const int big = 0x7FFFFFFF;
    int32_t rc = NQ_OK;
    e = hipMemcpyAsync(status, &big, 4, hipMemcpyHostToDevice, s);
    if (e == hipSuccess) {
        hipLaunchKernelGGL(gptq_prepare_kernel, dim3(1), dim3(64), 0, s, h_dev, k, damp_frac, dead, stats);
        hipLaunchKernelGGL(gptq_zero_dead_kernel, dim3(blocks_for(n * k)), dim3(256), 0, s, w_dev, n, k, dead);
        rc = launch_hinv_upper_f64(h_dev, k, u64, status, s);
    }
    int pivot = big;
    if (e == hipSuccess && rc == NQ_OK) {
        hipLaunchKernelGGL(f64_to_f32_kernel, dim3(blocks_for(kk)), dim3(256), 0, s, u64, u, kk);
        e = hipMemcpyAsync(&pivot, status, 4, hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipMemcpyAsync(stats_host, stats, 16, hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);
    }
    if (e == hipSuccess && rc == NQ_OK && pivot != big)
        rc = fail(NQ_ERR_INVALID, "cholesky_f64: not positive definite (pivot " + std::to_string(k - 1 - pivot) +
                                      " of the reversed matrix)");
    if (e == hipSuccess && rc == NQ_OK) {
        const size_t lds = (size_t)(GPTQ_BLOCK * GPTQ_BLOCK + ROWS_PER_WG * GPTQ_BLOCK) * 4;
        static LdsAttrOnce attr;
        e = set_max_lds_once(attr, reinterpret_cast<const void*>(gptq_rows_kernel), lds);
        if (e == hipSuccess) {
            hipLaunchKernelGGL(gptq_rows_kernel, dim3(blocks_for(n, ROWS_PER_WG)), dim3(64 * ROWS_PER_WG), lds, s,
                               w_dev, (int)n, k, u, q, d);
            hipLaunchKernelGGL(q4_0_pack_kernel, dim3(blocks_for(ngroups)), dim3(256), 0, s, q, d, blocks_dev, ngroups);
            e = hipGetLastError();
            if (e == hipSuccess) e = hipStreamSynchronize(s);
        }
    }
    cleanup();
    if (e != hipSuccess) return fail_hip(e, "gptq_q4_0");
    return rc;
}

// tr((W - What) H (W - What)^T) in fp64 (gptq.mojo:152-189); deq_dev = What as fp32 [n, k]
int32_t run_q4_0_objective(const float* w_dev, const float* deq_dev, int64_t n, int k, const double* h_dev,
                           double* out_host, hipStream_t s) {
    double *delta = nullptr, *dh = nullptr, *partial = nullptr;
    auto cleanup = [&]() { (void)hipFree(delta), (void)hipFree(dh), (void)hipFree(partial); };
    hipError_t e = hipMalloc((void**)&delta, (size_t)(n * k) * 8);
    if (e == hipSuccess) e = hipMalloc((void**)&dh, (size_t)(n * k) * 8);
    if (e == hipSuccess) e = hipMalloc((void**)&partial, (size_t)n * 8);
    if (e != hipSuccess) {
        cleanup();
        return fail_hip(e, "q4_0_objective alloc");
    }
    std::vector<double> host((size_t)n);
    hipLaunchKernelGGL(delta_kernel, dim3(blocks_for(n * k)), dim3(256), 0, s, w_dev, deq_dev, delta, n * k);
    e = hipMemsetAsync(dh, 0, (size_t)(n * k) * 8, s);
    int32_t rc = NQ_OK;
    if (e == hipSuccess) rc = dgemm(false, (int)n, k, k, 1.0, delta, k, h_dev, k, dh, k, false, s);
    if (e == hipSuccess && rc == NQ_OK) {
        hipLaunchKernelGGL(rowdot_kernel, dim3((unsigned)n), dim3(256), 0, s, dh, delta, partial, k);
        e = hipMemcpyAsync(host.data(), partial, (size_t)n * 8, hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);
    }
    cleanup();
    if (e != hipSuccess) return fail_hip(e, "q4_0_objective");
    if (rc) return rc;
    double sum = 0.0;
    for (double v : host) sum += v;
    *out_host = sum;
    return NQ_OK;
}

}  // namespace nq
