/*
 * vtl_oracle.c - CPU restatement of the INT8 quantized-linear arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY (see vtl_oracle.h).  Build with
 *   gcc -O3 -march=x86-64-v3 -ffp-contract=off -fno-fast-math -fopenmp
 * -ffp-contract=off matters: the epilogue is specified as separately rounded
 * multiply, multiply, add.
 *
 * What pins each function (all checks live in the CPU test-suite):
 *   vtl_ref_absmax_f32          reference vocabulary vectors
 *                               (tests/core/math_test.v:5-10 abs,
 *                               tests/core/reduction_test.v:49-54 max_axis,
 *                               stats/stats_test.v:228-240 max), numpy
 *                               np.abs().max(), sign/permutation invariance.
 *   vtl_ref_scale_from_absmax   numpy float32 division (IEEE single rounding).
 *   vtl_ref_quantize_one        hand-written round-half-even known answers,
 *                               exact rational arithmetic (fractions) on the
 *                               f32 quotient, numpy rint, tests/core/
 *                               math_op_test.v:103-108,117-122 divide_scalar.
 *   vtl_ref_quantize_f32_i8     the above + invariants (|x|==absmax -> +-127,
 *                               -128 never, power-of-two scale invariance,
 *                               |x - x_hat| <= scale/2).
 *   vtl_ref_dequantize_i8_f32   numpy float32 product.
 *   vtl_ref_gemm_i8_i32         numpy int64 matmul, la/la_test.v:30-37
 *                               (I.B = B), closed forms (all 127 -> K*16129,
 *                               alternating sign -> 0).
 *   vtl_ref_epilogue_f32        numpy float32 op-by-op evaluation, f64
 *                               bound, ReLU closed form.
 *   vtl_ref_linear_f32_via_f64  autograd_cuda/device_session_test.v:34-36
 *                               literals (y = [1.41, 3.22]), numpy f64 matmul.
 *                               Summation order of the un-vendored VSL GEMM
 *                               is unknown: parity unpinned beyond f64
 *                               rounding error.
 *   vtl_ref_matmul_f32/_f64     la/la_test.v:30-37 (I.B = B), numpy f64
 *                               matmul on explicit transposes, integer-valued
 *                               operands (every order of summation exact)
 *                               against numpy int64 matmul, the literals of
 *                               benchmarks/vs_numpy/matmul_bench.v:28-33 in
 *                               closed form.  Same caveat on VSL's order.
 *   vtl_ref_colsum_f32/_f64     math.fsum (exact sum, one rounding).
 *   vtl_ref_gemv_*              numpy f64 dot, integer-valued operands (exact).
 *   vtl_ref_sigmoid_*           closed forms (sigmoid(0) = 0.5, sigmoid(x) +
 *                               sigmoid(-x) = 1 to rounding), numpy's
 *                               1 / (1 + exp(-x)) op by op; saturation at
 *                               large |x|.  exp is the C library's, correct to
 *                               <= 1 ulp: results pinned to that.
 *   vtl_ref_linear_backward_*   autograd_cuda/device_session_test.v:52-60
 *                               operands worked by hand (dx = [0.3, 0.45,
 *                               0.6], dw = [[1,2,3],[0.5,1,1.5]], db = grad),
 *                               central finite differences of the f64 forward.
 */
#include "vtl_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int vtl_ref_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* abs via math.abs (math.v:11-16), running max with `val > best` as in
 * max_axis (reduction.v:163-232); starting from 0 is the same as starting
 * from the first |x| because |x| >= 0, and it makes NaN never selected. */
static float absmax_slice(const float *x, int64_t n)
{
    float best = 0.0f;
    for (int64_t i = 0; i < n; i++) {
        float a = fabsf(x[i]);
        if (a > best)
            best = a;
    }
    return best;
}

void vtl_ref_absmax_f32(const float *x, int64_t rows, int64_t cols, int per_row, float *out)
{
    if (per_row) {
        for (int64_t r = 0; r < rows; r++)
            out[r] = absmax_slice(x + r * cols, cols);
    } else {
        out[0] = absmax_slice(x, rows * cols);
    }
}

float vtl_ref_scale_from_absmax(float absmax)
{
    float s = absmax / 127.0f; /* one IEEE f32 division */
    return s;
}

int8_t vtl_ref_quantize_one(float x, float scale)
{
    /* divide_scalar works in T = f32 (math_op.v:103-111); round_to_even
     * widens to f64 (math.v:570-574), which is lossless, so rintf under the
     * default round-to-nearest mode gives the same integer. */
    float t = x / scale;
    float r = rintf(t);
    if (r != r)
        return 0; /* NaN (0/0, Inf/Inf, NaN input) */
    if (r < -127.0f)
        r = -127.0f; /* clamp: autograd/variable_ops.v:231-239 */
    else if (r > 127.0f)
        r = 127.0f;
    return (int8_t)(int)r;
}

void vtl_ref_quantize_with_scale(const float *x, const float *scale, int64_t rows, int64_t cols,
                                 int per_row, int8_t *q)
{
    for (int64_t r = 0; r < rows; r++) {
        float s = per_row ? scale[r] : scale[0];
        const float *xr = x + r * cols;
        int8_t *qr = q + r * cols;
        for (int64_t c = 0; c < cols; c++)
            qr[c] = vtl_ref_quantize_one(xr[c], s);
    }
}

void vtl_ref_quantize_f32_i8(const float *x, int64_t rows, int64_t cols, int per_row,
                             int8_t *q, float *scale_out)
{
    int64_t ns = per_row ? rows : 1;
    vtl_ref_absmax_f32(x, rows, cols, per_row, scale_out);
    for (int64_t i = 0; i < ns; i++)
        scale_out[i] = vtl_ref_scale_from_absmax(scale_out[i]);
    vtl_ref_quantize_with_scale(x, scale_out, rows, cols, per_row, q);
}

void vtl_ref_dequantize_i8_f32(const int8_t *q, const float *scale, int64_t rows, int64_t cols,
                               int per_row, float *x)
{
    for (int64_t r = 0; r < rows; r++) {
        float s = per_row ? scale[r] : scale[0];
        const int8_t *qr = q + r * cols;
        float *xr = x + r * cols;
        for (int64_t c = 0; c < cols; c++)
            xr[c] = (float)qr[c] * s;
    }
}

static void gemm_rows(const int8_t *A, const int8_t *Bt, int32_t *C,
                      int64_t m0, int64_t m1, int64_t N, int64_t K)
{
    for (int64_t m = m0; m < m1; m++) {
        const int8_t *a = A + m * K;
        for (int64_t n = 0; n < N; n++) {
            const int8_t *b = Bt + n * K;
            int32_t acc = 0;
            for (int64_t k = 0; k < K; k++)
                acc += (int32_t)a[k] * (int32_t)b[k];
            C[m * N + n] = acc;
        }
    }
}

void vtl_ref_gemm_i8_i32(const int8_t *A, const int8_t *Bt, int32_t *C,
                         int64_t M, int64_t N, int64_t K, int threads)
{
    if (threads <= 1) {
        gemm_rows(A, Bt, C, 0, M, N, K);
        return;
    }
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (int64_t m = 0; m < M; m++)
        gemm_rows(A, Bt, C, m, m + 1, N, K);
}

void vtl_ref_epilogue_f32(const int32_t *acc, const float *sa, int sa_per_row,
                          const float *sw, int sw_per_col, const float *bias,
                          float *Y, int64_t M, int64_t N, int relu)
{
    for (int64_t m = 0; m < M; m++) {
        float a = sa_per_row ? sa[m] : sa[0];
        for (int64_t n = 0; n < N; n++) {
            float w = sw_per_col ? sw[n] : sw[0];
            float s = a * w;                        /* rounded once */
            float v = (float)acc[m * N + n] * s;    /* rounded once */
            if (bias)
                v = v + bias[n];                    /* rounded once, no FMA */
            if (relu && v < 0.0f)
                v = 0.0f;
            Y[m * N + n] = v;
        }
    }
}

void vtl_ref_linear_i8_f32(const int8_t *A, const float *sa, int sa_per_row,
                           const int8_t *Wq, const float *sw, int sw_per_col,
                           const float *bias, float *Y,
                           int64_t M, int64_t N, int64_t K, int relu, int threads)
{
    int32_t *acc = (int32_t *)malloc((size_t)M * (size_t)N * sizeof(int32_t));
    vtl_ref_gemm_i8_i32(A, Wq, acc, M, N, K, threads);
    vtl_ref_epilogue_f32(acc, sa, sa_per_row, sw, sw_per_col, bias, Y, M, N, relu);
    free(acc);
}

void vtl_ref_linear_f32_dynquant(const float *X, const int8_t *Wq, const float *sw,
                                 const float *bias, float *Y,
                                 int64_t M, int64_t N, int64_t K, int relu, int threads)
{
    int8_t *xq = (int8_t *)malloc((size_t)M * (size_t)K);
    float *sx = (float *)malloc((size_t)M * sizeof(float));
    vtl_ref_quantize_f32_i8(X, M, K, 1, xq, sx);
    vtl_ref_linear_i8_f32(xq, sx, 1, Wq, sw, 1, bias, Y, M, N, K, relu, threads);
    free(xq);
    free(sx);
}

void vtl_ref_relu_f32(float *x, int64_t n)
{
    for (int64_t i = 0; i < n; i++)
        if (x[i] < 0.0f)
            x[i] = 0.0f;
}

void vtl_ref_linear_f32_via_f64(const float *X, const float *W, const float *bias, float *Y,
                                int64_t M, int64_t N, int64_t K)
{
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; k++)
                acc += (double)X[m * K + k] * (double)W[n * K + k];
            float y = (float)acc;   /* as_f32, la/la.v:51-53 */
            if (bias)
                y = y + bias[n];    /* Tensor.add in f32 */
            Y[m * N + n] = y;
        }
    }
}

#define VTL_REF_MATMUL(NAME, T)                                                              \
    void NAME(const T *A, const T *B, T *C, int64_t M, int64_t N, int64_t K, int trans_a,     \
              int trans_b, int threads)                                                       \
    {                                                                                         \
        const int64_t a_rs = trans_a ? 1 : K, a_ks = trans_a ? M : 1;                         \
        const int64_t b_ks = trans_b ? 1 : N, b_cs = trans_b ? K : 1;                         \
        (void)threads;                                                                        \
        _Pragma("omp parallel for schedule(static) num_threads(threads > 1 ? threads : 1)")   \
        for (int64_t m = 0; m < M; m++) {                                                     \
            for (int64_t n = 0; n < N; n++) {                                                 \
                double acc = 0.0;                                                             \
                for (int64_t k = 0; k < K; k++)                                               \
                    acc += (double)A[m * a_rs + k * a_ks] * (double)B[k * b_ks + n * b_cs];   \
                C[m * N + n] = (T)acc; /* as_f32 for f32, la/la.v:51-53 */                    \
            }                                                                                 \
        }                                                                                     \
    }
VTL_REF_MATMUL(vtl_ref_matmul_f32, float)
VTL_REF_MATMUL(vtl_ref_matmul_f64, double)

#define VTL_REF_COLSUM(NAME, T)                                   \
    void NAME(const T *x, int64_t rows, int64_t cols, T *out)     \
    {                                                             \
        for (int64_t c = 0; c < cols; c++) {                      \
            double acc = 0.0;                                     \
            for (int64_t r = 0; r < rows; r++)                    \
                acc += 1.0 * (double)x[r * cols + c];             \
            out[c] = (T)acc;                                      \
        }                                                         \
    }
VTL_REF_COLSUM(vtl_ref_colsum_f32, float)
VTL_REF_COLSUM(vtl_ref_colsum_f64, double)

#define VTL_REF_LINEAR_BACKWARD(NAME, T, MATMUL, COLSUM)                                          \
    void NAME(const T *grad, const T *x, const T *w, T *dx, T *dw, T *db, int64_t M, int64_t N,    \
              int64_t K, int threads)                                                              \
    {                                                                                              \
        if (dx) /* la.matmul(grad, weight), linear.v:69-70 */                                      \
            MATMUL(grad, w, dx, M, K, N, 0, 0, threads);                                           \
        if (dw) /* la.matmul(grad.t(), input), linear.v:72-73 */                                   \
            MATMUL(grad, x, dw, N, K, M, 1, 0, threads);                                           \
        if (db) /* la.matmul(ones[1,batch], grad), linear.v:75-79 */                               \
            COLSUM(grad, M, N, db);                                                                \
    }
VTL_REF_LINEAR_BACKWARD(vtl_ref_linear_backward_f32, float, vtl_ref_matmul_f32, vtl_ref_colsum_f32)
VTL_REF_LINEAR_BACKWARD(vtl_ref_linear_backward_f64, double, vtl_ref_matmul_f64, vtl_ref_colsum_f64)

#define VTL_REF_GEMV(NAME, T)                                                  \
    void NAME(const T *A, const T *x, T *y, int64_t rows, int64_t cols)        \
    {                                                                          \
        for (int64_t r = 0; r < rows; r++) {                                   \
            double acc = 0.0;                                                  \
            for (int64_t c = 0; c < cols; c++)                                 \
                acc += (double)A[r * cols + c] * (double)x[c];                 \
            y[r] = (T)acc;                                                     \
        }                                                                      \
    }
VTL_REF_GEMV(vtl_ref_gemv_f32, float)
VTL_REF_GEMV(vtl_ref_gemv_f64, double)

void vtl_ref_sigmoid_f32(const float *x, float *y, int64_t n)
{
    for (int64_t i = 0; i < n; i++) {
        const float e = (float)exp(-(double)x[i]); /* vtl.cast[T](math.exp(-vtl.cast[f64](val))) */
        y[i] = 1.0f / (1.0f + e);
    }
}

void vtl_ref_sigmoid_f64(const double *x, double *y, int64_t n)
{
    for (int64_t i = 0; i < n; i++)
        y[i] = 1.0 / (1.0 + exp(-x[i]));
}

void vtl_ref_relu_f64(double *x, int64_t n)
{
    for (int64_t i = 0; i < n; i++)
        if (x[i] < 0.0)
            x[i] = 0.0;
}

/* Row-parallel forms of the two bandwidth-bound routines, used only to time
 * the CPU baseline on all host cores.  Same arithmetic per element. */
void vtl_ref_quantize_f32_i8_mt(const float *x, int64_t rows, int64_t cols, int per_row,
                                int8_t *q, float *scale_out, int threads)
{
    if (threads <= 1) {
        vtl_ref_quantize_f32_i8(x, rows, cols, per_row, q, scale_out);
        return;
    }
    if (per_row) {
#pragma omp parallel for schedule(static) num_threads(threads)
        for (int64_t r = 0; r < rows; r++)
            vtl_ref_quantize_f32_i8(x + r * cols, 1, cols, 1, q + r * cols, scale_out + r);
        return;
    }
    float best = 0.0f;
#pragma omp parallel for schedule(static) num_threads(threads) reduction(max : best)
    for (int64_t r = 0; r < rows; r++) {
        float a = absmax_slice(x + r * cols, cols);
        if (a > best)
            best = a;
    }
    scale_out[0] = vtl_ref_scale_from_absmax(best);
#pragma omp parallel for schedule(static) num_threads(threads)
    for (int64_t r = 0; r < rows; r++)
        vtl_ref_quantize_with_scale(x + r * cols, scale_out, 1, cols, 0, q + r * cols);
}

void vtl_ref_dequantize_i8_f32_mt(const int8_t *q, const float *scale, int64_t rows, int64_t cols,
                                  int per_row, float *x, int threads)
{
    if (threads <= 1) {
        vtl_ref_dequantize_i8_f32(q, scale, rows, cols, per_row, x);
        return;
    }
#pragma omp parallel for schedule(static) num_threads(threads)
    for (int64_t r = 0; r < rows; r++)
        vtl_ref_dequantize_i8_f32(q + r * cols, per_row ? scale + r : scale, 1, cols, 0, x + r * cols);
}
