/*
 * vtl_oracle.h - CPU restatement of the INT8 quantized-linear arithmetic that
 * sits behind vtl.Tensor[T] / Sequential.linear().
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the
 * smoke check and the CPU-baseline leg of the benchmark may link or load it.
 * The product library (libvtlhip.so) never calls into it and has no CPU
 * fallback of its own.
 *
 * The reference (a pure-V library) has no composed INT8 path; the contract
 * below is composed from the reference's CPU vocabulary, cited per function.
 * All paths are relative to the reference tree.
 *
 * Spec decisions that the reference cannot settle (none of its tests reach
 * them) and that this oracle fixes:
 *   - NaN elements are ignored by absmax (max_axis's `val > best` compare,
 *     reduction.v:198-203, never selects a NaN that is not first); an
 *     all-NaN or empty slice has absmax 0.
 *   - absmax == 0  -> scale 0, every code 0, dequantized 0.
 *   - NaN quotient -> code 0 (what an x86 float->int cast followed by the
 *     narrowing to i8 yields on the reference's CPU path).
 *   - +-Inf input  -> absmax Inf, scale Inf, finite x -> 0, +-Inf -> NaN -> 0.
 *   - -128 is never produced.
 *
 * Pinning status (which independent check pins each function) is listed in
 * the header of vtl_oracle.c.
 */
#ifndef VTL_ORACLE_H
#define VTL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* absmax over the whole tensor (per_row == 0, out[1]) or per row
 * (per_row != 0, out[rows]).  abs: math.v:11-16; max: math.v:468-472,
 * max_axis: reduction.v:163-232, stats.max: stats/stats.v:401-407. */
void vtl_ref_absmax_f32(const float *x, int64_t rows, int64_t cols, int per_row, float *out);

/* scale = absmax / 127 in f32 (divide_scalar in T: math_op.v:103-111). */
float vtl_ref_scale_from_absmax(float absmax);

/* One code: clamp(round_half_even(x / scale), -127, 127).
 * divide_scalar math_op.v:103-111, round_to_even math.v:570-574,
 * clamp autograd/variable_ops.v:228-248. */
int8_t vtl_ref_quantize_one(float x, float scale);

/* Symmetric quantize: computes scales (1 or rows of them) and codes. */
void vtl_ref_quantize_f32_i8(const float *x, int64_t rows, int64_t cols, int per_row,
                             int8_t *q, float *scale_out);

/* Quantize with caller-supplied scales (1 or rows of them). */
void vtl_ref_quantize_with_scale(const float *x, const float *scale, int64_t rows, int64_t cols,
                                 int per_row, int8_t *q);

/* x_hat = f32(q) * scale (multiply_scalar math_op.v:137-145). */
void vtl_ref_dequantize_i8_f32(const int8_t *q, const float *scale, int64_t rows, int64_t cols,
                               int per_row, float *x);

/* C[M,N] (i32) = A[M,K] (i8, row-major) . Bt[N,K]^T (i8, row-major: the
 * weight as LinearLayer stores it, nn/layers/linear.v:10-16).  Shape rule
 * of la.matmul la/la.v:38-43.  threads <= 1: single thread (the reference is
 * single-threaded); otherwise OpenMP over rows. */
void vtl_ref_gemm_i8_i32(const int8_t *A, const int8_t *Bt, int32_t *C,
                         int64_t M, int64_t N, int64_t K, int threads);

/* Y[m,n] = fl(fl(fl((float)acc) * fl(sa[m]*sw[n])) + bias[n]), then optional
 * ReLU (x < 0 -> 0, nn/internal/activation.v:63-70).  sa has M entries when
 * sa_per_row else 1; sw has N entries when sw_per_col else 1; bias may be
 * NULL (no add at all).  Bias broadcast [1,N] over [M,N]: math_op.v:9-21. */
void vtl_ref_epilogue_f32(const int32_t *acc, const float *sa, int sa_per_row,
                          const float *sw, int sw_per_col, const float *bias,
                          float *Y, int64_t M, int64_t N, int relu);

/* gemm + epilogue in one call. */
void vtl_ref_linear_i8_f32(const int8_t *A, const float *sa, int sa_per_row,
                           const int8_t *Wq, const float *sw, int sw_per_col,
                           const float *bias, float *Y,
                           int64_t M, int64_t N, int64_t K, int relu, int threads);

/* Per-token dynamic quantization of X[M,K] followed by the int8 linear. */
void vtl_ref_linear_f32_dynquant(const float *X, const int8_t *Wq, const float *sw,
                                 const float *bias, float *Y,
                                 int64_t M, int64_t N, int64_t K, int relu, int threads);

/* ReLU in place (nn/internal/activation.v:63-70). */
void vtl_ref_relu_f32(float *x, int64_t n);

/* The reference's existing f32 Linear as documented: y = x.W^T + b through
 * f64 (la/la.v:44-53: as_f64 -> f64 GEMM -> as_f32; then Tensor.add,
 * nn/layers/linear_forward_f32.v:16-18), with the explicit transpose the
 * reference's own device session uses (autograd_cuda/device_session.v:38-46).
 * The f64 summation order inside the un-vendored VSL GEMM is unknown, so
 * values are pinned only up to f64 rounding: parity unpinned beyond that. */
void vtl_ref_linear_f32_via_f64(const float *X, const float *W, const float *bias, float *Y,
                                int64_t M, int64_t N, int64_t K);

/* C[M,N] = op(A) . op(B) the way la.matmul (la/la.v:38-55) and gate_matmul
 * (autograd/gates_blas.v:6-23) compute it: every element widened to f64, a
 * f64 GEMM (here: k ascending, one f64 accumulator per element), one rounding
 * to the tensor's type (as_f32 for f32; f64 stays).  trans_a == 0: A is
 * [M,K] row-major, else A is stored [K,M] (the caller's `.t()`, as in
 * MatMulGate.backward gates_blas.v:43-48 and LinearGate.backward
 * nn/gates/layers/linear.v:69-74); same for B ([K,N] / [N,K]).  threads > 1:
 * OpenMP over rows, same arithmetic.  Summation order inside VSL's GEMM
 * (vsl@v0.2.0-beta.1, not vendored) is unknown and is not even one order: the
 * reference's CI builds it both over its pure-V BLAS and over cblas
 * (.github/workflows/ci.yml:81-86,132-140), so the reference's own f32 results
 * are defined only up to the order of the f64 sum.  Parity unpinned beyond
 * that f64 rounding error (about 1e-16 relative before the one rounding). */
void vtl_ref_matmul_f32(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                        int trans_a, int trans_b, int threads);
void vtl_ref_matmul_f64(const double *A, const double *B, double *C, int64_t M, int64_t N, int64_t K,
                        int trans_a, int trans_b, int threads);

/* out[c] = sum over rows of x[r,c], summed in f64 and rounded once:
 * la.matmul(ones[1,M], grad), nn/gates/layers/linear.v:75-79. */
void vtl_ref_colsum_f32(const float *x, int64_t rows, int64_t cols, float *out);
void vtl_ref_colsum_f64(const double *x, int64_t rows, int64_t cols, double *out);

/* LinearGate.backward (nn/gates/layers/linear.v:57-79; f64 twin
 * autograd_cuda/linear_backward_f64.v): dx[M,K] = grad[M,N] . W[N,K],
 * dw[N,K] = grad^T . x[M,K], db[N] = ones[1,M] . grad.  Any output may be
 * NULL (that gradient is not required). */
void vtl_ref_linear_backward_f32(const float *grad, const float *x, const float *w, float *dx,
                                 float *dw, float *db, int64_t M, int64_t N, int64_t K, int threads);
void vtl_ref_linear_backward_f64(const double *grad, const double *x, const double *w, double *dx,
                                 double *dw, double *db, int64_t M, int64_t N, int64_t K, int threads);

/* y[r] = sum_c A[r,c] * x[c] through f64, one rounding (gemv_cuda
 * tensor_cuda_d_cuda.v:182-203; la.matmul arithmetic la/la.v:44-53). */
void vtl_ref_gemv_f32(const float *A, const float *x, float *y, int64_t rows, int64_t cols);
void vtl_ref_gemv_f64(const double *A, const double *x, double *y, int64_t rows, int64_t cols);

/* y = 1 / (1 + T(exp(-f64(x)))), sum and quotient in T
 * (nn/internal/activation.v:35-40). */
void vtl_ref_sigmoid_f32(const float *x, float *y, int64_t n);
void vtl_ref_sigmoid_f64(const double *x, double *y, int64_t n);

/* ReLU on f64 in place (nn/internal/activation.v:63-70). */
void vtl_ref_relu_f64(double *x, int64_t n);

/* Row-parallel forms (same arithmetic), for timing the CPU baseline on all cores. */
void vtl_ref_quantize_f32_i8_mt(const float *x, int64_t rows, int64_t cols, int per_row,
                                int8_t *q, float *scale_out, int threads);
void vtl_ref_dequantize_i8_f32_mt(const int8_t *q, const float *scale, int64_t rows, int64_t cols,
                                  int per_row, float *x, int threads);

int vtl_ref_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
