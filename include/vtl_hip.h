/*
 * vtl_hip.h - C ABI of libvtlhip.so, the MI355X (gfx950) backend of VTL's
 * INT8 quantized-linear path.
 *
 * The reference is a V library; V binds C with `fn C.name(...) int` plus
 * `#flag -lvtlhip` / `#include "vtl_hip.h"`.  Every entry point below is what
 * one of the reference's V call sites would bind; the site it replaces or
 * mirrors is cited (paths relative to the reference tree).
 *
 * Conventions (taken from the reference's CUDA call sites,
 * storage/cuda_d_cuda.v:39-42,74-77):
 *   - every function returns an int status, 0 = success; the V side turns a
 *     non-zero status into `error(...)` and the layer falls back to its CPU
 *     path (nn/layers/linear_forward_f32.v:8-11);
 *   - no exceptions, no aborts: null pointers, negative or mismatching sizes
 *     return VTL_HIP_ERR_INVALID_ARG;
 *   - all pointers given to compute entry points are DEVICE pointers obtained
 *     from vtl_hip_malloc (the owner is the V-side HipStorage, released
 *     explicitly as in storage/cuda_d_cuda.v:98-102); host memory is touched
 *     only by the memcpy calls, which block until the copy is done;
 *   - compute entry points enqueue on the library's current stream (the null
 *     stream unless vtl_hip_set_stream was called) and return without
 *     waiting; a later blocking memcpy or vtl_hip_sync orders after them;
 *   - matrices are dense row-major; weights are passed AS STORED by
 *     LinearLayer, `[out_features, in_features]` (nn/layers/linear.v:10-16),
 *     never as a transposed view;
 *   - one host thread per device; the library keeps no pointers to caller
 *     memory after a call returns;
 *   - a few entry points stage data in scratch memory the library owns (the
 *     K-split partial sums of the matmuls, vtl_hip_linear_i8_requant,
 *     vtl_hip_linear_f32_dynquant with workspace == NULL, int8 operands that
 *     need repacking).  There is one such buffer per purpose and device,
 *     shared by every stream: calls that use it must not overlap on a device,
 *     i.e. issue them on one stream (or order the streams yourself).  The
 *     buffers grow on demand, which waits for the whole device; while the
 *     current stream is being captured into a graph a call that would have to
 *     grow one returns VTL_HIP_ERR_UNSUPPORTED instead (pass a workspace of
 *     your own where the entry point takes one, use
 *     vtl_hip_linear_f32_dynquant_noalloc, or run the call once before
 *     capturing).  A buffer that a recorded graph uses is never freed: when a
 *     later call needs a larger one it gets a new buffer and the old one stays
 *     allocated until the process ends, so replays of the graph stay valid.
 */
#ifndef VTL_HIP_H
#define VTL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    VTL_HIP_OK = 0,
    VTL_HIP_ERR_INVALID_ARG = 1, /* null pointer, bad size, bad flag */
    VTL_HIP_ERR_NO_DEVICE = 2,   /* no usable GPU / bad device id */
    VTL_HIP_ERR_RUNTIME = 3,     /* a HIP runtime call failed */
    VTL_HIP_ERR_OUT_OF_MEMORY = 4,
    VTL_HIP_ERR_UNSUPPORTED = 5  /* shape outside what the kernels cover */
};

/* ---- device, memory, transfer ------------------------------------------ */

/* cuda.get_device(id) in storage/cuda_d_cuda.v:33. */
int vtl_hip_device_count(int *n);
int vtl_hip_set_device(int device_id);
/* Name and compute-unit count of the current device (diagnostics only). */
int vtl_hip_device_info(char *name, size_t name_cap, int *compute_units, int *clock_mhz);

/* C.cudaMalloc storage/cuda_d_cuda.v:39; C.cudaFree :100. */
int vtl_hip_malloc(void **dptr, size_t bytes);
int vtl_hip_free(void *dptr);

/* C.cudaMemcpy H2D storage/cuda_d_cuda.v:46, D2H :74,:90 (blocking). */
int vtl_hip_memcpy_h2d(void *dst_device, const void *src_host, size_t bytes);
int vtl_hip_memcpy_d2h(void *dst_host, const void *src_device, size_t bytes);
int vtl_hip_memcpy_d2d(void *dst_device, const void *src_device, size_t bytes);
/* Byte fill on the current stream, any alignment and size; done by a kernel,
 * so a caller's stream capture records a kernel node, not a memset node. */
int vtl_hip_memset(void *dst_device, int byte_value, size_t bytes);

/* Wait for everything enqueued on the current stream. */
int vtl_hip_sync(void);

/* Stream the compute entry points enqueue on (a hipStream_t, NULL = null
 * stream), kept per calling host thread like HIP's current device.  The
 * reference has no stream concept beyond the unused field at
 * storage/cuda_notd_cuda.v:9. */
int vtl_hip_set_stream(void *hip_stream);
int vtl_hip_get_stream(void **hip_stream);

/* Timing helpers (hipEvent on the current stream); the reference times with
 * wall-clock ticks, benchmarks/vs_numpy/matmul_bench.v:41-43. */
int vtl_hip_event_create(void **event);
int vtl_hip_event_destroy(void *event);
int vtl_hip_event_record(void *event);
int vtl_hip_event_elapsed_ms(void *start, void *stop, float *ms);

/* ---- quantization vocabulary -------------------------------------------- */

/* absmax_out[0] = max |x| over the tensor (per_row == 0) or absmax_out[r] =
 * max |x[r, :]| (per_row != 0).  NaN elements are ignored; empty -> 0.
 * The whole-tensor maximum is collected in a few bytes of device memory that the
 * library keeps per stream (for the first 16 streams of a device that make such
 * a call; calls on further streams, and calls recorded into a graph, clear and
 * use absmax_out itself, one launch more).  Calls on one stream are ordered;
 * calls on different streams do not disturb each other.
 * Replaces Tensor.abs (math.v:11-16) + max_axis (reduction.v:163-232) /
 * stats.max (stats/stats.v:401-407). */
int vtl_hip_absmax_f32(const float *x, int64_t rows, int64_t cols, int per_row,
                       float *absmax_out);

/* scale = absmax / 127 (f32 division); q = clamp(round_half_even(x / scale),
 * -127, 127) with NaN -> 0 and scale 0 -> all codes 0.  scale_out receives 1
 * (per_row == 0) or `rows` scales.  per_row != 0 is one launch; per_row == 0 is
 * one launch up to 65536 elements, two up to 2^24 (absmax as in
 * vtl_hip_absmax_f32, then a pass that derives the scale from it), four beyond
 * or where vtl_hip_absmax_f32 has no memory of its own for the stream.
 * Replaces divide_scalar (math_op.v:103-111)
 * + round_to_even (math.v:570-574) + clamp (autograd/variable_ops.v:228-248)
 * + as_i8 (cast.v:107-121). */
int vtl_hip_quantize_f32_i8(const float *x, int64_t rows, int64_t cols, int per_row,
                            int8_t *q, float *scale_out);

/* Same codes, but with scales the caller already holds on the device. */
int vtl_hip_quantize_with_scale_f32_i8(const float *x, const float *scale, int64_t rows,
                                       int64_t cols, int per_row, int8_t *q);

/* x[r,c] = f32(q[r,c]) * scale[r or 0].  Replaces as_f32 (cast.v:35) +
 * multiply_scalar (math_op.v:137-145). */
int vtl_hip_dequantize_i8_f32(const int8_t *q, const float *scale, int64_t rows, int64_t cols,
                              int per_row, float *x);

/* ---- matmul -------------------------------------------------------------- */

/* C[M,N] (i32) = A[M,K] (i8) . Bt[N,K]^T (i8), exact.  The int8 counterpart
 * of la.matmul (la/la.v:38-55) / gate_matmul (autograd/gates_blas.v:6-23) /
 * gemm_cuda (tensor_cuda_d_cuda.v:155-177) with the second operand given
 * K-contiguous.  K <= 131072 so that |acc| <= K * 127^2 < 2^31.  Any K and any
 * alignment; K % 16 == 0 with A and Bt 16-byte aligned spares a repacking pass
 * through scratch memory that the library allocates.  Outputs of more than
 * 2^32 elements are addressed in 64 bits; only min(M, 32) * N >= 2^32 (more
 * than 2^27 columns) can return VTL_HIP_ERR_UNSUPPORTED. */
int vtl_hip_gemm_i8_i32(const int8_t *A, const int8_t *Bt, int32_t *C, int M, int N, int K);

/* Y[m,n] = fl(fl(f32(acc) * fl(sa[m] * sw[n])) + bias[n]), ReLU if relu != 0
 * (x < 0 -> 0, nn/internal/activation.v:63-70).  sa: M scales when
 * sa_per_row else 1; sw: N scales when sw_per_col else 1; bias: N floats or
 * NULL (no addition).  The int8 form of linear_forward_f32
 * (nn/layers/linear_forward_f32.v:7-18): y = x.W^T + b with W as stored. */
int vtl_hip_linear_i8_f32(const int8_t *A, const float *sa, int sa_per_row,
                          const int8_t *Wq, const float *sw, int sw_per_col,
                          const float *bias, float *Y, int M, int N, int K, int relu);

/* The int8 linear whose output feeds the next quantized layer (Linear -> ReLU
 * -> Linear with activations requantized per token): y as
 * vtl_hip_linear_i8_f32 computes it, then every row of y quantized as
 * vtl_hip_quantize_f32_i8 with per_row = 1 would - codes Yq[M,N], scales
 * sy[M] - with the bits of those two calls.  Y receives the f32 rows when it
 * is not NULL.  The activation hand-off between layers of the reference's
 * device chain (DeviceGpuChain, autograd_cuda/device_session_gpu_d_cuda.v:9-55)
 * with the requantization that an int8 chain adds. */
int vtl_hip_linear_i8_requant(const int8_t *A, const float *sa, int sa_per_row,
                              const int8_t *Wq, const float *sw, int sw_per_col,
                              const float *bias, int relu, int8_t *Yq, float *sy, float *Y,
                              int M, int N, int K);

/* Per-token (row) quantization of X[M,K] on the fly, then the int8 linear
 * against per-output-channel quantized weights.  workspace: device scratch
 * of at least vtl_hip_linear_f32_dynquant_workspace(M, K) bytes, 16-byte
 * aligned, owned by the caller (the reference's DeviceSession keeps such
 * staging buffers, autograd_cuda/device_session.v:13-24); NULL (with size 0)
 * makes the library stage in a buffer of its own, one per device, grown on
 * demand.  Calls that may overlap on a device (several streams) need a
 * workspace each.  For 2 to 32 rows with K % 256 == 0 and K <= 8192 (most such
 * shapes from 128 weight rows on) and a workspace that starts on a 128-byte
 * boundary (anything vtl_hip_malloc returns), quantizer and linear are one
 * launch whose workgroups meet on a device counter that the library keeps per
 * stream, for the first 16 streams that make such a call; calls on further
 * streams, and calls made while the stream is being captured into a graph,
 * are two launches with the same results. */
size_t vtl_hip_linear_f32_dynquant_workspace(int M, int K);
int vtl_hip_linear_f32_dynquant(const float *X, const int8_t *Wq, const float *sw,
                                const float *bias, float *Y, int M, int N, int K, int relu,
                                void *workspace, size_t workspace_bytes);

/* vtl_hip_linear_f32_dynquant for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same arguments, arithmetic
 * and bits as vtl_hip_linear_f32_dynquant with workspace == NULL, but every
 * byte the call stages (activation codes and row scales, int32 partial sums
 * of a K split, repacked operands) lives in a static 32 MiB array that is part
 * of the library's code object, one per device: the call makes no hipMalloc /
 * hipFree.  A shape whose staging does not fit returns VTL_HIP_ERR_UNSUPPORTED
 * (vtl_hip_last_error() says how many bytes were missing) and leaves Y
 * untouched.  All calls on a device share that device's array, which keeps
 * the previous call's contents: calls that overlap on one device (several
 * streams, several host threads) race; calls on one stream are ordered.
 * vtl_hip_set_device resolves the array's device address, so a process that
 * captures graphs should call it (or this entry point once) beforehand. */
int vtl_hip_linear_f32_dynquant_noalloc(const float *X, const int8_t *Wq, const float *sw,
                                        const float *bias, float *Y, int M, int N, int K,
                                        int relu);

/* ---- f32 / f64 matmul with f64 accumulation ------------------------------ */

/* C[M,N] = op(A) . op(B) with every product and sum in f64 and one rounding
 * to the tensor's type: la.matmul (la/la.v:38-55: as_f64 -> f64 GEMM ->
 * as_f32) and gate_matmul (autograd/gates_blas.v:6-23).  trans_a == 0: A is
 * [M,K] row-major; otherwise A is stored [K,M] and used as its transpose (the
 * caller's `.t()`, gates_blas.v:43-48).  trans_b == 0: B is [K,N] row-major;
 * otherwise B is stored [N,K].  All matrices dense row-major.  K == 0 gives
 * zeros. */
int vtl_hip_matmul_f32(const float *A, const float *B, float *C, int M, int N, int K,
                       int trans_a, int trans_b);
int vtl_hip_matmul_f64(const double *A, const double *B, double *C, int M, int N, int K,
                       int trans_a, int trans_b);

/* The unquantized Linear forward, y = matmul(x, W^T) + b with W as stored
 * [N,K] (linear_forward_f32_cpu nn/layers/linear_forward_f32.v:16-18, f64
 * twin linear_forward_f64.v:7-26): matmul as above, then the bias added in the
 * tensor's type (Tensor.add, math_op.v:9-21); bias may be NULL; ReLU if
 * relu != 0. */
int vtl_hip_linear_f32(const float *X, const float *W, const float *bias, float *Y,
                       int M, int N, int K, int relu);
int vtl_hip_linear_f64(const double *X, const double *W, const double *bias, double *Y,
                       int M, int N, int K, int relu);

/* out[c] = sum_r x[r,c] in f64, rounded once: la.matmul(ones[1,rows], x), the
 * bias gradient of nn/gates/layers/linear.v:75-79. */
int vtl_hip_colsum_f32(const float *x, int64_t rows, int64_t cols, float *out);
int vtl_hip_colsum_f64(const double *x, int64_t rows, int64_t cols, double *out);

/* LinearGate.backward (nn/gates/layers/linear.v:57-79; the reference's device
 * forms: linear_backward_f64 autograd_cuda/linear_backward_cuda_d_cuda.v:9-36,
 * linear_backward_vulkan_f32 via linear_gate_backward_f32_d_vulkan.v:8-13):
 * dx[M,K] = grad[M,N] . W[N,K], dw[N,K] = grad^T . x[M,K], db[N] = column sums
 * of grad.  Any of dx, dw, db may be NULL (gradient not required). */
int vtl_hip_linear_backward_f32(const float *grad, const float *x, const float *W, float *dx,
                                float *dw, float *db, int M, int N, int K);
int vtl_hip_linear_backward_f64(const double *grad, const double *x, const double *W, double *dx,
                                double *dw, double *db, int M, int N, int K);

/* ReLU in place on the device (nn/internal/activation.v:63-70,
 * relu_cuda tensor_cuda_d_cuda.v:205-235). */
int vtl_hip_relu_f32(float *x, int64_t n);
int vtl_hip_relu_f64(double *x, int64_t n);

/* ---- generic tensor operations (tensor_cuda_d_cuda.v:182-270) -------------- */

/* y[rows] = A[rows, cols] . x[cols], products and sums in f64, one rounding to
 * the tensor's type (gemv_cuda, tensor_cuda_d_cuda.v:182-203). */
int vtl_hip_gemv_f32(const float *A, const float *x, float *y, int64_t rows, int64_t cols);
int vtl_hip_gemv_f64(const double *A, const double *x, double *y, int64_t rows, int64_t cols);

/* y = 1 / (1 + T(exp(-f64(x)))), the sum and the quotient in the tensor's type
 * (nn/internal/activation.v:35-40; sigmoid_cuda tensor_cuda_d_cuda.v:237-270).
 * y may be x. */
int vtl_hip_sigmoid_f32(const float *x, float *y, int64_t n);
int vtl_hip_sigmoid_f64(const double *x, double *y, int64_t n);

/* ---- diagnostics ---------------------------------------------------------- */

const char *vtl_hip_strerror(int status);
/* Text of the last HIP runtime error seen by this thread ("" if none). */
const char *vtl_hip_last_error(void);
const char *vtl_hip_version(void);
/* Which tile configuration and how many K ranges the int8 tile kernels' cost
 * model picks for an M x N x K product (pure host arithmetic, no device
 * needed), for vtl_hip_linear_i8_f32 / vtl_hip_gemm_i8_i32 (requant == 0) or
 * for vtl_hip_linear_i8_requant (requant != 0: its second kernel runs whatever
 * the split, so cutting K costs it less): config_index is what
 * VTL_HIP_GEMM_CONFIG takes ("<index>,<splits>"), tile_m x tile_n the block
 * tile.  A test and tuning aid (tests/ checks the choice against recorded
 * timings); products that take one of the special kernels (matrix-vector,
 * weight streaming, small products) never ask it.  No counterpart in the
 * reference. */
int vtl_hip_gemm_tile_choice(int M, int N, int K, int requant, int *config_index, int *tile_m, int *tile_n,
                             int *splits);

/* The library reads its tuning switches (environment variables VTL_HIP_*, used
 * by tests and tuning runs only) once, at the first call that looks at them;
 * this reads them again.  A test and tuning aid, not part of the path: launches
 * that run on other threads meanwhile see the old switches or the new ones. */
int vtl_hip_reload_env(void);

#ifdef __cplusplus
}
#endif
#endif
