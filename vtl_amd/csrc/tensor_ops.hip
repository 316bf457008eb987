// Device forms of the generic CudaTensor operations of the reference
// (tensor_cuda_d_cuda.v:182-270): matrix-vector product, ReLU and sigmoid, for
// f32 and f64 tensors.  All three are bound by HBM traffic.
#include "common.hpp"

namespace {

using vtlhip::check_launch;
using vtlhip::current_stream;

template <typename T>
struct alignas(16) Vec16 {
    static constexpr int N = 16 / (int)sizeof(T);
    T v[N];
};

__device__ __forceinline__ double wave_sum(double v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        v += __shfl_xor(v, off, 64);
    return v;
}

// y[r] = sum_c A[r,c] * x[c], products and sums in f64, one rounding to T
// (gemv_cuda, tensor_cuda_d_cuda.v:182-203; for f32 the arithmetic of la.matmul).
// WPR waves share one row; a 256-thread block covers 4 / WPR rows.
template <typename T, int WPR, bool VEC>
__global__ __launch_bounds__(256) void gemv_kernel(const T *__restrict__ A, const T *__restrict__ x,
                                                   T *__restrict__ y, int64_t rows, int64_t cols)
{
    __shared__ double part[4];
    constexpr int VN = Vec16<T>::N;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row = (int64_t)blockIdx.x * (4 / WPR) + wave / WPR;
    const int sub = wave % WPR;                      // this wave's share of the row
    double acc = 0.0;
    if (row < rows) {
        const T *__restrict__ a = A + row * cols;
        if (VEC) {
            const int64_t nv = cols / VN;
            for (int64_t i = sub * 64 + lane; i < nv; i += 64 * WPR) {
                const Vec16<T> av = *reinterpret_cast<const Vec16<T> *>(a + i * VN);
                const Vec16<T> xv = *reinterpret_cast<const Vec16<T> *>(x + i * VN);
#pragma unroll
                for (int j = 0; j < VN; ++j)
                    acc += (double)av.v[j] * (double)xv.v[j];
            }
            for (int64_t c = nv * VN + sub * 64 + lane; c < cols; c += 64 * WPR)
                acc += (double)a[c] * (double)x[c];
        } else {
            for (int64_t c = sub * 64 + lane; c < cols; c += 64 * WPR)
                acc += (double)a[c] * (double)x[c];
        }
    }
    acc = wave_sum(acc);
    if (WPR == 1) {
        if (lane == 0 && row < rows)
            y[row] = (T)acc;
        return;
    }
    if (lane == 0)
        part[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0 && row < rows)
        y[row] = (T)(((part[0] + part[1]) + part[2]) + part[3]);
}

// sigmoid: 1 / (1 + T(exp(-f64(x)))) with the sum and the quotient in T
// (nn/internal/activation.v:35-40); ReLU: x < 0 -> 0 (activation.v:63-70).
template <typename T, bool SIGMOID>
__global__ __launch_bounds__(256) void activation_kernel(const T *__restrict__ x, T *__restrict__ y, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n)
        return;
    const T v = x[i];
    if (SIGMOID)
        y[i] = T(1) / (T(1) + (T)exp(-(double)v));
    else
        y[i] = v < T(0) ? T(0) : v;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T>
int gemv_impl(const T *A, const T *x, T *y, int64_t rows, int64_t cols)
{
    if (rows < 0 || cols < 0)
        return VTL_HIP_ERR_INVALID_ARG;
    if (rows == 0)
        return VTL_HIP_OK;
    if (!y || (cols > 0 && (!A || !x)))
        return VTL_HIP_ERR_INVALID_ARG;
    hipStream_t st = current_stream();
    const bool vec = aligned16(A) && aligned16(x) && cols % (16 / (int)sizeof(T)) == 0;
    const bool wide = rows < 2048 && cols >= 2048;   // few long rows: a whole workgroup per row
    const int64_t blocks = wide ? rows : (rows + 3) / 4;
    if (blocks > 0x7fffffff)
        return VTL_HIP_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)blocks), block(256);
    if (wide && vec)
        hipLaunchKernelGGL((gemv_kernel<T, 4, true>), grid, block, 0, st, A, x, y, rows, cols);
    else if (wide)
        hipLaunchKernelGGL((gemv_kernel<T, 4, false>), grid, block, 0, st, A, x, y, rows, cols);
    else if (vec)
        hipLaunchKernelGGL((gemv_kernel<T, 1, true>), grid, block, 0, st, A, x, y, rows, cols);
    else
        hipLaunchKernelGGL((gemv_kernel<T, 1, false>), grid, block, 0, st, A, x, y, rows, cols);
    return check_launch("gemv_kernel");
}

template <typename T, bool SIGMOID>
int activation_impl(const T *x, T *y, int64_t n)
{
    if (n < 0 || (n > 0 && (!x || !y)))
        return VTL_HIP_ERR_INVALID_ARG;
    if (n == 0)
        return VTL_HIP_OK;
    const int64_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffff)
        return VTL_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((activation_kernel<T, SIGMOID>), dim3((unsigned)blocks), dim3(256), 0, current_stream(),
                       x, y, n);
    return check_launch("activation_kernel");
}

}  // namespace

extern "C" {

int vtl_hip_gemv_f32(const float *A, const float *x, float *y, int64_t rows, int64_t cols)
{
    return gemv_impl<float>(A, x, y, rows, cols);
}

int vtl_hip_gemv_f64(const double *A, const double *x, double *y, int64_t rows, int64_t cols)
{
    return gemv_impl<double>(A, x, y, rows, cols);
}

int vtl_hip_sigmoid_f32(const float *x, float *y, int64_t n) { return activation_impl<float, true>(x, y, n); }

int vtl_hip_sigmoid_f64(const double *x, double *y, int64_t n) { return activation_impl<double, true>(x, y, n); }

int vtl_hip_relu_f64(double *x, int64_t n) { return activation_impl<double, false>(x, x, n); }

}  // extern "C"
