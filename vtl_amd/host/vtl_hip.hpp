// C++ host-side mirror of the V binding of libvtlhip.so: HipStorage<T>,
// HipTensor<T> and the Linear hook, written against the C ABI only
// (include/vtl_hip.h; no HIP headers, no device code).  The reference's host
// language is V, a compiled language with no toolchain here; this header plays
// the role of storage/hip_d_hip.v, tensor_hip_d_hip.v and
// nn/layers/linear_hip_d_hip.v for C++ callers and for the test program.
//
// Error behaviour follows the reference's GPU call sites
// (storage/cuda_d_cuda.v:39-42,74-77): a non-zero status becomes an error
// (here: vtl::HipError), never an abort, and there is no CPU fallback in here.
#pragma once

#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "vtl_hip.h"

namespace vtl {

struct HipError : std::runtime_error {
    int status;
    HipError(const std::string &what, int st)
        : std::runtime_error(what + " failed with status " + std::to_string(st) + ": " + vtl_hip_strerror(st)),
          status(st) {}
};

inline void hip_check(int status, const char *what)
{
    if (status != VTL_HIP_OK)
        throw HipError(what, status);
}

// `@[params] HipParams{device_id int = 0}` (cf. CudaParams, storage/cuda_d_cuda.v:9-11)
struct HipParams {
    int device_id = 0;
};

// `HipStorage[T]{ptr voidptr; size int; count int; device_id int}`
// (cf. CudaStorage, storage/cuda_d_cuda.v:19-107).  Move-only; release() is
// explicit as in the reference, the destructor is a safety net.
template <typename T>
class HipStorage {
public:
    void *ptr = nullptr;
    size_t size = 0;   // bytes
    size_t count = 0;  // elements
    int device_id = 0;

    HipStorage() = default;
    HipStorage(size_t n, HipParams p = {}) : size(n * sizeof(T)), count(n), device_id(p.device_id)
    {
        hip_check(vtl_hip_set_device(p.device_id), "HipStorage: vtl_hip_set_device");
        if (size)
            hip_check(vtl_hip_malloc(&ptr, size), "HipStorage: vtl_hip_malloc");
    }
    // `(cpu &CpuStorage[T]) hip(params)`: allocate and copy, blocking
    static HipStorage from_cpu(const std::vector<T> &host, HipParams p = {})
    {
        HipStorage s(host.size(), p);
        if (s.size)
            hip_check(vtl_hip_memcpy_h2d(s.ptr, host.data(), s.size), "HipStorage.hip: vtl_hip_memcpy_h2d");
        return s;
    }
    HipStorage(const HipStorage &) = delete;
    HipStorage &operator=(const HipStorage &) = delete;
    HipStorage(HipStorage &&o) noexcept { *this = std::move(o); }
    HipStorage &operator=(HipStorage &&o) noexcept
    {
        if (this != &o) {
            release();
            ptr = o.ptr; size = o.size; count = o.count; device_id = o.device_id;
            o.ptr = nullptr; o.size = 0; o.count = 0;
        }
        return *this;
    }
    ~HipStorage() { release(); }

    // `.to_array() ![]T`
    std::vector<T> to_array() const
    {
        if (count && !ptr)
            throw HipError("HipStorage.to_array: null pointer", VTL_HIP_ERR_INVALID_ARG);
        std::vector<T> out(count);
        if (size)
            hip_check(vtl_hip_memcpy_d2h(out.data(), ptr, size), "HipStorage.to_array: vtl_hip_memcpy_d2h");
        return out;
    }
    std::vector<T> cpu() const { return to_array(); }
    void release() noexcept
    {
        if (ptr) {
            vtl_hip_free(ptr);
            ptr = nullptr;
        }
    }
};

// `HipTensor[T]{data; memory; size; shape; strides}` (cf. CudaTensor,
// tensor_cuda_d_cuda.v:13-60), row-major only.
template <typename T>
class HipTensor {
public:
    HipStorage<T> data;
    std::vector<int> shape;
    std::vector<int> strides;
    size_t size = 0;

    HipTensor() = default;
    HipTensor(std::vector<int> shp, HipParams p = {}) : shape(std::move(shp))
    {
        init_strides();
        data = HipStorage<T>(size, p);
    }
    // `(t &Tensor[T]) hip(params)`
    static HipTensor from_host(const std::vector<T> &host, std::vector<int> shp, HipParams p = {})
    {
        HipTensor t;
        t.shape = std::move(shp);
        t.init_strides();
        if (t.size != host.size())
            throw std::invalid_argument("HipTensor: shape does not match the number of elements");
        t.data = HipStorage<T>::from_cpu(host, p);
        return t;
    }
    std::vector<T> cpu() const { return data.to_array(); }
    void release() { data.release(); }
    int rank() const { return (int)shape.size(); }
    size_t numel() const { return size; }
    bool is_matrix() const { return rank() == 2; }
    bool is_vector() const { return rank() == 1; }
    bool is_square_matrix() const { return rank() == 2 && shape[0] == shape[1]; }

private:
    void init_strides()
    {
        size = 1;
        strides.assign(shape.size(), 1);
        for (int i = (int)shape.size() - 1; i >= 0; i--) {
            strides[i] = (int)size;
            size *= (size_t)shape[i];
        }
    }
};

inline int per_row_of(int axis)
{
    if (axis == -1)
        return 0;
    if (axis == 0)
        return 1;
    throw std::invalid_argument("axis: use -1 (whole tensor) or 0 (one scale per row)");
}

inline void matmul_shapes(const std::vector<int> &a, const std::vector<int> &bt, int &m, int &n, int &k)
{
    if (a.size() != 2 || bt.size() != 2)
        throw std::invalid_argument("Matrix expected");
    if (a[1] != bt[1])  // la.matmul, la/la.v:41-43
        throw std::invalid_argument("Invalid shapes for matrix multiplication");
    m = a[0]; n = bt[0]; k = a[1];
}

// `quantize_i8(axis) !(&HipTensor[i8], &HipTensor[f32])`
inline std::pair<HipTensor<int8_t>, HipTensor<float>> quantize_i8(const HipTensor<float> &x, int axis)
{
    if (!x.is_matrix())
        throw std::invalid_argument("Matrix expected");
    const int per_row = per_row_of(axis);
    HipParams p{x.data.device_id};
    HipTensor<int8_t> q({x.shape[0], x.shape[1]}, p);
    HipTensor<float> s({per_row ? x.shape[0] : 1}, p);
    hip_check(vtl_hip_quantize_f32_i8((const float *)x.data.ptr, x.shape[0], x.shape[1], per_row,
                                      (int8_t *)q.data.ptr, (float *)s.data.ptr),
              "vtl_hip_quantize_f32_i8");
    return {std::move(q), std::move(s)};
}

// `dequantize(scales, axis) !&HipTensor[f32]`
inline HipTensor<float> dequantize(const HipTensor<int8_t> &q, const HipTensor<float> &scales, int axis)
{
    if (!q.is_matrix())
        throw std::invalid_argument("Matrix expected");
    const int per_row = per_row_of(axis);
    if (scales.size != (size_t)(per_row ? q.shape[0] : 1))
        throw std::invalid_argument("dequantize: number of scales does not match");
    HipTensor<float> x({q.shape[0], q.shape[1]}, HipParams{q.data.device_id});
    hip_check(vtl_hip_dequantize_i8_f32((const int8_t *)q.data.ptr, (const float *)scales.data.ptr, q.shape[0],
                                        q.shape[1], per_row, (float *)x.data.ptr),
              "vtl_hip_dequantize_i8_f32");
    return x;
}

// `gemm_i8_hip(dst, a, b) !`
inline void gemm_i8_hip(HipTensor<int32_t> &dst, const HipTensor<int8_t> &a, const HipTensor<int8_t> &bt)
{
    int m, n, k;
    matmul_shapes(a.shape, bt.shape, m, n, k);
    if (dst.shape != std::vector<int>{m, n})
        throw std::invalid_argument("gemm_i8_hip: dst shape");
    hip_check(vtl_hip_gemm_i8_i32((const int8_t *)a.data.ptr, (const int8_t *)bt.data.ptr, (int32_t *)dst.data.ptr,
                                  m, n, k),
              "vtl_hip_gemm_i8_i32");
}

// `linear_forward_hip_f32(x, weights, bias) !&vtl.Tensor[f32]`: host tensors in,
// host tensor out (every GPU path of the reference returns host tensors,
// docs/DEVICE_MEMORY.md:9-16).  weights are [out, in] as stored, bias [1, out].
inline std::vector<float> linear_forward_hip_f32(const std::vector<float> &x, int m, int k,
                                                 const std::vector<float> &weights, int n,
                                                 const std::vector<float> *bias, bool relu = false)
{
    if (x.size() != (size_t)m * k || weights.size() != (size_t)n * k)
        throw std::invalid_argument("Invalid shapes for matrix multiplication");
    if (bias && bias->size() != (size_t)n)
        throw std::invalid_argument("bias: one entry per output feature expected");
    auto w_dev = HipTensor<float>::from_host(weights, {n, k});
    auto wq = quantize_i8(w_dev, 0);
    auto x_dev = HipTensor<float>::from_host(x, {m, k});
    HipStorage<float> b_dev;
    if (bias)
        b_dev = HipStorage<float>::from_cpu(*bias);
    HipTensor<float> y({m, n});
    // null workspace: the library stages the activation codes in its own buffer
    hip_check(vtl_hip_linear_f32_dynquant((const float *)x_dev.data.ptr, (const int8_t *)wq.first.data.ptr,
                                          (const float *)wq.second.data.ptr, (const float *)b_dev.ptr,
                                          (float *)y.data.ptr, m, n, k, relu ? 1 : 0, nullptr, 0),
              "vtl_hip_linear_f32_dynquant");
    return y.cpu();
}

// `linear_i8_hip(x_q, sx, w_q, sw, bias, relu) !&HipTensor[f32]`
inline HipTensor<float> linear_i8_hip(const HipTensor<int8_t> &x_q, const HipTensor<float> &sx,
                                      const HipTensor<int8_t> &w_q, const HipTensor<float> &sw,
                                      const HipStorage<float> *bias, bool relu)
{
    int m, n, k;
    matmul_shapes(x_q.shape, w_q.shape, m, n, k);
    HipTensor<float> y({m, n}, HipParams{x_q.data.device_id});
    hip_check(vtl_hip_linear_i8_f32((const int8_t *)x_q.data.ptr, (const float *)sx.data.ptr, sx.size == (size_t)m,
                                    (const int8_t *)w_q.data.ptr, (const float *)sw.data.ptr, sw.size == (size_t)n,
                                    bias ? (const float *)bias->ptr : nullptr, (float *)y.data.ptr, m, n, k,
                                    relu ? 1 : 0),
              "vtl_hip_linear_i8_f32");
    return y;
}

// `linear_i8_requant_hip(x_q, sx, w_q, sw, bias, relu) !(&HipTensor[i8], &HipTensor[f32])`:
// the hand-off between two int8 layers.
inline std::pair<HipTensor<int8_t>, HipTensor<float>> linear_i8_requant_hip(
    const HipTensor<int8_t> &x_q, const HipTensor<float> &sx, const HipTensor<int8_t> &w_q,
    const HipTensor<float> &sw, const HipStorage<float> *bias, bool relu)
{
    int m, n, k;
    matmul_shapes(x_q.shape, w_q.shape, m, n, k);
    HipParams p{x_q.data.device_id};
    HipTensor<int8_t> y_q({m, n}, p);
    HipTensor<float> sy({m}, p);
    hip_check(vtl_hip_linear_i8_requant((const int8_t *)x_q.data.ptr, (const float *)sx.data.ptr,
                                        sx.size == (size_t)m, (const int8_t *)w_q.data.ptr,
                                        (const float *)sw.data.ptr, sw.size == (size_t)n,
                                        bias ? (const float *)bias->ptr : nullptr, relu ? 1 : 0,
                                        (int8_t *)y_q.data.ptr, (float *)sy.data.ptr, nullptr, m, n, k),
              "vtl_hip_linear_i8_requant");
    return {std::move(y_q), std::move(sy)};
}

// `matmul_hip(a, b, trans_a, trans_b) !&HipTensor[T]`: la.matmul (la/la.v:38-55)
// on the device, f64 products and sums, one rounding to T (float or double).
template <typename T>
inline HipTensor<T> matmul_hip(const HipTensor<T> &a, const HipTensor<T> &b, bool trans_a = false,
                               bool trans_b = false)
{
    static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value, "f32 or f64");
    if (!a.is_matrix() || !b.is_matrix())
        throw std::invalid_argument("Matrix expected");
    const int m = trans_a ? a.shape[1] : a.shape[0], k = trans_a ? a.shape[0] : a.shape[1];
    const int k2 = trans_b ? b.shape[1] : b.shape[0], n = trans_b ? b.shape[0] : b.shape[1];
    if (k != k2)
        throw std::invalid_argument("Invalid shapes for matrix multiplication");
    HipTensor<T> c({m, n}, HipParams{a.data.device_id});
    if (std::is_same<T, float>::value)
        hip_check(vtl_hip_matmul_f32((const float *)a.data.ptr, (const float *)b.data.ptr, (float *)c.data.ptr, m,
                                     n, k, trans_a, trans_b),
                  "vtl_hip_matmul_f32");
    else
        hip_check(vtl_hip_matmul_f64((const double *)a.data.ptr, (const double *)b.data.ptr,
                                     (double *)c.data.ptr, m, n, k, trans_a, trans_b),
                  "vtl_hip_matmul_f64");
    return c;
}

// `gemv_hip(y, a, x) !` (cf. gemv_cuda, tensor_cuda_d_cuda.v:182-203): y = A . x.
template <typename T>
inline void gemv_hip(HipTensor<T> &y, const HipTensor<T> &a, const HipTensor<T> &x)
{
    static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value, "f32 or f64");
    if (a.rank() != 2 || x.rank() != 1 || y.rank() != 1)
        throw std::invalid_argument("gemv_hip: A must be rank-2, x and y must be rank-1");
    if (x.size != (size_t)a.shape[1] || y.size != (size_t)a.shape[0])
        throw std::invalid_argument("gemv_hip: shapes of A, x and y disagree");
    if (std::is_same<T, float>::value)
        hip_check(vtl_hip_gemv_f32((const float *)a.data.ptr, (const float *)x.data.ptr, (float *)y.data.ptr,
                                   a.shape[0], a.shape[1]),
                  "vtl_hip_gemv_f32");
    else
        hip_check(vtl_hip_gemv_f64((const double *)a.data.ptr, (const double *)x.data.ptr, (double *)y.data.ptr,
                                   a.shape[0], a.shape[1]),
                  "vtl_hip_gemv_f64");
}

// `sigmoid_hip() !&HipTensor[T]` (cf. sigmoid_cuda, tensor_cuda_d_cuda.v:237-270): a new tensor.
template <typename T>
inline HipTensor<T> sigmoid_hip(const HipTensor<T> &t)
{
    static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value, "f32 or f64");
    HipTensor<T> out(t.shape, HipParams{t.data.device_id});
    if (std::is_same<T, float>::value)
        hip_check(vtl_hip_sigmoid_f32((const float *)t.data.ptr, (float *)out.data.ptr, (int64_t)t.size),
                  "vtl_hip_sigmoid_f32");
    else
        hip_check(vtl_hip_sigmoid_f64((const double *)t.data.ptr, (double *)out.data.ptr, (int64_t)t.size),
                  "vtl_hip_sigmoid_f64");
    return out;
}

// `relu_hip() !` in place (cf. relu_cuda, tensor_cuda_d_cuda.v:205-235).
template <typename T>
inline void relu_hip(HipTensor<T> &t)
{
    static_assert(std::is_same<T, float>::value || std::is_same<T, double>::value, "f32 or f64");
    if (std::is_same<T, float>::value)
        hip_check(vtl_hip_relu_f32((float *)t.data.ptr, (int64_t)t.size), "vtl_hip_relu_f32");
    else
        hip_check(vtl_hip_relu_f64((double *)t.data.ptr, (int64_t)t.size), "vtl_hip_relu_f64");
}

// `linear_backward_hip_f32(grad, input, weight, bias_needs_grad) ![]&vtl.Tensor[f32]`
// (cf. linear_backward_vulkan_f32, nn/internal/linear_vulkan_backward_d_vulkan.v:9-38):
// host tensors in, {d_input[M,K], d_weight[N,K], d_bias[1,N]} out; d_bias is zeros
// when the bias needs no gradient.
inline std::vector<std::vector<float>> linear_backward_hip_f32(const std::vector<float> &grad, int m, int n,
                                                               const std::vector<float> &input, int k,
                                                               const std::vector<float> &weight,
                                                               bool bias_needs_grad)
{
    if (grad.size() != (size_t)m * n || input.size() != (size_t)m * k || weight.size() != (size_t)n * k)
        throw std::invalid_argument("linear_backward_hip_f32: shapes of grad, input and weight disagree");
    auto g_dev = HipTensor<float>::from_host(grad, {m, n});
    auto x_dev = HipTensor<float>::from_host(input, {m, k});
    auto w_dev = HipTensor<float>::from_host(weight, {n, k});
    HipTensor<float> dx({m, k}), dw({n, k});
    HipStorage<float> db;
    if (bias_needs_grad)
        db = HipStorage<float>((size_t)n);
    hip_check(vtl_hip_linear_backward_f32((const float *)g_dev.data.ptr, (const float *)x_dev.data.ptr,
                                          (const float *)w_dev.data.ptr, (float *)dx.data.ptr,
                                          (float *)dw.data.ptr, (float *)db.ptr, m, n, k),
              "vtl_hip_linear_backward_f32");
    return {dx.cpu(), dw.cpu(), bias_needs_grad ? db.to_array() : std::vector<float>((size_t)n, 0.0f)};
}

// Cheap fingerprint of a parameter tensor's contents: FNV-1a over the bit patterns of
// up to 64 elements at even strides plus the last one, and the element count.
inline uint64_t content_fingerprint(const std::vector<float> &t)
{
    const size_t n = t.size();
    uint64_t h = 0xcbf29ce484222325ULL ^ (uint64_t)n;
    auto mix = [&](float v) {
        uint32_t bits;
        memcpy(&bits, &v, sizeof bits);
        h = (h ^ bits) * 0x100000001b3ULL;
    };
    if (n) {
        const size_t step = n / 64 ? n / 64 : 1;
        size_t taken = 0;
        for (size_t i = 0; i < n && taken < 64; i += step, taken++)
            mix(t[i]);
        mix(t[n - 1]);
    }
    return h;
}

// `HipSession` (autograd_hip/hip_session_d_hip.v): per-Context device state of the
// INT8 path - the staging buffer of the activation quantization, the int8 weights of
// every layer that ran through it (`slot` names the layer) and the f32 rows the last
// layer left on the device for the next one.
//
// When the device copy of a layer's parameters is re-used: most of the reference's
// optimizers update `v.value` IN PLACE (SGD: nn/optimizers/sgd.v:46-53 ->
// nn/internal/optimizers.v:6-12 `value.set`; adagrad.v:60, adamw.v:95, rmsprop.v:81),
// only Adam assigns a new tensor (adam.v:115,136), so the identity of the weight tensor
// says nothing about its contents.  A forward that is not `frozen` (the Context is not
// no_grad and the weight Variable requires grad) uploads and quantizes the parameters
// again, as the reference's own device chain uploads them on every forward
// (autograd_cuda/device_session_gpu_d_cuda.v:107).  A `frozen` forward re-uses the copy
// only if it was made by a frozen forward from the same tensors and their content
// fingerprints are unchanged (an in-place checkpoint load is seen that way);
// invalidate() drops a copy explicitly.
class HipSession {
public:
    struct QuantizedWeights {
        const void *slot = nullptr, *source = nullptr, *bias_source = nullptr;
        uint64_t fingerprint = 0, bias_fingerprint = 0;
        bool frozen = false;
        HipTensor<int8_t> w_q;
        HipTensor<float> sw;
        HipStorage<float> bias;
    };
    bool enabled = false;
    bool keep_activations = true;   // VTL_HIP_ACTIVATIONS=1 in the V host
    std::vector<QuantizedWeights> layers;
    HipStorage<uint8_t> workspace;
    HipTensor<float> pending;
    bool has_pending = false;
    int quantize_count = 0;         // how often weights were (re)quantized: for tests

    void init_device()
    {
        int n = 0;
        enabled = vtl_hip_device_count(&n) == VTL_HIP_OK && n > 0;
    }
    void release()
    {
        layers.clear();
        workspace.release();
        pending.release();
        has_pending = false;
    }
    const HipStorage<uint8_t> &ensure_workspace(int m, int k)
    {
        const size_t need = vtl_hip_linear_f32_dynquant_workspace(m, k);
        if (!workspace.ptr || workspace.size < need)
            workspace = HipStorage<uint8_t>(need);
        return workspace;
    }
    // drops the device copy of one layer (slot) or of all layers (null)
    void invalidate(const void *slot = nullptr)
    {
        for (auto &l : layers)
            if (!slot || l.slot == slot)
                l.source = l.bias_source = nullptr;
    }
    // `weights` / `bias` are the host tensors' storage
    QuantizedWeights &quantized(const void *slot, const std::vector<float> &weights, int n, int k,
                                const std::vector<float> &bias, bool frozen)
    {
        QuantizedWeights *q = nullptr;
        for (auto &l : layers)
            if (l.slot == slot)
                q = &l;
        if (!q) {
            layers.emplace_back();
            q = &layers.back();
            q->slot = slot;
        }
        const bool trust = frozen && q->frozen;
        const uint64_t fp = content_fingerprint(weights), bfp = content_fingerprint(bias);
        if (!trust || q->source != (const void *)&weights || q->fingerprint != fp || !q->w_q.data.ptr) {
            auto w_dev = HipTensor<float>::from_host(weights, {n, k});
            auto qs = quantize_i8(w_dev, 0);
            q->w_q = std::move(qs.first);
            q->sw = std::move(qs.second);
            q->source = &weights;
            q->fingerprint = fp;
            quantize_count++;
        }
        if (!trust || q->bias_source != (const void *)&bias || q->bias_fingerprint != bfp || !q->bias.ptr) {
            q->bias = HipStorage<float>::from_cpu(bias);
            q->bias_source = &bias;
            q->bias_fingerprint = bfp;
        }
        q->frozen = frozen;
        return *q;
    }
    // `(mut s HipSession) linear_forward_f32(x, weights, bias, slot, input_gpu, frozen) !&vtl.Tensor[f32]`:
    // host rows out; the device rows stay pending for the next layer.  `input_gpu` is a
    // device activation taken from the previous layer (take_pending) or null; `frozen`
    // says that no optimizer can have touched the parameters (see the class comment).
    std::vector<float> linear_forward_f32(const std::vector<float> &x, int m, int k,
                                          const std::vector<float> &weights, int n,
                                          const std::vector<float> &bias, const void *slot,
                                          HipTensor<float> *input_gpu, bool frozen = false)
    {
        if (!enabled)
            throw HipError("hip session disabled", VTL_HIP_ERR_NO_DEVICE);
        if (x.size() != (size_t)m * k || weights.size() != (size_t)n * k)
            throw std::invalid_argument("Invalid shapes for matrix multiplication");
        pending.release();
        has_pending = false;
        QuantizedWeights &q = quantized(slot, weights, n, k, bias, frozen);
        const HipStorage<uint8_t> &ws = ensure_workspace(m, k);
        HipTensor<float> uploaded;
        const HipTensor<float> *x_dev = input_gpu;
        if (!x_dev) {
            uploaded = HipTensor<float>::from_host(x, {m, k});
            x_dev = &uploaded;
        } else if (x_dev->shape != std::vector<int>{m, k}) {
            throw std::invalid_argument("hip chain: input activation shape mismatch");
        }
        HipTensor<float> y({m, n});
        hip_check(vtl_hip_linear_f32_dynquant((const float *)x_dev->data.ptr, (const int8_t *)q.w_q.data.ptr,
                                              (const float *)q.sw.data.ptr, (const float *)q.bias.ptr,
                                              (float *)y.data.ptr, m, n, k, 0, ws.ptr, ws.size),
                  "vtl_hip_linear_f32_dynquant");
        std::vector<float> host = y.cpu();
        if (keep_activations) {
            pending = std::move(y);
            has_pending = true;
        }
        return host;
    }
    // `relu_forward_f32(x, input_gpu)`: ReLU in place on the device activation, kept pending
    std::vector<float> relu_forward_f32(HipTensor<float> &&input_gpu)
    {
        relu_hip(input_gpu);
        std::vector<float> host = input_gpu.cpu();
        pending = std::move(input_gpu);
        has_pending = true;
        return host;
    }
    // `session_bind_hip_activation`: the pending activation moves to the caller (the Variable)
    HipTensor<float> take_pending()
    {
        has_pending = false;
        return std::move(pending);
    }
    // `mlp_forward_i8(x, weights, biases, relu_after, slots)`: the whole chain on the device,
    // int8 codes handed from layer to layer (f32 rows for up to 32 tokens), f32 rows of the
    // last layer back to the host.
    // An inference call: the parameters count as frozen.
    std::vector<float> mlp_forward_i8(const std::vector<float> &x, int m,
                                      const std::vector<const std::vector<float> *> &weights,
                                      const std::vector<const std::vector<float> *> &biases,
                                      const std::vector<int> &dims, const std::vector<bool> &relu_after)
    {
        if (!enabled)
            throw HipError("hip session disabled", VTL_HIP_ERR_NO_DEVICE);
        const size_t nl = weights.size();
        if (nl == 0 || biases.size() != nl || relu_after.size() != nl || dims.size() != nl + 1)
            throw std::invalid_argument("mlp_forward_i8: one bias and ReLU flag per weight matrix expected");
        auto x_dev = HipTensor<float>::from_host(x, {m, dims[0]});
        if (m <= 32) {
            // A few tokens: every layer quantizes its input inside its own launch (one launch a
            // layer), so the activations stay f32 between the layers.  Same bits as below.
            // (Buffers are sized and kept until the end: freeing one waits for the device.)
            int widest = dims[0];
            for (size_t i = 1; i < nl; i++)
                widest = std::max(widest, dims[i]);
            const HipStorage<uint8_t> &ws = ensure_workspace(m, widest);
            std::vector<HipTensor<float>> acts;
            acts.push_back(std::move(x_dev));
            for (size_t i = 0; i < nl; i++) {
                QuantizedWeights &q = quantized(weights[i], *weights[i], dims[i + 1], dims[i], *biases[i], true);
                HipTensor<float> y({m, dims[i + 1]});
                hip_check(vtl_hip_linear_f32_dynquant((const float *)acts.back().data.ptr,
                                                      (const int8_t *)q.w_q.data.ptr, (const float *)q.sw.data.ptr,
                                                      (const float *)q.bias.ptr, (float *)y.data.ptr, m, dims[i + 1],
                                                      dims[i], relu_after[i] ? 1 : 0, ws.ptr, ws.size),
                          "vtl_hip_linear_f32_dynquant");
                acts.push_back(std::move(y));
            }
            return acts.back().cpu();
        }
        auto cur = quantize_i8(x_dev, 0);
        x_dev.release();
        for (size_t i = 0; i + 1 < nl; i++) {
            QuantizedWeights &q = quantized(weights[i], *weights[i], dims[i + 1], dims[i], *biases[i], true);
            cur = linear_i8_requant_hip(cur.first, cur.second, q.w_q, q.sw, &q.bias, relu_after[i]);
        }
        QuantizedWeights &q = quantized(weights[nl - 1], *weights[nl - 1], dims[nl], dims[nl - 1], *biases[nl - 1], true);
        return linear_i8_hip(cur.first, cur.second, q.w_q, q.sw, &q.bias, relu_after[nl - 1]).cpu();
    }
};

}  // namespace vtl
