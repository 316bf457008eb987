// Symmetric INT8 quantization vocabulary for gfx950: absmax, quantize,
// dequantize, ReLU.  All of it is HBM-bound streaming work: 16-byte loads per
// lane, coalesced across the 64-wide wavefront, one pass over the data where
// the row fits in registers, wavefront reductions through cross-lane moves and
// one LDS exchange per workgroup.
//
// Arithmetic contract (per element, f32):
//   absmax = max |x|            NaN ignored (v_max_f32 returns the non-NaN)
//   scale  = absmax / 127       IEEE division, correctly rounded
//   code   = clamp(rne(x / scale), -127, 127), NaN -> 0
//   x_hat  = f32(code) * scale
// The division is the correctly rounded one.  The quotient is first estimated
// with x * (1/scale); only when that estimate is too close to a rounding tie
// to decide the integer is the exact division evaluated (see quant_code).
#include <atomic>
#include <mutex>

#include "common.hpp"
#include "quant_device.hpp"

using namespace vtlhip;

namespace {

using namespace vtlhip::qdev;

// Elements of a row that starts at flat element `start` before the next
// multiple of four (where 16-byte loads of f32 and 4-byte stores of codes are
// aligned, the base pointers being aligned), at most the whole row.
__device__ __forceinline__ int row_head(int64_t start, int64_t cols)
{
    const int h = (int)((4 - (start & 3)) & 3);
    return h < cols ? h : (int)cols;
}

// ---- absmax ----------------------------------------------------------------

// A whole-tensor maximum is collected by atomic maxima of the workgroups.  On one address those
// queue up (6 to 7 ns each: 4096 x 4096 took 28 us with 2048 workgroups, against 8.8 us for the
// per-row kernel over the same bytes), so a set of kAbsmaxCells cells 128 bytes apart takes
// them, workgroup b using cell b % kAbsmaxCells, and whoever wants the maximum reads them all.
constexpr int kAbsmaxCells = 64;
constexpr int kCellStride = 32;   // in 4-byte units

// The maximum over a set of cells; every lane of the calling wave gets it.
__device__ __forceinline__ float absmax_of_cells(const unsigned *cells)
{
    return wave_max(__uint_as_float(cells[(threadIdx.x & (kAbsmaxCells - 1)) * kCellStride]));
}


// One workgroup per row, strided loop over the row.
template <int T, int VEC>
__global__ __launch_bounds__(T) void absmax_rows_kernel(const float *__restrict__ x, int64_t cols,
                                                        float *__restrict__ out)
{
    __shared__ float smem[T / 64];
    const int64_t row = blockIdx.x;
    const float *xr = x + row * cols;
    float m = 0.0f;
    if constexpr (VEC == 4) {
        // x is 16-byte aligned; a row of any length starts at most three
        // elements before a 16-byte boundary: scalar head, vector body, scalar tail
        const int head = row_head(row * cols, cols);
        const float4_t *xv = reinterpret_cast<const float4_t *>(xr + head);
        const int64_t nv = (cols - head) >> 2;
        if ((int)threadIdx.x < head)
            m = fabsf(xr[threadIdx.x]);
        if ((int)threadIdx.x < (int)((cols - head) & 3))
            m = fmaxf(m, fabsf(xr[head + (nv << 2) + threadIdx.x]));
        int64_t i = threadIdx.x;
        for (; i + 3 * T < nv; i += 4 * T) {  // four independent loads in flight per lane
            const float4_t v0 = __builtin_nontemporal_load(xv + i);
            const float4_t v1 = __builtin_nontemporal_load(xv + i + T);
            const float4_t v2 = __builtin_nontemporal_load(xv + i + 2 * T);
            const float4_t v3 = __builtin_nontemporal_load(xv + i + 3 * T);
            m = absmax4(absmax4(absmax4(absmax4(m, v0), v1), v2), v3);
        }
        for (; i < nv; i += T)
            m = absmax4(m, xv[i]);
    } else {
        for (int64_t i = threadIdx.x; i < cols; i += T)
            m = fmaxf(m, fabsf(xr[i]));
    }
    m = block_max<T>(m, smem);
    if (threadIdx.x == 0)
        out[row] = m;
}

// A few very long rows (16-byte aligned, a multiple of four long): a row is cut into pieces of
// piece_vecs 16-byte vectors, one workgroup each (block = row * pieces + piece), which meet in
// an atomic max on out_bits[row] (cleared before).  One workgroup per row, as above, leaves
// most of the chip idle there: 16 rows of 2^20 took 98 us.
template <int T>
__global__ __launch_bounds__(T) void absmax_rows_split_kernel(const float *__restrict__ x, int64_t cols,
                                                              unsigned pieces, int64_t piece_vecs,
                                                              unsigned *__restrict__ out_bits)
{
    __shared__ float smem[T / 64];
    const int64_t row = blockIdx.x / pieces;
    const int64_t piece = blockIdx.x % pieces;
    const float4_t *xv = reinterpret_cast<const float4_t *>(x + row * cols);
    const int64_t nv = cols >> 2;
    const int64_t end = (piece + 1) * piece_vecs < nv ? (piece + 1) * piece_vecs : nv;
    float m = 0.0f;
    int64_t i = piece * piece_vecs + threadIdx.x;
    for (; i + 3 * T < end; i += 4 * T) {
        const float4_t v0 = __builtin_nontemporal_load(xv + i);
        const float4_t v1 = __builtin_nontemporal_load(xv + i + T);
        const float4_t v2 = __builtin_nontemporal_load(xv + i + 2 * T);
        const float4_t v3 = __builtin_nontemporal_load(xv + i + 3 * T);
        m = absmax4(absmax4(absmax4(absmax4(m, v0), v1), v2), v3);
    }
    for (; i < end; i += T)
        m = absmax4(m, xv[i]);
    m = block_max<T>(m, smem);
    if (threadIdx.x == 0)
        atomicMax(out_bits + row, __float_as_uint(m));
}

// Whole-tensor absmax: grid-stride pass, one atomic max per workgroup on the
// bit pattern (non-negative floats order like unsigned integers).
// KEEP: ordinary loads, for a tensor that a second pass reads again while the last-level cache
// still holds it; otherwise non-temporal ones.
template <int T, bool KEEP = false>
__global__ __launch_bounds__(T) void absmax_flat_kernel(const float *__restrict__ x, int64_t n,
                                                        int vec_ok, unsigned *__restrict__ out_bits,
                                                        int cells)
{
    __shared__ float smem[T / 64];
    float m = 0.0f;
    const int64_t tid = (int64_t)blockIdx.x * T + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * T;
    if (vec_ok) {
        const float4_t *xv = reinterpret_cast<const float4_t *>(x);
        const int64_t nv = n >> 2;
        int64_t i = tid;
        for (; i + 3 * stride < nv; i += 4 * stride) {
            float4_t v0, v1, v2, v3;
            if constexpr (KEEP) {
                v0 = xv[i];
                v1 = xv[i + stride];
                v2 = xv[i + 2 * stride];
                v3 = xv[i + 3 * stride];
            } else {
                v0 = __builtin_nontemporal_load(xv + i);
                v1 = __builtin_nontemporal_load(xv + i + stride);
                v2 = __builtin_nontemporal_load(xv + i + 2 * stride);
                v3 = __builtin_nontemporal_load(xv + i + 3 * stride);
            }
            m = absmax4(absmax4(absmax4(absmax4(m, v0), v1), v2), v3);
        }
        for (; i < nv; i += stride)
            m = absmax4(m, xv[i]);
        if (tid < (n & 3))
            m = fmaxf(m, fabsf(x[(nv << 2) + tid]));
    } else {
        for (int64_t i = tid; i < n; i += stride)
            m = fmaxf(m, fabsf(x[i]));
    }
    m = block_max<T>(m, smem);
    if (threadIdx.x == 0)
        atomicMax(out_bits + (blockIdx.x % (unsigned)cells) * kCellStride, __float_as_uint(m));
}

__global__ void fill_u32_kernel(unsigned *p, unsigned v, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        p[i] = v;
}

__global__ void scale_from_absmax_kernel(float *inout, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        inout[i] = inout[i] / 127.0f;
}

// One wave: the maximum over a set of cells to *out, and the cells back to zero.
__global__ __launch_bounds__(64) void absmax_cells_reduce_kernel(unsigned *cells, float *out)
{
    const float m = absmax_of_cells(cells);
    cells[threadIdx.x * kCellStride] = 0u;
    if (threadIdx.x == 0)
        *out = m;
}

// ---- fused per-row absmax + quantize ---------------------------------------

// One workgroup per row; the row stays in registers between the absmax pass
// and the quantize pass, so HBM sees 4 bytes in and 1 byte out per element.
// Requires cols % 4 == 0 and cols <= 4 * T * NV.  NT: non-temporal loads and
// stores, for tensors far larger than the caches (16384^2: 209 us against 243 us
// with cached accesses); small tensors that the next kernel reads back are
// better left in the caches (the three-layer chain: 66 us against 69 us).
template <int T, int NV, bool NT>
__global__ __launch_bounds__(T) void quantize_rows_reg_kernel(const float *__restrict__ x,
                                                              int64_t cols, int8_t *__restrict__ q,
                                                              float *__restrict__ scale_out)
{
    __shared__ float smem[T / 64];
    const int64_t row = blockIdx.x;
    const float4_t *xv = reinterpret_cast<const float4_t *>(x + row * cols);
    unsigned *qv = reinterpret_cast<unsigned *>(q + row * cols);
    const int nv = (int)(cols >> 2);

    float4_t v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int idx = i * T + threadIdx.x;
        if (idx < nv)
            v[i] = NT ? __builtin_nontemporal_load(xv + idx) : xv[idx];
        else
            v[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    }
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; i++)
        m = absmax4(m, v[i]);
    m = block_max<T>(m, smem);

    const float scale = m / 127.0f;
    if (threadIdx.x == 0)
        scale_out[row] = scale;
    const QuantScale p = make_quant_scale(scale);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int idx = i * T + threadIdx.x;
        if (idx < nv) {
            if (NT)
                __builtin_nontemporal_store(quant4(v[i], p), qv + idx);
            else
                qv[idx] = quant4(v[i], p);
        }
    }
}

// Rows too long for registers, or not a multiple of four: two passes over the
// row inside one workgroup (the second pass mostly hits L2 / MALL).  T >= 4.
// Many short rows (cols % 4 == 0, cols <= 4 * SEG, 16-byte aligned): SEG = 16, 32 or 64 lanes
// hold a row, one 16-byte vector each, and a workgroup of 256 threads takes 256 / SEG rows.  A
// workgroup of one wave per row, as the kernel above does it for up to 256 columns, is bound by
// the rate at which workgroups start when there are this many rows (262144 rows of 16 or of
// 64: 59 us against 10.5 and 14.8 us; of 132: 75 us).
// QUANT false: only the rows' absmax, to scale_out.
template <int SEG, bool QUANT>
__global__ __launch_bounds__(256) void short_rows_kernel(const float *__restrict__ x, int64_t rows, int cols,
                                                         int8_t *__restrict__ q, float *__restrict__ scale_out)
{
    const int lane = (int)threadIdx.x % SEG;
    const int64_t row = (int64_t)blockIdx.x * (256 / SEG) + (int)threadIdx.x / SEG;
    const int nv = cols >> 2;
    const bool live = row < rows && lane < nv;
    const int64_t at = row * nv + lane;
    float4_t v = float4_t{0.f, 0.f, 0.f, 0.f};
    if (live)
        v = reinterpret_cast<const float4_t *>(x)[at];
    const float m = segment_max<SEG>(absmax4(0.0f, v));
    if constexpr (QUANT) {
        const float scale = m / 127.0f;
        if (lane == 0 && row < rows)
            scale_out[row] = scale;
        const QuantScale p = make_quant_scale(scale);
        if (live)
            reinterpret_cast<unsigned *>(q)[at] = quant4(v, p);
    } else {
        if (lane == 0 && row < rows)
            scale_out[row] = m;
    }
}

template <int T, int VEC>
__global__ __launch_bounds__(T) void quantize_rows_loop_kernel(const float *__restrict__ x,
                                                               int64_t cols, int8_t *__restrict__ q,
                                                               float *__restrict__ scale_out)
{
    __shared__ float smem[T / 64];
    const int64_t row = blockIdx.x;
    const float *xr = x + row * cols;
    int8_t *qr = q + row * cols;
    float m = 0.0f;
    // VEC == 4: x is 16-byte and q 4-byte aligned; scalar head up to the next
    // multiple of four of the flat index, vector body, scalar tail
    const int head = VEC == 4 ? row_head(row * cols, cols) : 0;
    const int64_t nv = (cols - head) >> 2;
    const int tail = (int)((cols - head) & 3);
    if constexpr (VEC == 4) {
        const float4_t *xv = reinterpret_cast<const float4_t *>(xr + head);
        if ((int)threadIdx.x < head)
            m = fabsf(xr[threadIdx.x]);
        if ((int)threadIdx.x < tail)
            m = fmaxf(m, fabsf(xr[head + (nv << 2) + threadIdx.x]));
        for (int64_t i = threadIdx.x; i < nv; i += T)
            m = absmax4(m, xv[i]);
    } else {
        for (int64_t i = threadIdx.x; i < cols; i += T)
            m = fmaxf(m, fabsf(xr[i]));
    }
    m = block_max<T>(m, smem);
    const float scale = m / 127.0f;
    if (threadIdx.x == 0)
        scale_out[row] = scale;
    const QuantScale p = make_quant_scale(scale);
    if constexpr (VEC == 4) {
        const float4_t *xv = reinterpret_cast<const float4_t *>(xr + head);
        unsigned *qv = reinterpret_cast<unsigned *>(qr + head);
        if ((int)threadIdx.x < head)
            qr[threadIdx.x] = (int8_t)quant_code(xr[threadIdx.x], p);
        if ((int)threadIdx.x < tail) {
            const int64_t i = head + (nv << 2) + threadIdx.x;
            qr[i] = (int8_t)quant_code(xr[i], p);
        }
        for (int64_t i = threadIdx.x; i < nv; i += T)
            qv[i] = quant4(xv[i], p);
    } else {
        for (int64_t i = threadIdx.x; i < cols; i += T)
            qr[i] = (int8_t)quant_code(xr[i], p);
    }
}

// ---- quantize with scales already on the device ----------------------------

// One workgroup per chunk of 4 * T * NV elements (VEC == 4) or T * NV
// (VEC == 1).  The grid is one-dimensional and chunk-major (block = row *
// chunks_per_row + chunk), so that workgroups dispatched back to back touch
// adjacent memory; per_row == 0 treats the tensor as one row of `cols` elements.
// FROM_ABSMAX (whole tensor only): `scale` points at a set of cells as absmax_flat_kernel
// leaves them; every workgroup derives the scale from their maximum, the first also stores the
// scale to scale_out and clears the set clear_cells (the one the next such call on this stream
// will collect its absmax in).
template <int T, int NV, int VEC, bool FROM_ABSMAX = false>
__global__ __launch_bounds__(T) void quantize_scaled_kernel(const float *__restrict__ x,
                                                            const float *__restrict__ scale,
                                                            int per_row, int64_t cols,
                                                            unsigned chunks_per_row,
                                                            int8_t *__restrict__ q,
                                                            float *__restrict__ scale_out = nullptr,
                                                            unsigned *__restrict__ clear_cells = nullptr)
{
    const int64_t row = per_row ? (int64_t)(blockIdx.x / chunks_per_row) : 0;
    const int64_t chunk = per_row ? (int64_t)(blockIdx.x % chunks_per_row) : (int64_t)blockIdx.x;
    const float *xr = x + row * cols;
    int8_t *qr = q + row * cols;
    float row_scale;
    if constexpr (FROM_ABSMAX) {
        row_scale = absmax_of_cells(reinterpret_cast<const unsigned *>(scale)) / 127.0f;
        if (blockIdx.x == 0 && threadIdx.x < kAbsmaxCells) {
            clear_cells[threadIdx.x * kCellStride] = 0u;
            if (threadIdx.x == 0)
                *scale_out = row_scale;
        }
    } else {
        row_scale = scale[row];
    }
    const QuantScale p = make_quant_scale(row_scale);
    if constexpr (VEC == 4) {
        const float4_t *xv = reinterpret_cast<const float4_t *>(xr);
        unsigned *qv = reinterpret_cast<unsigned *>(qr);
        const int64_t nv = cols >> 2;
        const int64_t base = chunk * (T * NV);
        float4_t v[NV];
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int64_t idx = base + i * T + threadIdx.x;
            if (idx < nv)
                v[i] = __builtin_nontemporal_load(xv + idx);
        }
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int64_t idx = base + i * T + threadIdx.x;
            if (idx < nv)
                __builtin_nontemporal_store(quant4(v[i], p), qv + idx);
        }
        // ragged tail of a flat tensor (cols % 4 elements)
        if (chunk == 0 && threadIdx.x < (cols & 3)) {
            const int64_t idx = (nv << 2) + threadIdx.x;
            qr[idx] = (int8_t)quant_code(xr[idx], p);
        }
    } else {
        const int64_t base = chunk * (T * NV);
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int64_t idx = base + i * T + threadIdx.x;
            if (idx < cols)
                qr[idx] = (int8_t)quant_code(xr[idx], p);
        }
    }
}

// Per-row scales over a matrix walked as ONE flat run of 16-byte vectors, each
// element looking up its row: for rows shorter than a workgroup's chunk (one
// workgroup per row would leave most lanes idle: 262144 rows of 256 ran at
// 1.3 TB/s) and for row lengths that are no multiple of four (rows then start
// at any alignment, the flat run does not).  cols >= 4, so a vector touches at
// most two rows.  The workgroup divides once in 64 bits, its lanes in 32.
struct FlatRows {
    int64_t base;   // first vector of the workgroup
    int64_t row_b;  // row of its first element
    unsigned off_b; // column of its first element
};

template <int T, int NV>
__device__ __forceinline__ FlatRows flat_rows_origin(unsigned cols)
{
    FlatRows f;
    f.base = (int64_t)blockIdx.x * (T * NV);
    const int64_t e = f.base << 2;
    f.row_b = e / cols;
    f.off_b = (unsigned)(e - f.row_b * cols);
    return f;
}

// Row and column of the first element of vector `local` of the workgroup.
__device__ __forceinline__ void flat_rows_locate(const FlatRows &f, unsigned cols, unsigned local, int64_t &row,
                                                 unsigned &col)
{
    const unsigned e = f.off_b + 4u * local;
    const unsigned r = e / cols;
    row = f.row_b + r;
    col = e - r * cols;
}

template <int T, int NV>
__global__ __launch_bounds__(T) void quantize_scaled_flat_rows_kernel(const float *__restrict__ x,
                                                                      const float *__restrict__ scale,
                                                                      unsigned cols, int64_t n,
                                                                      int8_t *__restrict__ q)
{
    const FlatRows f = flat_rows_origin<T, NV>(cols);
    const int64_t nv_total = n >> 2;
    const float4_t *xv = reinterpret_cast<const float4_t *>(x);
    unsigned *qv = reinterpret_cast<unsigned *>(q);
    float4_t v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int64_t idx = f.base + i * T + threadIdx.x;
        if (idx < nv_total)
            v[i] = __builtin_nontemporal_load(xv + idx);
    }
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int64_t idx = f.base + i * T + threadIdx.x;
        if (idx < nv_total) {
            int64_t row;
            unsigned col;
            flat_rows_locate(f, cols, (unsigned)(i * T) + threadIdx.x, row, col);
            const QuantScale p = make_quant_scale(scale[row]);
            unsigned packed;
            if (col + 4 <= cols) {
                packed = quant4(v[i], p);
            } else {  // the vector runs into the next row
                const QuantScale p1 = make_quant_scale(scale[row + 1]);
                const unsigned in0 = cols - col;  // 1..3 elements still in `row`
                packed = 0;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    packed |= (unsigned)(uint8_t)(int8_t)quant_code(v[i][e], (unsigned)e < in0 ? p : p1) << (8 * e);
            }
            __builtin_nontemporal_store(packed, qv + idx);
        }
    }
    // the last n % 4 elements of the matrix belong to its last row
    if (blockIdx.x == 0 && threadIdx.x < (unsigned)(n & 3)) {
        const int64_t i = (nv_total << 2) + threadIdx.x;
        q[i] = (int8_t)quant_code(x[i], make_quant_scale(scale[(n - 1) / cols]));
    }
}

template <int T, int NV>
__global__ __launch_bounds__(T) void dequantize_flat_rows_kernel(const int8_t *__restrict__ q,
                                                                 const float *__restrict__ scale, unsigned cols,
                                                                 int64_t n, float *__restrict__ x)
{
    const FlatRows f = flat_rows_origin<T, NV>(cols);
    const int64_t nv_total = n >> 2;
    const unsigned *qv = reinterpret_cast<const unsigned *>(q);
    float4_t *xv = reinterpret_cast<float4_t *>(x);
    unsigned c[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int64_t idx = f.base + i * T + threadIdx.x;
        c[i] = (idx < nv_total) ? __builtin_nontemporal_load(qv + idx) : 0u;
    }
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int64_t idx = f.base + i * T + threadIdx.x;
        if (idx < nv_total) {
            int64_t row;
            unsigned col;
            flat_rows_locate(f, cols, (unsigned)(i * T) + threadIdx.x, row, col);
            const float s0 = scale[row];
            const unsigned in0 = cols - col;  // elements of the vector still in `row` (>= 4: all)
            const float s1 = in0 < 4 ? scale[row + 1] : s0;
            const unsigned w = c[i];
            float4_t o;
            o.x = (float)((int)(w << 24) >> 24) * s0;
            o.y = (float)((int)(w << 16) >> 24) * (in0 > 1 ? s0 : s1);
            o.z = (float)((int)(w << 8) >> 24) * (in0 > 2 ? s0 : s1);
            o.w = (float)((int)w >> 24) * (in0 > 3 ? s0 : s1);
            __builtin_nontemporal_store(o, xv + idx);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < (unsigned)(n & 3)) {
        const int64_t i = (nv_total << 2) + threadIdx.x;
        x[i] = (float)q[i] * scale[(n - 1) / cols];
    }
}

// ---- dequantize -------------------------------------------------------------

// Same chunk-major block indexing as quantize_scaled_kernel.  Each lane reads four codes
// (4 bytes) and writes one 16-byte vector, so both sides stay coalesced.
template <int T, int NV, int VEC>
__global__ __launch_bounds__(T) void dequantize_kernel(const int8_t *__restrict__ q,
                                                       const float *__restrict__ scale, int per_row,
                                                       int64_t cols, unsigned chunks_per_row,
                                                       float *__restrict__ x)
{
    const int64_t row = per_row ? (int64_t)(blockIdx.x / chunks_per_row) : 0;
    const int64_t chunk = per_row ? (int64_t)(blockIdx.x % chunks_per_row) : (int64_t)blockIdx.x;
    const int8_t *qr = q + row * cols;
    float *xr = x + row * cols;
    const float s = scale[row];
    if constexpr (VEC == 4) {
        const unsigned *qv = reinterpret_cast<const unsigned *>(qr);
        float4_t *xv = reinterpret_cast<float4_t *>(xr);
        const int64_t nv = cols >> 2;
        const int64_t base = chunk * (T * NV);
        unsigned c[NV];
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int64_t idx = base + i * T + threadIdx.x;
            c[i] = (idx < nv) ? __builtin_nontemporal_load(qv + idx) : 0u;
        }
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int64_t idx = base + i * T + threadIdx.x;
            if (idx < nv) {
                const unsigned w = c[i];
                float4_t o;
                o.x = (float)((int)(w << 24) >> 24) * s;
                o.y = (float)((int)(w << 16) >> 24) * s;
                o.z = (float)((int)(w << 8) >> 24) * s;
                o.w = (float)((int)w >> 24) * s;
                __builtin_nontemporal_store(o, xv + idx);
            }
        }
        if (chunk == 0 && threadIdx.x < (cols & 3)) {
            const int64_t idx = (nv << 2) + threadIdx.x;
            xr[idx] = (float)qr[idx] * s;
        }
    } else {
        const int64_t base = chunk * (T * NV);
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int64_t idx = base + i * T + threadIdx.x;
            if (idx < cols)
                xr[idx] = (float)qr[idx] * s;
        }
    }
}

// ---- ReLU --------------------------------------------------------------------

__global__ __launch_bounds__(256) void relu_kernel(float *__restrict__ x, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) {
        const float v = x[i];
        if (v < 0.0f)  // NaN and -0.0 pass through, as on the CPU path
            x[i] = 0.0f;
    }
}

// Plain streaming copy, one 16-byte vector per lane; also the kernel of known
// traffic that hardware byte counters are calibrated against.
__global__ __launch_bounds__(256) void copy_kernel(const float4_t *__restrict__ src,
                                                   float4_t *__restrict__ dst, int64_t nv)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < nv)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

constexpr int64_t kMaxGridX = 2147483647LL;

int check_2d(const void *a, const void *b, int64_t rows, int64_t cols)
{
    if (!a || !b || rows < 0 || cols < 0)
        return VTL_HIP_ERR_INVALID_ARG;
    if (rows > kMaxGridX)
        return VTL_HIP_ERR_UNSUPPORTED;
    if (cols > 0 && rows > INT64_MAX / cols)
        return VTL_HIP_ERR_INVALID_ARG;
    return VTL_HIP_OK;
}

// Whole-tensor quantization in two launches.  The absmax pass needs cells that hold zero when
// it starts and the quantize pass must find the maximum in them: a cell in the caller's
// scale_out would have to be cleared by a launch of its own and turned into the scale by
// another.  Instead every stream index (vtlhip::stream_slot) owns two sets of cells in device
// memory that the library uses in turn: a call collects its maximum in one, and its quantize
// pass clears the other for the next call on that stream, whose launches come later in stream
// order.  (vtl_hip_absmax_f32 uses the set whose turn it is and clears it itself.)  All cells
// start as zero.  A call whose launches fail leaves the sets in an unknown state: the index
// then goes back to the forms that use the caller's memory only, for good.
constexpr int kCellSet = kAbsmaxCells * kCellStride;
__device__ unsigned g_absmax_cells[vtlhip::kStreamSlots * 2 * kCellSet];

struct AbsmaxCells {
    std::mutex lock;
    std::atomic<unsigned *> base{nullptr};   // device address of this device's g_absmax_cells
    unsigned char turn[vtlhip::kStreamSlots] = {};
    bool unusable[vtlhip::kStreamSlots] = {};
};

AbsmaxCells *absmax_cells_of_device()
{
    static AbsmaxCells cells[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)hipGetLastError();
        return nullptr;
    }
    AbsmaxCells &c = cells[dev];
    if (!c.base.load(std::memory_order_acquire)) {
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_absmax_cells)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        c.base.store(static_cast<unsigned *>(ptr), std::memory_order_release);
    }
    return &c;
}

// max |x| over n > 0 elements into a set of kAbsmaxCells cells that hold zero (the bits of a
// non-negative float).
int launch_absmax_cells(const float *x, int64_t n, unsigned *cells, bool keep_cached, hipStream_t s)
{
    // Up to 8 M elements: workgroups of 256 threads with 128 bytes per thread (1024 x 4096: 7.5
    // against 8.8 us for the form below).  Beyond: at most two workgroups of 1024 threads per
    // compute unit, which stream better (16384 x 16384: 372 against 424 us).
    const int vec_ok = aligned(x, 16) ? 1 : 0;
    const int64_t small = (n / 4 + 256 * 8 - 1) / (256 * 8);
    if (small <= 1024) {
        const dim3 grid((unsigned)(small < 1 ? 1 : small));
        if (keep_cached)
            hipLaunchKernelGGL((absmax_flat_kernel<256, true>), grid, dim3(256), 0, s, x, n, vec_ok, cells,
                               kAbsmaxCells);
        else
            hipLaunchKernelGGL((absmax_flat_kernel<256, false>), grid, dim3(256), 0, s, x, n, vec_ok, cells,
                               kAbsmaxCells);
    } else {
        int64_t blocks = (n / 4 + 1024 * 4 - 1) / (1024 * 4);
        if (blocks > 512)
            blocks = 512;
        if (keep_cached)
            hipLaunchKernelGGL((absmax_flat_kernel<1024, true>), dim3((unsigned)blocks), dim3(1024), 0, s, x, n,
                               vec_ok, cells, kAbsmaxCells);
        else
            hipLaunchKernelGGL((absmax_flat_kernel<1024, false>), dim3((unsigned)blocks), dim3(1024), 0, s, x, n,
                               vec_ok, cells, kAbsmaxCells);
    }
    return check_launch("absmax_flat_kernel");
}

// The same into the single cell *cell (caller's memory, cleared before).
int launch_absmax_flat(const float *x, int64_t n, unsigned *cell, hipStream_t s)
{
    // One address for every workgroup's atomic maximum: few, large workgroups (at most two of
    // 1024 threads per compute unit), small ones only while there are at most 512 of them.
    const int vec_ok = aligned(x, 16) ? 1 : 0;
    const int64_t small = (n / 4 + 256 * 4 - 1) / (256 * 4);
    if (small <= 512) {
        hipLaunchKernelGGL((absmax_flat_kernel<256, false>), dim3((unsigned)(small < 1 ? 1 : small)), dim3(256), 0, s,
                           x, n, vec_ok, cell, 1);
    } else {
        int64_t blocks = (n / 4 + 1024 * 4 - 1) / (1024 * 4);
        if (blocks > 512)
            blocks = 512;
        hipLaunchKernelGGL((absmax_flat_kernel<1024, false>), dim3((unsigned)blocks), dim3(1024), 0, s, x, n, vec_ok,
                           cell, 1);
    }
    return check_launch("absmax_flat_kernel");
}

int launch_fill_zero(float *p, int64_t n, hipStream_t st);

// Rows so few and so long that one workgroup per row leaves most compute units idle (measured:
// from 131072 columns on with up to 128 rows, the forms that cut a row into pieces win; 16 rows
// of 2^20: absmax 98 -> 12 us, quantize 211 -> 36 us).
inline bool few_long_rows(const float *x, int64_t rows, int64_t cols)
{
    return rows <= 128 && cols >= 131072 && cols % 4 == 0 && aligned(x, 16);
}

// Per-row absmax of such rows into out[rows]: clear, then the pieces' atomic maxima.
int launch_absmax_rows_split(const float *x, int64_t rows, int64_t cols, float *out, hipStream_t s)
{
    int st = launch_fill_zero(out, rows, s);
    if (st != VTL_HIP_OK)
        return st;
    // About 512 workgroups of 1024 threads in all (two per compute unit), a piece a multiple of
    // what a workgroup loads per step: the rows' maxima share a cache line or two, on which the
    // atomic maxima queue up (2048 workgroups of 256 threads: 32 us for 64 MiB, this: 12 us).
    constexpr int T = 1024;
    const int64_t step = 4 * T;
    const int64_t share = (rows * (cols >> 2) + 511) / 512;
    const int64_t piece_vecs = (share + step - 1) / step * step;
    const int64_t pieces = ((cols >> 2) + piece_vecs - 1) / piece_vecs;
    if (pieces * rows > kMaxGridX)
        return VTL_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((absmax_rows_split_kernel<T>), dim3((unsigned)(pieces * rows)), dim3(T), 0, s, x, cols,
                       (unsigned)pieces, piece_vecs, reinterpret_cast<unsigned *>(out));
    return check_launch("absmax_rows_split_kernel");
}

int launch_fill_zero(float *p, int64_t n, hipStream_t st)
{
    const int64_t blocks = (n + 255) / 256;
    hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, st,
                       reinterpret_cast<unsigned *>(p), 0u, n);
    return check_launch("fill_u32_kernel");
}

}  // namespace

namespace vtlhip {

// Device-to-device copy with the library's own kernel (16-byte aligned, size a
// multiple of 16); returns false when the shape does not qualify.
bool launch_copy(void *dst, const void *src, size_t bytes, hipStream_t st)
{
    if (!aligned(dst, 16) || !aligned(src, 16) || (bytes & 15))
        return false;
    const int64_t nv = (int64_t)(bytes >> 4);
    const int64_t blocks = (nv + 255) / 256;
    if (blocks > kMaxGridX)
        return false;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, st,
                       reinterpret_cast<const float4_t *>(src), reinterpret_cast<float4_t *>(dst), nv);
    return true;
}

// Per-row fused quantize; used by the C entry point and by the dynamic-quant
// linear.  Preconditions were checked by the caller.
int launch_quantize_rows(const float *x, int64_t rows, int64_t cols, int8_t *q, float *scale_out,
                         hipStream_t st)
{
    if (rows == 0)
        return VTL_HIP_OK;
    if (cols == 0)
        return launch_fill_zero(scale_out, rows, st);
    const bool vec = (cols % 4 == 0) && aligned(x, 16) && aligned(q, 4);
    const dim3 grid((unsigned)rows);
    const bool nt = rows * cols > ((int64_t)16 << 20);  // more than 64 MiB of f32
#define VTL_Q_REG(T, NV)                                                                               \
    do {                                                                                               \
        if (nt)                                                                                        \
            hipLaunchKernelGGL((quantize_rows_reg_kernel<T, NV, true>), grid, dim3(T), 0, st, x, cols, q, \
                               scale_out);                                                             \
        else                                                                                           \
            hipLaunchKernelGGL((quantize_rows_reg_kernel<T, NV, false>), grid, dim3(T), 0, st, x, cols, q, \
                               scale_out);                                                             \
    } while (0)
    // many short rows: several rows per wave
    if (vec && cols <= 256 && rows >= 4096) {
        // (ordinary loads and stores whatever the size: rows that are no whole cache lines make
        // non-temporal stores slower, 262144 rows of 160: 61 against 48 us)
        if (cols <= 64)
            hipLaunchKernelGGL((short_rows_kernel<16, true>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, x,
                               rows, (int)cols, q, scale_out);
        else if (cols <= 128)
            hipLaunchKernelGGL((short_rows_kernel<32, true>), dim3((unsigned)((rows + 7) / 8)), dim3(256), 0, st, x,
                               rows, (int)cols, q, scale_out);
        else
            hipLaunchKernelGGL((short_rows_kernel<64, true>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, x,
                               rows, (int)cols, q, scale_out);
        return check_launch("short_rows_kernel");
    }
    // Workgroup sizes measured best per row length: one wave while the row
    // fits a wave's registers (no LDS, no barrier), 256 threads up to 4096
    // columns, 512 up to 8192, 1024 beyond (e.g. 65536 rows of 4096: 303 us
    // with 1024 threads a row, 210 us with 256).
    if (vec && cols <= 4 * 64 * 1)
        VTL_Q_REG(64, 1);
    else if (vec && cols <= 4 * 64 * 2)
        VTL_Q_REG(64, 2);
    else if (vec && cols <= 4 * 64 * 4)
        VTL_Q_REG(64, 4);
    else if (vec && cols <= 4 * 256 * 2)
        VTL_Q_REG(256, 2);
    else if (vec && cols <= 4 * 256 * 4)
        VTL_Q_REG(256, 4);
    else if (vec && cols <= 4 * 512 * 4)
        VTL_Q_REG(512, 4);
    else if (vec && cols <= 4 * 1024 * 4)
        VTL_Q_REG(1024, 4);
    else if (vec && cols <= 4 * 1024 * 16)
        VTL_Q_REG(1024, 16);
    else if (aligned(x, 16) && aligned(q, 4) && cols > 4 * 256 * 4)
        hipLaunchKernelGGL((quantize_rows_loop_kernel<1024, 4>), grid, dim3(1024), 0, st, x, cols, q,
                           scale_out);
    else if (aligned(x, 16) && aligned(q, 4) && cols >= 1024)
        hipLaunchKernelGGL((quantize_rows_loop_kernel<256, 4>), grid, dim3(256), 0, st, x, cols, q,
                           scale_out);
    else if (aligned(x, 16) && aligned(q, 4) && cols >= 16)
        hipLaunchKernelGGL((quantize_rows_loop_kernel<64, 4>), grid, dim3(64), 0, st, x, cols, q,
                           scale_out);
    else
        hipLaunchKernelGGL((quantize_rows_loop_kernel<256, 1>), grid, dim3(256), 0, st, x, cols, q,
                           scale_out);
#undef VTL_Q_REG
    return check_launch("quantize_rows");
}

}  // namespace vtlhip

extern "C" {

int vtl_hip_absmax_f32(const float *x, int64_t rows, int64_t cols, int per_row, float *absmax_out)
{
    int st = check_2d(x, absmax_out, rows, cols);
    if (st != VTL_HIP_OK)
        return st;
    hipStream_t s = current_stream();
    if (per_row) {
        if (rows == 0)
            return VTL_HIP_OK;
        if (cols == 0)
            return launch_fill_zero(absmax_out, rows, s);
        if (few_long_rows(x, rows, cols))
            return launch_absmax_rows_split(x, rows, cols, absmax_out, s);
        if (aligned(x, 16) && cols % 4 == 0 && cols <= 256 && rows >= 4096) {   // many short rows
            if (cols <= 64)
                hipLaunchKernelGGL((short_rows_kernel<16, false>), dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, s,
                                   x, rows, (int)cols, nullptr, absmax_out);
            else if (cols <= 128)
                hipLaunchKernelGGL((short_rows_kernel<32, false>), dim3((unsigned)((rows + 7) / 8)), dim3(256), 0, s,
                                   x, rows, (int)cols, nullptr, absmax_out);
            else
                hipLaunchKernelGGL((short_rows_kernel<64, false>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s,
                                   x, rows, (int)cols, nullptr, absmax_out);
            return check_launch("short_rows_kernel");
        }
        const bool vec = aligned(x, 16);  // any row length: the kernel peels to the next 16-byte boundary
        if (vec && cols >= 8192)
            hipLaunchKernelGGL((absmax_rows_kernel<512, 4>), dim3((unsigned)rows), dim3(512), 0, s, x,
                               cols, absmax_out);
        else if (vec && cols >= 1024)
            hipLaunchKernelGGL((absmax_rows_kernel<256, 4>), dim3((unsigned)rows), dim3(256), 0, s, x,
                               cols, absmax_out);
        else if (vec)
            hipLaunchKernelGGL((absmax_rows_kernel<64, 4>), dim3((unsigned)rows), dim3(64), 0, s, x,
                               cols, absmax_out);
        else
            hipLaunchKernelGGL((absmax_rows_kernel<256, 1>), dim3((unsigned)rows), dim3(256), 0, s, x,
                               cols, absmax_out);
        return check_launch("absmax_rows_kernel");
    }
    const int64_t n = rows * cols;
    if (n > 0) {
        // into the stream's cells, then one wave takes their maximum to absmax_out and clears them
        const int slot = tuning().quant_four_launches ? -1 : vtlhip::stream_slot(s);
        AbsmaxCells *cells = slot >= 0 ? absmax_cells_of_device() : nullptr;
        if (cells) {
            std::lock_guard<std::mutex> hold(cells->lock);
            if (!cells->unusable[slot]) {
                unsigned *mine = cells->base.load(std::memory_order_acquire) +
                                 (slot * 2 + cells->turn[slot]) * kCellSet;
                st = launch_absmax_cells(x, n, mine, false, s);
                if (st == VTL_HIP_OK) {
                    hipLaunchKernelGGL(absmax_cells_reduce_kernel, dim3(1), dim3(64), 0, s, mine, absmax_out);
                    st = check_launch("absmax_cells_reduce_kernel");
                }
                if (st != VTL_HIP_OK)
                    cells->unusable[slot] = true;
                return st;
            }
        }
    }
    st = launch_fill_zero(absmax_out, 1, s);
    if (st != VTL_HIP_OK)
        return st;
    if (n == 0)
        return VTL_HIP_OK;
    return launch_absmax_flat(x, n, reinterpret_cast<unsigned *>(absmax_out), s);
}

int vtl_hip_quantize_with_scale_f32_i8(const float *x, const float *scale, int64_t rows,
                                       int64_t cols, int per_row, int8_t *q)
{
    int st = check_2d(x, q, rows, cols);
    if (st != VTL_HIP_OK)
        return st;
    if (!scale)
        return VTL_HIP_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0)
        return VTL_HIP_OK;
    hipStream_t s = current_stream();
    constexpr int T = 512, NV = 2;
    const int64_t row_len = per_row ? cols : rows * cols;
    const bool vec = aligned(x, 16) && aligned(q, 4) && (!per_row || cols % 4 == 0);
    const int64_t per_chunk = vec ? 4 * T * NV : T * NV;
    if (per_row && rows > 1 && cols >= 4 && cols < ((int64_t)1 << 31) - 4 * T * NV && aligned(x, 16) &&
        aligned(q, 4) && (cols < 4 * T * NV || cols % 4 != 0)) {
        const int64_t n = rows * cols;
        const int64_t nblocks = ((n >> 2) + T * NV - 1) / (T * NV);
        if (nblocks > kMaxGridX)
            return VTL_HIP_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((quantize_scaled_flat_rows_kernel<T, NV>), dim3((unsigned)(nblocks > 0 ? nblocks : 1)),
                           dim3(T), 0, s, x, scale, (unsigned)cols, n, q);
        return check_launch("quantize_scaled_flat_rows_kernel");
    }
    const int64_t chunks = (row_len + per_chunk - 1) / per_chunk;
    const int64_t blocks = per_row ? rows * chunks : chunks;
    if (chunks > kMaxGridX || blocks > kMaxGridX)
        return VTL_HIP_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)blocks);
    if (vec)
        hipLaunchKernelGGL((quantize_scaled_kernel<T, NV, 4>), grid, dim3(T), 0, s, x, scale,
                           per_row ? 1 : 0, row_len, (unsigned)chunks, q);
    else
        hipLaunchKernelGGL((quantize_scaled_kernel<T, NV, 1>), grid, dim3(T), 0, s, x, scale,
                           per_row ? 1 : 0, row_len, (unsigned)chunks, q);
    return check_launch("quantize_scaled_kernel");
}

int vtl_hip_quantize_f32_i8(const float *x, int64_t rows, int64_t cols, int per_row, int8_t *q,
                            float *scale_out)
{
    int st = check_2d(x, q, rows, cols);
    if (st != VTL_HIP_OK)
        return st;
    if (!scale_out)
        return VTL_HIP_ERR_INVALID_ARG;
    hipStream_t s = current_stream();
    if (per_row && few_long_rows(x, rows, cols) && aligned(q, 4)) {
        // a few very long rows: absmax by pieces, scales in place, then the chunked quantize pass
        st = launch_absmax_rows_split(x, rows, cols, scale_out, s);
        if (st != VTL_HIP_OK)
            return st;
        hipLaunchKernelGGL(scale_from_absmax_kernel, dim3((unsigned)((rows + 63) / 64)), dim3(64), 0, s, scale_out,
                           rows);
        st = check_launch("scale_from_absmax_kernel");
        if (st != VTL_HIP_OK)
            return st;
        return vtl_hip_quantize_with_scale_f32_i8(x, scale_out, rows, cols, 1, q);
    }
    if (per_row)
        return launch_quantize_rows(x, rows, cols, q, scale_out, s);
    // a small tensor is one "row" of the fused kernel: a single workgroup holds it
    // in registers between the absmax and the rounding pass, one launch instead of four
    const int64_t total = rows * cols;
    if (total > 0 && total <= 4 * 1024 * 16 && total % 4 == 0 && aligned(x, 16) && aligned(q, 4))
        return launch_quantize_rows(x, 1, total, q, scale_out, s);
    if (total > 0 && total <= ((int64_t)1 << 24)) {
        // whole tensor in two launches: absmax into one of the stream's two sets of cells, then
        // the quantize pass, whose workgroups derive the scale from them (1024 x 1024: 6.0
        // against 10.8 us for the four launches below, 4096 x 4096: 24.6 against 32.6 us).  Up
        // to 16 M elements: beyond, reading the cells in every workgroup costs more than the two
        // launches (8192 x 8192: 106 against 98 us).
        const int slot = tuning().quant_four_launches ? -1 : vtlhip::stream_slot(s);
        AbsmaxCells *cells = slot >= 0 ? absmax_cells_of_device() : nullptr;
        constexpr int T = 512, NV = 2;
        const bool vec = aligned(x, 16) && aligned(q, 4);
        const int64_t per_chunk = vec ? 4 * T * NV : T * NV;
        const int64_t chunks = (total + per_chunk - 1) / per_chunk;
        if (cells && chunks <= kMaxGridX) {
            std::lock_guard<std::mutex> hold(cells->lock);
            if (!cells->unusable[slot]) {
                unsigned *pair = cells->base.load(std::memory_order_acquire) + slot * 2 * kCellSet;
                unsigned *mine = pair + cells->turn[slot] * kCellSet;
                unsigned *next = pair + (cells->turn[slot] ^ 1) * kCellSet;
                // (ordinary loads: the second pass finds the tensor in the last-level cache)
                st = launch_absmax_cells(x, total, mine, true, s);
                if (st == VTL_HIP_OK) {
                    const dim3 grid((unsigned)chunks);
                    if (vec)
                        hipLaunchKernelGGL((quantize_scaled_kernel<T, NV, 4, true>), grid, dim3(T), 0, s, x,
                                           reinterpret_cast<const float *>(mine), 0, total, (unsigned)chunks, q,
                                           scale_out, next);
                    else
                        hipLaunchKernelGGL((quantize_scaled_kernel<T, NV, 1, true>), grid, dim3(T), 0, s, x,
                                           reinterpret_cast<const float *>(mine), 0, total, (unsigned)chunks, q,
                                           scale_out, next);
                    st = check_launch("quantize_scaled_kernel");
                }
                if (st == VTL_HIP_OK)
                    cells->turn[slot] ^= 1;
                else
                    cells->unusable[slot] = true;
                return st;
            }
        }
    }
    // whole tensor: absmax pass, scale in place, then the scaled quantize pass
    st = vtl_hip_absmax_f32(x, rows, cols, 0, scale_out);
    if (st != VTL_HIP_OK)
        return st;
    hipLaunchKernelGGL(scale_from_absmax_kernel, dim3(1), dim3(64), 0, s, scale_out, (int64_t)1);
    st = check_launch("scale_from_absmax_kernel");
    if (st != VTL_HIP_OK)
        return st;
    return vtl_hip_quantize_with_scale_f32_i8(x, scale_out, rows, cols, 0, q);
}

int vtl_hip_dequantize_i8_f32(const int8_t *q, const float *scale, int64_t rows, int64_t cols,
                              int per_row, float *x)
{
    int st = check_2d(q, x, rows, cols);
    if (st != VTL_HIP_OK)
        return st;
    if (!scale)
        return VTL_HIP_ERR_INVALID_ARG;
    if (rows == 0 || cols == 0)
        return VTL_HIP_OK;
    hipStream_t s = current_stream();
    // Write-dominated: small chunk-major workgroups (16 KiB of output each) keep
    // the stores of workgroups in flight adjacent in memory; measured best.
    constexpr int T = 512, NV = 2;
    const int64_t row_len = per_row ? cols : rows * cols;
    const bool vec = aligned(x, 16) && aligned(q, 4) && (!per_row || cols % 4 == 0);
    const int64_t per_chunk = vec ? 4 * T * NV : T * NV;
    if (per_row && rows > 1 && cols >= 4 && cols < ((int64_t)1 << 31) - 4 * T * NV && aligned(x, 16) &&
        aligned(q, 4) && (cols < 4 * T * NV || cols % 4 != 0)) {
        const int64_t n = rows * cols;
        const int64_t nblocks = ((n >> 2) + T * NV - 1) / (T * NV);
        if (nblocks > kMaxGridX)
            return VTL_HIP_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((dequantize_flat_rows_kernel<T, NV>), dim3((unsigned)(nblocks > 0 ? nblocks : 1)),
                           dim3(T), 0, s, q, scale, (unsigned)cols, n, x);
        return check_launch("dequantize_flat_rows_kernel");
    }
    const int64_t chunks = (row_len + per_chunk - 1) / per_chunk;
    const int64_t blocks = per_row ? rows * chunks : chunks;
    if (chunks > kMaxGridX || blocks > kMaxGridX)
        return VTL_HIP_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)blocks);
    if (vec)
        hipLaunchKernelGGL((dequantize_kernel<T, NV, 4>), grid, dim3(T), 0, s, q, scale, per_row ? 1 : 0,
                           row_len, (unsigned)chunks, x);
    else
        hipLaunchKernelGGL((dequantize_kernel<T, NV, 1>), grid, dim3(T), 0, s, q, scale, per_row ? 1 : 0,
                           row_len, (unsigned)chunks, x);
    return check_launch("dequantize_kernel");
}

int vtl_hip_relu_f32(float *x, int64_t n)
{
    if (!x || n < 0)
        return VTL_HIP_ERR_INVALID_ARG;
    if (n == 0)
        return VTL_HIP_OK;
    const int64_t blocks = (n + 255) / 256;
    if (blocks > kMaxGridX)
        return VTL_HIP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL(relu_kernel, dim3((unsigned)blocks), dim3(256), 0, current_stream(), x, n);
    return check_launch("relu_kernel");
}

}  // extern "C"
