// Dense matmul with f64 products and sums on the gfx950 f64 matrix cores, for
// f32 and f64 tensors: the device form of la.matmul (la/la.v:38-55) and
// gate_matmul (autograd/gates_blas.v:6-23), which widen every operand to f64,
// multiply with a f64 GEMM and round the result once to the tensor's type.
// Also the unquantized Linear forward (nn/layers/linear_forward_f32.v:16-18)
// and LinearGate.backward (nn/gates/layers/linear.v:69-79) built on it.
//
// One workgroup of WR x WC waves owns a BM x BN tile of C.  Both operands are
// staged through LDS in k-major form (As[k][m], Bs[k][n]) whatever their
// layout in memory, so that one 16- or 32-byte LDS read hands a lane the
// operands of all its 16x16x4 MFMA tiles for one k.  MFMA tile i of a wave
// holds the rows {TM * r + i : r = 0..15} of the wave's rows (and likewise for
// columns), which makes those reads and the final stores contiguous per lane.
#include "common.hpp"

#include <stdlib.h>

namespace {

using vtlhip::check_launch;
using vtlhip::current_stream;

typedef double double4_t __attribute__((ext_vector_type(4)));

struct MatmulArgs {
    const void *A;      // trans_a == 0: [M,K] row-major, else [K,M]
    const void *B;      // trans_b == 0: [K,N] row-major, else [N,K]
    void *C;            // [M,N] row-major
    const void *bias;   // N values added after rounding to the output type, or nullptr
    int M, N, K;
    int vec_a, vec_b, vec_c;   // base 16-byte aligned and leading dimension % 4 == 0
    int relu;
    int k_per_split;           // split-K launches: k range of one grid.y slice (multiple of 32)
    double *partial;           // split-K launches: [splits][M][N] unrounded sums
};

template <typename T>
struct alignas(16) Vec4 {
    T v[4];
};

// Four consecutive elements of a row-major matrix starting at (row, col);
// positions outside rows x cols read as zero.  GUARD == false: the caller
// knows that every position is inside and 16-byte aligned.
template <typename T, bool GUARD>
__device__ __forceinline__ Vec4<T> load4(const T *__restrict__ base, int ld, int rows, int cols, int row,
                                         int col, bool vec_ok)
{
    Vec4<T> out;
    if (!GUARD || (row < rows && col + 3 < cols && vec_ok)) {
        out = *reinterpret_cast<const Vec4<T> *>(base + (int64_t)row * ld + col);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            out.v[j] = (row < rows && col + j < cols) ? base[(int64_t)row * ld + col + j] : T(0);
    }
    return out;
}

// NT consecutive LDS elements (NT = 2 or 4, naturally aligned) widened to f64.
template <typename T, int NT>
__device__ __forceinline__ void read_operands(const T *__restrict__ p, double (&out)[NT])
{
    struct alignas(NT * sizeof(T) > 16 ? 16 : NT * sizeof(T)) Pack {
        T v[NT];
    };
    const Pack pk = *reinterpret_cast<const Pack *>(p);
#pragma unroll
    for (int i = 0; i < NT; ++i)
        out[i] = (double)pk.v[i];
}

// One operand tile of BK x BMN elements (k-major in LDS, row stride LDW).
// KMAJOR: the matrix is stored with the tile's m/n index contiguous ([K, MN]);
// otherwise it is stored [MN, K] and is transposed on the way into LDS.
template <typename T, int BK, int BMN, int LDW, int NT, bool KMAJOR, bool GUARD>
struct OperandTile {
    static constexpr int kGroups = BK * BMN / 4;           // 4-element groups per tile
    static constexpr int kPerThread = (kGroups + NT - 1) / NT;   // NT threads in the workgroup
    Vec4<T> regs[kPerThread];

    // k_total: the matrix's K (its leading dimension when stored [MN, K]);
    // k_limit <= k_total: positions with k >= k_limit read as zero.
    __device__ __forceinline__ void fetch(const T *__restrict__ base, int mn_total, int k_total, int k_limit,
                                          int mn0, int k0, bool vec_ok)
    {
        const int t = threadIdx.x;
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const int g = t + NT * i;
            if (kGroups % NT != 0 && g >= kGroups)
                break;
            if constexpr (KMAJOR) {
                const int krow = g / (BMN / 4), c4 = g % (BMN / 4);
                regs[i] = load4<T, GUARD>(base, mn_total, k_limit, mn_total, k0 + krow, mn0 + 4 * c4, vec_ok);
            } else {
                const int mn = g % BMN, kc = g / BMN;
                regs[i] = load4<T, GUARD>(base, k_total, mn_total, k_limit, mn0 + mn, k0 + 4 * kc, vec_ok);
            }
        }
    }

    __device__ __forceinline__ void stash(T *__restrict__ lds) const
    {
        const int t = threadIdx.x;
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const int g = t + NT * i;
            if (kGroups % NT != 0 && g >= kGroups)
                break;
            if constexpr (KMAJOR) {
                const int krow = g / (BMN / 4), c4 = g % (BMN / 4);
                *reinterpret_cast<Vec4<T> *>(lds + krow * LDW + 4 * c4) = regs[i];
            } else {
                const int mn = g % BMN, kc = g / BMN;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    lds[(4 * kc + j) * LDW + mn] = regs[i].v[j];
            }
        }
    }
};

// Workgroup barrier that orders LDS traffic only: unlike __syncthreads() it does
// not wait for outstanding global loads, so the operand loads issued two
// k-tiles ahead stay in flight across it.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// GUARD == false: M, N, K are whole tiles and every row is 16-byte aligned, so
// the loads and stores carry no bounds checks and the k-loop is straight-line code.
// SPLIT: grid.y slices K; each slice writes its unrounded f64 sums to g.partial.
// Workgroup = WR x WC waves, each with TM x TN MFMA tiles of 16x16:
// BM = 16 * TM * WR, BN = 16 * TN * WC.
template <typename T, int TM, int TN, int WR, int WC, bool TA, bool TB, bool GUARD, bool SPLIT>
__global__ __launch_bounds__(64 * WR * WC) void matmul_f64acc_kernel(const MatmulArgs g)
{
    constexpr int BM = 16 * TM * WR, BN = 16 * TN * WC, NT = 64 * WR * WC;
    // bytes of k per tile row: 64 (16 f32 / 8 f64); the small tile takes 128 to halve its barriers
    constexpr int BK = (BM * BN <= 64 * 64 ? 128 : 64) / (int)sizeof(T);
    constexpr int LDA = BM + 4, LDB = BN + 4;
    static_assert(TM == 2 || TM == 4, "wave tile is 32 or 64 rows");
    static_assert(TN == 2 || TN == 4, "wave tile is 32 or 64 columns");

    // Three LDS buffers per operand: while tile kt is multiplied, tile kt+1 is
    // written at the start of the step (its global loads were issued a step
    // earlier) and the one barrier per step sits before the last k-group, so
    // that the first operands of tile kt+1 are read from LDS under the last
    // MFMAs of tile kt and no MFMA waits for a barrier followed by an LDS read.
    __shared__ __attribute__((aligned(16))) T As[3][BK * LDA];
    __shared__ __attribute__((aligned(16))) T Bs[3][BK * LDB];

    const T *__restrict__ A = static_cast<const T *>(g.A);
    const T *__restrict__ B = static_cast<const T *>(g.B);
    const int tiles_n = (g.N + BN - 1) / BN;
    const int m0 = (int)(blockIdx.x / tiles_n) * BM;
    const int n0 = (int)(blockIdx.x % tiles_n) * BN;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = (wave / WC) * (16 * TM), wn = (wave % WC) * (16 * TN);
    const int r16 = lane & 15, kq = lane >> 4;

    // A as op(A)[M,K]: stored [K,M] when transposed (k-major already)
    OperandTile<T, BK, BM, LDA, NT, TA, GUARD> ta;
    // B as op(B)[K,N]: stored [K,N] when not transposed (k-major already)
    OperandTile<T, BK, BN, LDB, NT, !TB, GUARD> tb;

    double4_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
            acc[i][j] = double4_t{0.0, 0.0, 0.0, 0.0};

    const int k_begin = SPLIT ? (int)blockIdx.y * g.k_per_split : 0;
    const int k_end = SPLIT ? (k_begin + g.k_per_split < g.K ? k_begin + g.k_per_split : g.K) : g.K;
    const int ktiles = (k_end - k_begin + BK - 1) / BK;
    constexpr int S = BK / 4;   // k-groups (one MFMA step each) per tile
    const int aoff = wm + TM * r16 + kq * LDA, boff = wn + TN * r16 + kq * LDB;

    ta.fetch(A, g.M, g.K, k_end, m0, k_begin, g.vec_a != 0);
    tb.fetch(B, g.N, g.K, k_end, n0, k_begin, g.vec_b != 0);
    ta.stash(As[0]);
    tb.stash(Bs[0]);
    if (ktiles > 1) {
        ta.fetch(A, g.M, g.K, k_end, m0, k_begin + BK, g.vec_a != 0);
        tb.fetch(B, g.N, g.K, k_end, n0, k_begin + BK, g.vec_b != 0);
    }
    __syncthreads();
    double a[TM], b[TN];
    read_operands<T, TM>(As[0] + aoff, a);
    read_operands<T, TN>(Bs[0] + boff, b);

    int cur = 0;
    for (int kt = 0; kt < ktiles; ++kt) {
        const int nxt = cur == 2 ? 0 : cur + 1;
        if (kt + 1 < ktiles) {
            // buffer nxt was last read two steps ago; every wave has passed a barrier since
            ta.stash(As[nxt]);
            tb.stash(Bs[nxt]);
        }
        if (kt + 2 < ktiles) {
            ta.fetch(A, g.M, g.K, k_end, m0, k_begin + (kt + 2) * BK, g.vec_a != 0);
            tb.fetch(B, g.N, g.K, k_end, n0, k_begin + (kt + 2) * BK, g.vec_b != 0);
        }
#pragma unroll
        for (int s = 0; s < S; ++s) {
            double an[TM], bn[TN];
            if (s + 1 < S) {
                read_operands<T, TM>(As[cur] + aoff + 4 * (s + 1) * LDA, an);
                read_operands<T, TN>(Bs[cur] + boff + 4 * (s + 1) * LDB, bn);
            } else {
                lds_barrier();   // tile kt+1 is in LDS for every wave; global loads stay in flight
                read_operands<T, TM>(As[nxt] + aoff, an);
                read_operands<T, TN>(Bs[nxt] + boff, bn);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc[i][j], 0, 0, 0);
#pragma unroll
            for (int i = 0; i < TM; ++i)
                a[i] = an[i];
#pragma unroll
            for (int j = 0; j < TN; ++j)
                b[j] = bn[j];
        }
        cur = nxt;
    }

    if constexpr (SPLIT) {
        double *__restrict__ P = g.partial + (int64_t)blockIdx.y * g.M * g.N;
        const int pcol0 = n0 + wn + TN * r16;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = m0 + wm + TM * (4 * e + kq) + i;
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    if (!GUARD || (row < g.M && pcol0 + j < g.N))
                        P[(int64_t)row * g.N + pcol0 + j] = acc[i][j][e];
            }
        return;
    }
    T *__restrict__ C = static_cast<T *>(g.C);
    const T *__restrict__ bias = static_cast<const T *>(g.bias);
    const int col0 = n0 + wn + TN * r16;
    T bv[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
        bv[j] = (bias && (!GUARD || col0 + j < g.N)) ? bias[col0 + j] : T(0);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int row = m0 + wm + TM * (4 * e + kq) + i;
            if (GUARD && row >= g.M)
                continue;
            T out[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                T y = (T)acc[i][j][e];   // the one rounding to the tensor's type
                if (bias)
                    y = y + bv[j];       // Tensor.add in the tensor's type
                if (g.relu && y < T(0))
                    y = T(0);
                out[j] = y;
            }
            T *dst = C + (int64_t)row * g.N + col0;
            if (!GUARD || (g.vec_c && col0 + TN - 1 < g.N)) {
                if constexpr (TN == 4) {
                    Vec4<T> v;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        v.v[j] = out[j];
                    *reinterpret_cast<Vec4<T> *>(dst) = v;
                } else {
                    struct alignas(2 * sizeof(T)) Vec2 {
                        T v[2];
                    } v;
                    v.v[0] = out[0];
                    v.v[1] = out[1];
                    *reinterpret_cast<Vec2 *>(dst) = v;
                }
            } else {
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    if (col0 + j < g.N)
                        dst[j] = out[j];
            }
        }
    }
}

// Column sums with f64 accumulation: la.matmul(ones[1,M], grad) of
// nn/gates/layers/linear.v:75-79.  Block = 64 column groups x 4 row phases;
// grid.y splits the rows, each split writing f64 partial sums when there is
// more than one.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void colsum_kernel(const T *__restrict__ x, int64_t rows, int64_t cols,
                                                     int64_t rows_per_split, T *__restrict__ out,
                                                     double *__restrict__ partial)
{
    __shared__ double red[4][64 * VEC];
    const int cg = threadIdx.x & 63, ph = threadIdx.x >> 6;
    const int64_t c0 = ((int64_t)blockIdx.x * 64 + cg) * VEC;
    const int64_t r_begin = (int64_t)blockIdx.y * rows_per_split;
    const int64_t r_end = r_begin + rows_per_split < rows ? r_begin + rows_per_split : rows;
    double acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        acc[j] = 0.0;
    if (c0 < cols) {
        int64_t r = r_begin + ph;
        for (; r + 12 < r_end; r += 16) {
            T v[4][VEC];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                if constexpr (VEC == 4) {
                    const Vec4<T> t4 = *reinterpret_cast<const Vec4<T> *>(x + (r + 4 * u) * cols + c0);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        v[u][j] = t4.v[j];
                } else {
                    v[u][0] = x[(r + 4 * u) * cols + c0];
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int j = 0; j < VEC; ++j)
                    acc[j] += (double)v[u][j];
        }
        for (; r < r_end; r += 4) {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
                acc[j] += (double)x[r * cols + c0 + j];
        }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
        red[ph][cg * VEC + j] = acc[j];
    __syncthreads();
    if (ph == 0 && c0 < cols) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
            const double s = ((red[0][cg * VEC + j] + red[1][cg * VEC + j]) + red[2][cg * VEC + j]) +
                             red[3][cg * VEC + j];
            if (partial)
                partial[(int64_t)blockIdx.y * cols + c0 + j] = s;
            else
                out[c0 + j] = (T)s;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(256) void colsum_finalize_kernel(const double *__restrict__ partial, int splits,
                                                              int64_t cols, T *__restrict__ out)
{
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= cols)
        return;
    double s = 0.0;
    for (int i = 0; i < splits; ++i)
        s += partial[(int64_t)i * cols + c];
    out[c] = (T)s;
}

// Sums the K slices of a split launch in slice order, rounds once to T, then
// bias and ReLU as in the unsplit epilogue.
template <typename T>
__global__ __launch_bounds__(256) void matmul_splitk_finalize_kernel(const MatmulArgs g, int splits)
{
    const int64_t total = (int64_t)g.M * g.N;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total)
        return;
    double s = 0.0;
    for (int i = 0; i < splits; ++i)
        s += g.partial[(int64_t)i * total + idx];
    T y = (T)s;
    const T *__restrict__ bias = static_cast<const T *>(g.bias);
    if (bias)
        y = y + bias[idx % g.N];
    if (g.relu && y < T(0))
        y = T(0);
    static_cast<T *>(g.C)[idx] = y;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <typename T, int TM, int TN, int WR, int WC, bool GUARD, bool SPLIT>
int launch_tile_guard(const MatmulArgs &g, bool ta, bool tb, int splits, hipStream_t st)
{
    constexpr int BM = 16 * TM * WR, BN = 16 * TN * WC;
    const int64_t tiles = (int64_t)((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    if (tiles > 0x7fffffff)
        return VTL_HIP_ERR_UNSUPPORTED;
    const dim3 grid((unsigned)tiles, (unsigned)splits), block(64 * WR * WC);
    if (!ta && !tb)
        hipLaunchKernelGGL((matmul_f64acc_kernel<T, TM, TN, WR, WC, false, false, GUARD, SPLIT>), grid, block, 0,
                           st, g);
    else if (!ta && tb)
        hipLaunchKernelGGL((matmul_f64acc_kernel<T, TM, TN, WR, WC, false, true, GUARD, SPLIT>), grid, block, 0,
                           st, g);
    else if (ta && !tb)
        hipLaunchKernelGGL((matmul_f64acc_kernel<T, TM, TN, WR, WC, true, false, GUARD, SPLIT>), grid, block, 0,
                           st, g);
    else
        hipLaunchKernelGGL((matmul_f64acc_kernel<T, TM, TN, WR, WC, true, true, GUARD, SPLIT>), grid, block, 0,
                           st, g);
    return check_launch("matmul_f64acc_kernel");
}

// Shapes made of whole tiles with 16-byte aligned rows run without bounds checks.
template <typename T, int TM, int TN, int WR, int WC>
int launch_tile(const MatmulArgs &g, bool ta, bool tb, hipStream_t st)
{
    constexpr int BM = 16 * TM * WR, BN = 16 * TN * WC;
    const bool whole = g.M % BM == 0 && g.N % BN == 0 && g.K % 32 == 0 && g.K > 0 && g.vec_a && g.vec_b &&
                       g.vec_c;
    return whole ? launch_tile_guard<T, TM, TN, WR, WC, false, false>(g, ta, tb, 1, st)
                 : launch_tile_guard<T, TM, TN, WR, WC, true, false>(g, ta, tb, 1, st);
}

// Few output tiles and a long K: slice K over grid.y so that every SIMD holds
// several waves, f64 partial sums in the library's workspace, then one pass
// that adds the slices in order and rounds.
template <typename T, int TM, int TN, int WR, int WC>
int launch_split(MatmulArgs g, bool ta, bool tb, int splits, hipStream_t st)
{
    constexpr int BM = 16 * TM * WR, BN = 16 * TN * WC;
    const int per = ((g.K + splits - 1) / splits + 31) / 32 * 32;
    splits = (g.K + per - 1) / per;
    g.k_per_split = per;
    g.partial = static_cast<double *>(
        vtlhip::library_workspace((size_t)splits * (size_t)g.M * (size_t)g.N * sizeof(double)));
    if (!g.partial)
        return vtlhip::workspace_status();
    const bool whole = g.M % BM == 0 && g.N % BN == 0 && g.K % per == 0 && g.vec_a && g.vec_b;
    int rc = whole ? launch_tile_guard<T, TM, TN, WR, WC, false, true>(g, ta, tb, splits, st)
                   : launch_tile_guard<T, TM, TN, WR, WC, true, true>(g, ta, tb, splits, st);
    if (rc != VTL_HIP_OK)
        return rc;
    const int64_t blocks = ((int64_t)g.M * g.N + 255) / 256;
    hipLaunchKernelGGL((matmul_splitk_finalize_kernel<T>), dim3((unsigned)blocks), dim3(256), 0, st, g, splits);
    return check_launch("matmul_splitk_finalize_kernel");
}

template <typename T>
int matmul_impl(const T *a, const T *b, T *c, const T *bias, int m, int n, int k, int trans_a, int trans_b,
                int relu)
{
    if (m < 0 || n < 0 || k < 0)
        return VTL_HIP_ERR_INVALID_ARG;
    if (m == 0 || n == 0)
        return VTL_HIP_OK;
    if (!c || (k > 0 && (!a || !b)))
        return VTL_HIP_ERR_INVALID_ARG;
    MatmulArgs g;
    g.A = a;
    g.B = b;
    g.C = c;
    g.bias = bias;
    g.M = m;
    g.N = n;
    g.K = k;
    const int lda = trans_a ? m : k, ldb = trans_b ? k : n;
    g.vec_a = aligned16(a) && lda % 4 == 0;
    g.vec_b = aligned16(b) && ldb % 4 == 0;
    g.vec_c = aligned16(c) && n % 4 == 0;
    g.relu = relu;
    g.k_per_split = 0;
    g.partial = nullptr;
    hipStream_t st = current_stream();
    // Tile choice by a per-compute-unit estimate, in units of one 128x128 tile at
    // peak: a compute unit runs two big workgroups together at ~0.84 of peak and
    // a single one at ~0.75; the 64x64 tile kernel reaches 0.72 (four workgroups
    // per compute unit) to 0.78 (many) and quantizes four times finer over the
    // 256 compute units.  Constants fitted to measured times (with many tiles
    // the big one is 7-12 % faster, e.g. 11008x4096x256: 350 against 377 us).
    const int64_t big = (int64_t)((m + 127) / 128) * ((n + 127) / 128);
    const int64_t small = (int64_t)((m + 63) / 64) * ((n + 63) / 64);
    const int64_t c128 = (big + 255) / 256, c64 = (small + 255) / 256;
    const double t128 = (double)(c128 / 2) * (2.0 / 0.84) + (double)(c128 % 2) * (1.0 / 0.75);
    const double t64 = (double)c64 * 0.25 / (0.78 - 0.24 / (double)c64);
    // eight waves of 32x64 per 128x128 tile measured a few percent above four waves of 64x64
    const int tile_env = vtlhip::tuning().matmul_tile;   // VTL_HIP_MATMUL_TILE 128 / 64 forces the tile (tuning, tests)
    if (tile_env ? tile_env == 128 : t128 <= t64)
        return launch_tile<T, 2, 4, 4, 2>(g, trans_a != 0, trans_b != 0, st);
    const bool force = vtlhip::tuning().matmul_splits >= 0;   // VTL_HIP_MATMUL_SPLITS (tuning and tests)
    // Too few big tiles for the chip but a long K: cut K until about 512 big
    // workgroups exist (two per compute unit); measured 8-12 % faster than
    // the small tile with its own split (256x4096x11008: 428 -> 386 us).
    if (!force && m >= 128 && big >= 32 && k >= 2048) {
        int sp = 1;
        while (big * sp < 512 && sp < 16 && k / (2 * sp) >= 512)
            sp *= 2;
        if (sp > 1)
            return launch_split<T, 2, 4, 4, 2>(g, trans_a != 0, trans_b != 0, sp, st);
    }
    int splits = force ? vtlhip::tuning().matmul_splits : 1;
    if (!force && small <= 512 && k >= 2048) {
        splits = (int)(1024 / small);
        if (splits > k / 512)
            splits = k / 512;
        if (splits > 16)
            splits = 16;
    }
    if (splits > 1 && k >= 32 * splits)
        return launch_split<T, 2, 2, 2, 2>(g, trans_a != 0, trans_b != 0, splits, st);
    return launch_tile<T, 2, 2, 2, 2>(g, trans_a != 0, trans_b != 0, st);
}

template <typename T>
int colsum_impl(const T *x, int64_t rows, int64_t cols, T *out)
{
    if (rows < 0 || cols < 0)
        return VTL_HIP_ERR_INVALID_ARG;
    if (cols == 0)
        return VTL_HIP_OK;
    if (!out || (rows > 0 && !x))
        return VTL_HIP_ERR_INVALID_ARG;
    hipStream_t st = current_stream();
    const bool vec = aligned16(x) && cols % 4 == 0;
    const int per_block = vec ? 256 : 64;
    const int64_t col_blocks = (cols + per_block - 1) / per_block;
    if (col_blocks > 0x7fffffff)
        return VTL_HIP_ERR_UNSUPPORTED;
    // enough workgroups to fill the chip, but at least 64 rows per split
    int64_t splits = 1;
    if (col_blocks < 1024 && rows >= 128) {
        splits = 1024 / col_blocks;
        if (splits > rows / 64)
            splits = rows / 64;
        if (splits > 1024)
            splits = 1024;
        if (splits < 1)
            splits = 1;
    }
    const int64_t rows_per_split = splits > 1 ? (rows + splits - 1) / splits : rows;
    if (splits > 1)
        splits = (rows + rows_per_split - 1) / rows_per_split;
    double *partial = nullptr;
    if (splits > 1) {
        partial = static_cast<double *>(
            vtlhip::library_workspace((size_t)splits * (size_t)cols * sizeof(double)));
        if (!partial)
            return vtlhip::workspace_status();
    }
    const dim3 grid((unsigned)col_blocks, (unsigned)splits);
    if (vec)
        hipLaunchKernelGGL((colsum_kernel<T, 4>), grid, dim3(256), 0, st, x, rows, cols, rows_per_split, out,
                           partial);
    else
        hipLaunchKernelGGL((colsum_kernel<T, 1>), grid, dim3(256), 0, st, x, rows, cols, rows_per_split, out,
                           partial);
    int rc = check_launch("colsum_kernel");
    if (rc != VTL_HIP_OK || splits == 1)
        return rc;
    hipLaunchKernelGGL((colsum_finalize_kernel<T>), dim3((unsigned)((cols + 255) / 256)), dim3(256), 0, st,
                       partial, (int)splits, cols, out);
    return check_launch("colsum_finalize_kernel");
}

template <typename T>
int linear_backward_impl(const T *grad, const T *x, const T *w, T *dx, T *dw, T *db, int m, int n, int k)
{
    if (m < 0 || n < 0 || k < 0 || !grad)
        return VTL_HIP_ERR_INVALID_ARG;
    if ((dx && !w) || (dw && !x))
        return VTL_HIP_ERR_INVALID_ARG;
    int rc = VTL_HIP_OK;
    if (dx)   // [M,K] = grad[M,N] . W[N,K]
        rc = matmul_impl<T>(grad, w, dx, nullptr, m, k, n, 0, 0, 0);
    if (rc == VTL_HIP_OK && dw)   // [N,K] = grad^T[N,M] . x[M,K]
        rc = matmul_impl<T>(grad, x, dw, nullptr, n, k, m, 1, 0, 0);
    if (rc == VTL_HIP_OK && db)   // [1,N] = ones[1,M] . grad[M,N]
        rc = colsum_impl<T>(grad, m, n, db);
    return rc;
}

}  // namespace

extern "C" {

int vtl_hip_matmul_f32(const float *a, const float *b, float *c, int m, int n, int k, int trans_a,
                       int trans_b)
{
    return matmul_impl<float>(a, b, c, nullptr, m, n, k, trans_a, trans_b, 0);
}

int vtl_hip_matmul_f64(const double *a, const double *b, double *c, int m, int n, int k, int trans_a,
                       int trans_b)
{
    return matmul_impl<double>(a, b, c, nullptr, m, n, k, trans_a, trans_b, 0);
}

int vtl_hip_linear_f32(const float *x, const float *w, const float *bias, float *y, int m, int n, int k,
                       int relu)
{
    return matmul_impl<float>(x, w, y, bias, m, n, k, 0, 1, relu);
}

int vtl_hip_linear_f64(const double *x, const double *w, const double *bias, double *y, int m, int n, int k,
                       int relu)
{
    return matmul_impl<double>(x, w, y, bias, m, n, k, 0, 1, relu);
}

int vtl_hip_colsum_f32(const float *x, int64_t rows, int64_t cols, float *out)
{
    return colsum_impl<float>(x, rows, cols, out);
}

int vtl_hip_colsum_f64(const double *x, int64_t rows, int64_t cols, double *out)
{
    return colsum_impl<double>(x, rows, cols, out);
}

int vtl_hip_linear_backward_f32(const float *grad, const float *x, const float *w, float *dx, float *dw,
                                float *db, int m, int n, int k)
{
    return linear_backward_impl<float>(grad, x, w, dx, dw, db, m, n, k);
}

int vtl_hip_linear_backward_f64(const double *grad, const double *x, const double *w, double *dx,
                                double *dw, double *db, int m, int n, int k)
{
    return linear_backward_impl<double>(grad, x, w, dx, dw, db, m, n, k);
}

}  // extern "C"
