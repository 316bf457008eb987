// int8 x int8 -> int32 matmul with a fused f32 scale/bias/ReLU epilogue, for
// gfx950 (CDNA4): LDS-tiled, v_mfma_i32_32x32x32_i8, accumulators kept in
// registers until the epilogue, which converts and scales them in place.
//
// Operand layout: A[M,K] and Bt[N,K] are both K-contiguous, so both LDS tiles
// are "rows of K bytes" and a lane's MFMA operand is 16 consecutive K bytes of
// one row.  Integer accumulation is order-free, so the only requirement on the
// K order inside the instruction is that A and B use the same one.
#include "common.hpp"

using namespace vtlhip;

namespace vtlhip {
int launch_quantize_rows(const float *x, int64_t rows, int64_t cols, int8_t *q, float *scale_out,
                         hipStream_t st);
}

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BK = 128;  // bytes of K per LDS tile row (8 chunks of 16 bytes)

struct GemmArgs {
    const int8_t *A;   // [M,K]
    const int8_t *Bt;  // [N,K]
    void *out;         // int32_t[M,N] or float[M,N]
    const float *sa;
    const float *sw;
    const float *bias;
    int M, N, K;
    int sa_stride;  // 1: one scale per row of A, 0: one scale
    int sw_stride;  // 1: one scale per row of Bt, 0: one scale
    int relu;
};

// LDS address of 16-byte chunk `chunk` of tile row `row`.  The chunk index is
// XOR-swizzled with row bits so that the 16 lanes a ds_read_b128 serves per
// cycle (16 consecutive rows, same logical chunk) fall into distinct banks.
__device__ __forceinline__ int lds_off(int row, int chunk)
{
    return row * BK + (((chunk ^ (row >> 1)) & 7) << 4);
}

template <int BM, int BN, int WR, int WC, bool F32OUT, bool EDGE>
__global__ __launch_bounds__(64 * WR * WC) void gemm_i8_mfma_kernel(const GemmArgs g)
{
    constexpr int NT = 64 * WR * WC;
    constexpr int WM = BM / WR, WN = BN / WC;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int A_CH = BM * 8 / NT, B_CH = BN * 8 / NT;
    constexpr int ROWS_PER_PASS = NT / 8;
    static_assert(BM % (32 * WR) == 0 && BN % (32 * WC) == 0, "wave tile must be a multiple of 32");
    static_assert(A_CH >= 1 && B_CH >= 1 && (BM * 8) % NT == 0 && (BN * 8) % NT == 0, "copy split");

    extern __shared__ __attribute__((aligned(16))) char smem[];
    char *sA = smem;                // [2][BM * BK]
    char *sB = smem + 2 * BM * BK;  // [2][BN * BK]

    const int M = g.M, N = g.N, K = g.K;
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    const int total = tiles_m * tiles_n;

    // Workgroups are dealt round-robin to the 8 XCDs; renumber them so that
    // each XCD (own L2) works on a compact patch of the tile grid.
    int pid = blockIdx.x;
    if ((total & 7) == 0)
        pid = (pid & 7) * (total >> 3) + (pid >> 3);
    constexpr int GM = 8;
    const int group_size = GM * tiles_n;
    const int first_m = (pid / group_size) * GM;
    const int gm = min(tiles_m - first_m, GM);
    const int tile_m = first_m + (pid % group_size) % gm;
    const int tile_n = (pid % group_size) / gm;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wr = wave / WC, wc = wave % WC;

    // ---- global -> register -> LDS copy assignment ----
    const int cc = tid & 7;   // 16-byte chunk inside the 128-byte row
    const int cr = tid >> 3;  // first row this thread copies
    v4i ra[A_CH], rb[B_CH];

    auto gload = [&](int kt) {
        const int kbyte = kt * BK + cc * 16;
#pragma unroll
        for (int i = 0; i < A_CH; i++) {
            int row = m0 + cr + i * ROWS_PER_PASS;
            if (EDGE)
                row = min(row, M - 1);
            const v4i *p = reinterpret_cast<const v4i *>(g.A + (int64_t)row * K + kbyte);
            if (EDGE)
                ra[i] = (kbyte < K) ? *p : v4i{0, 0, 0, 0};
            else
                ra[i] = *p;
        }
#pragma unroll
        for (int i = 0; i < B_CH; i++) {
            int row = n0 + cr + i * ROWS_PER_PASS;
            if (EDGE)
                row = min(row, N - 1);
            const v4i *p = reinterpret_cast<const v4i *>(g.Bt + (int64_t)row * K + kbyte);
            if (EDGE)
                rb[i] = (kbyte < K) ? *p : v4i{0, 0, 0, 0};
            else
                rb[i] = *p;
        }
    };
    auto lstore = [&](int buf) {
        char *a = sA + buf * (BM * BK);
        char *b = sB + buf * (BN * BK);
#pragma unroll
        for (int i = 0; i < A_CH; i++)
            *reinterpret_cast<v4i *>(a + lds_off(cr + i * ROWS_PER_PASS, cc)) = ra[i];
#pragma unroll
        for (int i = 0; i < B_CH; i++)
            *reinterpret_cast<v4i *>(b + lds_off(cr + i * ROWS_PER_PASS, cc)) = rb[i];
    };

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0;

    const int frow = lane & 31;  // row inside a 32-row MFMA operand
    const int fch = lane >> 5;   // which 16-byte half of the 32-byte K step

    auto compute = [&](int buf) {
        const char *a = sA + buf * (BM * BK) + 0;
        const char *b = sB + buf * (BN * BK) + 0;
#pragma unroll
        for (int s = 0; s < BK / 32; s++) {
            v4i af[TM], bf[TN];
            const int ch = s * 2 + fch;
#pragma unroll
            for (int i = 0; i < TM; i++)
                af[i] = *reinterpret_cast<const v4i *>(a + lds_off(wr * WM + i * 32 + frow, ch));
#pragma unroll
            for (int j = 0; j < TN; j++)
                bf[j] = *reinterpret_cast<const v4i *>(b + lds_off(wc * WN + j * 32 + frow, ch));
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
    };

    const int KT = (K + BK - 1) / BK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int kt = 0; kt < KT; kt++) {
        const bool more = kt + 1 < KT;
        if (more)
            gload(kt + 1);
        compute(kt & 1);
        if (more)
            lstore((kt + 1) & 1);
        __syncthreads();
    }

    // ---- epilogue: accumulator register r of lane l holds
    //      row 8*(r/4) + 4*(l/32) + r%4, column l%32 of its 32x32 tile ----
    const int col_in = lane & 31;
    const int row_in = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int n = n0 + wc * WN + j * 32 + col_in;
        const bool n_ok = !EDGE || n < N;
        float w = 0.f, bv = 0.f;
        if (F32OUT && n_ok) {
            w = g.sw[(int64_t)n * g.sw_stride];
            if (g.bias)
                bv = g.bias[n];
        }
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = m0 + wr * WM + i * 32 + 8 * (r >> 2) + row_in + (r & 3);
                if (EDGE && !(n_ok && m < M))
                    continue;
                const int64_t o = (int64_t)m * N + n;
                if (F32OUT) {
                    const float s = g.sa[(int64_t)m * g.sa_stride] * w;
                    float y = (float)acc[i][j][r] * s;
                    if (g.bias)
                        y = y + bv;
                    if (g.relu && y < 0.0f)
                        y = 0.0f;
                    reinterpret_cast<float *>(g.out)[o] = y;
                } else {
                    reinterpret_cast<int32_t *>(g.out)[o] = acc[i][j][r];
                }
            }
        }
    }
}

// Any shape, any alignment: one output per thread.  Only used when K is not a
// multiple of 16 or a pointer is not 16-byte aligned.
template <bool F32OUT>
__global__ __launch_bounds__(256) void gemm_i8_naive_kernel(const GemmArgs g)
{
    const int n = blockIdx.x * 16 + (threadIdx.x & 15);
    const int m = blockIdx.y * 16 + (threadIdx.x >> 4);
    if (m >= g.M || n >= g.N)
        return;
    const int8_t *a = g.A + (int64_t)m * g.K;
    const int8_t *b = g.Bt + (int64_t)n * g.K;
    int acc = 0;
    for (int k = 0; k < g.K; k++)
        acc += (int)a[k] * (int)b[k];
    const int64_t o = (int64_t)m * g.N + n;
    if (F32OUT) {
        const float s = g.sa[(int64_t)m * g.sa_stride] * g.sw[(int64_t)n * g.sw_stride];
        float y = (float)acc * s;
        if (g.bias)
            y = y + g.bias[n];
        if (g.relu && y < 0.0f)
            y = 0.0f;
        reinterpret_cast<float *>(g.out)[o] = y;
    } else {
        reinterpret_cast<int32_t *>(g.out)[o] = acc;
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int BM, int BN, int WR, int WC, bool F32OUT, bool EDGE>
int launch_tile(const GemmArgs &g, hipStream_t st)
{
    auto kern = gemm_i8_mfma_kernel<BM, BN, WR, WC, F32OUT, EDGE>;
    constexpr int lds = 2 * (BM + BN) * BK;
    static bool attr_done = false;  // one host thread per device
    if (!attr_done) {
        VTL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        attr_done = true;
    }
    const int tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(64 * WR * WC), lds, st, g);
    return check_launch("gemm_i8_mfma_kernel");
}

template <int BM, int BN, int WR, int WC, bool F32OUT>
int launch_tile_edge(const GemmArgs &g, hipStream_t st)
{
    const bool edge = (g.M % BM) || (g.N % BN) || (g.K % BK);
    return edge ? launch_tile<BM, BN, WR, WC, F32OUT, true>(g, st)
                : launch_tile<BM, BN, WR, WC, F32OUT, false>(g, st);
}

template <bool F32OUT>
int launch_gemm(const GemmArgs &g, hipStream_t st)
{
    if ((g.K % 16) || !aligned16(g.A) || !aligned16(g.Bt)) {
        const dim3 grid((unsigned)((g.N + 15) / 16), (unsigned)((g.M + 15) / 16));
        if (grid.y > 65535)
            return VTL_HIP_ERR_UNSUPPORTED;
        hipLaunchKernelGGL((gemm_i8_naive_kernel<F32OUT>), grid, dim3(256), 0, st, g);
        return check_launch("gemm_i8_naive_kernel");
    }
    // Tile choice: the largest tile that still yields about one workgroup per
    // compute unit; small problems trade tile efficiency for occupancy.
    const int64_t t256 = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
    const int64_t t128 = (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128);
    if (g.M > 128 && t256 >= 200)
        return launch_tile_edge<256, 256, 2, 2, F32OUT>(g, st);
    if (g.M > 64 && t128 >= 128)
        return launch_tile_edge<128, 128, 2, 2, F32OUT>(g, st);
    if (g.M > 32)
        return launch_tile_edge<64, 64, 2, 2, F32OUT>(g, st);
    return launch_tile_edge<32, 64, 1, 2, F32OUT>(g, st);
}

int check_gemm_args(const void *A, const void *Bt, const void *out, int M, int N, int K)
{
    if (!A || !Bt || !out || M < 0 || N < 0 || K < 0)
        return VTL_HIP_ERR_INVALID_ARG;
    if (K > 131072)  // |acc| <= K * 127^2 must stay below 2^31
        return VTL_HIP_ERR_UNSUPPORTED;
    return VTL_HIP_OK;
}

}  // namespace

extern "C" {

int vtl_hip_gemm_i8_i32(const int8_t *A, const int8_t *Bt, int32_t *C, int M, int N, int K)
{
    int st = check_gemm_args(A, Bt, C, M, N, K);
    if (st != VTL_HIP_OK)
        return st;
    if (M == 0 || N == 0)
        return VTL_HIP_OK;
    if (K == 0)
        return VTL_HIP_ERR_UNSUPPORTED;  // la.matmul has no empty inner dimension either
    GemmArgs g{A, Bt, C, nullptr, nullptr, nullptr, M, N, K, 0, 0, 0};
    return launch_gemm<false>(g, current_stream());
}

int vtl_hip_linear_i8_f32(const int8_t *A, const float *sa, int sa_per_row, const int8_t *Wq,
                          const float *sw, int sw_per_col, const float *bias, float *Y, int M, int N,
                          int K, int relu)
{
    int st = check_gemm_args(A, Wq, Y, M, N, K);
    if (st != VTL_HIP_OK)
        return st;
    if (!sa || !sw)
        return VTL_HIP_ERR_INVALID_ARG;
    if (M == 0 || N == 0)
        return VTL_HIP_OK;
    if (K == 0)
        return VTL_HIP_ERR_UNSUPPORTED;  // la.matmul rejects empty inner dimensions as well
    GemmArgs g{A, Wq, Y, sa, sw, bias, M, N, K, sa_per_row ? 1 : 0, sw_per_col ? 1 : 0, relu ? 1 : 0};
    return launch_gemm<true>(g, current_stream());
}

size_t vtl_hip_linear_f32_dynquant_workspace(int M, int K)
{
    if (M <= 0 || K <= 0)
        return 0;
    // int8 codes of X, rounded up to 256 bytes, then M row scales
    const size_t codes = (((size_t)M * (size_t)K) + 255) & ~(size_t)255;
    return codes + (size_t)M * sizeof(float);
}

int vtl_hip_linear_f32_dynquant(const float *X, const int8_t *Wq, const float *sw, const float *bias,
                                float *Y, int M, int N, int K, int relu, void *workspace,
                                size_t workspace_bytes)
{
    int st = check_gemm_args(X, Wq, Y, M, N, K);
    if (st != VTL_HIP_OK)
        return st;
    if (!sw || !workspace)
        return VTL_HIP_ERR_INVALID_ARG;
    if (M == 0 || N == 0)
        return VTL_HIP_OK;
    if (K == 0)
        return VTL_HIP_ERR_UNSUPPORTED;
    if (workspace_bytes < vtl_hip_linear_f32_dynquant_workspace(M, K) ||
        (reinterpret_cast<uintptr_t>(workspace) & 15))
        return VTL_HIP_ERR_INVALID_ARG;
    int8_t *xq = reinterpret_cast<int8_t *>(workspace);
    const size_t codes = (((size_t)M * (size_t)K) + 255) & ~(size_t)255;
    float *sx = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + codes);
    st = launch_quantize_rows(X, M, K, xq, sx, current_stream());
    if (st != VTL_HIP_OK)
        return st;
    GemmArgs g{xq, Wq, Y, sx, sw, bias, M, N, K, 1, 1, relu ? 1 : 0};
    return launch_gemm<true>(g, current_stream());
}

}  // extern "C"
