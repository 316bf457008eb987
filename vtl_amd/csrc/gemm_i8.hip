// int8 x int8 -> int32 matmul with a fused f32 scale/bias/ReLU epilogue, for
// gfx950 (CDNA4): LDS-tiled, v_mfma_i32_32x32x32_i8, operand tiles loaded from
// global memory straight into LDS, accumulators kept in registers until the
// epilogue, which converts and scales them in place.
//
// Operand layout: A[M,K] and Bt[N,K] are both K-contiguous, so both LDS tiles
// are "rows of K bytes" and a lane's MFMA operand is 16 consecutive K bytes of
// one row.  Integer accumulation is order-free, so the only requirement on the
// K order inside the instruction is that A and B use the same one.
#include <stdio.h>
#include <stdlib.h>

#include <atomic>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "quant_device.hpp"

using namespace vtlhip;

namespace vtlhip {
int launch_quantize_rows(const float *x, int64_t rows, int64_t cols, int8_t *q, float *scale_out,
                         hipStream_t st);
}

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float f4 __attribute__((ext_vector_type(4)));

#define VTL_GPTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define VTL_LPTR(p) ((__attribute__((address_space(3))) void *)(p))

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
    int splits;         // K is cut into this many ranges, one workgroup each (1 = no split)
    int32_t *partials;  // [splits][M][N] int32 partial sums when splits > 1
    const float *xf32;  // f32 activations [M,K] for the kernel that quantizes them itself
    int cached_out;     // f32 epilogue of the 256x256 tile: cached instead of non-temporal stores
    // When set, the launch leaves raw int32 sums in `partials` (also without a K split) and a
    // row kernel applies the epilogue and quantizes each output row: codes here, row scales in
    // requant_scales, the f32 rows in `out` unless that is null.
    int8_t *requant_codes;
    float *requant_scales;
    // Set by the launcher when the tile kernel itself applies the epilogue of a requantizing
    // linear (no K split): [tiles along N][M] maxima of |y| over each tile's columns, which
    // the tile kernel writes beside the f32 rows and requant_rows_wide_kernel reduces.
    float *row_absmax_parts;
    // Weight-streaming kernel that quantizes the f32 activations xf32 itself, into stage_codes
    // and stage_scales (which A and sa name too): M workgroups do, and count themselves in
    // counter sync_slot; the others wait (at most spin_limit polls) until it reads stage_target.
    int8_t *stage_codes;
    float *stage_scales;
    int sync_slot;
    int spin_limit;
    unsigned stage_target;
    // Weight-streaming kernel with up to 32 rows (every weight is read once): read the weights
    // with non-temporal loads.  Set by the size of the matrix, see stream_weights_from.
    int stream_weights;
};

// LDS tiles are rows of BK bytes (BK/16 chunks of 16 bytes).  The chunk index
// is XOR-swizzled with row bits so that the 16 lanes a ds_read_b128 serves per
// cycle (16 consecutive rows, same logical chunk) fall into 16 distinct
// 16-byte bank groups of the 64-bank LDS.
template <int BK>
__device__ __forceinline__ int swizzle(int row)
{
    return BK == 128 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}

template <int BK>
__device__ __forceinline__ int lds_off(int row, int chunk)
{
    return row * BK + (((chunk ^ swizzle<BK>(row)) & (BK / 16 - 1)) << 4);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Workgroups are dealt round-robin to the 8 XCDs; renumber them so that each
// XCD (own L2) works on a compact patch of the tile grid (XCD x holds
// total/8 tiles, one more when x < total%8), then walk the grid in groups of
// 8 tile rows.
__device__ __forceinline__ void tile_of_block(int tiles_m, int tiles_n, int block, int &tile_m, int &tile_n)
{
    const int total = tiles_m * tiles_n;
    const int xcd = block & 7, rest = total & 7;
    const int pid = xcd * (total >> 3) + min(xcd, rest) + (block >> 3);
    constexpr int GM = 8;
    const int group_size = GM * tiles_n;
    const int first_m = (pid / group_size) * GM;
    const int gm = min(tiles_m - first_m, GM);
    tile_m = first_m + (pid % group_size) % gm;
    tile_n = (pid % group_size) / gm;
}

// Scales and bias of a block tile, fetched by the threads of the workgroup before the K loop
// (thread t takes rows / columns t, t + NT, ...) and put into LDS by the epilogue: read only
// then, they add a memory latency to the end of every workgroup.  Used by the 256x256 tile
// (4096^3: 0.3 to 1 us earlier); the smaller tiles measured no better with it and read them
// in the epilogue.
template <int BM>
constexpr bool kScalesAhead = BM == 256;

template <int BM, int BN, int NT>
struct EpilogueScales {
    float sa[(BM + NT - 1) / NT], sw[(BN + NT - 1) / NT], bias[(BN + NT - 1) / NT];
};

template <int BM, int BN, int NT, bool EDGE>
__device__ __forceinline__ void fetch_scales(EpilogueScales<BM, BN, NT> &e, const GemmArgs &g, int m0, int n0)
{
#pragma unroll
    for (int i = 0; i < (BM + NT - 1) / NT; i++) {
        const int t = (int)threadIdx.x + i * NT;
        const int m = EDGE ? min(m0 + t, g.M - 1) : m0 + t;
        e.sa[i] = t < BM ? g.sa[(int64_t)m * g.sa_stride] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < (BN + NT - 1) / NT; i++) {
        const int t = (int)threadIdx.x + i * NT;
        const int n = EDGE ? min(n0 + t, g.N - 1) : n0 + t;
        e.sw[i] = t < BN ? g.sw[(int64_t)n * g.sw_stride] : 0.0f;
        e.bias[i] = (t < BN && g.bias) ? g.bias[n] : 0.0f;
    }
}

// Epilogue shared by the tiled kernels.  Accumulator register r of lane l of a
// 32x32 MFMA tile holds row 8*(r/4) + 4*(l/32) + r%4, column l%32.  The scale
// and bias slices of the block tile are staged in LDS (free once the K loop is
// over); every output element is
//     y = fl(fl(f32(acc) * fl(sa*sw)) + bias), then ReLU,
// evaluated in that order with separately rounded operations.
template <int BM, int BN, int WM, int WN, bool F32OUT, bool EDGE, int NT, bool ROWMAX = false>
__device__ __forceinline__ void epilogue(v16i (&acc)[WM / 32][WN / 32], const GemmArgs &g, int m0, int n0,
                                         int wr, int wc, char *smem, const EpilogueScales<BM, BN, NT> &pre)
{
    constexpr int TM = WM / 32, TN = WN / 32;
    const int lane = threadIdx.x & 63;
    const int col_in = lane & 31, row_in = (lane >> 5) * 4;
    const int M = g.M, N = g.N;
    if constexpr (!F32OUT) {
        int32_t *tile_out = reinterpret_cast<int32_t *>(g.out) + ((int64_t)m0 * N + n0);
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int nl = wc * WN + j * 32 + col_in;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ml = wr * WM + i * 32 + 8 * (r >> 2) + row_in + (r & 3);
                    if (EDGE && (m0 + ml >= M || n0 + nl >= N))
                        continue;
                    tile_out[(unsigned)ml * (unsigned)N + (unsigned)nl] = acc[i][j][r];
                }
            }
        }
    } else {
        float *s_sa = reinterpret_cast<float *>(smem);  // [BM]
        float *s_sw = s_sa + BM;                        // [BN]
        float *s_bias = s_sw + BN;                      // [BN]
        __syncthreads();  // every wave is done with the operand tiles
        if constexpr (kScalesAhead<BM>) {
#pragma unroll
            for (int i = 0; i < (BM + NT - 1) / NT; i++)
                if ((int)threadIdx.x + i * NT < BM)
                    s_sa[threadIdx.x + i * NT] = pre.sa[i];
#pragma unroll
            for (int i = 0; i < (BN + NT - 1) / NT; i++)
                if ((int)threadIdx.x + i * NT < BN) {
                    s_sw[threadIdx.x + i * NT] = pre.sw[i];
                    s_bias[threadIdx.x + i * NT] = pre.bias[i];
                }
        } else {
            for (int t = threadIdx.x; t < BM; t += NT) {
                const int m = EDGE ? min(m0 + t, M - 1) : m0 + t;
                s_sa[t] = g.sa[(int64_t)m * g.sa_stride];
            }
            for (int t = threadIdx.x; t < BN; t += NT) {
                const int n = EDGE ? min(n0 + t, N - 1) : n0 + t;
                s_sw[t] = g.sw[(int64_t)n * g.sw_stride];
                s_bias[t] = g.bias ? g.bias[n] : 0.0f;
            }
        }
        __syncthreads();
        // ROWMAX: max |y| of every row of the wave tile over this lane's columns
        float rmax[ROWMAX ? TM : 1][16];
        if constexpr (ROWMAX) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    rmax[i][r] = 0.0f;
        }
        // The bias / ReLU switches are uniform: branch once, not per element.
        auto store_tile = [&](auto has_bias_t, auto relu_t, auto nt_t) {
            constexpr bool HAS_BIAS = decltype(has_bias_t)::value;
            constexpr bool RELU = decltype(relu_t)::value;
            constexpr bool NT_STORE = decltype(nt_t)::value;
            // uniform tile origin + 32-bit in-tile offsets keep the address math to one add per store
            float *tile_out = reinterpret_cast<float *>(g.out) + ((int64_t)m0 * N + n0);
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int nl = wc * WN + j * 32 + col_in;
                const float w = s_sw[nl];
                const float bv = s_bias[nl];
#pragma unroll
                for (int i = 0; i < TM; i++) {
#pragma unroll
                    for (int rq = 0; rq < 4; rq++) {
                        const int ml = wr * WM + i * 32 + 8 * rq + row_in;
                        const f4 a4 = *reinterpret_cast<const f4 *>(s_sa + ml);
#pragma unroll
                        for (int k = 0; k < 4; k++) {
                            if (EDGE && (m0 + ml + k >= M || n0 + nl >= N))
                                continue;
                            const float s = a4[k] * w;
                            float y = (float)acc[i][j][rq * 4 + k] * s;
                            if (HAS_BIAS)
                                y = y + bv;
                            if (RELU && y < 0.0f)
                                y = 0.0f;
                            if constexpr (ROWMAX)
                                rmax[i][rq * 4 + k] = fmaxf(rmax[i][rq * 4 + k], fabsf(y));
                            float *dst = tile_out + ((unsigned)(ml + k) * (unsigned)N + (unsigned)nl);
                            if (NT_STORE)
                                __builtin_nontemporal_store(y, dst);
                            else
                                *dst = y;
                        }
                        // keep the compiler from hoisting every scale read of the tile to the
                        // top of the epilogue, which costs more registers than there are
                        asm volatile("" ::: "memory");
                    }
                }
            }
        };
        using T_ = std::true_type;
        using F_ = std::false_type;
        // The output is written once and not read by this kernel: non-temporal
        // stores keep it from displacing operand tiles in the caches (2048^3
        // -13 %, 8192^3 -4 %, 1024x4096^2 -6 %).  The exception, measured: a
        // single round of 256x256 tiles, where every workgroup stores at the
        // very end and cached stores let the kernel finish 2.5 % earlier.
        auto store_all = [&](auto nt_t) {
            if (g.bias != nullptr) {
                if (g.relu)
                    store_tile(T_{}, T_{}, nt_t);
                else
                    store_tile(T_{}, F_{}, nt_t);
            } else {
                if (g.relu)
                    store_tile(F_{}, T_{}, nt_t);
                else
                    store_tile(F_{}, F_{}, nt_t);
            }
        };
        if constexpr (ROWMAX) {
            store_all(F_{});   // the rows are read back by the next launch: cached stores
            // Row maxima of the block tile: over the 32 lanes that hold a row's columns (DPP, the
            // first five steps of wave_max: lanes 31 and 63 end up with their half's maximum),
            // then over the waves side by side through LDS (behind the staged scales).
            float *s_rm = s_bias + BN;   // [WN tiles along the row = BN / WN][BM]
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float v = rmax[i][r];
                    v = vtlhip::qdev::dpp_max_step<0xB1, 0xF>(v);
                    v = vtlhip::qdev::dpp_max_step<0x4E, 0xF>(v);
                    v = vtlhip::qdev::dpp_max_step<0x141, 0xF>(v);
                    v = vtlhip::qdev::dpp_max_step<0x140, 0xF>(v);
                    v = vtlhip::qdev::dpp_max_step<0x142, 0xA>(v);
                    if ((lane & 31) == 31)
                        s_rm[wc * BM + wr * WM + i * 32 + 8 * (r >> 2) + row_in + (r & 3)] = v;
                }
            __syncthreads();
            const int tile_n = n0 / BN;
            for (int t = threadIdx.x; t < BM; t += NT) {
                float v = s_rm[t];
#pragma unroll
                for (int c = 1; c < BN / WN; c++)
                    v = fmaxf(v, s_rm[c * BM + t]);
                if (m0 + t < M)
                    g.row_absmax_parts[(int64_t)tile_n * M + m0 + t] = v;
            }
        } else if constexpr (BM == 256 && BN == 256) {
            if (g.cached_out)
                store_all(F_{});
            else
                store_all(T_{});
        } else {
            store_all(T_{});
        }
    }
}

// Sixteen zero bytes in device memory: what lanes past the end of K load.
__device__ __attribute__((aligned(16))) int8_t g_zero_chunk[16];

// Main kernel.  Operand tiles go from global memory straight into LDS
// (global_load_lds_dwordx4, no register staging): a wave instruction fills
// 1 KiB of LDS in lane order, so the XOR swizzle is applied on the global side
// (each lane fetches the chunk that belongs at its LDS slot).  NSTAGE tiles are
// in flight.  MFMA operands are double-buffered in registers, the per-tile
// barrier sits before the last k-step of a tile so that its latency and the
// first operand reads of the next tile hide behind that step's MFMAs, and the
// loads that refill the freed stage are issued a few at a time between MFMAs.
// Requires K % BK == 0; with EDGE rows past M / N are clamped on load and masked
// on store; with KTAIL (and EDGE) K % 16 == 0 is enough: the chunks of the last
// tile that lie past K are loaded as zeros.
template <int BM, int BN, int BK, int NSTAGE, int WR, int WC, bool F32OUT, bool EDGE, bool SPLIT, bool ROWMAX = false,
          bool KTAIL = false>
__global__ __launch_bounds__(64 * WR * WC) void gemm_i8_dma_kernel(const GemmArgs g)
{
    static_assert(EDGE || !KTAIL, "a partial last K tile is handled by the kernels that also clamp rows");
    constexpr int NW = WR * WC, NT = 64 * NW;
    constexpr int WM = BM / WR, WN = BN / WC, TM = WM / 32, TN = WN / 32;
    constexpr int CPR = BK / 16;   // 16-byte chunks per tile row
    constexpr int RPI = 64 / CPR;  // tile rows one wave instruction fills
    constexpr int A_PW = BM / RPI / NW, B_PW = BN / RPI / NW;  // wave instructions per wave per tile
    constexpr int LPT = A_PW + B_PW;
    constexpr int KS = BK / 32;  // MFMA k-steps per tile
    constexpr int STAGE = (BM + BN) * BK;
    static_assert(KS % 2 == 0, "operand double buffering assumes an even number of k-steps");
    static_assert(BM % (RPI * NW) == 0 && BN % (RPI * NW) == 0, "copy split");
    static_assert(NSTAGE >= 2, "at least two stages");

    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int M = g.M, N = g.N, K = g.K;
    // block -> (output tile, K range): consecutive blocks are the K ranges of one tile
    const int nsplit = SPLIT ? g.splits : 1;
    const int split = SPLIT ? (int)(blockIdx.x % nsplit) : 0;
    int tile_m, tile_n;
    tile_of_block((M + BM - 1) / BM, (N + BN - 1) / BN, SPLIT ? (int)(blockIdx.x / nsplit) : (int)blockIdx.x,
                  tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // the wave's index: uniform, so kept in a scalar register
    const int wr = w / WC, wc = w % WC;
    const int kt_all = KTAIL ? (K + BK - 1) / BK : K / BK;  // KTAIL: the last tile may be partial in K
    const int kt_begin = SPLIT ? (int)((int64_t)kt_all * split / nsplit) : 0;
    const int kt_end = SPLIT ? (int)((int64_t)kt_all * (split + 1) / nsplit) : kt_all;

    // ---- global -> LDS ----
    const int lrow = RPI * w + lane / CPR;                  // tile row of this lane for j = 0
    const int lc = (lane % CPR) ^ swizzle<BK>(lrow);        // logical chunk it fetches (same for all j)
    // A load address is a uniform 64-bit part (operand, first row of the tile, K offset and,
    // without EDGE, the rows of load j) plus the lane's 32-bit offset from that row (at most
    // 255 rows of K <= 131072 bytes), which is the form the load instruction takes a scalar base
    // and a vector offset for: no vector arithmetic per load in the K loop.  With EDGE the
    // offsets differ per load, rows past M / N being clamped.
    unsigned oa[EDGE ? A_PW : 1], ob[EDGE ? B_PW : 1];
    if constexpr (EDGE) {
#pragma unroll
        for (int j = 0; j < A_PW; j++)
            oa[j] = (unsigned)(min(m0 + lrow + j * RPI * NW, M - 1) - m0) * (unsigned)K + (unsigned)(lc * 16);
#pragma unroll
        for (int j = 0; j < B_PW; j++)
            ob[j] = (unsigned)(min(n0 + lrow + j * RPI * NW, N - 1) - n0) * (unsigned)K + (unsigned)(lc * 16);
    } else {
        oa[0] = ob[0] = (unsigned)lrow * (unsigned)K + (unsigned)(lc * 16);
    }
    const int8_t *const a0 = g.A + (int64_t)m0 * K;
    const int8_t *const b0 = g.Bt + (int64_t)n0 * K;
    const int64_t jstride = (int64_t)RPI * NW * K;
    // The address of the zero chunk, made opaque to the compiler: left to itself it fetches the
    // address from the global offset table inside the K loop and waits for that scalar load in
    // every iteration.
    const int8_t *zero_chunk = g_zero_chunk;
    if constexpr (KTAIL)
        asm volatile("" : "+s"(zero_chunk));
    // Global source of load d (A rows first, then B) of the tile at K offset ko.
    // With KTAIL, a lane whose 16-byte chunk lies past K reads zeros instead
    // (K % 16 == 0, so a chunk is inside or outside as a whole).  That costs a
    // compare per tile and two selects per load and lane in the K loop (1.5 to
    // 2 us of a 12 us launch), so kernels for ragged M or N with a whole number
    // of K tiles are built without it.
    auto source = [&](int d, int64_t ko) -> const int8_t * {
        const int8_t *p;
        if (d < A_PW)
            p = (a0 + ko + (EDGE ? 0 : d * jstride)) + (uint64_t)oa[EDGE ? d : 0];
        else
            p = (b0 + ko + (EDGE ? 0 : (d - A_PW) * jstride)) + (uint64_t)ob[EDGE ? d - A_PW : 0];
        if constexpr (KTAIL) {
            if (ko + lc * 16 >= K)
                p = zero_chunk;
        }
        return p;
    };
    auto issue = [&](int kt, int st) {
        char *sa_ = smem + st * STAGE;
        char *sb_ = sa_ + BM * BK;
        const int64_t ko = (int64_t)(kt_begin + kt) * BK;
#pragma unroll
        for (int j = 0; j < A_PW; j++)
            __builtin_amdgcn_global_load_lds(VTL_GPTR(source(j, ko)), VTL_LPTR(sa_ + (w + NW * j) * 1024), 16, 0, 0);
#pragma unroll
        for (int j = 0; j < B_PW; j++)
            __builtin_amdgcn_global_load_lds(VTL_GPTR(source(A_PW + j, ko)), VTL_LPTR(sb_ + (w + NW * j) * 1024), 16,
                                             0, 0);
    };

    EpilogueScales<BM, BN, NT> pre;
    if constexpr (F32OUT && !SPLIT && kScalesAhead<BM>)
        fetch_scales<BM, BN, NT, EDGE>(pre, g, m0, n0);

    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                acc[i][j][r] = 0;

    // ---- LDS -> MFMA operands ----
    const int frow = lane & 31;  // row inside a 32-row operand
    const int fh = lane >> 5;    // which 16-byte half of the 32-byte k-step
    int foff[KS];
#pragma unroll
    for (int s = 0; s < KS; s++)
        foff[s] = lds_off<BK>(frow, 2 * s + fh);  // rows 32 apart share the swizzle
    const int a_base = wr * WM * BK, b_base = BM * BK + wc * WN * BK;
    v4i af[2][TM], bf[2][TN];
    auto lfrag = [&](int st, int s, int buf) {
        const char *sbase = smem + st * STAGE;
#pragma unroll
        for (int j = 0; j < TN; j++)
            bf[buf][j] = *reinterpret_cast<const v4i *>(sbase + b_base + j * 32 * BK + foff[s]);
#pragma unroll
        for (int i = 0; i < TM; i++)
            af[buf][i] = *reinterpret_cast<const v4i *>(sbase + a_base + i * 32 * BK + foff[s]);
    };
    auto mma = [&](int buf) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[buf][i], bf[buf][j], acc[i][j], 0, 0, 0);
    };
    // One k-step in a fixed instruction order: MFMA q, then one operand read of
    // the following k-step (stage rd_st, k-step rd_s, into register set rd_buf;
    // B tiles first, then A: the MFMAs run A-tile-major, so the first of them
    // needs both B tiles and only the first A tile), then this MFMA's share of the loads d0..d1-1 of
    // tile `tile` into stage st.  Why the loads are handed out like this: when
    // every wave issues all of its loads in one burst right after the barrier,
    // they pile up in front of the compute unit's one address unit (16 cycles
    // per wave instruction) and the in-order waves wait behind them instead of
    // issuing MFMAs - measured 93.9 k against 83.5 k cycles for the K loop of
    // the 256x256 tile at K = 4096.
    auto step_fixed = [&](int buf, int rd_st, int rd_s, int rd_buf, int tile, int st, int d0, int d1) {
        constexpr int NM = TM * TN, NR = TM + TN;
        const int per = (d1 - d0 + NM - 1) / NM;  // loads after each MFMA
        const char *rbase = smem + rd_st * STAGE;
        char *sa_ = smem + st * STAGE;
        char *sb_ = sa_ + BM * BK;
        const int64_t ko = (int64_t)(kt_begin + tile) * BK;
        auto read_one = [&](int r) {
            if (r < TN)
                bf[rd_buf][r] = *reinterpret_cast<const v4i *>(rbase + b_base + r * 32 * BK + foff[rd_s]);
            else
                af[rd_buf][r - TN] =
                    *reinterpret_cast<const v4i *>(rbase + a_base + (r - TN) * 32 * BK + foff[rd_s]);
        };
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int q = 0; q < NM; q++) {
            acc[q / TN][q % TN] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[buf][q / TN], bf[buf][q % TN],
                                                                        acc[q / TN][q % TN], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (q < NR)
                read_one(q);
#pragma unroll
            for (int d = 0; d < LPT; d++) {
                if (d >= d0 + q * per && d < d0 + (q + 1) * per && d < d1) {
                    if (d < A_PW)
                        __builtin_amdgcn_global_load_lds(VTL_GPTR(source(d, ko)),
                                                         VTL_LPTR(sa_ + (w + NW * d) * 1024), 16, 0, 0);
                    else
                        __builtin_amdgcn_global_load_lds(VTL_GPTR(source(d, ko)),
                                                         VTL_LPTR(sb_ + (w + NW * (d - A_PW)) * 1024), 16, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int r = NM; r < NR; r++)
            read_one(r);
    };
    // scheduling hint: spread the TM+TN LDS reads of the next k-step between
    // the TM*TN MFMAs of the current one
    auto interleave = [&]() {
        constexpr int NR = TM + TN, NM = TM * TN;
        if constexpr (NM >= NR) {
#pragma unroll
            for (int r = 0; r < NR; r++) {
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);        // one LDS read
                __builtin_amdgcn_sched_group_barrier(0x008, NM / NR, 0);  // MFMAs
            }
        }
    };

    // A k-step without loads.  Wave tiles with more MFMAs than operand reads (the 256x256
    // block tile) take the fixed order too - one read after each MFMA, so that every read has
    // several MFMAs of slack before its first use (4096^3 -1.5 %, 8192^3 -2 %, 3000^3 -5 %);
    // small wave tiles have no such slack and issue all reads first (fixed order: 2 % slower).
    auto plain_step = [&](int buf, int rd_st, int rd_s, int rd_buf) {
        if constexpr (TM * TN > TM + TN) {
            step_fixed(buf, rd_st, rd_s, rd_buf, 0, 0, 0, 0);
        } else {
            lfrag(rd_st, rd_s, rd_buf);
            mma(buf);
            interleave();
        }
    };

    const int KT = kt_end - kt_begin;
#pragma unroll
    for (int st = 0; st < NSTAGE; st++)
        if (st < KT)
            issue(st, st);
    if (KT >= NSTAGE)
        wait_vmcnt<(NSTAGE - 1) * LPT>();
    else
        wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    lfrag(0, 0, 0);
    int st_c = 0;
    // One tile but the last: k-steps 0..KS-2, hand-over, last k-step.  The
    // stage that the hand-over of tile kt frees takes tile kt + NSTAGE; its
    // loads are spread over SPREAD k-steps, the first share in the last k-step
    // of tile kt (with_issue), the others in the first k-steps of tile kt + 1
    // (with_prev, seen from that tile).  With two stages the tile is needed
    // again one tile later, so everything goes into the one k-step; with more,
    // three k-steps measured best (four delays the last share too much when the
    // operands come from HBM, as in a split-K launch).
    constexpr int SPREAD = NSTAGE >= 3 ? (KS < 3 ? KS : 3) : 1;
    auto tile_step = [&](auto with_prev, auto with_issue, int kt) {
        const int st_p = (st_c == 0) ? NSTAGE - 1 : st_c - 1;
#pragma unroll
        for (int s = 0; s < KS - 1; s++) {
            if (decltype(with_prev)::value && s + 1 < SPREAD) {
                step_fixed(s & 1, st_c, s + 1, (s + 1) & 1, kt - 1 + NSTAGE, st_p, (s + 1) * LPT / SPREAD,
                           (s + 2) * LPT / SPREAD);
            } else {
                plain_step(s & 1, st_c, s + 1, (s + 1) & 1);
            }
        }
        // every operand read of this tile has been issued: wait for them, make
        // sure the next tile has landed, and hand this tile's buffer over
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const int st_n = (st_c + 1 == NSTAGE) ? 0 : st_c + 1;
        if (decltype(with_issue)::value || kt + NSTAGE - 1 < KT)
            wait_vmcnt<(NSTAGE - 2) * LPT>();
        else
            wait_vmcnt<0>();
        __builtin_amdgcn_s_barrier();
        if constexpr (decltype(with_issue)::value) {
            step_fixed((KS - 1) & 1, st_n, 0, 0, kt + NSTAGE, st_c, 0, LPT / SPREAD);
        } else {
            plain_step((KS - 1) & 1, st_n, 0, 0);
        }
        st_c = st_n;
    };
    using Yes = std::true_type;
    using No = std::false_type;
    using Prev = std::integral_constant<bool, (SPREAD > 1)>;
    int kt = 0;
    if (NSTAGE < KT) {
        tile_step(No{}, Yes{}, 0);
        for (kt = 1; kt + NSTAGE < KT; kt++)
            tile_step(Prev{}, Yes{}, kt);
        // kt == KT - NSTAGE: the rest of the last tile's loads, no new tile
        tile_step(Prev{}, No{}, kt);
        kt++;
    }
    for (; kt < KT - 1; kt++)
        tile_step(No{}, No{}, kt);
#pragma unroll
    for (int s = 0; s < KS - 1; s++)
        plain_step(s & 1, st_c, s + 1, (s + 1) & 1);
    mma((KS - 1) & 1);

    if constexpr (SPLIT) {
        // raw partial sums of this K range; splitk_finalize_kernel adds the ranges up
        GemmArgs gp = g;
        gp.out = g.partials + (int64_t)split * M * N;
        epilogue<BM, BN, WM, WN, false, EDGE, NT>(acc, gp, m0, n0, wr, wc, smem, pre);
    } else {
        epilogue<BM, BN, WM, WN, F32OUT, EDGE, NT, ROWMAX>(acc, g, m0, n0, wr, wc, smem, pre);
    }
}

// Sums the int32 partial results of a split-K launch (exact, order-free) and
// applies the epilogue.  VEC consecutive outputs of one row per thread, n
// fastest (VEC = 4 needs N % 4 == 0 and 16-byte aligned buffers).
template <bool F32OUT, int VEC>
__global__ __launch_bounds__(256) void splitk_finalize_kernel(const GemmArgs g)
{
    const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    const int64_t mn = (int64_t)g.M * g.N;
    if (idx >= mn)
        return;
    int acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; j++)
        acc[j] = 0;
#pragma unroll 4
    for (int s = 0; s < g.splits; s++) {   // independent loads: several K ranges in flight per thread
        const int32_t *p = g.partials + (int64_t)s * mn + idx;
        if (VEC == 4) {
            const v4i v = *reinterpret_cast<const v4i *>(p);
#pragma unroll
            for (int j = 0; j < VEC; j++)
                acc[j] += v[j];
        } else {
            acc[0] += p[0];
        }
    }
    if (F32OUT) {
        const int m = (int)(idx / g.N), n = (int)(idx % g.N);
        const float sa = g.sa[(int64_t)m * g.sa_stride];
        float y[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            const float sc = sa * g.sw[(int64_t)(n + j) * g.sw_stride];
            y[j] = (float)acc[j] * sc;
            if (g.bias)
                y[j] = y[j] + g.bias[n + j];
            if (g.relu && y[j] < 0.0f)
                y[j] = 0.0f;
        }
        float *out = reinterpret_cast<float *>(g.out) + idx;
        if (VEC == 4) {
            *reinterpret_cast<vtlhip::qdev::float4_t *>(out) = vtlhip::qdev::float4_t{y[0], y[1], y[2], y[3]};
        } else {
            out[0] = y[0];
        }
    } else {
        int32_t *out = reinterpret_cast<int32_t *>(g.out) + idx;
        if (VEC == 4) {
            *reinterpret_cast<v4i *>(out) = v4i{acc[0], acc[1], acc[2], acc[3]};
        } else {
            out[0] = acc[0];
        }
    }
}

// Epilogue and per-row requantization in one pass over the int32 sums: one
// workgroup per output row adds the K ranges up (exact), applies
// y = fl(fl(f32(acc) * fl(sa * sw)) + bias) and ReLU as the other epilogues do,
// keeps the row in registers (4 * NV consecutive-by-four columns per thread,
// N <= 4 * T * NV, N % 4 == 0), takes its absmax and writes the codes the row
// quantizer would write for that f32 row (same arithmetic, same bits), its
// scale, and the f32 row itself when asked for.
template <int T, int NV>
__global__ __launch_bounds__(T) void finalize_requant_kernel(const GemmArgs g)
{
    constexpr int NW = T / 64;
    __shared__ float red[NW];
    const int m = blockIdx.x, N = g.N;
    const int64_t mn = (int64_t)g.M * N;
    // every load of the kernel is issued up front - the row scale, the column scales and bias
    // of this thread's columns, then the int32 sums of all K ranges - so that the kernel is one
    // memory latency deep, not three
    const float sa = g.sa[(int64_t)m * g.sa_stride];
    f4 swv[NV], bv[NV];
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int n = 4 * (v * T + (int)threadIdx.x);
        swv[v] = f4{0.f, 0.f, 0.f, 0.f};
        bv[v] = f4{0.f, 0.f, 0.f, 0.f};
        if (n < N) {
            swv[v] = g.sw_stride ? *reinterpret_cast<const f4 *>(g.sw + n) : f4{g.sw[0], g.sw[0], g.sw[0], g.sw[0]};
            if (g.bias)
                bv[v] = *reinterpret_cast<const f4 *>(g.bias + n);
        }
    }
    v4i acc[NV];
    const int32_t *p0 = g.partials + (int64_t)m * N + 4 * (int)threadIdx.x;
#pragma unroll
    for (int v = 0; v < NV; v++)
        acc[v] = 4 * (v * T + (int)threadIdx.x) < N ? *reinterpret_cast<const v4i *>(p0 + 4 * v * T) : v4i{0, 0, 0, 0};
#pragma unroll 4
    for (int s = 1; s < g.splits; s++) {
        v4i t[NV];
#pragma unroll
        for (int v = 0; v < NV; v++)
            t[v] = 4 * (v * T + (int)threadIdx.x) < N ? *reinterpret_cast<const v4i *>(p0 + (int64_t)s * mn + 4 * v * T)
                                                      : v4i{0, 0, 0, 0};
#pragma unroll
        for (int v = 0; v < NV; v++)
            acc[v] += t[v];
    }
    f4 y[NV];
    float am = 0.0f;
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int n = 4 * (v * T + (int)threadIdx.x);
        y[v] = f4{0.f, 0.f, 0.f, 0.f};
        if (n < N) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float sc = sa * swv[v][j];
                float t = (float)acc[v][j] * sc;
                if (g.bias)
                    t = t + bv[v][j];
                if (g.relu && t < 0.0f)
                    t = 0.0f;
                y[v][j] = t;
            }
            am = vtlhip::qdev::absmax4(am, y[v]);
        }
    }
    am = vtlhip::qdev::wave_max(am);
    if ((threadIdx.x & 63) == 0)
        red[threadIdx.x >> 6] = am;
    __syncthreads();
    am = red[0];
#pragma unroll
    for (int i = 1; i < NW; i++)
        am = fmaxf(am, red[i]);
    const float sy = am / 127.0f;
    const vtlhip::qdev::QuantScale qp = vtlhip::qdev::make_quant_scale(sy);
    if (threadIdx.x == 0)
        g.requant_scales[m] = sy;
#pragma unroll
    for (int v = 0; v < NV; v++) {
        const int n = 4 * (v * T + (int)threadIdx.x);
        if (n < N) {
            const int64_t o = (int64_t)m * N + n;
            *reinterpret_cast<unsigned *>(g.requant_codes + o) = vtlhip::qdev::quant4(y[v], qp);
            if (g.out)
                *reinterpret_cast<f4 *>(reinterpret_cast<float *>(g.out) + o) = y[v];
        }
    }
}

inline bool requant_rows_fit(int N)
{
    return N % 4 == 0 && N <= 16384;
}

int launch_finalize_requant(const GemmArgs &g, hipStream_t st)
{
    const dim3 grid((unsigned)g.M);
    // one workgroup per row and often few rows: large workgroups keep more loads in flight
    if (g.N <= 1024)
        hipLaunchKernelGGL((finalize_requant_kernel<256, 1>), grid, dim3(256), 0, st, g);
    else if (g.N <= 2048)
        hipLaunchKernelGGL((finalize_requant_kernel<512, 1>), grid, dim3(512), 0, st, g);
    else if (g.N <= 4096)
        hipLaunchKernelGGL((finalize_requant_kernel<1024, 1>), grid, dim3(1024), 0, st, g);
    else if (g.N <= 8192)
        hipLaunchKernelGGL((finalize_requant_kernel<1024, 2>), grid, dim3(1024), 0, st, g);
    else
        hipLaunchKernelGGL((finalize_requant_kernel<1024, 4>), grid, dim3(1024), 0, st, g);
    return check_launch("finalize_requant_kernel");
}

// Second half of a requantizing linear whose tile kernel applied the epilogue itself: the
// f32 rows are there, and per row one partial maximum of |y| per tile along N.  A workgroup
// takes 4096 columns of one row: it reduces the row's partial maxima (a few hundred bytes,
// every workgroup of the row redoes it), derives the row scale exactly as the row quantizer
// does and writes the codes of its columns.  Needs N % 4 == 0 and 16-byte aligned rows.
__global__ __launch_bounds__(256) void requant_rows_wide_kernel(const float *__restrict__ y,
                                                                const float *__restrict__ parts, int tiles_n, int M,
                                                                int N, int8_t *__restrict__ codes,
                                                                float *__restrict__ scales)
{
    __shared__ float red[4];
    const int m = blockIdx.y;
    const int n = (int)blockIdx.x * 4096 + 4 * (int)threadIdx.x;
    const f4 *row = reinterpret_cast<const f4 *>(y + (int64_t)m * N);
    f4 v[4];
#pragma unroll
    for (int i = 0; i < 4; i++)   // in flight while the maxima are reduced
        v[i] = n + 1024 * i < N ? row[(n + 1024 * i) >> 2] : f4{0.f, 0.f, 0.f, 0.f};
    float am = 0.0f;
    for (int t = threadIdx.x; t < tiles_n; t += 256)
        am = fmaxf(am, parts[(int64_t)t * M + m]);
    am = vtlhip::qdev::block_max<256>(am, red);
    const float sy = am / 127.0f;
    const vtlhip::qdev::QuantScale qp = vtlhip::qdev::make_quant_scale(sy);
    if (blockIdx.x == 0 && threadIdx.x == 0)
        scales[m] = sy;
    unsigned *out = reinterpret_cast<unsigned *>(codes + (int64_t)m * N);
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (n + 1024 * i < N)
            out[(n + 1024 * i) >> 2] = vtlhip::qdev::quant4(v[i], qp);
}

// Workgroup barrier that orders LDS traffic only: unlike __syncthreads() it does
// not wait for outstanding global loads, so direct-to-LDS weight loads issued
// earlier stay in flight across it.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// ---- activations quantized inside the weight-streaming launch ----------------
//
// A decode-shaped linear on f32 activations used to be two launches, the row quantizer and the
// weight-streaming kernel; the first cost 3.2 us in front of a 12 us kernel, nearly all of it
// launch latency.  Here one launch does both.  Its first M workgroups ("producers",
// dispatched first) quantize one activation row each into the staging buffer and count
// themselves in the slot's counter; the other workgroups start their weight stream, wait
// until the counter has reached the value the host computed for this launch, and then read
// codes and scales as they would after a quantizer launch (N = 14336, K = 4096: 14.4 against
// 16.0 us with 8 rows, 16.8 against 18.8 us with 32).  Splitting a row's conversion over
// several producers, or giving every XCD producers and a staging copy of its own (nothing
// then leaves an L2), measured slower: both read the cold activations more often.
//
// Coherence.  The chip has eight L2 caches (one per XCD) that do not snoop each other, and a
// release or acquire fence of device scope writes back or invalidates a whole L2: a few tenths
// of a microsecond each, 40 us for the ~900 waves of such a launch (measured).  So no fence is
// used.  Producers store codes and scales with device-scope stores, which go through their
// L2 to memory, wait until those are acknowledged (s_waitcnt vmcnt(0), then the workgroup
// barrier) and only then count themselves; the counter is touched with device-scope atomics
// only, which are carried out at the memory side.  A waiting workgroup cannot hold a stale
// copy of the staging buffer: every cache was invalidated when the launch began and nothing
// reads the buffer before the count is complete (a workgroup that gives up waiting writes
// the same values before it reads them), so its ordinary loads miss and fetch what the
// producers wrote.
//
// The counter only ever grows: the host keeps, per slot, the sum of the producers of all
// launches so far, so nothing needs clearing between launches; a launch recorded into a
// graph would replay a stale target, so this form is not used while the stream is capturing.
// There are 64 copies of the counter, 256 bytes apart; every producer adds to all of them (one
// wave instruction) and a waiting workgroup polls one: 448 workgroups polling a single
// address took longer than the quantizer launch this replaces.  The wait is bounded: after
// spin_limit polls a workgroup quantizes all M rows itself (the same values into the same
// places) and goes on, so the launch drains whatever the order in which workgroups start.
// Launches that share a slot must not overlap.
constexpr int kStageSlots = vtlhip::kStreamSlots;
constexpr int kStageCopies = 64;
constexpr int kStageMaxK = 8192;
__device__ unsigned g_stage_count[kStageSlots * kStageCopies * 64];

__device__ __forceinline__ void stage_store(unsigned *p, unsigned v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void wait_memory_acknowledged()
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// One row of K floats (K % 4 == 0, K <= 8192) by a workgroup of NT threads: scale = absmax / 127,
// codes as the row quantizer makes them, stored through to memory; a thread returns when its
// stores are acknowledged.  `red` holds NT / 64 floats; the caller puts a barrier between two
// calls.
template <int NT>
__device__ __forceinline__ void stage_quantize_row(const float *x, int K, int8_t *q, float *scale_out, float *red)
{
    constexpr int NV = kStageMaxK / 4 / NT;
    const vtlhip::qdev::float4_t *xv = reinterpret_cast<const vtlhip::qdev::float4_t *>(x);
    unsigned *qv = reinterpret_cast<unsigned *>(q);
    const int nv = K >> 2;
    vtlhip::qdev::float4_t v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int idx = i * NT + (int)threadIdx.x;
        v[i] = idx < nv ? xv[idx] : vtlhip::qdev::float4_t{0.f, 0.f, 0.f, 0.f};
    }
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < NV; i++)
        m = vtlhip::qdev::absmax4(m, v[i]);
    m = vtlhip::qdev::block_max<NT>(m, red);
    const float scale = m / 127.0f;
    if (threadIdx.x == 0)
        stage_store(reinterpret_cast<unsigned *>(scale_out), __float_as_uint(scale));
    const vtlhip::qdev::QuantScale p = vtlhip::qdev::make_quant_scale(scale);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int idx = i * NT + (int)threadIdx.x;
        if (idx < nv)
            stage_store(qv + idx, vtlhip::qdev::quant4(v[i], p));
    }
    wait_memory_acknowledged();
}

// Weight-streaming kernel for M <= 32 (decode-shaped linear): bound by reading
// the weight matrix once, so the design goal is bytes in flight and long
// contiguous reads, not MFMA rate.  (With more activation rows grid.y walks
// blocks of 32 of them: the form used for small outputs with a long K, see
// skinny_blocks_waves.)  A workgroup owns 32 weight rows (128 KiB of
// contiguous memory when K = 4096); its NWAVE waves split K between them and
// each wave runs a PRIVATE software pipeline - its own LDS ring of STAGES
// slots (32 rows x 256 bytes of Wq plus the activation rows that exist),
// filled by its own direct-to-LDS loads and released by its own vmcnt waits -
// so there is no workgroup barrier in the K loop at all.  Reads are 256 bytes
// per row per step: measured, 128-byte pieces at row stride reach 5.4 TB/s on
// this matrix, 256-byte pieces 7.8 TB/s.  The waves' int32 partial tiles are
// added up through LDS at the end (exact), then the f32 epilogue runs.
// MFMA operand A = weight rows (n), operand B = activation rows (m), so a
// lane ends up with four consecutive n of one m: 16-byte stores along Y rows.
// Only the 8*XJ activation rows that can exist (M <= 8*XJ) are loaded; lanes
// of absent rows re-read existing ones and their output columns are never
// stored.  Requires K % 256 == 0; rows past N are clamped on load and masked
// on store.
template <int NWAVE, int STAGES, int XJ, bool F32OUT, bool STAGEQ = false>
__global__ __launch_bounds__(64 * NWAVE) void linear_skinny_kernel(const GemmArgs g)
{
    static_assert(!STAGEQ || STAGES == 2, "the staged form counts its first loads for a ring of two slots");
    constexpr int BK = 256;
    constexpr int WCHUNK = 32 * BK;              // 8 KiB of weights per slot
    constexpr int XROWS = 8 * XJ;
    constexpr int SLOT = WCHUNK + XROWS * BK;
    constexpr int WLOADS = 8, XLOADS = 2 * XJ;   // wave instructions (4 rows x 256 bytes each)
    constexpr int LOADS = WLOADS + XLOADS;
    constexpr int KS = BK / 32;                  // MFMA k-steps per slot
    static_assert((STAGES - 1) * LOADS <= 63, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const int M = g.M, N = g.N, K = g.K;
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform in a wave: a scalar, and with it the ring addresses
    __shared__ float s_red[NWAVE];
    __shared__ int s_ready;
    int bx = blockIdx.x;
    unsigned *const counter = g_stage_count + g.sync_slot * (kStageCopies * 64);
    if constexpr (STAGEQ) {
        if (bx < M) {   // producer: one activation row, then gone
            stage_quantize_row<64 * NWAVE>(g.xf32 + (int64_t)bx * K, K, g.stage_codes + (int64_t)bx * K,
                                           g.stage_scales + bx, s_red);
            __syncthreads();   // every thread's share of the row is in memory
            if (tid < kStageCopies)
                __hip_atomic_fetch_add(counter + tid * 64, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
        bx -= M;
    }
    const int n0 = bx * 32;
    const int m0 = blockIdx.y * 32;   // more than 32 activation rows: one block of 32 per grid row
    char *ring = smem + w * (STAGES * SLOT);

    // K range of this wave, in 256-byte chunks
    const int kc_all = K / BK;
    const int kc_begin = (int)((int64_t)kc_all * w / NWAVE);
    const int kc_end = (int)((int64_t)kc_all * (w + 1) / NWAVE);
    const int KC = kc_end - kc_begin;

    // global -> LDS: instruction j covers tile rows 4j .. 4j+3, 16 lanes per 256-byte row;
    // LDS rows are 256 bytes, 16-byte chunk index XOR (row & 15)
    const int lrow = lane >> 4;
    const int8_t *pw[WLOADS];
    const int8_t *px[XLOADS];
#pragma unroll
    for (int j = 0; j < WLOADS; j++) {
        const int row = lrow + 4 * j;
        const int lc = (lane & 15) ^ (row & 15);
        pw[j] = g.Bt + (int64_t)min(n0 + row, N - 1) * K + (int64_t)kc_begin * BK + lc * 16;
    }
#pragma unroll
    for (int j = 0; j < XLOADS; j++) {
        const int row = lrow + 4 * j;
        const int lc = (lane & 15) ^ (row & 15);
        px[j] = g.A + (int64_t)min(m0 + row, M - 1) * K + (int64_t)kc_begin * BK + lc * 16;
    }
    auto issue_w = [&](int c, int st) {
        char *sw_ = ring + st * SLOT;
        const int64_t ko = (int64_t)c * BK;
        // (the cache policy is part of the instruction: one copy of the loads for each)
        if (g.stream_weights) {
#pragma unroll
            for (int j = 0; j < WLOADS; j++)
                __builtin_amdgcn_global_load_lds(VTL_GPTR(pw[j] + ko), VTL_LPTR(sw_ + j * 1024), 16, 0, 2);
        } else {
#pragma unroll
            for (int j = 0; j < WLOADS; j++)
                __builtin_amdgcn_global_load_lds(VTL_GPTR(pw[j] + ko), VTL_LPTR(sw_ + j * 1024), 16, 0, 0);
        }
    };
    auto issue_x = [&](int c, int st) {
        char *sx_ = ring + st * SLOT + WCHUNK;
        const int64_t ko = (int64_t)c * BK;
#pragma unroll
        for (int j = 0; j < XLOADS; j++)
            __builtin_amdgcn_global_load_lds(VTL_GPTR(px[j] + ko), VTL_LPTR(sx_ + j * 1024), 16, 0, 0);
    };
    auto issue = [&](int c, int st) {
        issue_w(c, st);
        issue_x(c, st);
    };

    v16i acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        acc0[r] = 0;
        acc1[r] = 0;
    }
    const int frow = lane & 31, fh = lane >> 5;
    const int xrow = frow & (XROWS - 1);  // absent activation rows alias existing ones
    int woff[KS], xoff[KS];
#pragma unroll
    for (int s = 0; s < KS; s++) {
        woff[s] = frow * BK + ((((2 * s + fh) ^ frow) & 15) << 4);
        xoff[s] = xrow * BK + ((((2 * s + fh) ^ xrow) & 15) << 4);
    }

    // The scales and bias of the outputs this thread will write are asked for now, ahead of the
    // weight stream: read in the epilogue they would add a memory latency to the end of every
    // workgroup.  (They are older than every ring load, so the ring's vmcnt waits cover them.)
    constexpr int ITEMS = 256 / (64 * NWAVE);   // (m, 4 x n) outputs per thread
    float e_sa[F32OUT ? ITEMS : 1], e_sw[F32OUT ? ITEMS : 1][4], e_bias[F32OUT ? ITEMS : 1][4];
    if constexpr (F32OUT) {
#pragma unroll
        for (int it = 0; it < ITEMS; it++) {
            const int item = tid + it * 64 * NWAVE;
            const int m = m0 + (item >> 3), n = n0 + (item & 7) * 4;
            if constexpr (!STAGEQ)
                e_sa[it] = m < M ? g.sa[(int64_t)m * g.sa_stride] : 0.0f;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const bool in = m < M && n + k < N;
                e_sw[it][k] = in ? g.sw[(int64_t)(n + k) * g.sw_stride] : 0.0f;
                e_bias[it][k] = (in && g.bias) ? g.bias[n + k] : 0.0f;
            }
        }
    }
    if constexpr (STAGEQ) {
        // the weights of every ring slot are under way while the activations are being made
#pragma unroll
        for (int st = 0; st < STAGES; st++)
            if (st < KC)
                issue_w(st, st);
        if (tid == 0) {
            int seen = 0;
            const unsigned *mine = counter + (bx % kStageCopies) * 64;
            for (int spin = 0;; spin++) {
                const unsigned now = __hip_atomic_load(mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((int)(now - g.stage_target) >= 0) {
                    seen = 1;
                    break;
                }
                if (spin >= g.spin_limit)
                    break;
                __builtin_amdgcn_s_sleep(1);
            }
            s_ready = seen;
        }
        lds_barrier();
        if (!s_ready) {   // not seen in time: this workgroup makes the rows itself
            for (int r = 0; r < M; r++) {
                stage_quantize_row<64 * NWAVE>(g.xf32 + (int64_t)r * K, K, g.stage_codes + (int64_t)r * K,
                                               g.stage_scales + r, s_red);
                __syncthreads();
            }
        }
        asm volatile("" ::: "memory");   // the loads below stay below
        if constexpr (F32OUT) {
#pragma unroll
            for (int it = 0; it < ITEMS; it++) {
                const int m = m0 + ((tid + it * 64 * NWAVE) >> 3);
                e_sa[it] = m < M ? g.sa[m] : 0.0f;
            }
        }
#pragma unroll
        for (int st = 0; st < STAGES; st++)
            if (st < KC)
                issue_x(st, st);
    } else {
#pragma unroll
        for (int st = 0; st < STAGES - 1; st++)
            if (st < KC)
                issue(st, st);
    }
    int st_c = 0, st_l = STAGES - 1;
    for (int c = 0; c < KC; c++) {
        if (STAGEQ && c == 0) {
            // Both slots were filled above, the weight loads first (W0 W1 X0 X1): chunk 0 is
            // there when only X1 is outstanding.
            if (KC > 1)
                wait_vmcnt<XLOADS>();
            else
                wait_vmcnt<0>();
        } else if (c + STAGES - 1 < KC) {
            issue(c + STAGES - 1, st_l);
            wait_vmcnt<(STAGES - 1) * LOADS>();  // chunk c has landed
        } else {
            wait_vmcnt<0>();
        }
        const char *sw_ = ring + st_c * SLOT;
        const char *sx_ = sw_ + WCHUNK;
        v4i wf[KS], xf[KS];
#pragma unroll
        for (int s = 0; s < KS; s++) {
            wf[s] = *reinterpret_cast<const v4i *>(sw_ + woff[s]);
            xf[s] = *reinterpret_cast<const v4i *>(sx_ + xoff[s]);
        }
#pragma unroll
        for (int s = 0; s < KS; s += 2) {
            acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[s], xf[s], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[s + 1], xf[s + 1], acc1, 0, 0, 0);
        }
        // the reads of this slot are complete before it is refilled in the next iteration
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        st_c = (st_c + 1 == STAGES) ? 0 : st_c + 1;
        st_l = (st_l + 1 == STAGES) ? 0 : st_l + 1;
    }

    // ---- add the waves' partial tiles up through LDS: part[wave][m][n] ----
    __syncthreads();  // every wave is done with its ring
    int *part = reinterpret_cast<int *>(smem);
    {
        const int m = lane & 31, nb = (lane >> 5) * 4;
#pragma unroll
        for (int rq = 0; rq < 4; rq++) {
            v4i v;
#pragma unroll
            for (int k = 0; k < 4; k++)
                v[k] = acc0[rq * 4 + k] + acc1[rq * 4 + k];
            *reinterpret_cast<v4i *>(part + w * 1024 + m * 32 + 8 * rq + nb) = v;
        }
    }
    __syncthreads();
    // 256 (m, 4 x n) items; 8 threads cover the 128-byte row segment of one m
#pragma unroll
    for (int it = 0; it < ITEMS; it++) {
        const int item = tid + it * 64 * NWAVE;
        const int ml = item >> 3, nq = (item & 7) * 4;
        v4i sum = *reinterpret_cast<const v4i *>(part + ml * 32 + nq);
#pragma unroll
        for (int ww = 1; ww < NWAVE; ww++)
            sum += *reinterpret_cast<const v4i *>(part + ww * 1024 + ml * 32 + nq);
        const int m = m0 + ml;
        if (m >= M)
            continue;
        const int n = n0 + nq;
        const int64_t o = (int64_t)m * N + n;
        if constexpr (F32OUT) {
            const float a = e_sa[it];
            float y[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int k = 0; k < 4; k++) {
                if (n + k < N) {
                    const float sc = a * e_sw[it][k];
                    float v = (float)sum[k] * sc;
                    if (g.bias)
                        v = v + e_bias[it][k];
                    if (g.relu && v < 0.0f)
                        v = 0.0f;
                    y[k] = v;
                }
            }
            if (n + 3 < N && (N & 3) == 0) {
                *reinterpret_cast<f4 *>(reinterpret_cast<float *>(g.out) + o) = f4{y[0], y[1], y[2], y[3]};
            } else {
#pragma unroll
                for (int k = 0; k < 4; k++)
                    if (n + k < N)
                        reinterpret_cast<float *>(g.out)[o + k] = y[k];
            }
        } else {
            if (n + 3 < N && (N & 3) == 0) {
                *reinterpret_cast<v4i *>(reinterpret_cast<int32_t *>(g.out) + o) = sum;
            } else {
#pragma unroll
                for (int k = 0; k < 4; k++)
                    if (n + k < N)
                        reinterpret_cast<int32_t *>(g.out)[o + k] = sum[k];
            }
        }
    }
}

// Sum of an int over the 64 lanes of a wave, the same value returned to every
// lane: cross-lane moves inside the VALU (DPP) instead of six trips through the
// LDS crossbar.  Quads, half rows and rows by mirroring, then lane 15 of each
// row into the next row and lane 31 into the upper half; lane 63 holds the sum.
__device__ __forceinline__ int wave_sum_i32(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, false);  // row_half_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, false);  // row_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);  // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast:31 into rows 2 and 3
    return __builtin_amdgcn_readlane(v, 63);
}

// Single token (M = 1): a matrix-vector product bound by reading Wq once, done
// without LDS staging and without MFMA.  With DYNQ the row arrives as f32 and
// every workgroup quantizes it itself (K floats from L2, the arithmetic of the
// row quantizer, codes exchanged through LDS) while the first weight rows of
// its waves are already in flight; otherwise the codes and their scale are
// read as given.  Each lane keeps its 16-byte pieces of the codes in registers
// (KV of them, K <= 1024 * KV) for all rows.  A wave owns a run of consecutive
// weight rows: a row is up to KV fully coalesced 1 KiB loads straight into
// registers (cached loads: between launches the weights stay in the last-level
// cache, non-temporal ones measured 20-40 % slower), two rows are in flight
// while the current one goes through 4 * KV dot4 instructions and a
// cross-lane sum.  Requires K % 16 == 0, the row and Wq 16-byte aligned.
template <int KV, int NWAVE, bool DYNQ, bool F32OUT, bool WNT = false>
__global__ __launch_bounds__(64 * NWAVE) void linear_gemv_kernel(const GemmArgs g)
{
    constexpr int T = 64 * NWAVE;
    constexpr int XV = (256 * KV + T - 1) / T;  // float4 of x per thread
    constexpr int DEPTH = 2, RING = DEPTH + 1;
    __shared__ float red[NWAVE];
    __shared__ __attribute__((aligned(16))) int8_t xq[DYNQ ? 1024 * KV : 16];
    const int N = g.N, K = g.K;
    const int kv = K >> 4;  // 16-byte pieces of a row
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // rows are dealt out cyclically: wave i of W takes rows i, i + W, i + 2 W, ... so that at any
    // moment the waves of the chip read one contiguous stretch of the matrix
    const int64_t W = (int64_t)gridDim.x * NWAVE;
    const int64_t r0 = (int64_t)blockIdx.x * NWAVE + w, r1 = N;

    // the activations are asked for first: behind the weight rows they would wait for all of them
    f4 xr[XV];
    if constexpr (DYNQ) {
        const f4 *xv = reinterpret_cast<const f4 *>(g.xf32);
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const int idx = i * T + threadIdx.x;
            xr[i] = idx < (K >> 2) ? xv[idx] : f4{0.f, 0.f, 0.f, 0.f};
        }
    }
    v4i wb[RING][KV];
    auto load_row = [&](int64_t r, v4i (&dst)[KV]) {
        const v4i *p = reinterpret_cast<const v4i *>(g.Bt + r * K) + lane;
#pragma unroll
        for (int j = 0; j < KV; j++)
            dst[j] = (64 * j + lane < kv) ? (WNT ? __builtin_nontemporal_load(p + 64 * j) : p[64 * j]) : v4i{0, 0, 0, 0};
    };
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
        if (r0 + d * W < r1)
            load_row(r0 + d * W, wb[d]);

    v4i xc[KV];
    float sx;
    if constexpr (DYNQ) {
        float m = 0.0f;
#pragma unroll
        for (int i = 0; i < XV; i++)
            m = vtlhip::qdev::absmax4(m, xr[i]);
        m = vtlhip::qdev::wave_max(m);
        if (lane == 0)
            red[w] = m;
        lds_barrier();
        float am = red[0];
#pragma unroll
        for (int i = 1; i < NWAVE; i++)
            am = fmaxf(am, red[i]);
        sx = am / 127.0f;
        const vtlhip::qdev::QuantScale qp = vtlhip::qdev::make_quant_scale(sx);
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const int idx = i * T + threadIdx.x;
            if (idx < 256 * KV)  // pieces past K are written as zeros
                reinterpret_cast<unsigned *>(xq)[idx] = vtlhip::qdev::quant4(xr[i], qp);
        }
        lds_barrier();
#pragma unroll
        for (int j = 0; j < KV; j++)
            xc[j] = reinterpret_cast<const v4i *>(xq)[64 * j + lane];
    } else {
        sx = F32OUT ? g.sa[0] : 0.0f;
        const v4i *p = reinterpret_cast<const v4i *>(g.A) + lane;
#pragma unroll
        for (int j = 0; j < KV; j++)
            xc[j] = (64 * j + lane < kv) ? p[64 * j] : v4i{0, 0, 0, 0};
    }

    // lane u of the wave looks after its u-th row: scale and bias are fetched now, the sum is
    // parked in the lane when the row is done, the epilogue runs once after the loop
    const int64_t my_row = r0 + (int64_t)lane * W;
    const bool mine = my_row < r1;
    float swv = 0.0f, bv = 0.0f;
    if (F32OUT && mine) {
        swv = g.sw[my_row * g.sw_stride];
        if (g.bias)
            bv = g.bias[my_row];
    }
    int res = 0, it = 0;
    for (int64_t rb = r0; rb < r1; rb += RING * W) {
#pragma unroll
        for (int u = 0; u < RING; u++) {
            const int64_t r = rb + u * W;
            if (r >= r1)
                break;
            if (r + DEPTH * W < r1)
                load_row(r + DEPTH * W, wb[(u + DEPTH) % RING]);
            int acc = 0;
#pragma unroll
            for (int j = 0; j < KV; j++)
#pragma unroll
                for (int c = 0; c < 4; c++)
                    acc = __builtin_amdgcn_sdot4(wb[u][j][c], xc[j][c], acc, false);
            acc = wave_sum_i32(acc);
            res = (lane == it) ? acc : res;
            it++;
        }
    }
    if (mine) {
        if constexpr (F32OUT) {
            const float sc = sx * swv;
            float y = (float)res * sc;
            if (g.bias)
                y = y + bv;
            if (g.relu && y < 0.0f)
                y = 0.0f;
            reinterpret_cast<float *>(g.out)[my_row] = y;
        } else {
            reinterpret_cast<int32_t *>(g.out)[my_row] = res;
        }
    }
}


template <int CTRL>
__device__ __forceinline__ int dpp_move(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}

// MR per-lane partial sums (one per activation row) of the 64 lanes, added up
// so that lane l ends with the wave's total for row l % MR.  Each folding step
// halves the number of values a lane carries: the lanes of a pair keep one half
// each and hand the other half over, so 8 rows cost 4 + 2 + 1 exchanges and
// one more per remaining lane bit, instead of six per row.
template <int MR>
__device__ __forceinline__ int fold_rows(int (&a)[MR], int lane)
{
    if constexpr (MR == 1) {
        return a[0];
    } else {
        constexpr int H = MR / 2;
        const bool hi = (lane & H) != 0;
        int b[H];
#pragma unroll
        for (int i = 0; i < H; i++) {
            const int send = hi ? a[i] : a[i + H], keep = hi ? a[i + H] : a[i];
            if constexpr (MR == 8)
                b[i] = keep + dpp_move<0x141>(send);  // row_half_mirror: lane l of 8 <-> 7 - l
            else if constexpr (MR == 4)
                b[i] = keep + dpp_move<0x4E>(send);   // quad_perm [2,3,0,1]
            else
                b[i] = keep + dpp_move<0xB1>(send);   // quad_perm [1,0,3,2]
        }
        return fold_rows<H>(b, lane);
    }
}

template <int MR>
__device__ __forceinline__ int wave_sum_rows(int (&a)[MR], int lane)
{
    int v = fold_rows<MR>(a, lane);
    if constexpr (MR < 4)
        v += dpp_move<0x4E>(v);   // lanes l and l ^ 2
    if constexpr (MR < 8)
        v += dpp_move<0x124>(v);  // row_ror:4
    v += dpp_move<0x128>(v);      // row_ror:8
    // rows of 16 lanes: odd rows against even rows, then the upper half against the lower one
    const auto r16 = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    v = r16[0] + r16[1];
    const auto r32 = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return r32[0] + r32[1];
}

// A few tokens (2 <= M <= MR, MR = 2, 4 or 8): the single-token kernel with MR
// rows of codes in registers (16 * KV * MR bytes per lane), so every weight
// row, loaded once and straight into registers, meets all of them: 4 * KV * MR
// dot4 instructions and one folded cross-lane sum per weight row.  With DYNQ
// every workgroup quantizes the MR activation rows itself, all threads sharing
// the work (the arithmetic of the row quantizer), and the codes are exchanged
// through LDS.  Sums are parked
// 64 / MR weight rows at a time (lane l: row l % MR, weight row l / MR of the
// batch) and then scaled and stored.  Requires K % 16 == 0, K <= 1024 * KV,
// operands 16-byte aligned.
template <int KV, int MR, int DEPTH, bool DYNQ, bool F32OUT, bool WNT = false>
__global__ __launch_bounds__(512) void linear_gemv_rows_kernel(const GemmArgs g)
{
    constexpr int NWAVE = 8;
    constexpr int RING = DEPTH + 1;
    constexpr int SLOTS = 64 / MR;
    __shared__ float s_sa[MR], s_rinv[MR];
    __shared__ unsigned s_amax[MR];
    __shared__ int s_fast[MR];
    __shared__ __attribute__((aligned(16))) int8_t xq[DYNQ ? MR * 1024 * KV : 16];
    const int M = g.M, N = g.N, K = g.K;
    const int kv = K >> 4;  // 16-byte pieces of a row
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t W = (int64_t)gridDim.x * NWAVE;
    const int64_t r0 = (int64_t)blockIdx.x * NWAVE + w, r1 = N;

    // The activations are asked for first: behind the weight rows they would wait for all of them.
    // The MR rows are one flat run of 256 * KV * MR float4 pieces dealt out to the 512 threads, so
    // the 64 pieces of a wave instruction belong to one row.
    constexpr int PIECES = 256 * KV;                      // float4 per (padded) row
    constexpr int XV = DYNQ ? (MR * PIECES) / 512 : 1;    // pieces per thread
    static_assert(!DYNQ || (MR * PIECES) % 512 == 0, "whole pieces per thread");
    f4 xr[XV];
    if constexpr (DYNQ) {
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const int f = i * 512 + (int)threadIdx.x, row = f / PIECES, col = f % PIECES;
            xr[i] = (row < M && col < (K >> 2))
                        ? reinterpret_cast<const f4 *>(g.xf32 + (int64_t)row * K)[col]
                        : f4{0.f, 0.f, 0.f, 0.f};
        }
    }
    v4i wb[RING][KV];
    auto load_row = [&](int64_t r, v4i (&dst)[KV]) {
        const v4i *p = reinterpret_cast<const v4i *>(g.Bt + r * K) + lane;
#pragma unroll
        for (int j = 0; j < KV; j++)
            dst[j] = (64 * j + lane < kv) ? (WNT ? __builtin_nontemporal_load(p + 64 * j) : p[64 * j]) : v4i{0, 0, 0, 0};
    };
#pragma unroll
    for (int d = 0; d < DEPTH; d++)
        if (r0 + d * W < r1)
            load_row(r0 + d * W, wb[d]);

    v4i xc[MR][KV];
    if constexpr (DYNQ) {
        // absmax of a row: non-negative floats order like their bit patterns, so an integer
        // maximum in LDS collects the waves' shares in any order
        if (threadIdx.x < MR)
            s_amax[threadIdx.x] = 0u;
        lds_barrier();
#pragma unroll
        for (int i = 0; i < XV; i++) {
            const float m = vtlhip::qdev::wave_max(vtlhip::qdev::absmax4(0.0f, xr[i]));
            if (lane == 0)
                atomicMax(&s_amax[(i * 512 + (int)threadIdx.x) / PIECES], __float_as_uint(m));
        }
        lds_barrier();
        if (threadIdx.x < MR) {
            const float sx = __uint_as_float(s_amax[threadIdx.x]) / 127.0f;
            const vtlhip::qdev::QuantScale qp = vtlhip::qdev::make_quant_scale(sx);
            s_sa[threadIdx.x] = sx;
            s_rinv[threadIdx.x] = qp.rinv;
            s_fast[threadIdx.x] = qp.fast ? 1 : 0;
        }
        lds_barrier();
#pragma unroll
        for (int i = 0; i < XV; i++) {  // pieces past K and rows past M are written as zeros
            const int f = i * 512 + (int)threadIdx.x, row = f / PIECES;
            // one row per wave instruction: scalar values, so the choice of path is a scalar branch
            vtlhip::qdev::QuantScale qp;
            qp.scale = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(s_sa[row])));
            qp.rinv = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(s_rinv[row])));
            qp.fast = __builtin_amdgcn_readfirstlane(s_fast[row]) != 0;
            reinterpret_cast<unsigned *>(xq)[f] = vtlhip::qdev::quant4(xr[i], qp);
        }
        lds_barrier();
#pragma unroll
        for (int m = 0; m < MR; m++)
#pragma unroll
            for (int j = 0; j < KV; j++)
                xc[m][j] = reinterpret_cast<const v4i *>(xq)[m * 64 * KV + 64 * j + lane];
    } else {
#pragma unroll
        for (int m = 0; m < MR; m++) {
            const v4i *p = reinterpret_cast<const v4i *>(g.A + (int64_t)(m < M ? m : 0) * K) + lane;
#pragma unroll
            for (int j = 0; j < KV; j++)
                xc[m][j] = (m < M && 64 * j + lane < kv) ? p[64 * j] : v4i{0, 0, 0, 0};
        }
    }

    const int my_m = lane % MR, my_slot = lane / MR;
    float sav = 0.0f;
    if (F32OUT && my_m < M)
        sav = DYNQ ? s_sa[my_m] : g.sa[my_m * g.sa_stride];
    int res = 0, it = 0;
    // scale and bias of the weight row this lane parks next are fetched a batch ahead
    float swv = 0.0f, bv = 0.0f;
    auto fetch_scales = [&](int it0) {
        const int64_t n = r0 + (int64_t)(it0 + my_slot) * W;
        if (F32OUT && my_m < M && n < r1) {
            swv = g.sw[n * g.sw_stride];
            if (g.bias)
                bv = g.bias[n];
        }
    };
    fetch_scales(0);
    // weight rows it0 .. it0 + SLOTS - 1 of this wave's sequence are parked: scale and store them
    auto flush = [&](int it0) {
        const int64_t n = r0 + (int64_t)(it0 + my_slot) * W;
        if (my_m < M && n < r1 && it0 + my_slot < it) {
            const int64_t o = (int64_t)my_m * N + n;
            if constexpr (F32OUT) {
                const float sc = sav * swv;
                float y = (float)res * sc;
                if (g.bias)
                    y = y + bv;
                if (g.relu && y < 0.0f)
                    y = 0.0f;
                reinterpret_cast<float *>(g.out)[o] = y;
            } else {
                reinterpret_cast<int32_t *>(g.out)[o] = res;
            }
        }
    };
    for (int64_t rb = r0; rb < r1; rb += RING * W) {
#pragma unroll
        for (int u = 0; u < RING; u++) {
            const int64_t r = rb + u * W;
            if (r >= r1)
                break;
            if (r + DEPTH * W < r1)
                load_row(r + DEPTH * W, wb[(u + DEPTH) % RING]);
            int acc[MR];
#pragma unroll
            for (int m = 0; m < MR; m++)
                acc[m] = 0;
#pragma unroll
            for (int j = 0; j < KV; j++)
#pragma unroll
                for (int c = 0; c < 4; c++)
#pragma unroll
                    for (int m = 0; m < MR; m++)
                        acc[m] = __builtin_amdgcn_sdot4(wb[u][j][c], xc[m][j][c], acc[m], false);
            const int tot = wave_sum_rows<MR>(acc, lane);
            res = (my_slot == it % SLOTS) ? tot : res;
            it++;
            if (it % SLOTS == 0) {
                flush(it - SLOTS);
                fetch_scales(it);
            }
        }
    }
    if (it % SLOTS != 0)
        flush(it - it % SLOTS);
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

// Copies `rows` rows of K bytes into rows of Kp >= K bytes (Kp % 4 == 0), zero
// filled: four destination bytes per thread.
__global__ __launch_bounds__(256) void pad_rows_i8_kernel(const int8_t *__restrict__ src, int64_t rows, int K,
                                                         int8_t *__restrict__ dst, int Kp)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int q = Kp >> 2;
    if (i >= rows * q)
        return;
    const int64_t row = i / q;
    const int c = (int)(i - row * q) * 4;
    const int8_t *s = src + row * K;
    unsigned w = 0;
#pragma unroll
    for (int b = 0; b < 4; b++)
        if (c + b < K)
            w |= (unsigned)(uint8_t)s[c + b] << (8 * b);
    reinterpret_cast<unsigned *>(dst)[i] = w;
}

// Small products (up to a few hundred 32x32 output tiles): nothing is reused
// often enough to stage, so each wave feeds the MFMA straight from global memory.
// One workgroup per 32x32 tile; its NW waves split the K steps (U steps of loads
// in flight per wave) and the partial tiles meet in LDS.  With sixteen waves a
// tile with K = 4096 is two rounds of loads per wave, so a product like
// 256x1024x4096 (256 tiles, one per compute unit) is one launch whose length is
// a couple of memory latencies, instead of a K-split launch plus the pass that
// adds the partial sums.  Needs K % 16 == 0 and 16-byte aligned operands.
template <bool F32OUT, int NW, int U>
__global__ __launch_bounds__(64 * NW) void gemm_i8_small_kernel(const GemmArgs g)
{
    __shared__ int red[NW][16][64];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tiles_n = (g.N + 31) / 32;
    const int m0 = (int)(blockIdx.x / tiles_n) * 32, n0 = (int)(blockIdx.x % tiles_n) * 32;
    const int r = lane & 31, half = lane >> 5;
    // rows past the edge repeat the last row; their results are never stored
    const int arow = m0 + r < g.M ? m0 + r : g.M - 1;
    const int brow = n0 + r < g.N ? n0 + r : g.N - 1;
    const int8_t *__restrict__ ap = g.A + (int64_t)arow * g.K + 16 * half;
    const int8_t *__restrict__ bp = g.Bt + (int64_t)brow * g.K + 16 * half;
    const int steps = (g.K + 31) / 32;
    const int per = (steps + NW - 1) / NW;
    const int t0 = wave * per, t1 = t0 + per < steps ? t0 + per : steps;
    v16i acc;
#pragma unroll
    for (int i = 0; i < 16; ++i)
        acc[i] = 0;
    const v4i zero = {0, 0, 0, 0};
    for (int t = t0; t < t1; t += U) {   // U steps of loads in flight
        v4i a[U], b[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = 32 * (t + u);
            // K % 32 == 16: the upper half of the last step is empty
            const bool in = t + u < t1 && k + 16 * half < g.K;
            a[u] = in ? *reinterpret_cast<const v4i *>(ap + k) : zero;
            b[u] = in ? *reinterpret_cast<const v4i *>(bp + k) : zero;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u], b[u], acc, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i)
        red[wave][i][lane] = acc[i];
    __syncthreads();
    for (int o = threadIdx.x; o < 1024; o += 64 * NW) {
        const int reg = o >> 6, l = o & 63;
        int sum = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w)
            sum += red[w][reg][l];
        // accumulator register reg of lane l: row 8 * (reg / 4) + 4 * (l / 32) + reg % 4, column l % 32
        const int m = m0 + 8 * (reg >> 2) + 4 * (l >> 5) + (reg & 3), n = n0 + (l & 31);
        if (m >= g.M || n >= g.N)
            continue;
        const int64_t idx = (int64_t)m * g.N + n;
        if (F32OUT) {
            const float sc = g.sa[(int64_t)m * g.sa_stride] * g.sw[(int64_t)n * g.sw_stride];
            float y = (float)sum * sc;
            if (g.bias)
                y = y + g.bias[n];
            if (g.relu && y < 0.0f)
                y = 0.0f;
            reinterpret_cast<float *>(g.out)[idx] = y;
        } else {
            reinterpret_cast<int32_t *>(g.out)[idx] = sum;
        }
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// A flag per device: kernel attributes are per device, the library may serve several.  Atomic,
// so that two host threads that meet at a kernel's first launch do not race on the flag itself
// (setting the attribute twice is harmless).
using DoneFlag = std::atomic<bool>;
template <typename V>
struct PerDevice {
    V v[64] = {};
    V &get()
    {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
            (void)hipGetLastError();
            dev = 0;
        }
        return v[dev];
    }
};

template <typename Kern>
int launch_with_lds(Kern kern, DoneFlag &attr_done, int lds, int tiles, int threads, const GemmArgs &g,
                    hipStream_t st, const char *name)
{
    if (!attr_done.load(std::memory_order_acquire)) {
        VTL_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        attr_done.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(threads), lds, st, g);
    return check_launch(name);
}

template <int BM, int BN, int BK, int NSTAGE, int WR, int WC, bool F32OUT>
int launch_dma(GemmArgs g, int splits, hipStream_t st)
{
    constexpr int lds = NSTAGE * (BM + BN) * BK;
    static_assert(lds >= (BM + 2 * BN + (BN / 32) * BM) * 4, "epilogue staging fits in the operand buffers");
    static_assert((NSTAGE - 1) * ((BM + BN) / (64 / (BK / 16)) / (WR * WC)) <= 63, "vmcnt is a 6-bit counter");
    const int tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    const int kt_all = (g.K + BK - 1) / BK;
    if (splits > kt_all)
        splits = kt_all;
    if (splits < 1)
        splits = 1;
    g.splits = splits;
    const bool requant = F32OUT && g.requant_codes != nullptr;
    if (splits > 1 || requant) {
        g.partials = static_cast<int32_t *>(
            vtlhip::library_workspace((size_t)splits * (size_t)g.M * (size_t)g.N * sizeof(int32_t)));
        if (!g.partials)
            return vtlhip::workspace_status();
    }
    static PerDevice<DoneFlag> done_flags[12];
    DoneFlag *done[12];
    for (int i = 0; i < 12; i++)
        done[i] = &done_flags[i].get();
    const bool ktail = (g.K % BK) != 0;
    const bool edge = (g.M % BM) || (g.N % BN) || ktail;
    g.cached_out = tiles <= 256 ? 1 : 0;  // one round of workgroups
    int rc;
    if (requant && splits == 1) {
        // No K split.  Either the tile kernel applies the epilogue itself, leaves the f32 rows
        // (in the caller's Y, or in the scratch plane) with one partial row maximum per tile, and
        // a wide kernel quantizes them; or it leaves int32 sums and one workgroup per row does
        // epilogue and quantization.  Measured, the second form is the faster one everywhere
        // (256x11008x4096: 25.8 against 26.8 us, 128x14336x4096: 21.9 against 23.5 us,
        // 256x16384x1024: 17.7 against 22.3 us; with the f32 rows wanted as well the gap is
        // 0.6 to 1 us): the reduction in the tile kernel's epilogue and the second kernel's
        // dependent loads cost more than the one-workgroup-per-row kernel's idle lanes.  So it
        // is the default; VTL_HIP_REQUANT_WIDE=1 selects the first form (tests keep both exact).
        constexpr bool kRowMaxTile = BM >= 64 && BM <= 128 && BN >= 64;   // the instantiated shapes
        const int tiles_n = (g.N + BN - 1) / BN;
        bool wide = kRowMaxTile && tuning().requant_wide > 0;
        if constexpr (kRowMaxTile) {
            if (wide) {
                const size_t plane = (size_t)g.M * (size_t)g.N * sizeof(float);
                char *ws = static_cast<char *>(
                    vtlhip::library_workspace(plane + (size_t)tiles_n * (size_t)g.M * sizeof(float)));
                if (!ws)
                    return vtlhip::workspace_status();
                GemmArgs gf = g;
                gf.out = g.out ? g.out : reinterpret_cast<void *>(ws);
                gf.row_absmax_parts = reinterpret_cast<float *>(ws + plane);
                if (ktail)
                    rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, true, true, false, true, true>,
                                         *done[8], lds, tiles, 64 * WR * WC, gf, st, "gemm_i8_dma_kernel");
                else if (edge)
                    rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, true, true, false, true>,
                                         *done[6], lds, tiles, 64 * WR * WC, gf, st, "gemm_i8_dma_kernel");
                else
                    rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, true, false, false, true>,
                                         *done[7], lds, tiles, 64 * WR * WC, gf, st, "gemm_i8_dma_kernel");
                if (rc != VTL_HIP_OK)
                    return rc;
                const dim3 grid((unsigned)((g.N + 4095) / 4096), (unsigned)g.M);
                if (grid.y > 65535)
                    return VTL_HIP_ERR_UNSUPPORTED;
                hipLaunchKernelGGL(requant_rows_wide_kernel, grid, dim3(256), 0, st,
                                   reinterpret_cast<const float *>(gf.out), gf.row_absmax_parts, tiles_n, g.M, g.N,
                                   g.requant_codes, g.requant_scales);
                return check_launch("requant_rows_wide_kernel");
            }
        }
        // the int32 sums of the whole K go to the scratch plane the row kernel reads
        GemmArgs gi = g;
        gi.out = g.partials;
        if (ktail)
            rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, false, true, false, false, true>,
                                 *done[9], lds, tiles, 64 * WR * WC, gi, st, "gemm_i8_dma_kernel");
        else if (edge)
            rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, false, true, false>, *done[4], lds,
                                 tiles, 64 * WR * WC, gi, st, "gemm_i8_dma_kernel");
        else
            rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, false, false, false>, *done[5], lds,
                                 tiles, 64 * WR * WC, gi, st, "gemm_i8_dma_kernel");
        return rc != VTL_HIP_OK ? rc : launch_finalize_requant(g, st);
    }
    // the partial sums of a split launch are int32 whatever the final type is
    if (splits > 1 && ktail)
        rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, false, true, true, false, true>, *done[10],
                             lds, tiles * splits, 64 * WR * WC, g, st, "gemm_i8_dma_kernel");
    else if (splits > 1 && edge)
        rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, false, true, true>, *done[0], lds,
                             tiles * splits, 64 * WR * WC, g, st, "gemm_i8_dma_kernel");
    else if (splits > 1)
        rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, false, false, true>, *done[1], lds,
                             tiles * splits, 64 * WR * WC, g, st, "gemm_i8_dma_kernel");
    else if (ktail)
        rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, F32OUT, true, false, false, true>,
                             *done[11], lds, tiles, 64 * WR * WC, g, st, "gemm_i8_dma_kernel");
    else if (edge)
        rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, F32OUT, true, false>, *done[2], lds,
                             tiles, 64 * WR * WC, g, st, "gemm_i8_dma_kernel");
    else
        rc = launch_with_lds(gemm_i8_dma_kernel<BM, BN, BK, NSTAGE, WR, WC, F32OUT, false, false>, *done[3], lds,
                             tiles, 64 * WR * WC, g, st, "gemm_i8_dma_kernel");
    if (rc != VTL_HIP_OK || splits == 1)
        return rc;
    if (requant)
        return launch_finalize_requant(g, st);
    const int64_t mn = (int64_t)g.M * g.N;
    if (g.N % 4 == 0 && aligned16(g.out) && aligned16(g.partials)) {
        hipLaunchKernelGGL((splitk_finalize_kernel<F32OUT, 4>), dim3((unsigned)((mn / 4 + 255) / 256)), dim3(256), 0,
                           st, g);
    } else {
        hipLaunchKernelGGL((splitk_finalize_kernel<F32OUT, 1>), dim3((unsigned)((mn + 255) / 256)), dim3(256), 0, st,
                           g);
    }
    return check_launch("splitk_finalize_kernel");
}

// The DMA-kernel instantiations, smallest tile first.
struct TileConfig {
    int bm, bn;
    float step_cycles;  // one 128-byte K step of one workgroup: max(MFMA time, L2->LDS fill at ~40 B/clk)
    int wgs_per_cu;     // workgroups that fit a compute unit's LDS together
    float busy_chip;    // factor on step_cycles when the whole chip runs such steps at once
};
constexpr TileConfig kTileConfigs[] = {
    {32, 64, 352.f, 1, 3.7f}, {32, 128, 483.f, 2, 1.07f},
    {64, 64, 410.f, 2, 1.06f},   // four stages
    {64, 128, 575.f, 2, 1.1f},
    {128, 64, 518.f, 1, 1.2f},  // four stages
    {128, 128, 1068.f, 2, 0.86f},
    {128, 128, 636.f, 1, 1.45f},  // four stages, eight waves: alone on its compute unit, for launches of one round
    {256, 256, 1996.f, 1, 0.83f}};
constexpr int kNumTileConfigs = 8;

// The epilogue addresses a tile's elements as a 32-bit offset (row in tile x N
// + column in tile) from the tile's origin: a tile shape qualifies only while
// the largest such offset fits.
inline bool tile_offsets_fit(const TileConfig &c, int M, int N)
{
    const int64_t rows = c.bm < M ? c.bm : M;
    return rows * (int64_t)N + c.bn <= (int64_t)0xffffffffLL;
}

template <bool F32OUT>
int launch_config(int idx, const GemmArgs &g, int splits, hipStream_t st)
{
    if (idx < 0 || idx >= kNumTileConfigs || !tile_offsets_fit(kTileConfigs[idx], g.M, g.N))
        return VTL_HIP_ERR_UNSUPPORTED;  // more than 2^32 / 32 output columns: no tile shape qualifies
    switch (idx) {
    case 0: return launch_dma<32, 64, 128, 8, 1, 2, F32OUT>(g, splits, st);
    case 1: return launch_dma<32, 128, 128, 4, 1, 4, F32OUT>(g, splits, st);
    case 2: return launch_dma<64, 64, 128, 4, 2, 2, F32OUT>(g, splits, st);
    case 3: return launch_dma<64, 128, 128, 3, 2, 2, F32OUT>(g, splits, st);
    case 4: return launch_dma<128, 64, 128, 4, 2, 2, F32OUT>(g, splits, st);
    case 5: return launch_dma<128, 128, 128, 2, 2, 2, F32OUT>(g, splits, st);
    case 6: return launch_dma<128, 128, 128, 4, 2, 4, F32OUT>(g, splits, st);
    default: return launch_dma<256, 256, 128, 2, 2, 4, F32OUT>(g, splits, st);
    }
}

// Picks the tile and the number of K ranges that minimise a simple cost
// model, the larger of
//   latency:    rounds of workgroups over the resident slots x K steps per workgroup x step cost
//   throughput: all K steps of all workgroups x step cost x busy-chip factor / 256 compute units
// plus, for split K, the extra launch and the pass over the partial sums.  For the
// requantizing linear, whose second kernel runs whatever the split, only the planes of
// partial sums that kernel has to read count.
// The constants were fitted (random search, least mean log regret) to exhaustive timing
// sweeps of every tile and split count, each shape timed once with the same weights every
// launch (up to 256 MB of them then stay in the last-level cache) and once with the weights
// taken from enough copies in turn that every launch streams them from HBM, since which tile
// wins can depend on that: 87 shapes from 40x11008x4096 to 8192^3, 153 with a ragged M
// (33 ... 520 rows against nine weight matrices), and 90 through the requantizing entry
// (48 ... 2048 rows), the shapes of the decode and MLP-chain workloads weighted six-fold.
// Mean regret against the fastest measured entry 1.1 % cached and 1.2 % from HBM (worst 29 %:
// 2048^3 through the requantizing entry, cached); the constants this replaces, fitted before
// the kernels for ragged shapes were sped up, were at 5.4 % and 4.3 % on the same data, worst
// 45 % and 53 % (config 6 with a K split chosen for 65 ... 400 rows and K >= 8192).
void choose_config(int M, int N, int K, int &best_idx, int &best_splits, bool requant = false)
{
    const int kt_all = (K + 127) / 128;
    float best = 3.0e38f;
    best_idx = -1;  // stays so when no tile shape can address the output (see tile_offsets_fit)
    best_splits = 1;
    for (int i = 0; i < kNumTileConfigs; i++) {
        const TileConfig &c = kTileConfigs[i];
        if (i > 0 && kTileConfigs[i - 1].bm >= M && c.bm > kTileConfigs[i - 1].bm)
            break;  // a taller tile would only add padding rows
        if (!tile_offsets_fit(c, M, N))
            continue;
        const int64_t tiles = (int64_t)((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
        // More than one round of 256x256 tiles with a short K: each round pays the long fill and
        // the 256 KiB store of a tile that owns its compute unit, while two 128x128 tiles per
        // compute unit overlap theirs (8192x8192x1024: 97 against 104 us, 6144x6144x2048: 90
        // against 98 us).
        if (c.bm == 256 && K <= 2048 && tiles > 256)
            continue;
        for (int s = 1; s <= 16; s *= 2) {
            if (s > 1 && kt_all / s < 4)
                break;
            const int64_t rounds = (tiles * s + 256 * c.wgs_per_cu - 1) / (256 * c.wgs_per_cu);
            const int steps = (kt_all + s - 1) / s;
            const float fixed = c.bm == 256 ? 4865.f : 6058.f;   // fill and store of one workgroup
            const float latency = (float)rounds * ((float)steps * c.step_cycles + fixed);
            const float throughput = (float)tiles * (float)s * (float)steps * c.step_cycles * c.busy_chip / 256.f + fixed;
            float cost = latency > throughput ? latency : throughput;
            if (requant)
                cost += (float)s * (float)M * (float)N * 4.0f / 636.f;
            else if (s > 1)
                cost += 4084.f + (float)s * (float)M * (float)N * 4.0f / 606.f;
            if (cost < best) {
                best = cost;
                best_idx = i;
                best_splits = s;
            }
        }
    }
}

// Waves (K ranges) per workgroup for up to 32 rows against 2048 weight rows or more.  From a
// sweep of M = 2 .. 32, N = 2048 .. 14336, K = 1024 .. 11008, cached and from HBM: four waves
// up to 256 workgroups (N <= 8192: half the chip or less would otherwise run two waves each;
// 12 x 2048 x 4096 5.9 -> 4.8 us, 16 x 4096 x 8192 9.1 -> 6.8 us) and whenever K >= 8192
// (6 x 14336 x 8192 from HBM 26.4 -> 21.5 us); two waves for more workgroups with a shorter K,
// where the smaller LDS footprint keeps every workgroup resident (24 x 11008 x 4096: 9.7 against
// 10.6 us).  Mean regret against the best of both over the sweep 1.1 % cached, 2.1 % from HBM.
inline int skinny_waves_few_rows(int N, int K)
{
    return ((N <= 8192 && K >= 2048) || K >= 8192) ? 4 : 2;
}

// Whether a decode kernel reads an N x K weight matrix with non-temporal loads: from `mib` MiB
// on.  A model made of such matrices does not stay in the 256 MB last-level cache from one
// step to the next, and streaming from HBM the loads are worth 2 to 8 % (N = 14336, K = 4096:
// 1 row 11.7 -> 11.1 us, 8 rows 14.4 -> 13.7 us, 32 rows 16.6 -> 16.1 us).  The price is paid by
// a caller who repeats the launch on one matrix that would have stayed in that cache: nothing
// for the single-row kernel (it gains there too, 10.1 -> 9.2 us), but 12 to 23 % for the
// weight-streaming kernel on matrices of 32 to 45 MiB and 0 to 12 % on larger ones, which is
// why it and the few-token kernel (2 to 8 rows: 3 to 6 % from HBM, 12 % behind on a repeated
// matrix of 32 to 45 MiB) start at 48 MiB and the single-row kernel at 8 (below, it is level or
// 5 % behind).  A caller whose model is made of smaller matrices and does not fit that cache
// lowers the first limit with VTL_HIP_STREAM_WEIGHTS_MIB (16 for 4096 x 4096 and up).
inline bool stream_weights_from(int N, int K, int mib) { return (int64_t)N * K >= ((int64_t)mib << 20); }

template <int NWAVE, int STAGES, int XJ, bool F32OUT, bool STAGEQ = false>
int launch_skinny_cfg(const GemmArgs &g_in, hipStream_t st)
{
    GemmArgs g = g_in;
    g.stream_weights = (g.M <= 32 && stream_weights_from(g.N, g.K, tuning().stream_weights_mib)) ? 1 : 0;   // (one block of rows: every weight is read once)
    constexpr int lds = NWAVE * STAGES * (8192 + XJ * 2048);
    static_assert(lds >= NWAVE * 4096, "room for the partial tiles");
    static PerDevice<DoneFlag> done_flag;
    DoneFlag &done = done_flag.get();
    // STAGEQ: M <= 32, and in front the workgroups that quantize the activation rows
    const dim3 grid((unsigned)((g.N + 31) / 32 + (STAGEQ ? g.M : 0)),
                    STAGEQ ? 1u : (unsigned)((g.M + 31) / 32));
    if (grid.y > 65535)
        return VTL_HIP_ERR_UNSUPPORTED;
    if (!done.load(std::memory_order_acquire)) {
        VTL_HIP_TRY(hipFuncSetAttribute(
            reinterpret_cast<const void *>(linear_skinny_kernel<NWAVE, STAGES, XJ, F32OUT, STAGEQ>),
            hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        done.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL((linear_skinny_kernel<NWAVE, STAGES, XJ, F32OUT, STAGEQ>), grid, dim3(64 * NWAVE), lds, st, g);
    return check_launch("linear_skinny_kernel");
}

// Where the launch that quantizes the activations itself beats quantizer + linear, from a sweep
// of N = 128 .. 14336, K = 1024 .. 8192, M = 2 .. 32 (weights cached and from HBM): with
// thousands of weight rows whenever K <= 4096 (0.3 to 2.2 us of 6 to 19 us), with K = 8192 only
// from about 12288 rows on (with fewer rows the wait for 8192-element rows is not hidden: 14.4
// against 12.9 us at 8 x 4096 x 8192); below 2048 weight rows, where the linear is the four-wave
// form, for K = 1024 .. 4096 (7.3 -> 5.0 us at 16 x 512 x 1024, 8.1 -> 7.2 us at 16 x 1024 x 4096).
// `few_token_kernel`: the matrix-vector kernel for 2 to 8 rows (behind a quantizer launch)
// would take the product; it keeps it except below 2048 rows and on the largest matrices.
inline bool stage_inside_launch_faster(int M, int N, int K, bool few_token_kernel)
{
    if (M > 32 || K % 256 != 0 || K > kStageMaxK)
        return false;
    if (N < 2048)   // (3 or 4 rows of more than 2048 elements stay with the matrix-vector kernel: within 0.5 us either way)
        return N >= 128 && K >= 1024 && K <= 4096 && (M >= 5 || K <= 2048);
    if (few_token_kernel && !(N >= 12288 && K <= 4096))
        return false;
    // (rows of 8192 elements: with 8 of them the producers' one row each is not hidden, 8 x 14336 x
    // 8192 23.1 against 21.9 us; with 16 and 32 the launch is long enough, 23.5 against 24.5 us)
    return K <= 4096 || (N >= 12288 && M > 8);
}

// The instances of the kernel that quantizes the activations itself, by row count.
inline int launch_skinny_staged_cfg(const GemmArgs &g, hipStream_t st)
{
    if (g.N < 2048 || skinny_waves_few_rows(g.N, g.K) == 4) {   // K over four waves, as launch_skinny does for these
        if (g.M <= 8)
            return launch_skinny_cfg<4, 2, 1, true, true>(g, st);
        if (g.M <= 16)
            return launch_skinny_cfg<4, 2, 2, true, true>(g, st);
        return launch_skinny_cfg<4, 2, 4, true, true>(g, st);
    }
    if (g.M <= 8)
        return launch_skinny_cfg<2, 2, 1, true, true>(g, st);
    if (g.M <= 16)
        return launch_skinny_cfg<2, 2, 2, true, true>(g, st);
    return launch_skinny_cfg<2, 2, 4, true, true>(g, st);
}

// Host side of the launch that quantizes the activations itself.  Its workgroups meet on a
// counter that only grows, so the host has to know what every earlier launch added to it and
// launches that share a counter must run one after the other: each stream gets a counter of
// its own (the index vtlhip::stream_slot gives it: one of the first kStageSlots streams per
// device that ask), and the value it will reach is kept beside it.  No counter is handed out
// while the stream is being captured (a replay would wait for a value that was reached long
// ago), nor when the capture state cannot be queried.
struct StageCounters {
    std::mutex lock;
    unsigned counted[kStageSlots] = {};
};

// The weight-streaming launch that quantizes the f32 activations g.xf32 itself, into
// g.stage_codes / g.stage_scales (which g.A / g.sa name too).  M <= 32, K <= kStageMaxK.
// `launched` is false when the stream has no counter: nothing was enqueued then and the
// caller takes the two-launch path.
inline int launch_skinny_staged(GemmArgs g, hipStream_t st, bool &launched)
{
    static PerDevice<StageCounters> counters;
    StageCounters &c = counters.get();
    std::lock_guard<std::mutex> hold(c.lock);
    const int slot = vtlhip::stream_slot(st);
    launched = slot >= 0;
    if (!launched)
        return VTL_HIP_OK;
    g.sync_slot = slot;
    g.spin_limit = tuning().stage_spin;
    g.stage_target = c.counted[slot] + (unsigned)g.M;
    const int rc = launch_skinny_staged_cfg(g, st);
    if (rc == VTL_HIP_OK)
        c.counted[slot] = g.stage_target;
    return rc;
}


// nwave: K ranges (waves) per workgroup.  Two waves and two ring slots measured best for the
// decode shapes (M <= 32 against thousands of weight rows): the small LDS footprint keeps every
// workgroup of the grid resident at once, and that parallelism hides latency better than a
// deeper ring per wave does.  Four waves are for grids of at most one workgroup per compute
// unit, where the K split is the only parallelism left.
template <bool F32OUT>
int launch_skinny(const GemmArgs &g, int nwave, hipStream_t st)
{
    if (nwave == 4) {
        if (g.M <= 8)
            return launch_skinny_cfg<4, 2, 1, F32OUT>(g, st);
        if (g.M <= 16)
            return launch_skinny_cfg<4, 2, 2, F32OUT>(g, st);
        return launch_skinny_cfg<4, 2, 4, F32OUT>(g, st);
    }
    if (g.M <= 8)
        return launch_skinny_cfg<2, 2, 1, F32OUT>(g, st);
    if (g.M <= 16)
        return launch_skinny_cfg<2, 2, 2, F32OUT>(g, st);
    return launch_skinny_cfg<2, 2, 4, F32OUT>(g, st);
}

// The weight-streaming kernel on blocks of 32 activation rows x 32 weight rows (grid.y walks
// the row blocks) for small outputs with a long K: every block is a workgroup whose waves cut
// K between them, so a product like 256x1024x4096 (256 blocks, one per compute unit) is one
// launch of 6.1 us where the tile kernels need a K split and a second launch to fill the chip
// (10.0 us); 33x4096x2048 4.9 against 8.1 us, 256x1024x11008 10.9 against 13.7 us.  Returns
// the number of waves per workgroup (4: at most one round of workgroups, one per compute unit;
// the tuning knob can ask for 2 or 8), or 0 where the tile kernels are as fast or
// faster (short K: everything is launch-bound; more blocks: the tiles' operand reuse wins;
// few blocks with a very long K: the tile kernels' finer K split wins).  Measured over
// K = 256 ... 8192 and 4 ... 1024 blocks.
inline int skinny_blocks_waves(int M, int N, int K)
{
    if (tuning().skinny_tiled >= 0)   // 1 / 0 force the choice (tests, tuning)
        return tuning().skinny_tiled != 0 ? tuning().skinny_waves : 0;
    const int64_t blocks = (int64_t)((M + 31) / 32) * ((N + 31) / 32);
    if (K < 1024)
        return 0;
    // Timed again with the two routes alternating (after an idle gap the first timing of a launch
    // this short reads several percent high): up to 256 blocks 0.61 to 0.86 of the tile kernels'
    // time for K <= 4096 and 0.61 to 0.93 at K = 8192 from 64 blocks on (level below that); with
    // 257 to 512 blocks, two waves each, 8 to 12 % behind at K = 1024, 0 to 9 % behind at K = 2048
    // and level at K = 4096, so that range went back to the tile kernels.
    if (blocks <= 256)
        return (K <= 4096 || blocks >= 64) ? 4 : 0;
    return 0;
}

// Waves of the single-token kernel's grid: no more than the chip holds at once, sixteen per
// compute unit up to 6144 codes a row, eight beyond (the codes and three weight rows of a wave
// take 150 to 250 registers then).
inline int gemv_max_waves(int K) { return K <= 6144 ? 4096 : 2048; }

// Single-token linear (M = 1, K % 16 == 0, K <= 14336, operands 16-byte aligned).
template <bool DYNQ, bool F32OUT>
int launch_gemv(const GemmArgs &g_in, hipStream_t st)
{
    const GemmArgs &g = g_in;
    constexpr int NWAVE = 8;
    // every wave the same number of rows
    const int max_waves = gemv_max_waves(g.K);
    const int rows_per_wave = (g.N + max_waves - 1) / max_waves;
    if (rows_per_wave > 64)   // more rows than a wave has lanes to park their sums in
        return VTL_HIP_ERR_UNSUPPORTED;
    const int64_t waves = (g.N + rows_per_wave - 1) / rows_per_wave;
    const dim3 grid((unsigned)((waves + NWAVE - 1) / NWAVE)), block(64 * NWAVE);
    const bool wnt = stream_weights_from(g.N, g.K, 8);   // the cache policy is part of the load instruction
#define VTL_GEMV(KV)                                                                                        \
    do {                                                                                                    \
        if (wnt)                                                                                            \
            hipLaunchKernelGGL((linear_gemv_kernel<KV, NWAVE, DYNQ, F32OUT, true>), grid, block, 0, st, g); \
        else                                                                                                \
            hipLaunchKernelGGL((linear_gemv_kernel<KV, NWAVE, DYNQ, F32OUT, false>), grid, block, 0, st, g); \
    } while (0)
    switch ((g.K + 1023) / 1024) {
    case 1: VTL_GEMV(1); break;
    case 2: VTL_GEMV(2); break;
    case 3: VTL_GEMV(3); break;
    case 4: VTL_GEMV(4); break;
    case 5:
    case 6: VTL_GEMV(6); break;
    case 7:
    case 8: VTL_GEMV(8); break;
    case 9:
    case 10:
    case 11: VTL_GEMV(11); break;
    default: VTL_GEMV(14); break;
    }
#undef VTL_GEMV
    return check_launch("linear_gemv_kernel");
}

// A few tokens (2 <= M <= 8): rows of up to 11264 (2 tokens), 8192 (4) or 4096 (8) codes.
template <int KV, int MR, bool DYNQ, bool F32OUT>
int launch_gemv_rows_kv(const GemmArgs &g, hipStream_t st)
{
    constexpr int NWAVE = 8;
    // Codes and weight rows live in registers, which limits the waves a SIMD holds; with few
    // waves a third weight row in flight per wave keeps enough bytes on their way from HBM.
    constexpr int DEPTH = (MR * KV >= 16 && 4 * KV * (MR + 4) + 40 <= 256) ? 3 : 2;
    constexpr int REGS = 4 * KV * (MR + DEPTH + 1) + 40;
    // a workgroup of 8 waves puts two on every SIMD: whole workgroups only
    constexpr int OCC = 512 / REGS >= 8 ? 8 : (512 / REGS >= 2 ? (512 / REGS) & ~1 : 2);
    const int rows_per_wave = (g.N + 1024 * OCC - 1) / (1024 * OCC);  // every wave the same number of rows
    const int64_t waves = (g.N + rows_per_wave - 1) / rows_per_wave;
    const dim3 grid((unsigned)((waves + NWAVE - 1) / NWAVE)), block(64 * NWAVE);
    if constexpr (DYNQ && MR * KV > 8) {
        return VTL_HIP_ERR_UNSUPPORTED;  // not routed here: a quantizer launch of its own is cheaper
    } else {
        if (stream_weights_from(g.N, g.K, tuning().stream_weights_mib))   // (the cache policy is part of the load instruction)
            hipLaunchKernelGGL((linear_gemv_rows_kernel<KV, MR, DEPTH, DYNQ, F32OUT, true>), grid, block, 0, st, g);
        else
            hipLaunchKernelGGL((linear_gemv_rows_kernel<KV, MR, DEPTH, DYNQ, F32OUT, false>), grid, block, 0, st, g);
        return check_launch("linear_gemv_rows_kernel");
    }
}

template <int MR, bool DYNQ, bool F32OUT>
int launch_gemv_rows_mr(const GemmArgs &g, hipStream_t st)
{
    const int kv = (g.K + 1023) / 1024;
    if (kv <= 1)
        return launch_gemv_rows_kv<1, MR, DYNQ, F32OUT>(g, st);
    if (kv <= 2)
        return launch_gemv_rows_kv<2, MR, DYNQ, F32OUT>(g, st);
    if (kv <= 4)
        return launch_gemv_rows_kv<4, MR, DYNQ, F32OUT>(g, st);
    if constexpr (MR <= 4) {
        if (kv <= 8)
            return launch_gemv_rows_kv<8, MR, DYNQ, F32OUT>(g, st);
    }
    if constexpr (MR <= 2) {
        if (kv <= 11)
            return launch_gemv_rows_kv<11, MR, DYNQ, F32OUT>(g, st);
    }
    return VTL_HIP_ERR_UNSUPPORTED;  // not reached: see gemv_rows_applies
}

template <bool DYNQ, bool F32OUT>
int launch_gemv_rows(const GemmArgs &g, hipStream_t st)
{
    if (g.M <= 2)
        return launch_gemv_rows_mr<2, DYNQ, F32OUT>(g, st);
    if (g.M <= 4)
        return launch_gemv_rows_mr<4, DYNQ, F32OUT>(g, st);
    return launch_gemv_rows_mr<8, DYNQ, F32OUT>(g, st);
}

// The codes of the MR rows stay in registers: at most 32 pieces of 16 bytes per lane (22 for two rows:
// their weight rows are longer).
inline bool gemv_rows_applies(const void *rows, const void *w, int M, int N, int K)
{
    return M >= 2 && M <= 8 && K % 16 == 0 && K >= 256 && K <= (M <= 2 ? 11264 : (M <= 4 ? 8192 : 4096)) &&
           aligned16(rows) &&
           aligned16(w) && !tuning().no_gemv;
}

// Where the few-token kernel beats the MFMA weight-streaming kernel (measured, N = 64 ... 28672,
// K = 256 ... 8192): its dot4 work grows with M * N * K while the other's does not, but it has no
// LDS staging and a lower fixed cost.  Shapes the other kernel cannot take (K % 256 != 0) come here.
// `against_staged_launch`: the narrower rule by which the f32 entry decides between quantizer +
// this kernel and the weight-streaming launch that quantizes the rows itself (its sweep was made
// with that rule; the one launch keeps shapes there that this kernel wins as a plain linear).
inline bool gemv_rows_faster(int M, int N, int K, bool against_staged_launch = false)
{
    if (tuning().gemv_rows >= 0)   // 1 / 0 force the choice (tests, tuning)
        return tuning().gemv_rows != 0;
    if (M <= 2 || K % 256 != 0 || N < 2048)   // few weight rows: never slower, 1.8x faster from K = 4096 on
        return true;
    if (against_staged_launch)
        return M <= 4 ? (K >= 2048 || N <= 8192) : (int64_t)N * K <= ((int64_t)4 << 20);
    // As a plain int8 linear, timed with the two kernels alternating (N = 512 ... 14336, K = 1024
    // ... 8192, cached / from HBM): 3 and 4 rows 0.72 to 0.93 of the other kernel's time up to
    // 8192 x 4096 and level beyond; 5 to 8 rows 0.80 to 0.94 / 0.89 to 1.0 up to N * K = 8 M
    // (6 x 2048 x 4096: 4.7 against 5.9 us), level at 16 M, and 1.1 to 1.25 from 14336 x 1024 on.
    if (M <= 4)
        return true;
    return (int64_t)N * K <= ((int64_t)8 << 20);
}

// Quantizing the rows inside every workgroup of the few-token kernel costs about 15 instructions
// per element and workgroup; past 8192 elements (rows rounded up to 2, 4 or 8) a quantizer launch
// of its own is cheaper.
inline bool gemv_rows_fused_quant_faster(int M, int N, int K)
{
    const int mr = M <= 2 ? 2 : (M <= 4 ? 4 : 8);
    if (tuning().gemv_rows >= 0)   // only the instantiated sizes can be forced
        return tuning().gemv_rows != 0 && (int64_t)mr * ((K + 1023) / 1024) <= 8;
    return (int64_t)mr * K <= 8192 && (mr < 8 || (int64_t)N * K <= (int64_t)4 << 20);
}

// A wave parks one sum per lane, so it can own at most 64 rows: N <= 64 * waves of the grid.
inline bool gemv_applies(const void *row, const void *w, int N, int K)
{
    return K % 16 == 0 && K <= 14336 && N <= 64 * gemv_max_waves(K) && aligned16(row) && aligned16(w) &&
           !tuning().no_gemv;
}

// Where one workgroup per 32x32 tile, fed straight from global memory, beats the tile kernels:
// few tiles and a short K (nothing to stage), and up to a chip's worth of tiles with a long K,
// which the tile kernels could only fill the chip with by cutting K (a second launch).
inline bool small_product_faster(int64_t t32, int K)
{
    // (up to 128 tiles below K = 1024, where the 32 x 32-block route does not go: 256 x 512 x 512
    // 3.8 against 4.5 us on the tile kernels)
    return (t32 <= 64 && K <= 2048) || (t32 <= 128 && K < 1024);
}
inline int small_product_waves(int64_t t32, int K)
{
    (void)t32;
    return K <= 2048 ? 4 : (K <= 4096 ? 8 : 16);
}

template <bool F32OUT>
int launch_gemm(const GemmArgs &g_in, hipStream_t st)
{
    GemmArgs g = g_in;
    if ((g.K % 16) || !aligned16(g.A) || !aligned16(g.Bt)) {
        // The fast kernels read 16-byte chunks of rows that start 16-byte
        // aligned.  A tiny product is done one output per thread; anything
        // else is first copied into zero-padded rows of the library's scratch
        // (one more pass over the int8 operands: e.g. 1024x4096x4090 takes
        // 21 ms output-per-thread and well under 0.1 ms this way).
        const dim3 grid((unsigned)((g.N + 15) / 16), (unsigned)((g.M + 15) / 16));
        if ((int64_t)g.M * g.N * g.K <= (int64_t)1 << 20 && grid.y <= 65535) {
            hipLaunchKernelGGL((gemm_i8_naive_kernel<F32OUT>), grid, dim3(256), 0, st, g);
            return check_launch("gemm_i8_naive_kernel");
        }
        const int Kp = (g.K + 15) & ~15;
        const size_t a_bytes = ((size_t)g.M * Kp + 255) & ~(size_t)255;
        const size_t b_bytes = (size_t)g.N * Kp;
        int8_t *ws = static_cast<int8_t *>(vtlhip::library_workspace(a_bytes + b_bytes, 2));
        if (!ws)
            return vtlhip::workspace_status();
        const int64_t ta = (int64_t)g.M * (Kp / 4), tb = (int64_t)g.N * (Kp / 4);
        if ((ta + 255) / 256 > 0x7fffffff || (tb + 255) / 256 > 0x7fffffff)
            return VTL_HIP_ERR_UNSUPPORTED;
        hipLaunchKernelGGL(pad_rows_i8_kernel, dim3((unsigned)((ta + 255) / 256)), dim3(256), 0, st, g.A,
                           (int64_t)g.M, g.K, ws, Kp);
        hipLaunchKernelGGL(pad_rows_i8_kernel, dim3((unsigned)((tb + 255) / 256)), dim3(256), 0, st, g.Bt,
                           (int64_t)g.N, g.K, ws + a_bytes, Kp);
        const int rc = check_launch("pad_rows_i8_kernel");
        if (rc != VTL_HIP_OK)
            return rc;
        g.A = ws;
        g.Bt = ws + a_bytes;
        g.K = Kp;
    }
    // one row: matrix-vector product (very short rows go to the small-product kernel)
    const Tuning &tn = tuning();
    const bool config_set = tn.gemm_config >= 0, small_set = tn.gemm_small >= 0;
    if (g.M == 1 && g.K >= 256 && gemv_applies(g.A, g.Bt, g.N, g.K) && !config_set && !small_set)
        return launch_gemv<false, F32OUT>(g, st);
    if (gemv_rows_applies(g.A, g.Bt, g.M, g.N, g.K) && gemv_rows_faster(g.M, g.N, g.K) && !config_set && !small_set)
        return launch_gemv_rows<false, F32OUT>(g, st);
    if (g.K % 256 == 0 && g.M <= 32 && g.N >= 2048 && !config_set)
        return launch_skinny<F32OUT>(g, skinny_waves_few_rows(g.N, g.K), st);  // weight streaming: enough row blocks to fill the chip
    if (g.K % 256 == 0 && !config_set && !small_set) {
        const int nwave = skinny_blocks_waves(g.M, g.N, g.K);
        if (nwave)
            return launch_skinny<F32OUT>(g, nwave == 2 ? 2 : 4, st);
    }
    const int64_t t32 = (int64_t)((g.M + 31) / 32) * ((g.N + 31) / 32);
    // VTL_HIP_GEMM_SMALL 1 / 0 forces the choice (tests, tuning); 4, 8, 16 also the number of waves
    if (small_set ? tn.gemm_small != 0 : small_product_faster(t32, g.K)) {
        if (t32 > 0x7fffffff)
            return VTL_HIP_ERR_UNSUPPORTED;
        const int nw = tn.gemm_small >= 4 ? tn.gemm_small : small_product_waves(t32, g.K);
        const dim3 grid((unsigned)t32);
        if (nw >= 16)
            hipLaunchKernelGGL((gemm_i8_small_kernel<F32OUT, 16, 8>), grid, dim3(1024), 0, st, g);
        else if (nw >= 8)
            hipLaunchKernelGGL((gemm_i8_small_kernel<F32OUT, 8, 8>), grid, dim3(512), 0, st, g);
        else
            hipLaunchKernelGGL((gemm_i8_small_kernel<F32OUT, 4, 4>), grid, dim3(256), 0, st, g);
        return check_launch("gemm_i8_small_kernel");
    }
    int idx, splits;
    choose_config(g.M, g.N, g.K, idx, splits);
    if (config_set && tn.gemm_config < kNumTileConfigs) {  // tuning knob VTL_HIP_GEMM_CONFIG "<tile index>,<splits>"
        idx = tn.gemm_config;
        splits = tn.gemm_splits;
    }
    return launch_config<F32OUT>(idx, g, splits, st);
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
    GemmArgs g{A, Bt, C, nullptr, nullptr, nullptr, M, N, K, 0, 0, 0, 1, nullptr, nullptr, 0};
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
    GemmArgs g{A, Wq, Y, sa, sw, bias, M, N, K, sa_per_row ? 1 : 0, sw_per_col ? 1 : 0, relu ? 1 : 0, 1, nullptr, nullptr, 0};
    return launch_gemm<true>(g, current_stream());
}

int vtl_hip_linear_i8_requant(const int8_t *A, const float *sa, int sa_per_row, const int8_t *Wq,
                              const float *sw, int sw_per_col, const float *bias, int relu, int8_t *Yq,
                              float *sy, float *Y, int M, int N, int K)
{
    int st = check_gemm_args(A, Wq, Yq, M, N, K);
    if (st != VTL_HIP_OK)
        return st;
    if (!sa || !sw || !sy)
        return VTL_HIP_ERR_INVALID_ARG;
    if (M == 0 || N == 0)
        return VTL_HIP_OK;
    if (K == 0)
        return VTL_HIP_ERR_UNSUPPORTED;
    GemmArgs g{A, Wq, Y, sa, sw, bias, M, N, K, sa_per_row ? 1 : 0, sw_per_col ? 1 : 0, relu ? 1 : 0, 1, nullptr, nullptr, 0};
    if (M > 32 && K % 16 == 0 && aligned16(A) && aligned16(Wq) && requant_rows_fit(N) && aligned16(Yq) &&
        (!Y || aligned16(Y)) && (!sw_per_col || aligned16(sw)) && (!bias || aligned16(bias)) &&
        // a caller who wants the f32 rows anyway provides the staging: past 256 MiB of int32 sums
        // the two-pass route through Y needs no scratch of the library's
        !(Y && (size_t)M * (size_t)N * sizeof(int32_t) > ((size_t)256 << 20)) &&
        !tuning().no_fused_requant) {
        // tile kernel leaves int32 sums, one row kernel does epilogue + quantization
        int idx, splits;
        choose_config(M, N, K, idx, splits, true);
        const Tuning &tn = tuning();
        const bool config_set = tn.gemm_config >= 0 && tn.gemm_config < kNumTileConfigs;
        if (config_set) {   // VTL_HIP_GEMM_CONFIG, as in launch_gemm
            idx = tn.gemm_config;
            splits = tn.gemm_splits;
        }
        // Without a K split and with a large output the two launches below are the faster
        // pair: the row kernel of this form reads, per output element, the int32 sum and the
        // column's scale and bias (12 bytes, two thirds of them the same vectors again for
        // every row), the row quantizer behind the f32 linear 4.  From about 2.6 M outputs on
        // that outweighs the tile kernel's cheaper store: 4096^3 85 -> 75 us, 1024 x 11008 x
        // 4096 64 -> 59 us, 384 x 11008 x 4096 36.0 -> 33.3 us, 256 x 11008 x 4096 23.2 -> 22.4
        // us; below, this form is 2 to 5 % ahead (256 x 6144 x 4096: 16.0 against 16.9 us).
        const bool separate_faster = splits == 1 && !config_set && tn.requant_wide <= 0 &&
                                     (int64_t)M * N >= ((int64_t)5 << 19);
        if (!separate_faster) {
            g.requant_codes = Yq;
            g.requant_scales = sy;
            return launch_config<true>(idx, g, splits, current_stream());
        }
    }
    // any other shape: the f32 rows (in the library's staging buffer when the caller wants none),
    // then the row quantizer
    if (!Y) {
        Y = static_cast<float *>(vtlhip::library_workspace((size_t)M * (size_t)N * sizeof(float), 1));
        if (!Y)
            return vtlhip::workspace_status();
        g.out = Y;
    }
    st = launch_gemm<true>(g, current_stream());
    if (st != VTL_HIP_OK)
        return st;
    return launch_quantize_rows(Y, M, N, Yq, sy, current_stream());
}

int vtl_hip_gemm_tile_choice(int M, int N, int K, int requant, int *config_index, int *tile_m, int *tile_n,
                             int *splits)
{
    if (!config_index || !tile_m || !tile_n || !splits || M <= 0 || N <= 0 || K <= 0)
        return VTL_HIP_ERR_INVALID_ARG;
    int idx, s;
    choose_config(M, N, K, idx, s, requant != 0);
    if (idx < 0)
        return VTL_HIP_ERR_UNSUPPORTED;
    *config_index = idx;
    *tile_m = kTileConfigs[idx].bm;
    *tile_n = kTileConfigs[idx].bn;
    *splits = s;
    return VTL_HIP_OK;
}


size_t vtl_hip_linear_f32_dynquant_workspace(int M, int K)
{
    if (M <= 0 || K <= 0)
        return 0;
    // int8 codes of X, then M row scales, each rounded up to 256 bytes: a buffer of this size that
    // starts on a cache line owns every line it touches (the launch that quantizes the rows
    // itself relies on nothing else living in those lines)
    const size_t codes = (((size_t)M * (size_t)K) + 255) & ~(size_t)255;
    return codes + (((size_t)M * sizeof(float) + 255) & ~(size_t)255);
}

int vtl_hip_linear_f32_dynquant(const float *X, const int8_t *Wq, const float *sw, const float *bias,
                                float *Y, int M, int N, int K, int relu, void *workspace,
                                size_t workspace_bytes)
{
    int st = check_gemm_args(X, Wq, Y, M, N, K);
    if (st != VTL_HIP_OK)
        return st;
    if (!sw)
        return VTL_HIP_ERR_INVALID_ARG;
    if (M == 0 || N == 0)
        return VTL_HIP_OK;
    if (K == 0)
        return VTL_HIP_ERR_UNSUPPORTED;
    if (workspace && (workspace_bytes < vtl_hip_linear_f32_dynquant_workspace(M, K) ||
                      (reinterpret_cast<uintptr_t>(workspace) & 15)))
        return VTL_HIP_ERR_INVALID_ARG;
    if (M == 1 && gemv_applies(X, Wq, N, K) && !tuning().no_fused_decode) {
        // a single token: quantized inside the matrix-vector kernel, one launch instead of two
        // (N = 14336, K = 4096: 9.5 us against 12.8 us).  The workspace stays unused.
        // VTL_HIP_NO_FUSED_DECODE forces the two-launch path (tests).
        GemmArgs g{nullptr, Wq, Y, nullptr, sw, bias, M, N, K, 1, 1, relu ? 1 : 0, 1, nullptr, X, 0};
        return launch_gemv<true, true>(g, current_stream());
    }
    if (gemv_rows_applies(X, Wq, M, N, K) && gemv_rows_fused_quant_faster(M, N, K) && !tuning().no_fused_decode) {
        // a few tokens and short rows: same, each workgroup quantizes the rows itself
        GemmArgs g{nullptr, Wq, Y, nullptr, sw, bias, M, N, K, 1, 1, relu ? 1 : 0, 1, nullptr, X, 0};
        return launch_gemv_rows<true, true>(g, current_stream());
    }
    const bool staged = stage_inside_launch_faster(M, N, K, gemv_rows_applies(X, Wq, M, N, K) && gemv_rows_faster(M, N, K, true)) &&
                        aligned16(X) && aligned16(Wq) && tuning().gemm_config < 0 && !tuning().no_fused_decode;
    if (!workspace) {   // no caller scratch: stage in the library's own buffer
        workspace = vtlhip::library_workspace(vtl_hip_linear_f32_dynquant_workspace(M, K), 1);
        if (!workspace)
            return vtlhip::workspace_status();
    }
    int8_t *xq = reinterpret_cast<int8_t *>(workspace);
    const size_t codes = (((size_t)M * (size_t)K) + 255) & ~(size_t)255;
    float *sx = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + codes);
    if (staged && (reinterpret_cast<uintptr_t>(workspace) & 127) == 0) {
        // a few tokens: quantized inside the weight-streaming launch (N = 14336, K = 4096, M = 8:
        // 14.4 us against 16.0 us).  Its workgroups read the staging buffer as soon as the rows
        // are counted and rely on no cache holding an older copy of those lines, which holds
        // when nothing else shares them: the buffer starts on a cache line (anything from
        // vtl_hip_malloc does) and its size is a whole number of them.
        GemmArgs g{xq, Wq, Y, sx, sw, bias, M, N, K, 1, 1, relu ? 1 : 0, 1, nullptr, X, 0};
        g.stage_codes = xq;
        g.stage_scales = sx;
        bool launched = false;
        st = launch_skinny_staged(g, current_stream(), launched);
        if (launched || st != VTL_HIP_OK)
            return st;
    }
    st = launch_quantize_rows(X, M, K, xq, sx, current_stream());
    if (st != VTL_HIP_OK)
        return st;
    GemmArgs g{xq, Wq, Y, sx, sw, bias, M, N, K, 1, 1, relu ? 1 : 0, 1, nullptr, nullptr, 0};
    return launch_gemm<true>(g, current_stream());
}

int vtl_hip_linear_f32_dynquant_noalloc(const float *X, const int8_t *Wq, const float *sw, const float *bias,
                                        float *Y, int M, int N, int K, int relu)
{
    void *base = vtlhip::static_scratch();   // device address of this device's array, resolved once
    if (!base)
        return VTL_HIP_ERR_RUNTIME;
    // Everything the call stages - activation codes and row scales, partial sums of a K split,
    // repacked operands - is cut from the static array in the order it is asked for; a call that
    // needs more than the array holds returns VTL_HIP_ERR_UNSUPPORTED (kernels that only fill
    // earlier pieces of the scratch may have been enqueued by then; Y is not written).
    vtlhip::ScratchArena arena(base, vtlhip::kStaticScratchBytes);
    return vtl_hip_linear_f32_dynquant(X, Wq, sw, bias, Y, M, N, K, relu, nullptr, 0);
}

}  // extern "C"
