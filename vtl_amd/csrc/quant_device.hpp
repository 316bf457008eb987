// Device-side pieces of the symmetric INT8 quantizer shared by the streaming
// kernels and the fused decode kernel: wave / workgroup max, the correctly
// rounded code of one element, packing.  Arithmetic contract in quant.hip.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace vtlhip {
namespace qdev {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef int int4_t __attribute__((ext_vector_type(4)));

// Max over the 64 lanes of a wave, returned to every lane: cross-lane moves
// inside the VALU (DPP) - quads, half rows and rows by mirroring, then lane 15
// of each row into the next row and lane 31 into the upper half; lane 63 holds
// the result.  Lanes a move does not reach see 0, the identity for the
// non-negative values this is used on.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_max_step(float v)
{
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false);
    return fmaxf(v, __int_as_float(t));
}

__device__ __forceinline__ float wave_max(float v)
{
    v = dpp_max_step<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v = dpp_max_step<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v = dpp_max_step<0x141, 0xF>(v);  // row_half_mirror
    v = dpp_max_step<0x140, 0xF>(v);  // row_mirror
    v = dpp_max_step<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
    v = dpp_max_step<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Max over each group of SEG = 16, 32 or 64 consecutive lanes (a DPP row, two, or the wave),
// returned to every lane of the group.
template <int SEG>
__device__ __forceinline__ float segment_max(float v)
{
    static_assert(SEG == 16 || SEG == 32 || SEG == 64, "a DPP row, two, or the wave");
    if constexpr (SEG == 64)
        return wave_max(v);
    v = dpp_max_step<0xB1, 0xF>(v);
    v = dpp_max_step<0x4E, 0xF>(v);
    v = dpp_max_step<0x141, 0xF>(v);
    v = dpp_max_step<0x140, 0xF>(v);
    if constexpr (SEG == 32)
        v = fmaxf(v, __shfl_xor(v, 16));
    return v;
}

// Max over the workgroup; every thread gets the result.  smem holds T/64
// floats and is used once per kernel.
template <int T>
__device__ __forceinline__ float block_max(float v, float *smem)
{
    v = wave_max(v);
    if constexpr (T > 64) {
        const int w = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0)
            smem[w] = v;
        __syncthreads();
        float r = smem[0];
#pragma unroll
        for (int i = 1; i < T / 64; i++)
            r = fmaxf(r, smem[i]);
        v = r;
    }
    return v;
}

__device__ __forceinline__ float absmax4(float m, float4_t v)
{
    m = fmaxf(m, fabsf(v.x));
    m = fmaxf(m, fabsf(v.y));
    m = fmaxf(m, fabsf(v.z));
    m = fmaxf(m, fabsf(v.w));
    return m;
}

// Saturating f32 -> i32 conversion; NaN converts to 0 in hardware.
__device__ __forceinline__ int cvt_i32_sat(float r)
{
    int i;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(i) : "v"(r));
    return i;
}

struct QuantScale {
    float scale;
    float rinv;  // 1/scale when `fast`
    bool fast;   // scale and 1/scale are normal numbers with headroom
};

__device__ __forceinline__ QuantScale make_quant_scale(float scale)
{
    QuantScale p;
    p.scale = scale;
    p.fast = (scale >= 0x1p-100f) && (scale <= 0x1p100f);
    p.rinv = p.fast ? (1.0f / scale) : 0.0f;
    return p;
}

// Half-width of the band around k + 0.5 inside which the estimated quotient
// cannot decide the rounding.  For |x/scale| <= 128 the estimate
// fl(x * fl(1/scale)) is within 2^-16 of the true quotient and the correctly
// rounded quotient within 2^-18, so 2^-14 leaves a factor of three.  Larger
// quotients clamp to +-127 whichever way they round.
constexpr float kTieBand = 0x1p-14f;

__device__ __forceinline__ int quant_code(float x, const QuantScale &p)
{
    float r;
    if (p.fast) {
        const float t = x * p.rinv;
        r = rintf(t);
        if (__builtin_expect(fabsf(t - r) >= 0.5f - kTieBand, 0))
            r = rintf(x / p.scale);
    } else {
        r = rintf(x / p.scale);  // 0/0, x/Inf, subnormal scales: exact path
    }
    const int i = cvt_i32_sat(r);
    return min(max(i, -127), 127);
}

__device__ __forceinline__ unsigned pack4(int a, int b, int c, int d)
{
    return (unsigned)(a & 0xff) | ((unsigned)(b & 0xff) << 8) | ((unsigned)(c & 0xff) << 16) |
           ((unsigned)d << 24);
}

__device__ __forceinline__ unsigned quant4(float4_t v, const QuantScale &p)
{
    return pack4(quant_code(v.x, p), quant_code(v.y, p), quant_code(v.z, p), quant_code(v.w, p));
}

}  // namespace qdev
}  // namespace vtlhip
