// Measurement aid of bench.py, built into its own small library and not part
// of libvtlhip.so: nothing but the int8 MFMA of the matmul kernels, so that a
// run can time what the matrix cores sustain on given operand bits.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// 16 independent 32x32 accumulators per wave fed from registers that are loaded
// once (8 operand vectors per lane from `operands`, 32 KiB), four waves on every
// SIMD of the chip.  With constant operands this loop runs at the nominal rate,
// with random ones at whatever the power limit leaves.
__global__ __launch_bounds__(256) void mfma_i8_probe_kernel(const int8_t *__restrict__ operands, int iterations,
                                                            int32_t *sink)
{
    const v4i *in = reinterpret_cast<const v4i *>(operands) + threadIdx.x * 8;
    v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a[i] = in[i];
        b[i] = in[4 + i];
    }
    v16i acc[16];
#pragma unroll
    for (int i = 0; i < 16; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            acc[i][r] = 0;
    for (int it = 0; it < iterations; it++) {
#pragma unroll
        for (int i = 0; i < 16; i++)
            acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i & 3], b[i >> 2], acc[i], 0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 16; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            s += acc[i][r];
    if (s == 0x7fffffff)   // keeps the loop alive; practically never true
        sink[0] = s;
}

// The same loop with fresh operands for every instruction: 32 A and 32 B
// fragments per lane stay in registers (256 VGPRs, one wave per SIMD) and the
// 64 instructions of an iteration walk through all of them, so that no two
// consecutive instructions share an operand register, as in a matmul kernel
// whose operands change with every k-step.  `operands`: 256 KiB (64 fragments
// of 16 bytes for each of the 256 threads of a workgroup).
__global__ __launch_bounds__(256) void mfma_i8_probe_rotating_kernel(const int8_t *__restrict__ operands,
                                                                     int iterations, int32_t *sink)
{
    const v4i *in = reinterpret_cast<const v4i *>(operands) + threadIdx.x * 64;
    v4i a[32], b[32];
#pragma unroll
    for (int i = 0; i < 32; i++) {
        a[i] = in[i];
        b[i] = in[32 + i];
    }
    v16i acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            acc[i][r] = 0;
    for (int it = 0; it < iterations; it++) {
#pragma unroll
        for (int u = 0; u < 64; u++)
            acc[u & 7] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[u & 31], b[(u * 7 + (u >> 5) * 3) & 31], acc[u & 7],
                                                               0, 0, 0);
    }
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int r = 0; r < 16; r++)
            s += acc[i][r];
    if (s == 0x7fffffff)   // keeps the loop alive; practically never true
        sink[0] = s;
}

// 1024 workgroups of 4 waves, each wave `iterations` times 16 instructions of
// 32x32x32: ops = 1024 * 4 * 16 * iterations * 65536.  `operands`: 32 KiB on the
// device, 16-byte aligned; `sink`: one int32 on the device; `stream`: a
// hipStream_t or NULL.  Returns 0, 1 for bad arguments, 3 when the launch fails.
extern "C" int vtl_bench_probe_mfma_i8(const int8_t *operands, int iterations, int32_t *sink, void *stream)
{
    if (!operands || !sink || iterations < 0 || (reinterpret_cast<uintptr_t>(operands) & 15))
        return 1;
    hipLaunchKernelGGL(mfma_i8_probe_kernel, dim3(1024), dim3(256), 0, (hipStream_t)stream, operands, iterations,
                       sink);
    return hipGetLastError() == hipSuccess ? 0 : 3;
}

// 1024 workgroups of 4 waves, each wave `iterations` times 64 instructions:
// ops = 1024 * 4 * 64 * iterations * 65536.  `operands`: 256 KiB on the device.
extern "C" int vtl_bench_probe_mfma_i8_rotating(const int8_t *operands, int iterations, int32_t *sink, void *stream)
{
    if (!operands || !sink || iterations < 0 || (reinterpret_cast<uintptr_t>(operands) & 15))
        return 1;
    hipLaunchKernelGGL(mfma_i8_probe_rotating_kernel, dim3(1024), dim3(256), 0, (hipStream_t)stream, operands,
                       iterations, sink);
    return hipGetLastError() == hipSuccess ? 0 : 3;
}
