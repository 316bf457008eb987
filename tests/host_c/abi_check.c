/* The boundary is a C ABI: this file is plain C99 and includes only the
 * library's header.  It calls a few entry points that need no device and
 * takes the address of every compute entry point with its declared type, so
 * a signature that stops being valid C, or a symbol that is no longer
 * exported with C linkage, fails the build or the link. */
#include <stdio.h>
#include <string.h>

#include "vtl_hip.h"

int main(void)
{
    int (*quantize)(const float *, int64_t, int64_t, int, int8_t *, float *) = vtl_hip_quantize_f32_i8;
    int (*dequantize)(const int8_t *, const float *, int64_t, int64_t, int, float *) = vtl_hip_dequantize_i8_f32;
    int (*gemm)(const int8_t *, const int8_t *, int32_t *, int, int, int) = vtl_hip_gemm_i8_i32;
    int (*linear)(const int8_t *, const float *, int, const int8_t *, const float *, int, const float *, float *,
                  int, int, int, int) = vtl_hip_linear_i8_f32;
    int (*requant)(const int8_t *, const float *, int, const int8_t *, const float *, int, const float *, int,
                   int8_t *, float *, float *, int, int, int) = vtl_hip_linear_i8_requant;
    int (*dynquant)(const float *, const int8_t *, const float *, const float *, float *, int, int, int, int,
                    void *, size_t) = vtl_hip_linear_f32_dynquant;
    int (*matmul)(const float *, const float *, float *, int, int, int, int, int) = vtl_hip_matmul_f32;
    int (*backward)(const float *, const float *, const float *, float *, float *, float *, int, int, int) =
        vtl_hip_linear_backward_f32;
    int failures = 0;
    if (!quantize || !dequantize || !gemm || !linear || !requant || !dynquant || !matmul || !backward)
        failures++;
    if (strcmp(vtl_hip_strerror(VTL_HIP_OK), "success") != 0)
        failures++;
    if (quantize(NULL, 1, 1, 1, NULL, NULL) != VTL_HIP_ERR_INVALID_ARG)
        failures++;
    if (gemm(NULL, NULL, NULL, 0, 0, 0) != VTL_HIP_ERR_INVALID_ARG)
        failures++;
    if (vtl_hip_free(NULL) != VTL_HIP_OK)
        failures++;
    if (vtl_hip_linear_f32_dynquant_workspace(4, 16) < 4 * 16 + 4 * sizeof(float))
        failures++;
    if (failures)
        printf("C ABI check: %d failure(s)\n", failures);
    else
        printf("C ABI check: ok (%s)\n", vtl_hip_version());
    return failures ? 1 : 0;
}
