/* Walks every function of the CPU oracle over ragged shapes with exactly sized
 * heap buffers; built with -fsanitize=address,undefined so that an access past
 * a buffer, a misaligned access, a signed overflow or an out-of-range float to
 * int conversion inside the oracle stops the program.  Values are checked only
 * loosely here (the parity tests pin them): what this program looks for is
 * undefined behaviour. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "vtl_oracle.h"

static uint64_t state = 0x9e3779b97f4a7c15ull;
static uint32_t rnd(void)
{
    state ^= state << 13;
    state ^= state >> 7;
    state ^= state << 17;
    return (uint32_t)(state >> 16);
}
static float rndf(void) { return (float)((int32_t)rnd() % 2001 - 1000) / 250.0f; }

static void *buf(size_t n, size_t elem)
{
    void *p = malloc(n > 0 ? n * elem : 1);   /* exactly sized: one element more is an error */
    if (!p) {
        fprintf(stderr, "out of memory\n");
        exit(2);
    }
    return p;
}

static int fails = 0;
#define CHECK(c)                                                       \
    do {                                                               \
        if (!(c)) {                                                    \
            fprintf(stderr, "line %d: %s\n", __LINE__, #c);            \
            fails++;                                                   \
        }                                                              \
    } while (0)

static void quant_case(int64_t rows, int64_t cols, int special)
{
    const int64_t n = rows * cols;
    float *x = buf(n, 4), *xh = buf(n, 4), *am = buf(rows ? rows : 1, 4), *sc = buf(rows ? rows : 1, 4);
    int8_t *q = buf(n, 1), *q2 = buf(n, 1);
    for (int64_t i = 0; i < n; i++)
        x[i] = rndf();
    if (special && n > 0) {   /* values the conversion to int8 must survive */
        const float sp[] = {NAN, INFINITY, -INFINITY, 3.0e38f, -3.0e38f, 1e-45f, -0.0f, 0.5f, 1.5f, 2.5f};
        for (int64_t i = 0; i < n && i < 10; i++)
            x[(i * 7) % n] = sp[i];
    }
    for (int per_row = 0; per_row < 2; per_row++) {
        vtl_ref_absmax_f32(x, rows, cols, per_row, am);
        vtl_ref_quantize_f32_i8(x, rows, cols, per_row, q, sc);
        vtl_ref_quantize_with_scale(x, sc, rows, cols, per_row, q2);
        CHECK(memcmp(q, q2, (size_t)n) == 0);
        vtl_ref_dequantize_i8_f32(q, sc, rows, cols, per_row, xh);
        vtl_ref_quantize_f32_i8_mt(x, rows, cols, per_row, q2, sc, 3);
        CHECK(memcmp(q, q2, (size_t)n) == 0);
        vtl_ref_dequantize_i8_f32_mt(q, sc, rows, cols, per_row, xh, 3);
        for (int64_t i = 0; i < n; i++)
            CHECK(q[i] != -128);
    }
    free(x), free(xh), free(am), free(sc), free(q), free(q2);
}

static void linear_case(int64_t M, int64_t N, int64_t K, int extreme)
{
    int8_t *a = buf(M * K, 1), *w = buf(N * K, 1);
    float *sa = buf(M, 4), *sw = buf(N, 4), *bias = buf(N, 4), *y = buf(M * N, 4), *y2 = buf(M * N, 4);
    float *xf = buf(M * K, 4);
    int32_t *c = buf(M * N, 4);
    for (int64_t i = 0; i < M * K; i++) {
        a[i] = extreme ? (int8_t)((i & 1) ? 127 : -127) : (int8_t)((int)(rnd() % 255) - 127);
        xf[i] = rndf();
    }
    for (int64_t i = 0; i < N * K; i++)
        w[i] = extreme ? (int8_t)127 : (int8_t)((int)(rnd() % 255) - 127);
    for (int64_t i = 0; i < M; i++)
        sa[i] = 0.01f + 0.001f * (float)(i % 7);
    for (int64_t i = 0; i < N; i++) {
        sw[i] = 0.02f + 0.001f * (float)(i % 5);
        bias[i] = rndf();
    }
    for (int threads = 1; threads <= 3; threads += 2) {
        vtl_ref_gemm_i8_i32(a, w, c, M, N, K, threads);
        vtl_ref_epilogue_f32(c, sa, 1, sw, 1, bias, y, M, N, 1);
        vtl_ref_linear_i8_f32(a, sa, 1, w, sw, 1, bias, y2, M, N, K, 1, threads);
        CHECK(memcmp(y, y2, (size_t)(M * N) * 4) == 0);
        vtl_ref_epilogue_f32(c, sa, 0, sw, 0, NULL, y, M, N, 0);
        vtl_ref_linear_f32_dynquant(xf, w, sw, bias, y, M, N, K, 0, threads);
        vtl_ref_linear_f32_dynquant(xf, w, sw, NULL, y, M, N, K, 1, threads);
    }
    vtl_ref_relu_f32(y, M * N);
    free(a), free(w), free(sa), free(sw), free(bias), free(y), free(y2), free(xf), free(c);
}

static void matmul_case(int64_t M, int64_t N, int64_t K)
{
    float *a = buf(M * K, 4), *b = buf(K * N, 4), *c = buf(M * N, 4), *g = buf(M * N, 4);
    float *dx = buf(M * K, 4), *dw = buf(N * K, 4), *db = buf(N, 4), *w = buf(N * K, 4), *bias = buf(N, 4);
    double *ad = buf(M * K, 8), *bd = buf(K * N, 8), *cd = buf(M * N, 8), *gd = buf(M * N, 8);
    double *dxd = buf(M * K, 8), *dwd = buf(N * K, 8), *dbd = buf(N, 8), *wd = buf(N * K, 8);
    for (int64_t i = 0; i < M * K; i++)
        ad[i] = a[i] = rndf();
    for (int64_t i = 0; i < K * N; i++)
        wd[i] = w[i] = bd[i] = b[i] = rndf();
    for (int64_t i = 0; i < M * N; i++)
        gd[i] = g[i] = rndf();
    for (int64_t i = 0; i < N; i++)
        bias[i] = rndf();
    for (int ta = 0; ta < 2; ta++)
        for (int tb = 0; tb < 2; tb++) {
            /* the same buffers read as [M,K] / [K,M] and [K,N] / [N,K]: sizes agree either way */
            vtl_ref_matmul_f32(a, b, c, M, N, K, ta, tb, 1 + 2 * ta);
            vtl_ref_matmul_f64(ad, bd, cd, M, N, K, ta, tb, 1 + 2 * tb);
        }
    vtl_ref_linear_f32_via_f64(a, w, bias, c, M, N, K);
    vtl_ref_linear_f32_via_f64(a, w, NULL, c, M, N, K);
    vtl_ref_colsum_f32(g, M, N, db);
    vtl_ref_colsum_f64(gd, M, N, dbd);
    vtl_ref_linear_backward_f32(g, a, w, dx, dw, db, M, N, K, 2);
    vtl_ref_linear_backward_f32(g, a, w, NULL, dw, NULL, M, N, K, 1);
    vtl_ref_linear_backward_f64(gd, ad, wd, dxd, dwd, dbd, M, N, K, 2);
    vtl_ref_linear_backward_f64(gd, ad, wd, dxd, NULL, NULL, M, N, K, 1);
    if (K > 0) {
        float *yv = buf(M, 4);
        double *yd = buf(M, 8);
        vtl_ref_gemv_f32(a, b, yv, M, K);   /* b has K * N >= K elements when N >= 1 */
        vtl_ref_gemv_f64(ad, bd, yd, M, K);
        free(yv), free(yd);
    }
    vtl_ref_sigmoid_f32(g, c, M * N);
    vtl_ref_sigmoid_f64(gd, cd, M * N);
    vtl_ref_relu_f64(gd, M * N);
    free(a), free(b), free(c), free(g), free(dx), free(dw), free(db), free(w), free(bias);
    free(ad), free(bd), free(cd), free(gd), free(dxd), free(dwd), free(dbd), free(wd);
}

int main(void)
{
    const int64_t qshapes[][2] = {{0, 0}, {0, 5}, {3, 0}, {1, 1}, {1, 7}, {7, 1}, {5, 33}, {64, 65}, {3, 1023},
                                  {2, 4097}};
    for (size_t i = 0; i < sizeof qshapes / sizeof qshapes[0]; i++)
        for (int special = 0; special < 2; special++)
            quant_case(qshapes[i][0], qshapes[i][1], special);
    const int64_t lshapes[][3] = {{1, 1, 1}, {1, 5, 16}, {3, 2, 17}, {33, 65, 48}, {7, 9, 255}, {64, 31, 130},
                                  {2, 3, 4099}};
    for (size_t i = 0; i < sizeof lshapes / sizeof lshapes[0]; i++)
        for (int extreme = 0; extreme < 2; extreme++)
            linear_case(lshapes[i][0], lshapes[i][1], lshapes[i][2], extreme);
    /* the longest K the library accepts: K * 127^2 must stay below 2^31 (no signed overflow) */
    linear_case(1, 2, 131072, 1);
    const int64_t mshapes[][3] = {{1, 1, 1}, {2, 3, 5}, {17, 9, 33}, {5, 64, 7}, {31, 2, 129}};
    for (size_t i = 0; i < sizeof mshapes / sizeof mshapes[0]; i++)
        matmul_case(mshapes[i][0], mshapes[i][1], mshapes[i][2]);
    CHECK(vtl_ref_quantize_one(NAN, 1.0f) == 0);
    CHECK(vtl_ref_quantize_one(INFINITY, 1.0f) == 127);
    CHECK(vtl_ref_quantize_one(-3.0e38f, 1e-30f) == -127);
    CHECK(vtl_ref_quantize_one(0.0f, 0.0f) == 0);   /* an all-zero slice: scale 0, 0 / 0 -> code 0 */
    CHECK(vtl_ref_scale_from_absmax(127.0f) == 1.0f);
    CHECK(vtl_ref_max_threads() >= 1);
    if (fails) {
        fprintf(stderr, "oracle under sanitizers: %d checks failed\n", fails);
        return 1;
    }
    printf("oracle under sanitizers: ok\n");
    return 0;
}
