"""GPU parity of the int8 matmul and the fused f32 epilogue through the C ABI.

Bar: int32 accumulators bit-exact; f32 outputs within 1e-5 relative of the
oracle applying the same scales (the kernels keep the oracle's operation
order, so equality is asserted as well).
"""
import numpy as np
import pytest

import oracle
from helpers import CPU_THREADS, KAT, dev, rel_err, raw_device_buffer, h2d, d2h
from vtl_amd import capi, workloads
from vtl_amd.tensor import HipTensor, gemm_i8_hip, linear_i8_hip

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("guard_bands")]

F32_REL_TOL = 1e-5   # tolerance stated for dequantized f32 outputs


def _gemm(a, bt):
    A, B = dev(a), dev(bt)
    Cm = HipTensor.empty([a.shape[0], bt.shape[0]], np.int32)
    gemm_i8_hip(Cm, A, B)
    out = Cm.cpu()
    for h in (A, B, Cm):
        h.release()
    return out


def test_identity_vector_from_reference_tests(hip):
    v = KAT["reference_vocabulary"]["matmul_identity"]           # la/la_test.v:30-37
    a = np.array(v["a"], np.int8)
    b = np.array(v["b"], np.int8)
    assert np.array_equal(_gemm(a, np.ascontiguousarray(b.T)), np.array(v["out"], np.int32))


@pytest.mark.parametrize("k", KAT["gemm_closed_forms"]["k_values"])
def test_closed_forms(hip, k):
    ones = np.full((40, k), 127, np.int8)
    assert np.all(_gemm(ones, ones) == k * 16129)
    assert np.all(_gemm(ones, -ones) == -k * 16129)
    alt = np.tile(np.array([1, -1], np.int8), k // 2)[None, :].repeat(5, 0)
    assert np.all(_gemm(alt, np.ones((70, k), np.int8)) == 0)
    n_eye = min(k, 96)
    eye = np.eye(k, dtype=np.int8)[:n_eye] * 127
    b = (np.arange(33 * k, dtype=np.int64).reshape(33, k) % 255 - 127)
    assert np.array_equal(_gemm(eye, b.astype(np.int8)), 127 * b[:, :n_eye].T)


def test_maximum_k_accumulates_without_overflow(hip):
    k = 131072                                                   # K * 127^2 = 2 114 060 288 < 2^31
    a = np.full((2, k), 127, np.int8)
    assert np.all(_gemm(a, a) == k * 16129)
    assert np.all(_gemm(a, -a) == -k * 16129)


SHAPES = [(1, 1, 16), (1, 64, 4096), (8, 128, 256), (33, 65, 48), (17, 19, 23), (64, 256, 784),
          (128, 128, 128), (256, 256, 128), (256, 512, 512), (300, 200, 144), (257, 255, 1040),
          (512, 768, 384), (96, 11008 // 8, 640), (1024, 1024, 256), (5, 7, 1), (2, 3, 17),
          # K a multiple of 16 but not of the 128-byte tile depth, on every tile size
          (300, 300, 48), (40, 2100, 400), (64, 2100, 400), (130, 2100, 2000), (1100, 1100, 1936), (2100, 2100, 272)]


@pytest.mark.parametrize("mnk", SHAPES)
def test_gemm_and_linear_match_oracle(hip, mnk):
    m, n, k = mnk
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k, seed=m * 31 + n * 17 + k)
    ref = oracle.gemm_i8_i32(a, bt, threads=CPU_THREADS)
    assert np.array_equal(_gemm(a, bt), ref)
    A, B = dev(a), dev(bt)
    for sa_v, sb_v, bias_v, relu in [(sa, sb, bias, False), (sa, sb, bias, True), (sa[:1], sb, None, False),
                                     (sa, sb[:1], bias, True), (sa[:1], sb[:1], None, False)]:
        dsa, dsb = dev(sa_v), dev(sb_v)
        dbias = dev(bias_v) if bias_v is not None else None
        y = linear_i8_hip(A, dsa, B, dsb, dbias, relu=relu)
        got = y.cpu()
        want = oracle.epilogue(ref, sa_v, sb_v, bias_v, relu=relu)
        assert rel_err(got, want) <= F32_REL_TOL
        assert np.array_equal(got, want)
        for h in (dsa, dsb, y) + ((dbias,) if dbias is not None else ()):
            h.release()
    A.release()
    B.release()


def test_unaligned_operands_take_the_generic_kernel(hip):
    a, bt, sa, sb, bias = workloads.square_int8_gemm(20, 24, 64, seed=5)
    abuf, bbuf = raw_device_buffer(a.size + 64), raw_device_buffer(bt.size + 64)
    cbuf = raw_device_buffer(20 * 24 * 4)
    h2d(abuf.ptr + 3, a)
    h2d(bbuf.ptr + 5, bt)
    capi.call("vtl_hip_gemm_i8_i32", abuf.ptr + 3, bbuf.ptr + 5, cbuf.ptr, 20, 24, 64)
    assert np.array_equal(d2h(cbuf.ptr, (20, 24), np.int32), oracle.gemm_i8_i32(a, bt))
    for h in (abuf, bbuf, cbuf):
        h.release()


@pytest.mark.parametrize("mnk", [(300, 200, 1000), (8, 2048, 4090), (64, 256, 777), (1100, 520, 2001),
                                 (256, 1024, 1024), (20, 2304, 512)])
def test_odd_k_and_unaligned_operands_are_repacked(hip, mnk):
    """K that is no multiple of 16, and operands / outputs at odd addresses: the
    library pads the rows into its own scratch and runs the fast kernels; results
    are the oracle's bit for bit (int32 and the f32 epilogue)."""
    m, n, k = mnk
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k, seed=m + n + k)
    ref = oracle.gemm_i8_i32(a, bt, threads=CPU_THREADS)
    want = oracle.epilogue(ref, sa, sb, bias, relu=True)
    abuf, bbuf = raw_device_buffer(a.size + 64), raw_device_buffer(bt.size + 64)
    cbuf, ybuf = raw_device_buffer(m * n * 4 + 64), raw_device_buffer(m * n * 4 + 64)
    dsa, dsb, dbias = dev(sa), dev(sb), dev(bias)
    for off_a, off_b, off_c in ((0, 0, 0), (3, 5, 4), (16, 1, 12)):
        h2d(abuf.ptr + off_a, a)
        h2d(bbuf.ptr + off_b, bt)
        capi.call("vtl_hip_gemm_i8_i32", abuf.ptr + off_a, bbuf.ptr + off_b, cbuf.ptr + off_c, m, n, k)
        assert np.array_equal(d2h(cbuf.ptr + off_c, (m, n), np.int32), ref), (off_a, off_b, off_c)
        capi.call("vtl_hip_linear_i8_f32", abuf.ptr + off_a, dsa.ptr, 1, bbuf.ptr + off_b, dsb.ptr, 1, dbias.ptr,
                  ybuf.ptr + off_c, m, n, k, 1)
        assert np.array_equal(d2h(ybuf.ptr + off_c, (m, n), np.float32), want), (off_a, off_b, off_c)
    for h in (abuf, bbuf, cbuf, ybuf, dsa, dsb, dbias):
        h.release()


def test_shape_mismatch_is_reported_like_la_matmul(hip):
    A, B = dev(np.zeros((4, 32), np.int8)), dev(np.zeros((6, 48), np.int8))
    Cm = HipTensor.empty([4, 6], np.int32)
    with pytest.raises(ValueError, match="Invalid shapes for matrix multiplication"):   # la/la.v:41-43
        gemm_i8_hip(Cm, A, B)
    with pytest.raises(ValueError, match="dst shape"):
        gemm_i8_hip(HipTensor.empty([4, 5], np.int32), A, dev(np.zeros((6, 32), np.int8)))


def test_square_gemm_config_full_size(hip):
    """Config 3 at its real size 4096^3: full oracle parity on a band of rows,
    exact row/column checksums and linearity over the whole product."""
    m = n = k = 4096
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k)
    A, B = dev(a), dev(bt)
    Cm = HipTensor.empty([m, n], np.int32)
    gemm_i8_hip(Cm, A, B)
    c = Cm.cpu()
    band = np.r_[0:96, 2000:2096, m - 64:m]
    ref_band = oracle.gemm_i8_i32(a[band], bt, threads=CPU_THREADS)
    assert np.array_equal(c[band], ref_band)
    # checksums: 1^T C = (1^T A) B^T and C 1 = A (B^T 1), in int64
    a64, b64 = a.astype(np.int64), bt.astype(np.int64)
    assert np.array_equal(c.sum(axis=0, dtype=np.int64), a64.sum(axis=0) @ b64.T)
    assert np.array_equal(c.sum(axis=1, dtype=np.int64), a64 @ b64.sum(axis=0))
    # linearity in the second operand: C(A, B1 + B2) = C(A, B1) + C(A, B2)
    b1 = (bt // 2).astype(np.int8)
    b2 = (bt - b1).astype(np.int8)
    B1, B2 = dev(b1), dev(b2)
    C1, C2 = HipTensor.empty([m, n], np.int32), HipTensor.empty([m, n], np.int32)
    gemm_i8_hip(C1, A, B1)
    gemm_i8_hip(C2, A, B2)
    assert np.array_equal(C1.cpu() + C2.cpu(), c)
    # fused epilogue over the whole output against the oracle epilogue on the
    # (already verified) accumulators
    dsa, dsb, dbias = dev(sa), dev(sb), dev(bias)
    y = linear_i8_hip(A, dsa, B, dsb, dbias).cpu()
    want = oracle.epilogue(c, sa, sb, bias)
    assert rel_err(y, want) <= F32_REL_TOL
    assert np.array_equal(y, want)
    for h in (A, B, Cm, B1, B2, C1, C2, dsa, dsb, dbias):
        h.release()


# Shapes chosen to reach every kernel family: the weight-streaming kernel
# (M <= 32, N >= 2048, K % 256 == 0) with ragged N and M, split-K launches
# (few output tiles, long K) with uneven K ranges, and the register-staged
# tile kernel (K % 128 != 0).
ROUTED_SHAPES = [(1, 2048, 256), (1, 5, 256), (1, 4099, 4080), (1, 9000, 5120), (1, 300, 8192), (1, 2048, 8448),
                 (1, 9000, 9232), (1, 4097, 11264), (1, 8192, 14336), (1, 100, 14352), (1, 3000, 16384),
                 (1, 262200, 256),      # more rows than the matrix-vector kernel deals out
                 # rows longer than 6144 codes run on half as many waves: 64 rows per wave is the
                 # most a wave can park (131072 rows), one row more leaves the matrix-vector kernel
                 (1, 131072, 6160), (1, 131073, 6160), (1, 152064, 8192),

                 (3, 2050, 256), (8, 2048, 4096), (9, 2048, 768), (16, 2047, 1280),
                 (17, 2077, 1280), (32, 4096, 512), (31, 14336, 256), (5, 3001, 4096),
                 (256, 1024, 4096), (256, 512, 11008), (64, 128, 11008), (128, 256, 8192), (40, 200, 5504),
                 (100, 300, 1360), (256, 256, 1040)]
# small products: one 32x32 tile per workgroup fed straight from global memory
# (at most 64 tiles, K <= 2048), incl. K % 32 == 16, single rows and columns
SMALL_SHAPES = [(64, 256, 784), (1, 1, 16), (2, 3, 16), (33, 65, 48), (64, 64, 2048), (31, 1, 1008),
                (1, 97, 2032), (256, 256, 512), (100, 300, 1360), (256, 256, 1040)]


@pytest.mark.parametrize("small", ["0", "1", None])
@pytest.mark.parametrize("mnk", SMALL_SHAPES)
def test_small_product_kernel_and_its_alternatives(hip, mnk, small, knobs):
    """VTL_HIP_GEMM_SMALL=1 forces the small-product kernel, 0 the tile kernels the
    same shapes used before it existed, unset the library's own choice."""
    if small is None:
        knobs.delenv("VTL_HIP_GEMM_SMALL", raising=False)
    else:
        knobs.setenv("VTL_HIP_GEMM_SMALL", small)
    m, n, k = mnk
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k, seed=m * 17 + n * 5 + k)
    ref = oracle.gemm_i8_i32(a, bt, threads=CPU_THREADS)
    assert np.array_equal(_gemm(a, bt), ref)
    A, B, dsa, dsb, dbias = dev(a), dev(bt), dev(sa), dev(sb), dev(bias)
    for relu, b_dev, b_host in ((True, dbias, bias), (False, None, None)):
        y = linear_i8_hip(A, dsa, B, dsb, b_dev, relu=relu)
        assert np.array_equal(y.cpu(), oracle.epilogue(ref, sa, sb, b_host, relu=relu))
        y.release()
    for h in (A, B, dsa, dsb, dbias):
        h.release()


@pytest.mark.parametrize("mnk", ROUTED_SHAPES)
def test_every_kernel_family_matches_oracle(hip, mnk):
    m, n, k = mnk
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k, seed=m * 131 + n * 7 + k)
    ref = oracle.gemm_i8_i32(a, bt, threads=CPU_THREADS)
    assert np.array_equal(_gemm(a, bt), ref)
    A, B, dsa, dsb, dbias = dev(a), dev(bt), dev(sa), dev(sb), dev(bias)
    for relu, b_dev, b_host in ((True, dbias, bias), (False, None, None)):
        y = linear_i8_hip(A, dsa, B, dsb, b_dev, relu=relu)
        got = y.cpu()
        want = oracle.epilogue(ref, sa, sb, b_host, relu=relu)
        assert rel_err(got, want) <= F32_REL_TOL and np.array_equal(got, want)
        y.release()
    for h in (A, B, dsa, dsb, dbias):
        h.release()


# few-token kernel (2 <= M <= 8 rows of codes held in registers): every row count, every
# row-length class (K <= 1024, 2048, 4096, 8192), K % 16 == 0 only, ragged N, more weight rows
# than one batch of parked sums per wave (at K = 256 there are 8192 waves, a batch is 64 / MR
# weight rows per wave: the last two shapes need two and three batches)
FEW_TOKEN_SHAPES = [(2, 2048, 256), (2, 3001, 1008), (2, 2050, 2048), (2, 2048, 4096), (2, 2049, 8192),
                    (3, 2048, 1024), (4, 4099, 1040), (4, 2048, 4096), (3, 2051, 8192), (4, 2048, 5120),
                    (5, 2048, 512), (8, 2050, 2032), (7, 2048, 4096), (6, 5000, 3088), (8, 40000, 256),
                    (2, 140000, 272), (4, 70001, 256), (8, 70001, 256), (5, 140000, 256),
                    # few weight rows: fewer rows than waves, a single row, ragged everything
                    (2, 1, 256), (3, 7, 4096), (8, 64, 1024), (4, 100, 8192), (7, 1000, 272), (2, 1536, 4096),
                    # two tokens with long rows (up to 11264 codes), and just past that limit
                    (2, 2048, 9232), (2, 4099, 11008), (2, 300, 11264), (2, 2048, 11280)]


@pytest.mark.parametrize("rows_kernel", ["1", "0", None])
@pytest.mark.parametrize("mnk", FEW_TOKEN_SHAPES)
def test_few_token_kernel_and_its_alternatives(hip, mnk, rows_kernel, knobs):
    """VTL_HIP_GEMV_ROWS=1 forces the few-token kernel wherever it applies, 0 keeps it
    off, unset is the library's own choice: int32 sums and f32 epilogue are those of the oracle."""
    if rows_kernel is None:
        knobs.delenv("VTL_HIP_GEMV_ROWS", raising=False)
    else:
        knobs.setenv("VTL_HIP_GEMV_ROWS", rows_kernel)
    m, n, k = mnk
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k, seed=m * 31 + n * 3 + k)
    ref = oracle.gemm_i8_i32(a, bt, threads=CPU_THREADS)
    assert np.array_equal(_gemm(a, bt), ref)
    A, B, dsa, dsb, dbias = dev(a), dev(bt), dev(sa), dev(sb), dev(bias)
    for relu, b_dev, b_host in ((True, dbias, bias), (False, None, None)):
        y = linear_i8_hip(A, dsa, B, dsb, b_dev, relu=relu)
        assert np.array_equal(y.cpu(), oracle.epilogue(ref, sa, sb, b_host, relu=relu))
        y.release()
    # one scale for all rows of A and one for all of W
    y = linear_i8_hip(A, dev(sa[:1]), B, dev(sb[:1]), dbias, relu=False)
    assert np.array_equal(y.cpu(), oracle.epilogue(ref, sa[:1], sb[:1], bias))
    for h in (A, B, dsa, dsb, dbias, y):
        h.release()


# the weight-streaming kernel on blocks of 32 activation rows x 32 weight rows (small outputs
# with a long K, M > 32; also M <= 32 against few weight rows): whole and ragged blocks in both
# directions, one block, one round of workgroups and two, every row-count class of a block
# (<= 8, <= 16, <= 32 rows in the last block), K of one chunk per wave and of uneven shares
ROW_BLOCK_SHAPES = [(256, 1024, 4096), (250, 1000, 4096), (33, 4096, 2048), (64, 64, 4096), (100, 2500, 1024),
                    (40, 31, 1024), (65, 33, 1280), (72, 96, 2304), (48, 50, 11008), (300, 40, 768),
                    (16, 1024, 4096), (5, 500, 2048), (32, 64, 1024), (1000, 32, 1024)]


@pytest.mark.parametrize("waves", ["4", "2", "0", None])
@pytest.mark.parametrize("mnk", ROW_BLOCK_SHAPES)
def test_row_block_weight_streaming_kernel_and_its_alternatives(hip, mnk, waves, knobs):
    """VTL_HIP_SKINNY_TILED=1 forces the kernel (with VTL_HIP_SKINNY_WAVES waves a workgroup),
    0 keeps it off, unset is the library's own choice: same int32 sums, same f32 rows."""
    if waves is None:
        knobs.delenv("VTL_HIP_SKINNY_TILED", raising=False)
    elif waves == "0":
        knobs.setenv("VTL_HIP_SKINNY_TILED", "0")
    else:
        knobs.setenv("VTL_HIP_SKINNY_WAVES", waves)
        knobs.setenv("VTL_HIP_SKINNY_TILED", "1")
    m, n, k = mnk
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k, seed=m * 37 + n * 11 + k)
    ref = oracle.gemm_i8_i32(a, bt, threads=CPU_THREADS)
    assert np.array_equal(_gemm(a, bt), ref)
    A, B, dsa, dsb, dbias = dev(a), dev(bt), dev(sa), dev(sb), dev(bias)
    for relu, b_dev, b_host in ((True, dbias, bias), (False, None, None)):
        y = linear_i8_hip(A, dsa, B, dsb, b_dev, relu=relu)
        assert np.array_equal(y.cpu(), oracle.epilogue(ref, sa, sb, b_host, relu=relu))
        y.release()
    for h in (A, B, dsa, dsb, dbias):
        h.release()


@pytest.mark.parametrize("k", [2432, 2448, 80])   # 19 K steps of 128; the same plus a 16-byte tail; one partial step
def test_forced_split_k_is_exact(hip, knobs, k):
    """Every tile configuration with 1, 2, 3 and 8 K ranges gives the same int32 result
    (uneven ranges for every split count)."""
    m, n = 96, 384
    a, bt, sa, sb, bias = workloads.square_int8_gemm(m, n, k, seed=77)
    ref = oracle.gemm_i8_i32(a, bt, threads=CPU_THREADS)
    want = oracle.epilogue(ref, sa, sb, bias)
    A, B, dsa, dsb, dbias = dev(a), dev(bt), dev(sa), dev(sb), dev(bias)
    for idx in range(8):
        for splits in (1, 2, 3, 8):
            knobs.setenv("VTL_HIP_GEMM_CONFIG", f"{idx},{splits}")
            assert np.array_equal(_gemm(a, bt), ref), (idx, splits)
            y = linear_i8_hip(A, dsa, B, dsb, dbias)
            assert np.array_equal(y.cpu(), want), (idx, splits)
            y.release()
    knobs.delenv("VTL_HIP_GEMM_CONFIG")
    for h in (A, B, dsa, dsb, dbias):
        h.release()
