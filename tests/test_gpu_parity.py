"""GPU parity: every kernel, through the C ABI, against the CPU oracle on the same seeded
inputs.  Integer results (packed nibbles, int32 accumulators) must be bit-exact; fp16
outputs are compared bit-exactly too (the bar is 1e-3 relative; the kernels mirror the
reference's per-operator rounding, so equality is expected and asserted)."""
import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip(dev):
    from duqlinear4bitcuda_amd import _HIP

    return _HIP


def _say(*a):
    print(*a, flush=True)


# ---------------------------------------------------------------- quantizers
@pytest.mark.parametrize("M,K", [(1, 64), (3, 72), (16, 4096), (5, 33), (7, 1), (64, 11008), (2, 8)])
@pytest.mark.parametrize("qmax", [6, 7])
def test_sym_quant_given_scale(hip, dev, M, K, qmax):
    _say("sym_quant", M, K, qmax)
    x = cases.acts_outliers(M, K, seed=10 + M + K)
    s = orc.sym_scales(x)
    want = orc.sym_quant(x, s, qmax)
    got = hip.sym_quant(cases.t(x, dev), cases.t(s, dev), qmax=qmax).cpu().numpy()
    assert got.shape == want.shape
    assert np.array_equal(got, want)


def test_sym_quant_exhaustive_fp16(hip, dev):
    """Every finite and non-finite binary16 input against a set of scales: pins the
    division + rounding + clamp bit for bit."""
    allx = np.arange(65536, dtype=np.uint16).view(np.float16)
    scales = np.array([1.0, 0.5, 3.0, 0.1, 7.0, 1e-3, 6e-5, 5.96e-8, 1.001, 0.333, 65504.0, 0.0, 123.4, 0.7197,
                       np.inf, 2.5e-4], dtype=np.float16)
    x = np.tile(allx, (len(scales), 1))
    s = scales.reshape(-1, 1)
    for qmax in (6, 7):
        want = orc.sym_quant(x, s, qmax)
        got = hip.sym_quant(cases.t(x, dev), cases.t(s, dev), qmax=qmax).cpu().numpy()
        bad = np.argwhere(got != want)
        assert bad.size == 0, f"first mismatches (row, byte): {bad[:8]}"


def test_asym_quant_exhaustive_fp16(hip, dev):
    allx = np.arange(65536, dtype=np.uint16).view(np.float16)
    scales = np.array([1.0, 0.4, 0.0133, 2.0, 1e-3, 0.0, 100.0, 0.25], dtype=np.float16)
    zeros = np.array([0.0, 7.0, 15.0, -3.0, 8.0, np.inf, 2048.0, 3.0], dtype=np.float16)
    x = np.tile(allx, (len(scales), 1))
    want = orc.asym_quant(x, scales.reshape(-1, 1), zeros.reshape(-1, 1))
    got = hip.asym_quant(cases.t(x, dev), cases.t(scales.reshape(-1, 1), dev),
                         cases.t(zeros.reshape(-1, 1), dev)).cpu().numpy()
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"first mismatches (row, byte): {bad[:8]}"


@pytest.mark.parametrize("M,K", [(4, 64), (3, 40), (16, 4096), (5, 33)])
def test_dual_and_asym_quant_given_scale(hip, dev, M, K):
    _say("dual/asym quant", M, K)
    x = cases.acts_uniform(M, K, seed=20 + M + K)
    rng = np.random.default_rng(M * 1000 + K)
    s1 = rng.uniform(0.05, 1.0, (M, 1)).astype(np.float16)
    s2 = rng.uniform(0.05, 1.0, (M, 1)).astype(np.float16)
    z1 = rng.integers(0, 8, (M, 1)).astype(np.float16)
    z2 = (rng.integers(0, 16, (M, 1)) + 0.5).astype(np.float16)
    d = dev
    got = hip.sym_dual_quant(cases.t(x, d), cases.t(s1, d), cases.t(s2, d)).cpu().numpy()
    assert np.array_equal(got, orc.sym_dual_quant(x, s1, s2))
    got = hip.asym_quant(cases.t(x, d), cases.t(s1, d), cases.t(z1, d)).cpu().numpy()
    assert np.array_equal(got, orc.asym_quant(x, s1, z1))
    got = hip.asym_dual_quant(cases.t(x, d), cases.t(s1, d), cases.t(z1, d), cases.t(s2, d), cases.t(z2, d)).cpu().numpy()
    assert np.array_equal(got, orc.asym_dual_quant(x, s1, z1, s2, z2))


@pytest.mark.parametrize("M,K", [(1, 4096), (16, 4096), (4, 11008), (33, 64), (2048, 4096), (3, 28672), (128, 8192),
                                 (5, 32), (2, 65536 + 64)])
def test_quantize_rows_sym(hip, dev, M, K):
    _say("quantize_rows_sym", M, K)
    x = cases.acts_outliers(M, K, seed=30 + M + K)
    if M > 2:
        x[1, :] = 0  # an all-zero token: scale 0, codes 0
    if M > 8:
        x[2, 5] = np.nan          # NaN statistic: every code of the row becomes 0
        x[3, 7] = np.inf          # inf statistic: scale inf, codes 0
        x[4, :] = 0
        x[4, 9] = 6e-8            # max/7 underflows to a zero scale on a non-zero row
        x[5, :] *= 1e-4           # a subnormal-range row
    for qmax, clip in ((6, 1.0), (7, 1.0), (6, 0.9), (6, 0.5), (3, 1.0)):
        s_want = orc.sym_scales(x, clip)
        q_want = orc.sym_quant(x, s_want, qmax)
        q, s = hip.quantize_rows_sym(cases.t(x, dev), clip=clip, qmax=qmax)
        assert cases.bits_equal(s.cpu().numpy(), s_want)
        assert np.array_equal(q.cpu().numpy(), q_want)


@pytest.mark.parametrize("M,K", [(1, 4096), (16, 4096), (512, 4096), (4, 11008), (3, 28672), (9, 64)])
def test_quantize_rows_asym(hip, dev, M, K):
    _say("quantize_rows_asym", M, K)
    x = cases.acts_uniform(M, K, seed=40 + M + K)
    if M > 2:
        x[1, :] = cases.acts_normal(1, K, seed=5)[0]  # a signed row
    if M > 3:
        x[2, :] = 1.5  # max == min: scale 0
    if M > 8:
        x[3, :] = x[3, :] * 0.01 + 900.0   # large offset: zero point far above 480
        x[4, 3] = np.inf
        x[5, :] = -x[5, :]                 # all negative
    s_want, z_want = orc.asym_scales_zeros(x)
    q_want = orc.asym_quant(x, s_want, z_want)
    q, s, z = hip.quantize_rows_asym(cases.t(x, dev))
    assert cases.bits_equal(s.cpu().numpy(), s_want)
    assert cases.bits_equal(z.cpu().numpy(), z_want)
    assert np.array_equal(q.cpu().numpy(), q_want)


def test_quantize_rows_magnitude_sweep(hip, dev):
    """Rows of every magnitude binary16 holds, clip ratios on both sides of the point where the lower clamp starts to
    act (row maximum over scale = 8.5) and upper bounds below, at and above 7: the kernel decides per row which
    clamps it can leave out, and every such decision has to give the oracle's codes."""
    M, K = 4096, 64
    _say("quantize_rows magnitude sweep", M, K)
    rng = np.random.default_rng(77)
    mag = np.exp2(rng.uniform(-24.0, 15.9, (M, 1)))
    with np.errstate(over="ignore"):  # the largest rows overflow to inf here and there: those rows are cases too
        x = (rng.standard_normal((M, K)) * mag).astype(np.float16)
        x[::7] = np.round(x[::7] / mag[::7] * 3.0) * (mag[::7] / 3.0).astype(np.float16)  # many exact ties
    xt = cases.t(x, dev)
    for qmax, clip in ((6, 1.0), (7, 1.0), (7, 0.83), (7, 0.82), (6, 0.8), (7, 0.5), (2, 1.0), (7, 1.2)):
        s_want = orc.sym_scales(x, clip)
        q_want = orc.sym_quant(x, s_want, qmax)
        q, s = hip.quantize_rows_sym(xt, clip=clip, qmax=qmax)
        assert cases.bits_equal(s.cpu().numpy(), s_want), (qmax, clip)
        bad = np.argwhere(q.cpu().numpy() != q_want)
        assert bad.size == 0, f"qmax {qmax} clip {clip}: first mismatches (row, byte) {bad[:8]}"
    for shift in (0.0, 0.37, -2.5):
        with np.errstate(over="ignore", invalid="ignore"):
            xa = (x.astype(np.float32) + shift * mag).astype(np.float16)
        s_want, z_want = orc.asym_scales_zeros(xa)
        q_want = orc.asym_quant(xa, s_want, z_want)
        q, s, z = hip.quantize_rows_asym(cases.t(xa, dev))
        assert cases.bits_equal(s.cpu().numpy(), s_want), shift
        assert cases.bits_equal(z.cpu().numpy(), z_want), shift
        bad = np.argwhere(q.cpu().numpy() != q_want)
        assert bad.size == 0, f"shift {shift}: first mismatches (row, byte) {bad[:8]}"


# ---------------------------------------------------------------- GEMM
def _rand_packed(rng, rows, K):
    return rng.integers(0, 256, (rows, K // 2), dtype=np.uint8)


@pytest.mark.parametrize("M,N,K", [
    (1, 16, 64), (1, 4096, 4096), (4, 4096, 4096), (16, 11008, 4096), (16, 40, 128), (7, 33, 192),
    (17, 64, 64), (64, 64, 128), (65, 130, 192), (100, 257, 320), (128, 256, 4096), (300, 520, 1024),
    (2048, 4096, 256), (256, 4096, 11008), (130, 1000, 64), (16, 16, 8192), (2, 48, 28672), (7, 48, 28672),
    (9, 40000, 64), (16, 33000, 192), (12, 17000, 8192), (5, 100, 16384),
    # one to four rows: dot kernel (one row; two rows with K > 4096; up to four with K > 16384), skinny otherwise
    (2, 512, 8192), (2, 300, 4096), (3, 300, 20480), (4, 64, 28672), (3, 1000, 2048), (4, 520, 8192), (1, 77, 20480),
    # ring kernel: 17..64 rows (2, 3, 4 row blocks; several row groups when K is long) and long rows up to 16
    (17, 4096, 4096), (33, 300, 8192), (64, 520, 11008), (48, 4099, 1024), (40, 64, 16384), (16, 300, 11008),
    (9, 4096, 16384), (64, 11008, 4096), (50, 1000, 4160),
    # ring kernel with several row groups: 65..256 rows of a narrow or short problem
    (100, 1000, 4096), (200, 520, 8192), (90, 300, 11008), (256, 1024, 8192),
    # stream kernel on 64 x 128 tiles (one round of 64..256 of them), tiles that end inside M, N and K
    (128, 4096, 4096), (65, 4100, 320), (130, 8000, 4160), (200, 3000, 8192), (500, 4099, 448), (512, 4096, 1024),
    # and on 128 x 128 tiles (one round where 64 x 128 tiles need two)
    (700, 4000, 1024), (650, 4100, 1088),
])
def test_matmul_bit_exact(hip, dev, M, N, K):
    _say("matmul", M, N, K)
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a = _rand_packed(rng, M, K)
    b = _rand_packed(rng, N, K)
    want = orc.matmul_s4(a, b)
    got = hip.matmul(cases.t(a, dev), cases.t(b, dev)).cpu().numpy()
    bad = np.argwhere(got != want)
    assert bad.size == 0, f"{len(bad)} mismatches, first (m, n): {bad[:8]} got {got[tuple(bad[0])]} want {want[tuple(bad[0])]}"


def test_matmul_extremes(hip, dev):
    """all -8 x all -8 = 64*K; -8 x 7 = -56*K; one-hot rows select single products."""
    K = 4096
    a = np.full((32, K // 2), 0x88, np.uint8)
    b = np.full((48, K // 2), 0x88, np.uint8)
    got = hip.matmul(cases.t(a, dev), cases.t(b, dev)).cpu().numpy()
    assert np.all(got == 64 * K)
    b7 = np.full((48, K // 2), 0x77, np.uint8)
    got = hip.matmul(cases.t(a, dev), cases.t(b7, dev)).cpu().numpy()
    assert np.all(got == -56 * K)
    # one-hot: A row m has +1 at k = 37*m+5 only
    M, N = 24, 40
    aq = np.zeros((M, K), np.int8)
    for m in range(M):
        aq[m, 37 * m + 5] = 1
    rng = np.random.default_rng(3)
    bq = rng.integers(-8, 8, (N, K)).astype(np.int8)
    got = hip.matmul(cases.t(orc.pack_i4(aq), dev), cases.t(orc.pack_i4(bq), dev)).cpu().numpy()
    want = np.stack([bq[:, 37 * m + 5] for m in range(M)]).astype(np.int32)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- dequant + fused
def _epi_inputs(rng, M, N):
    sr = rng.uniform(0.01, 1.0, (M, 1)).astype(np.float16)
    zr = rng.integers(0, 16, (M, 1)).astype(np.float16)
    sc1 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    sc2 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    zc1 = rng.integers(0, 16, (N, 1)).astype(np.float16)
    zc2 = rng.integers(0, 16, (N, 1)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    return sr, zr, sc1, zc1, sc2, zc2, bias


@pytest.mark.parametrize("M,N", [(1, 16), (16, 4096), (33, 130), (7, 11), (512, 4096)])
def test_dequant_kernels(hip, dev, M, N):
    _say("dequant", M, N)
    rng = np.random.default_rng(M + N)
    acc = rng.integers(-70000, 70000, (M, N)).astype(np.int32)
    acc.flat[:8] = [65519, 65520, -65519, -65520, 2049, 2051, 0, -1]
    sr, zr, sc1, zc1, sc2, zc2, _ = _epi_inputs(rng, M, N)
    d = dev
    T = lambda a: cases.t(a, d)
    assert cases.bits_equal(hip.sym_dequant(T(acc), T(sr), T(sc1), 32).cpu().numpy(), orc.sym_dequant(acc, sr, sc1))
    assert cases.bits_equal(hip.sym_dual_dequant(T(acc), T(sr), T(sc1), T(sc2), 32).cpu().numpy(),
                            orc.sym_dual_dequant(acc, sr, sc1, sc2))
    assert cases.bits_equal(hip.asym_dequant(T(acc), T(sr), T(zr), T(sc1), T(zc1), 32).cpu().numpy(),
                            orc.asym_dequant(acc, sr, zr, sc1, zc1))
    assert cases.bits_equal(
        hip.asym_dual_dequant(T(acc), T(sr), T(zr), T(sc1), T(zc1), T(sc2), T(zc2), 32).cpu().numpy(),
        orc.asym_dual_dequant(acc, sr, zr, sc1, zc1, sc2, zc2))


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (16, 4096, 4096), (16, 50, 128), (100, 257, 320), (512, 4096, 4096),
                                   (130, 1000, 64),
                                   # the stream kernel at its three tile heights, aligned and ragged epilogues:
                                   # 64 rows (1024 x 4096, 900 x 4100), 32 rows (200 x 2051), 128 rows (1100 x 8200)
                                   (1024, 4096, 512), (900, 4100, 128), (200, 2051, 192), (1100, 8200, 320),
                                   # and on its 64 x 128 tiles
                                   (128, 4096, 512), (300, 3100, 320), (250, 8190, 384), (100, 4097, 1088),
                                   # and on its 128 x 128 tiles
                                   (700, 4000, 1024), (650, 4100, 1088),
                                   # the short-row kernel (K <= 256): whole-line and ragged epilogues, every step count
                                   (300, 1024, 64), (520, 2048, 256), (1000, 520, 192), (65, 4096, 128),
                                   # two to four rows on either decode kernel
                                   (2, 512, 8192), (3, 300, 20480), (4, 1000, 4096), (2, 300, 4096),
                                   # ring kernel
                                   (33, 300, 8192), (64, 520, 11008), (48, 4099, 1024), (16, 300, 11008), (20, 4096, 4096),
                                   (100, 1000, 4096), (200, 520, 8192)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_fused_forward_equals_unfused_and_oracle(hip, dev, M, N, K, with_bias):
    _say("fused", M, N, K, with_bias)
    rng = np.random.default_rng(M * 11 + N * 5 + K)
    a = _rand_packed(rng, M, K)
    b = _rand_packed(rng, N, K)
    sr, zr, sc1, zc1, sc2, zc2, bias = _epi_inputs(rng, M, N)
    acc = orc.matmul_s4(a, b)
    T = lambda v: cases.t(v, dev)
    tb = T(bias) if with_bias else None

    def fin(y):
        return orc.add_bias(y, bias) if with_bias else y

    got = hip.linear4bit_forward(hip.EPI_SYM, T(a), T(sr), None, T(b), T(sc1), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.sym_dequant(acc, sr, sc1)))
    got = hip.linear4bit_forward(hip.EPI_ASYM, T(a), T(sr), T(zr), T(b), T(sc1), T(zc1), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.asym_dequant(acc, sr, zr, sc1, zc1)))
    got = hip.linear4bit_forward(hip.EPI_SYM_DUAL, T(a), T(sr), None, T(b), T(sc1), None, T(sc2), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.sym_dual_dequant(acc, sr, sc1, sc2)))
    got = hip.linear4bit_forward(hip.EPI_ASYM_DUAL, T(a), T(sr), T(zr), T(b), T(sc1), T(zc1), T(sc2), T(zc2),
                                 bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.asym_dual_dequant(acc, sr, zr, sc1, zc1, sc2, zc2)))


@pytest.mark.parametrize("M,N,K,with_bias", [(4090, 4088, 4160, True), (4096, 4090, 4096, False)])
def test_stream_kernel_256_row_tiles(hip, dev, M, N, K, with_bias):
    """The stream kernel's 256 x 256 tiles (problems with at least one per CU): ragged last row tile, a last column
    tile that ends inside a 32-column fragment, an odd number of 64-element row segments, whole-line and
    per-element epilogues; int32 accumulators, the four reference epilogues and the row-sum one against the oracle
    over the whole output."""
    _say("256-row tiles", M, N, K, with_bias)
    assert hip.gemm_kernel_for(M, N, K) == 6 and hip.gemm_stream_tile_for(M, N, K) == 256256
    rng = np.random.default_rng(M + N + K)
    a = _rand_packed(rng, M, K)
    b = _rand_packed(rng, N, K)
    sr, zr, sc1, zc1, sc2, zc2, bias = _epi_inputs(rng, M, N)
    acc = orc.matmul_s4(a, b)
    T = lambda v: cases.t(v, dev)
    A, B = T(a), T(b)
    tb = T(bias) if with_bias else None
    fin = (lambda y: orc.add_bias(y, bias)) if with_bias else (lambda y: y)
    assert np.array_equal(hip.matmul(A, B).cpu().numpy(), acc)
    got = hip.linear4bit_forward(hip.EPI_SYM, A, T(sr), None, B, T(sc1), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.sym_dequant(acc, sr, sc1)))
    got = hip.linear4bit_forward(hip.EPI_ASYM, A, T(sr), T(zr), B, T(sc1), T(zc1), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.asym_dequant(acc, sr, zr, sc1, zc1)))
    got = hip.linear4bit_forward(hip.EPI_SYM_DUAL, A, T(sr), None, B, T(sc1), None, T(sc2), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.sym_dual_dequant(acc, sr, sc1, sc2)))
    got = hip.linear4bit_forward(hip.EPI_ASYM_DUAL, A, T(sr), T(zr), B, T(sc1), T(zc1), T(sc2), T(zc2), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.asym_dual_dequant(acc, sr, zr, sc1, zc1, sc2, zc2)))
    rs_row = rng.integers(-8 * K, 8 * K, (M,)).astype(np.int32)
    adj = rng.integers(-8 * K, 8 * K, (N,)).astype(np.int32)
    got = hip.linear4bit_forward_rowsum(A, T(sr), T(zr), T(rs_row), B, T(sc1), T(zc1), T(adj), tb).cpu().numpy()
    assert cases.bits_equal(got, orc.asym_rowsum_dequant(acc, sr, zr, rs_row, sc1, zc1, adj, bias if with_bias else None))
