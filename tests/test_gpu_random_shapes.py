"""Seeded random shapes through the C ABI: the hand-picked shapes of the other GPU tests sit on the
kernels' known boundaries; these draw M, N, K from log-uniform ranges (K a multiple of the path's
granule, M and N anything) so that a launch rule or a tail that nobody thought of still meets the oracle.
Bit-exact, as everywhere."""
import numpy as np
import pytest

from oracle import duq_oracle as orc
from tests import cases


@pytest.fixture(scope="module")
def hip(dev):
    from duqlinear4bitcuda_amd import _HIP
    return _HIP


def _draw(rng, n, k_granule, k_max, mn_max):
    out = []
    for _ in range(n):
        m = int(np.exp(rng.uniform(0, np.log(mn_max[0]))))
        nn = int(np.exp(rng.uniform(0, np.log(mn_max[1]))))
        k = k_granule * max(1, int(np.exp(rng.uniform(0, np.log(k_max // k_granule)))))
        # keep the oracle's float64 GEMM in seconds
        while m * nn * k > 3e9:
            nn = max(1, nn // 2)
        out.append((max(1, m), max(1, nn), k))
    return out


SHAPES4 = _draw(np.random.default_rng(2024), 28, 64, 16384, (1500, 9000))
# every other shape also fits the 6-bit float path (N % 16 == 0, K % 128 == 0)
SHAPES4 = [(m, -(-n // 16) * 16, -(-k // 128) * 128) if i % 2 else (m, n, k) for i, (m, n, k) in enumerate(SHAPES4)]
SHAPES8 = _draw(np.random.default_rng(2025), 24, 32, 8192, (1500, 9000))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", SHAPES4)
def test_random_shapes_4bit(hip, dev, M, N, K):
    print("4bit", M, N, K, flush=True)
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a = rng.integers(0, 256, (M, K // 2), dtype=np.uint8)
    b = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    sr = rng.uniform(0.01, 1.0, (M, 1)).astype(np.float16)
    zr = rng.integers(0, 16, (M, 1)).astype(np.float16)
    sc = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    zc = rng.integers(0, 16, (N, 1)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    T = lambda v: cases.t(v, dev)
    acc = orc.matmul_s4(a, b)
    assert np.array_equal(hip.matmul(T(a), T(b)).cpu().numpy(), acc)
    want_sym = orc.add_bias(orc.sym_dequant(acc, sr, sc), bias)
    want_asym = orc.asym_dequant(acc, sr, zr, sc, zc)
    got = hip.linear4bit_forward(hip.EPI_SYM, T(a), T(sr), None, T(b), T(sc), bias=T(bias)).cpu().numpy()
    assert cases.bits_equal(got, want_sym)
    got = hip.linear4bit_forward(hip.EPI_ASYM, T(a), T(sr), T(zr), T(b), T(sc), T(zc)).cpu().numpy()
    assert cases.bits_equal(got, want_asym)
    if K % 128 == 0 and N % 16 == 0:   # the same on the 6-bit float matrix path
        xs, ws = hip.activation_shadow_bf6(T(a)), hip.weight_shadow_bf6(T(b))
        got = hip.linear4bit_forward_bf6(hip.EPI_SYM, xs, T(sr), None, ws, T(sc), bias=T(bias)).cpu().numpy()
        assert cases.bits_equal(got, want_sym)
        got = hip.linear4bit_forward_bf6(hip.EPI_ASYM, xs, T(sr), T(zr), ws, T(sc), T(zc)).cpu().numpy()
        assert cases.bits_equal(got, want_asym)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", SHAPES8)
def test_random_shapes_8bit(hip, dev, M, N, K):
    print("8bit", M, N, K, flush=True)
    rng = np.random.default_rng(M * 5 + N * 11 + K)
    a = rng.integers(-128, 128, (M, K)).astype(np.int8)
    b = rng.integers(-128, 128, (N, K)).astype(np.int8)
    sr = rng.uniform(0.01, 1.0, (M, 1)).astype(np.float32)
    zr = np.rint(rng.uniform(-10, 126, (M, 1))).astype(np.float32)
    sc = rng.uniform(0.0001, 0.01, (N, 1)).astype(np.float32)
    zc = np.rint(rng.uniform(-60, 10, (N, 1))).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    T = lambda v: cases.t(v, dev)
    acc = orc.matmul_s8(a, b).astype(np.int32)
    assert np.array_equal(hip.matmul_8bit(T(a), T(b)).cpu().numpy(), acc)
    want = (orc.asym_dequant_hprec(acc, sr, zr, sc, zc) + bias[None, :]).astype(np.float32)
    got = hip.linear8bit_forward(T(a), T(sr), T(zr), T(b), T(sc), T(zc), T(bias)).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    got = hip.linear8bit_forward(T(a), T(sr), T(zr), hip.weight_tile_8bit(T(b)), T(sc), T(zc), T(bias),
                                 tiled_rows=N).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _draw_decode(rng, n):
    """Decode-sized shapes for the entry points that take binary16 rows: one launch or two depends on M, N and K
    together, so the draws spread over all three (a few rows, narrow to very wide layers, short to long rows)."""
    out = []
    for i in range(n):
        m = int(rng.integers(1, 18))
        nn = int(np.exp(rng.uniform(np.log(8), np.log(40000))))
        k = 64 * int(np.exp(rng.uniform(0, np.log(256))))
        while m * nn * k > 2e9:
            nn = max(1, nn // 2)
        out.append((m, nn, k, i % 6))
    return out


SHAPES_FP16IN = _draw_decode(np.random.default_rng(2026), 42)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K,mode", SHAPES_FP16IN)
def test_random_shapes_fp16_input(hip, dev, M, N, K, mode):
    """quantizer + GEMM + dequant from binary16 rows (duq_quantize_linear4bit_forward / ..._forward_asym), every
    epilogue mode, with a zero row and a row that holds an infinity now and then: the oracle's bits."""
    print("fp16-in", M, N, K, "mode", mode, "one launch" if hip.quantize_linear4bit_one_launch(M, N, K) else "two", flush=True)
    rng = np.random.default_rng(M * 13 + N * 3 + K + mode)
    x = (cases.acts_outliers if mode in (0, 2) else cases.acts_uniform)(M, K, seed=int(rng.integers(1 << 30)))
    if rng.random() < 0.3:
        x[rng.integers(M)] = 0
    if rng.random() < 0.2:
        x[rng.integers(M), rng.integers(K)] = np.float16(np.inf)
    wq = rng.integers(0, 256, (N, K // 2)).astype(np.uint8)
    s1 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    s2 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    z1 = rng.integers(-8, 8, (N, 1)).astype(np.float16)
    z2 = rng.integers(-8, 8, (N, 1)).astype(np.float16)
    a1 = rng.integers(-8 * K, 8 * K, (N,)).astype(np.int32)
    a2 = rng.integers(-8 * K, 8 * K, (N,)).astype(np.int32)
    bias = rng.standard_normal(N).astype(np.float16) if rng.random() < 0.5 else None
    T = lambda v: None if v is None else cases.t(v, dev)
    X = T(x)
    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        if mode == 0:
            clip, qmax = (1.0, 6) if rng.random() < 0.6 else (0.9, 7)
            got = hip.quantize_linear4bit_forward(X, T(wq), T(s1), None, T(bias), clip, qmax)
            want = orc.linear4bit_sq_forward(x, wq, s1, bias, clip, qmax)[0]
        elif mode == 2:
            got = hip.quantize_linear4bit_forward(X, T(wq), T(s1), T(s2), T(bias))
            want = orc.linear4bit_dusq_forward(x, wq, s1, s2, bias)[0]
        elif mode == 1:
            got = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM, X, T(wq), T(s1), T(z1 + 8), bias=T(bias))
            want = orc.linear4bit_asq_forward(x, wq, s1, z1 + 8, bias)[0]
        elif mode == 3:
            got = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM_DUAL, X, T(wq), T(s1), T(z1 + 8), T(s2), T(z2 + 8), bias=T(bias))
            want = orc.linear4bit_duasq_forward(x, wq, s1, z1 + 8, s2, z2 + 8, bias)[0]
        elif mode == 4:
            got = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM_ROWSUM, X, T(wq), T(s1), T(z1), None, None, T(a1), T(bias))
            want = orc.linear4bit_asq_rowsum_forward(x, wq, s1, z1, a1, bias)[0]
        else:
            got = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM_DUAL_ROWSUM, X, T(wq), T(s1), T(z1), T(s2), T(z2), T(a1),
                                                       T(bias), w_rowsum_adj_2=T(a2))
            want = orc.linear4bit_duasq_rowsum_forward(x, wq, s1, z1, s2, z2, a1, a2, bias)[0]
    assert cases.bits_equal(got.cpu().numpy().reshape(M, N), want)
