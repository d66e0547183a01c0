"""Asymmetric forward with exact zero-point correction (row sums).  The reference has no such
path, so parity is against the definition in include/duq_hip.h restated by the oracle; the
oracle itself is pinned here by the integer identity and by dequantize-then-matmul in float64
(a dropped term, a wrong sign or a transposed operand fails both)."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from tests import cases


def _ints(z):
    return np.rint(np.asarray(z, np.float64)).astype(np.int64)


# ------------------------------------------------------------------ oracle pins (CPU)
@pytest.mark.parametrize("M,N,K,seed", [(5, 7, 64, 0), (3, 4, 192, 1), (8, 2, 64, 2)])
def test_oracle_rowsum_identity_and_closed_form(M, N, K, seed):
    rng = np.random.default_rng(seed)
    x = (rng.random((M, K)) * 6 - (seed == 1) * 2).astype(np.float16)   # nonnegative skew; one case crosses zero
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    wq, ws, wz, adj = orc.weight_asym_shifted_from_linear(w)
    y, acc, qx, sx, zx, rx = orc.linear4bit_asq_rowsum_forward(x, wq, ws, wz, adj)

    # shifted storage == unshifted codes / zeros minus 8
    s0, z0 = orc.asym_scales_zeros(x)
    u = orc.asym_quant_values(x, s0, z0)
    cx = orc.unpack_i4(qx, signed=True).astype(np.int64)
    assert np.array_equal(cx, u.astype(np.int64) - 8)
    assert np.array_equal(orc.asym_quant(x, s0, z0) ^ 0x88, qx)
    assert np.array_equal(_ints(zx), _ints(z0) - 8) and np.array_equal(sx, s0)
    assert np.array_equal(rx, cx.sum(axis=1))

    # integer identity, term by term from a brute-force triple loop
    cw = orc.unpack_i4(wq, signed=True).astype(np.int64)
    zxi, zwi = _ints(zx).reshape(-1), _ints(wz).reshape(-1)
    want_corr = np.zeros((M, N), np.int64)
    for m in range(M):
        for n in range(N):
            want_corr[m, n] = sum(int(cx[m, k] - zxi[m]) * int(cw[n, k] - zwi[n]) for k in range(K))
    corr = acc.astype(np.int64) - zxi[:, None] * adj.astype(np.int64)[None, :] - zwi[None, :] * rx.astype(np.int64)[:, None]
    assert np.array_equal(corr, want_corr)

    # y is s_x * s_w * corr rounded: within one binary16 + one float32 rounding of the exact product
    exact = sx.astype(np.float64) * ws.astype(np.float64).reshape(1, -1) * want_corr
    assert np.all(np.abs(y.astype(np.float64) - exact) <= np.abs(exact) * (2.0 ** -11 + 2.0 ** -23) + 6e-8)
    # and it is the product of the dequantized operands
    ref = (sx.astype(np.float64) * (cx - zxi[:, None])) @ (ws.astype(np.float64) * (cw - zwi[:, None])).T
    assert np.allclose(exact, ref, rtol=1e-12, atol=0)

    # the point of the mode: close to the real product, where the reference-faithful path is not
    true = x.astype(np.float64) @ w.astype(np.float64).T
    err = np.abs(y.astype(np.float64) - true).max() / np.abs(true).max()
    y_ref_mode, *_ = orc.linear4bit_asq_forward(x, *orc.weight_asym_from_linear(w))
    err_ref_mode = np.abs(y_ref_mode.astype(np.float64) - true).max() / np.abs(true).max()
    assert err < 0.25 and err < err_ref_mode


def test_oracle_rowsum_bias_and_wrapping():
    acc = np.array([[2 ** 31 - 5, -7]], np.int32)
    sr = np.array([[0.5]], np.float16); zr = np.array([[-3.0]], np.float16); rr = np.array([10], np.int32)
    sc = np.array([0.25, 2.0], np.float16); zc = np.array([1.0, -2.0], np.float16); ac = np.array([4, -6], np.int32)
    y = orc.asym_rowsum_dequant(acc, sr, zr, rr, sc, zc, ac, bias=np.array([1.0, 0.5], np.float16))
    # column 0: 2^31-5 + 12 - 10 wraps to -2^31 - 3 + ... ; computed by hand in Python integers
    c0 = ((2 ** 31 - 5) - (-3) * 4 - 1 * 10 + 2 ** 31) % 2 ** 32 - 2 ** 31
    c1 = -7 - (-3) * (-6) - (-2) * 10
    want0 = np.float16(np.float32(c0) * np.float32(0.125)) + np.float16(1.0)
    want1 = np.float16(np.float16(np.float32(c1) * np.float32(1.0)) + np.float16(0.5))
    assert y[0, 1] == want1 and (y[0, 0] == want0 or (np.isinf(y[0, 0]) and np.isinf(want0)))
    assert c1 == -5


@pytest.mark.parametrize("M,N,K,seed", [(5, 7, 64, 0), (3, 4, 192, 1), (8, 2, 64, 2)])
def test_oracle_dual_rowsum_identity_and_closed_form(M, N, K, seed):
    """Dual-uniform row-sum mode: the two corrections are the brute-force sums over their own k ranges, y is the
    float64 product of the dequantized operands up to the stated roundings, and the weight preparation quantizes
    each range with its own true min/max."""
    rng = np.random.default_rng(seed)
    x = (rng.random((M, K)) * 6 - (seed == 1) * 2).astype(np.float16)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float16)
    w[:, :10] *= 8                      # the first ten input columns on another scale: what the layer is for
    wq, s1, z1, s2, z2, a1, a2 = orc.weight_asym_dual_shifted_from_linear(w)
    y, acc, qx, sx, zx, rx = orc.linear4bit_duasq_rowsum_forward(x, wq, s1, z1, s2, z2, a1, a2)
    cx = orc.unpack_i4(qx, signed=True).astype(np.int64)
    cw = orc.unpack_i4(wq, signed=True).astype(np.int64)
    zxi, z1i, z2i = _ints(zx).reshape(-1), _ints(z1).reshape(-1), _ints(z2).reshape(-1)
    # weight preparation: every range is asym_quant_shifted of that range alone
    for lo, hi, s, z, a in ((0, 10, s1, z1, a1), (10, K, s2, z2, a2)):
        q_r, s_r, z_r, _ = orc.asym_quant_shifted(np.ascontiguousarray(w[:, lo:hi]))
        assert np.array_equal(orc.unpack_i4(q_r, signed=True), cw[:, lo:hi]) and np.array_equal(s_r, s) and np.array_equal(z_r, z)
        assert np.array_equal(a, cw[:, lo:hi].sum(axis=1) - (hi - lo) * _ints(z).reshape(-1))
    # the two corrections, term by term from brute-force loops
    want_l = np.zeros((M, N), np.int64)
    want_r = np.zeros((M, N), np.int64)
    for m in range(M):
        for n in range(N):
            want_l[m, n] = sum(int(cx[m, k] - zxi[m]) * int(cw[n, k] - z1i[n]) for k in range(10))
            want_r[m, n] = sum(int(cx[m, k] - zxi[m]) * int(cw[n, k] - z2i[n]) for k in range(10, K))
    acc_l = cx[:, :10] @ cw[:, :10].T
    rxl = cx[:, :10].sum(axis=1)
    corr_l = acc_l - zxi[:, None] * a1.astype(np.int64)[None, :] - z1i[None, :] * rxl[:, None]
    corr_r = (acc.astype(np.int64) - acc_l) - zxi[:, None] * a2.astype(np.int64)[None, :] - z2i[None, :] * (rx.astype(np.int64) - rxl)[:, None]
    assert np.array_equal(corr_l, want_l) and np.array_equal(corr_r, want_r)
    # y against the exact value: two float32 products, one float32 sum, one binary16 rounding
    sx64 = sx.astype(np.float64)
    e1 = sx64 * s1.astype(np.float64).reshape(1, -1) * want_l
    e2 = sx64 * s2.astype(np.float64).reshape(1, -1) * want_r
    exact = e1 + e2
    bound = (np.abs(e1) + np.abs(e2)) * 2.0 ** -22 + np.abs(exact) * 2.0 ** -11 + 6e-8
    assert np.all(np.abs(y.astype(np.float64) - exact) <= bound)
    # exact is the product of the dequantized operands
    wd = np.concatenate([s1.astype(np.float64) * (cw[:, :10] - z1i[:, None]), s2.astype(np.float64) * (cw[:, 10:] - z2i[:, None])], axis=1)
    ref = (sx64 * (cx - zxi[:, None])) @ wd.T
    assert np.allclose(exact, ref, rtol=1e-12, atol=1e-300)
    # the point of the mode: close to the real product, where the reference's epilogue is not
    true = x.astype(np.float64) @ w.astype(np.float64).T
    err = np.abs(y.astype(np.float64) - true).max() / np.abs(true).max()
    assert err < 0.25
    # swapping the two pairs (a plausible mistake) must show
    y_swapped = orc.asym_dual_rowsum_dequant(acc, qx, sx, zx, rx, wq, s2, z2, s1, z1, a2, a1)
    assert not np.array_equal(y_swapped, y)


def test_oracle_dual_rowsum_hand_case():
    """One row, one column, K = 64, every quantity small enough to do by hand."""
    cxv = np.zeros(64, np.int8); cwv = np.zeros(64, np.int8)
    cxv[:12] = [1, -2, 3, 0, 7, -8, 1, 1, 2, -3, 5, 4]
    cwv[:12] = [2, 2, -1, 5, 1, 1, 0, -4, 3, 3, -2, 6]
    qx, qw = orc.pack_i4(cxv[None, :], sym=True), orc.pack_i4(cwv[None, :], sym=True)
    acc = orc.matmul_s4(qx, qw)
    acc_l = 2 - 4 - 3 + 0 + 7 - 8 + 0 - 4 + 6 - 9          # first ten products
    assert acc[0, 0] == acc_l + (-10 + 24)
    rx = int(cxv.sum()); rxl = 1 - 2 + 3 + 0 + 7 - 8 + 1 + 1 + 2 - 3
    zx, z1, z2 = -8, 3, -2
    a1 = int(cwv[:10].sum()) - 10 * z1
    a2 = int(cwv[10:].sum()) - 54 * z2
    corr_l = acc_l - zx * a1 - z1 * rxl
    corr_r = 14 - zx * a2 - z2 * (rx - rxl)
    H = lambda v: np.array([[v]], np.float16)
    y = orc.asym_dual_rowsum_dequant(acc, qx, H(0.5), H(zx), np.array([rx], np.int32), qw, H(0.25), H(z1), H(2.0), H(z2),
                                     np.array([a1], np.int32), np.array([a2], np.int32), bias=np.array([1.5], np.float16))
    want = np.float16(np.float16(np.float32(corr_l) * np.float32(0.125) + np.float32(corr_r) * np.float32(1.0)) + np.float16(1.5))
    assert y[0, 0] == want
    assert (corr_l, corr_r) == (acc_l + 8 * a1 - 3 * rxl, 14 + 8 * a2 + 2 * (rx - rxl))


def test_abi_validation_rowsum_entries():
    from duqlinear4bitcuda_amd import _lib
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    P = (ctypes.addressof(buf) + 15) & ~15
    assert lib.duq_quantize_rows_asym_shifted(P, 2, 64, P, P, P, None, None) == -1
    assert lib.duq_quantize_rows_asym_shifted(P, 2, 48, P, P, P, P, None) == -2
    assert lib.duq_quantize_rows_asym_shifted(P, 0, 64, None, None, None, None, None) == 0
    assert lib.duq_linear4bit_forward_rowsum(P, P, P, None, P, P, P, P, None, 4, 4, 64, P, None) == -1
    assert lib.duq_linear4bit_forward_rowsum(P, P, P, P, P, P, P, P, None, 4, 4, 96, P, None) == -3
    assert lib.duq_asym_rowsum_dequant_host(P, P, P, P, P, P, None, None, 4, 4, P, None) == -1
    dual = lambda *a: lib.duq_asym_dual_rowsum_dequant_host(*a)
    assert dual(P, P, P, P, P, P, P, P, P, P, P, None, None, 4, 4, 64, P, None) == -1
    assert dual(P, P, P, P, P, P, P, P, P, P, P, P, None, 4, 4, 96, P, None) == -3
    assert dual(P, P + 8, P, P, P, P, P, P, P, P, P, P, None, 4, 4, 64, P, None) == -5
    assert dual(None, None, None, None, None, None, None, None, None, None, None, None, None, 0, 4, 64, None, None) == 0


# ------------------------------------------------------------------ GPU parity
@pytest.fixture(scope="module")
def hip(dev):
    from duqlinear4bitcuda_amd import _HIP
    return _HIP


@pytest.mark.gpu
@pytest.mark.parametrize("M,K", [(1, 64), (16, 4096), (300, 1024), (2048, 4096), (3, 11008), (2, 66048), (40, 32)])
def test_gpu_quantize_rows_asym_shifted(hip, dev, M, K):
    print("asym_shifted", M, K, flush=True)
    x = cases.acts_uniform(M, K, seed=M + K) if K % 3 else cases.acts_outliers(M, K, seed=M + K)
    wq, ws, wz, wr = orc.asym_quant_shifted(x)
    q, s, z, r = hip.quantize_rows_asym_shifted(cases.t(x, dev))
    assert np.array_equal(q.cpu().numpy(), wq)
    assert cases.bits_equal(s.cpu().numpy(), ws) and cases.bits_equal(z.cpu().numpy(), wz)
    assert np.array_equal(r.cpu().numpy(), wr)
    # the unshifted kernel still gives the unshifted form
    q0, s0, z0 = hip.quantize_rows_asym(cases.t(x, dev))
    assert np.array_equal(q0.cpu().numpy() ^ 0x88, wq)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (4, 1000, 512), (16, 4096, 4096), (9, 300, 8192), (48, 96, 256),
                                   (100, 257, 320), (512, 4096, 4096), (300, 1000, 4160), (2048, 4096, 1024),
                                   (900, 4100, 128), (200, 2051, 192), (48, 4099, 1024), (33, 300, 8192), (12, 300, 11008),
                                   (520, 2048, 256), (300, 1024, 64)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_gpu_rowsum_forward(hip, dev, M, N, K, with_bias):
    """Every GEMM kernel family (dot, skinny, tile, stream; aligned and ragged epilogues) in row-sum mode:
    fused == unfused == oracle, bit for bit."""
    print("rowsum forward", M, N, K, with_bias, flush=True)
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    x = cases.acts_uniform(M, K, seed=M + N + K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    wq, ws, wz, adj = orc.weight_asym_shifted_from_linear(w)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float16) if with_bias else None
    want, acc, qx, sx, zx, rx = orc.linear4bit_asq_rowsum_forward(x, wq, ws, wz, adj, bias)
    T = lambda v: cases.t(v, dev)
    q, s, z, r = hip.quantize_rows_asym_shifted(T(x))
    got = hip.linear4bit_forward_rowsum(q, s, z, r, T(wq), T(ws), T(wz), T(adj), None if bias is None else T(bias))
    assert cases.bits_equal(got.cpu().numpy(), want)
    acc_gpu = hip.matmul(q, T(wq))
    assert np.array_equal(acc_gpu.cpu().numpy(), acc)
    unfused = hip.asym_rowsum_dequant(acc_gpu, s, z, r, T(ws), T(wz), T(adj), None if bias is None else T(bias))
    assert cases.bits_equal(unfused.cpu().numpy(), want)


@pytest.mark.gpu
def test_gpu_rowsum_module_config4(dev):
    """Config 4 (M=512, K=N=4096, activations ~U[0,6]) through the module: weights prepared on the
    device, forward equals the oracle, and the result is close to the fp16 layer it replaces."""
    from duqlinear4bitcuda_amd.nn import Linear4bitASQRowSum
    M, K, N = 512, 4096, 4096
    x = cases.acts_uniform(M, K, seed=4)
    g = torch.Generator().manual_seed(44)
    lin = torch.nn.Linear(K, N, bias=True).half()
    with torch.no_grad():
        lin.weight.copy_((torch.randn(N, K, generator=g) * 0.02).half())
        lin.bias.copy_(torch.randn(N, generator=g).half())
    mod = Linear4bitASQRowSum.from_linear(lin.to(dev))
    w = lin.weight.detach().cpu().numpy()
    wq, ws, wz, adj = orc.weight_asym_shifted_from_linear(w)
    assert np.array_equal(mod.weight.cpu().numpy(), wq)
    assert cases.bits_equal(mod.weight_scales.cpu().numpy(), ws) and cases.bits_equal(mod.weight_zeros.cpu().numpy(), wz)
    assert np.array_equal(mod.weight_rowsum.cpu().numpy(), adj)
    y = mod(cases.t(x, dev).view(2, 256, K))
    assert y.shape == (2, 256, N)
    want, *_ = orc.linear4bit_asq_rowsum_forward(x, wq, ws, wz, adj, lin.bias.detach().cpu().numpy())
    assert cases.bits_equal(y.view(M, N).cpu().numpy(), want)
    mod.fused = False
    assert cases.bits_equal(mod(cases.t(x, dev)).cpu().numpy(), want)
    true = x.astype(np.float64) @ w.astype(np.float64).T + lin.bias.detach().cpu().numpy().astype(np.float64)
    rel = np.linalg.norm(want.astype(np.float64) - true) / np.linalg.norm(true)
    y_ref_mode, *_ = orc.linear4bit_asq_forward(x, *orc.weight_asym_from_linear(w), bias=lin.bias.detach().cpu().numpy())
    rel_ref_mode = np.linalg.norm(y_ref_mode.astype(np.float64) - true) / np.linalg.norm(true)
    assert rel < 0.25 and rel < 0.5 * rel_ref_mode, (rel, rel_ref_mode)  # 4-bit x 4-bit noise, not a broken correction


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(128, 4096, 512), (300, 3104, 320), (700, 4000, 1024), (1024, 4096, 320), (65, 8192, 448),
                                   (1, 64, 64), (7, 130, 128), (48, 1000, 256), (300, 1027, 320), (512, 4096, 4096),
                                   (33, 4100, 1024), (2050, 96, 64)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_gpu_dual_rowsum_dequant(hip, dev, M, N, K, with_bias):
    """The dual-uniform row-sum epilogue through the C ABI against the oracle: aligned and ragged widths, more
    than one column block, more rows than one row group."""
    print("dual rowsum", M, N, K, with_bias, flush=True)
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    x = cases.acts_uniform(M, K, seed=M + N + K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    w[:, :10] *= 6
    wq, s1, z1, s2, z2, a1, a2 = orc.weight_asym_dual_shifted_from_linear(w)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float16) if with_bias else None
    want, acc, qx, sx, zx, rx = orc.linear4bit_duasq_rowsum_forward(x, wq, s1, z1, s2, z2, a1, a2, bias)
    T = lambda v: cases.t(v, dev)
    q, s, z, r = hip.quantize_rows_asym_shifted(T(x))
    acc_gpu = hip.matmul(q, T(wq))
    assert np.array_equal(acc_gpu.cpu().numpy(), acc)
    got = hip.asym_dual_rowsum_dequant(acc_gpu, q, s, z, r, T(wq), T(s1), T(z1), T(s2), T(z2), T(a1), T(a2),
                                       None if bias is None else T(bias))
    assert cases.bits_equal(got.cpu().numpy(), want)
    # GEMM + epilogue through one entry point (one launch where the GEMM kernel of the shape applies it itself)
    got = hip.linear4bit_forward_dual_rowsum(q, s, z, r, T(wq), T(s1), T(z1), T(s2), T(z2), T(a1), T(a2),
                                             None if bias is None else T(bias))
    assert cases.bits_equal(got.cpu().numpy(), want)


@pytest.mark.gpu
def test_gpu_dual_rowsum_wide_factors(hip, dev):
    """Row-sum terms outside the signed 24-bit range (no genuine layer has them; the arrays are inputs): the fused
    kernel leaves its 24-bit multiplier path and still gives the oracle's wrapping 32-bit arithmetic, like the
    stand-alone epilogue."""
    M, N, K = 128, 4096, 512
    print("dual rowsum wide factors", M, N, K, flush=True)
    rng = np.random.default_rng(99)
    x = cases.acts_uniform(M, K, seed=7)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    wq, s1, z1, s2, z2, a1, a2 = orc.weight_asym_dual_shifted_from_linear(w)
    T = lambda v: cases.t(v, dev)
    q, s, z, r = hip.quantize_rows_asym_shifted(T(x))
    acc = hip.matmul(q, T(wq))
    for which in ("adj", "rowsum"):
        a1w, a2w, rw = a1.copy(), a2.copy(), r.cpu().numpy().copy()
        if which == "adj":
            a1w[5] = 2 ** 30 + 12345
            a2w[4000] = -(2 ** 29) - 7
        else:
            rw[77] = 2 ** 31 - 5
        want = orc.asym_dual_rowsum_dequant(acc.cpu().numpy(), q.cpu().numpy(), s.cpu().numpy(), z.cpu().numpy(), rw, wq,
                                            s1, z1, s2, z2, a1w, a2w)
        got = hip.linear4bit_forward_dual_rowsum(q, s, z, T(rw), T(wq), T(s1), T(z1), T(s2), T(z2), T(a1w), T(a2w))
        assert cases.bits_equal(got.cpu().numpy(), want), which
        got = hip.asym_dual_rowsum_dequant(acc, q, s, z, T(rw), T(wq), T(s1), T(z1), T(s2), T(z2), T(a1w), T(a2w))
        assert cases.bits_equal(got.cpu().numpy(), want), which


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(512, 4096, 4096), (100, 4096, 512), (300, 3104, 384), (2048, 1024, 1024), (70, 8192, 128),
                                   (1100, 4096, 256), (200, 512, 640)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_gpu_dual_rowsum_on_the_6bit_float_path(hip, dev, M, N, K, with_bias):
    """The dual-uniform row-sum epilogue inside the 6-bit float GEMM (128-, 64-row and 64 x 128 tiles, ragged M, N
    ending inside a tile, one chunk and several) against the oracle, and row-sum terms outside the signed 24-bit
    range (the kernel then leaves its 24-bit multiplier)."""
    print("dual rowsum fp6", M, N, K, with_bias, flush=True)
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    x = cases.acts_uniform(M, K, seed=M + N + K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    w[:, :10] *= 6
    wq, s1, z1, s2, z2, a1, a2 = orc.weight_asym_dual_shifted_from_linear(w)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float16) if with_bias else None
    want, acc, qx, sx, zx, rx = orc.linear4bit_duasq_rowsum_forward(x, wq, s1, z1, s2, z2, a1, a2, bias)
    T = lambda v: cases.t(v, dev)
    q, b6, s, z, r = hip.quantize_rows_asym_bf6(T(x), shifted=True, with_q=True)
    assert np.array_equal(q.cpu().numpy(), qx) and np.array_equal(r.cpu().numpy(), rx)
    W = T(wq)
    W6 = hip.weight_shadow_bf6(W)
    B = None if bias is None else T(bias)
    got = hip.linear4bit_forward_dual_rowsum_bf6(b6, q, s, z, r, W6, W, T(s1), T(z1), T(s2), T(z2), T(a1), T(a2), B)
    assert cases.bits_equal(got.cpu().numpy(), want)
    if with_bias and M <= 512:
        a1w, a2w, rw = a1.copy(), a2.copy(), rx.copy()
        a1w[5] = 2 ** 30 + 12345
        a2w[N - 3] = -(2 ** 29) - 7
        rw[M // 2] = 2 ** 31 - 5
        want = orc.asym_dual_rowsum_dequant(acc, qx, sx, zx, rw, wq, s1, z1, s2, z2, a1w, a2w, bias)
        got = hip.linear4bit_forward_dual_rowsum_bf6(b6, q, s, z, T(rw), W6, W, T(s1), T(z1), T(s2), T(z2), T(a1w), T(a2w), B)
        assert cases.bits_equal(got.cpu().numpy(), want)


def test_dual_rowsum_fused_shapes_and_validation():
    """Which shapes the fused entry point runs as one launch (no workspace), and its argument checks."""
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    ws = lib.duq_linear4bit_dual_rowsum_workspace_bytes
    assert ws(512, 4096, 4096) == 0 and ws(128, 4096, 512) == 0 and ws(2048, 4096, 4096) == 0 and ws(700, 4000, 1024) == 0
    assert ws(16, 4096, 4096) == 0 and ws(1, 64, 64) == 0 and ws(64, 11008, 4096) == 0   # decode kernels apply it too
    assert ws(100, 1000, 4096) == 100 * 1000 * 4    # ring kernel
    assert ws(300, 1028, 320) == 300 * 1028 * 4     # N % 8 != 0
    assert ws(512, 4096, 256) == 512 * 4096 * 4     # short rows
    assert ws(0, 4096, 4096) == 0
    P = 0x1000
    f = lib.duq_linear4bit_forward_dual_rowsum
    args = lambda M, N, K, y=P, w=None, nb=0: (P, P, P, P, P, P, P, P, P, P, P, None, M, N, K, y, w, nb, None)
    assert f(*args(100, 64, 100)) == -3                      # K % 64
    assert f(*args(100, 64, 128, y=None)) == -1
    assert f(*args(100, 64, 128, y=P + 2)) == -5
    assert f(*args(100, 64, 128)) == -1                      # needs a workspace
    assert f(*args(100, 64, 128, w=P, nb=100)) == -2         # too small
    assert f(*args(0, 64, 128)) == 0


@pytest.mark.gpu
def test_gpu_dual_rowsum_module_config4(dev):
    """Config 4 (M=512, K=N=4096, activations ~U[0,6]) through LinearQuant4bitDUASQRowSum: weights prepared on the
    device equal the oracle's, the forward equals the oracle, and the result is close to the fp16 layer it
    replaces, where the reference's dual-uniform epilogue is not."""
    from duqlinear4bitcuda_amd.nn import LinearQuant4bitDUASQRowSum
    M, K, N = 512, 4096, 4096
    x = cases.acts_uniform(M, K, seed=4)
    g = torch.Generator().manual_seed(45)
    lin = torch.nn.Linear(K, N, bias=True).half()
    with torch.no_grad():
        wt = torch.randn(N, K, generator=g) * 0.02
        wt[:, :10] *= 6                                  # outlier input channels in the first range
        lin.weight.copy_(wt.half())
        lin.bias.copy_(torch.randn(N, generator=g).half())
    mod = LinearQuant4bitDUASQRowSum.from_linear(lin.to(dev))
    w = lin.weight.detach().cpu().numpy()
    wq, s1, z1, s2, z2, a1, a2 = orc.weight_asym_dual_shifted_from_linear(w)
    assert np.array_equal(mod.weight.cpu().numpy(), wq)
    for name, want in (("weight_scales_1", s1), ("weight_zeros_1", z1), ("weight_scales_2", s2), ("weight_zeros_2", z2)):
        assert cases.bits_equal(getattr(mod, name).cpu().numpy(), want), name
    assert np.array_equal(mod.weight_rowsum_1.cpu().numpy(), a1) and np.array_equal(mod.weight_rowsum_2.cpu().numpy(), a2)
    y = mod(cases.t(x, dev).view(2, 256, K))
    assert y.shape == (2, 256, N)
    b = lin.bias.detach().cpu().numpy()
    want, *_ = orc.linear4bit_duasq_rowsum_forward(x, wq, s1, z1, s2, z2, a1, a2, b)
    assert cases.bits_equal(y.view(M, N).cpu().numpy(), want)
    true = x.astype(np.float64) @ w.astype(np.float64).T + b.astype(np.float64)
    rel = np.linalg.norm(want.astype(np.float64) - true) / np.linalg.norm(true)
    # the reference's layer on the same weights (its own preparation and epilogue)
    from duqlinear4bitcuda_amd.nn import LinearQuant4bitDUASQ
    ref_mod = LinearQuant4bitDUASQ.from_linear(lin.cpu()).to(dev)
    y_ref = ref_mod(cases.t(x, dev)).float().cpu().numpy().astype(np.float64)
    rel_ref = np.linalg.norm(y_ref - true) / np.linalg.norm(true)
    print("relative error: dual row-sum", rel, "reference dual epilogue", rel_ref, flush=True)
    assert rel < 0.25 and rel < 0.5 * rel_ref, (rel, rel_ref)
    # state_dict round trip
    other = LinearQuant4bitDUASQRowSum(K, N, bias=True).to(dev)
    other.load_state_dict(mod.state_dict())
    assert torch.equal(other(cases.t(x, dev)).view(torch.int16), y.view(M, N).view(torch.int16))
    # the same layer on the 6-bit float matrix path: same bits
    other.enable_fp6()
    assert other._fp6_wanted(M)
    assert torch.equal(other(cases.t(x, dev)).view(torch.int16), y.view(M, N).view(torch.int16))
