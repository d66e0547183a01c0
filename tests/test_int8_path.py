"""The 8-bit asymmetric layer (LinearQuant8bitASQ of the reference): float32 activations ->
int8 codes -> int8 x int8 GEMM -> float32 dequant.  CPU tests pin the oracle's restatement by
hand-computed cases, exact rational arithmetic with one explicit rounding per operator, brute
force and torch's CPU operators (an independent implementation of the same IEEE operations);
GPU tests compare the HIP kernels, through the C ABI, bit for bit with the oracle."""
import ctypes
from fractions import Fraction

import numpy as np
import pytest

from oracle import duq_oracle as orc

F32 = np.float32


# ------------------------------------------------------------------ helpers for the pins
def rn_f32(fr: Fraction) -> float:
    """Exact rational -> nearest binary32 (ties to even), normal range only."""
    if fr == 0:
        return 0.0
    sign = -1 if fr < 0 else 1
    fr = abs(fr)
    e = 0
    while fr >= 2 ** 24:
        fr /= 2
        e += 1
    while fr < 2 ** 23:
        fr *= 2
        e -= 1
    n, rem = divmod(fr.numerator, fr.denominator)
    twice = 2 * rem
    if twice > fr.denominator or (twice == fr.denominator and n % 2 == 1):
        n += 1
    assert -126 - 23 <= e <= 127 - 23
    return sign * float(n) * 2.0 ** e


def test_rn_f32_helper_agrees_with_numpy_on_exact_doubles():
    rng = np.random.default_rng(1)
    for v in rng.standard_normal(200) * 10.0 ** rng.integers(-5, 6, 200):
        assert rn_f32(Fraction(float(v))) == float(F32(v))
    assert rn_f32(Fraction(2 ** 24 + 1)) == float(2 ** 24)          # tie -> even
    assert rn_f32(Fraction(2 ** 24 + 3)) == float(2 ** 24 + 4)


# ------------------------------------------------------------------ oracle pins (CPU)
def test_asym_quant_8bit_hand_cases():
    def q(x, s, z):
        return int(orc.asym_quant_8bit(np.array([[x]], F32), np.array([s], F32), np.array([z], F32))[0, 0])

    assert q(5.0, 1.0, 0.0) == 5 and q(5.0, 0.5, 3.0) == 13
    assert q(-4.0, 1.0, 3.0) == 0 and q(200.0, 1.0, 0.0) == 126              # clamp to [0, 126]
    assert q(2.5, 1.0, 0.0) == 2 and q(3.5, 1.0, 0.0) == 4                   # ties to even
    # the quotient passes through binary16 (spacing 1/16 in [64, 128)): 101.49 -> 101.5 -> 102; directly, 101
    assert q(101.49, 1.0, 0.0) == 102
    # spacing 1/512 in [2, 4): 3.4995 -> 3.5 -> 4; directly, 3
    assert q(3.4995, 1.0, 0.0) == 4
    # the zero point passes through binary16 too: 2049 is a tie between 2048 and 2050 -> 2048
    assert q(-2000.0, 1.0, 2049.0) == 48
    # overflow of binary16 -> inf -> INT_MAX; the int add wraps
    assert q(1e30, 1.0, 0.0) == 126 and q(1e30, 1.0, 5.0) == 0 and q(-1e30, 1.0, 5.0) == 0
    assert q(70000.0, 1.0, 0.0) == 126 and q(65519.0, 1.0, -65504.0) == 0    # 65519 -> 65504 (no overflow yet)
    assert q(float("nan"), 1.0, 7.0) == 7                                    # NaN -> 0
    out = orc.asym_quant_8bit(np.zeros((2, 3), F32), np.ones(2, F32), np.zeros(2, F32))
    assert out.dtype == np.int8 and out.shape == (2, 3)


def test_asym_quant_8bit_against_torch_cpu():
    import torch
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((37, 300)) * 3).astype(F32)
    s, z = orc.asym8_scales_zeros(x)
    got = orc.asym_quant_8bit(x, s, z)
    xt, st, zt = torch.from_numpy(x), torch.from_numpy(s), torch.from_numpy(z)
    qi = (xt / st).to(torch.float16).to(torch.float32).round().to(torch.int64)
    zi = zt.to(torch.float16).to(torch.float32).round().to(torch.int64)
    want = torch.clamp(qi + zi, 0, 126).to(torch.int8).numpy()
    assert np.array_equal(got, want)
    assert got.min() == 0 and got.max() == 126


def test_asym8_scales_zeros_hand_and_torch():
    import torch
    s, z = orc.asym8_scales_zeros(np.array([[-1.0, 0.0, 3.0]], F32))
    assert s.shape == z.shape == (1, 1) and s.dtype == z.dtype == F32
    assert abs(float(s[0, 0]) - 4 / 127) < 1e-8 and float(z[0, 0]) == 32.0      # 1 / (4/127) = 31.75
    rng = np.random.default_rng(3)
    x = (rng.standard_normal((50, 129)) * rng.uniform(0.01, 50, (50, 1))).astype(F32)
    # the quotient form is what torch computes on a CPU
    s, z = orc.asym8_scales_zeros(x, device_division=False)
    xt = torch.from_numpy(x)
    lo, hi = xt.min(dim=-1, keepdim=True)[0], xt.max(dim=-1, keepdim=True)[0]
    st = (hi - lo) / 127
    zt = (-lo / st).round()
    assert np.array_equal(s, st.numpy()) and np.array_equal(z, zt.numpy())
    # both forms in exact rational arithmetic, one rounding per operator; the device form multiplies by
    # float32(1/127) (the GPU test compares it with torch's own result on the device)
    inv = rn_f32(Fraction(1, 127))
    assert inv == float(F32(1.0) / F32(127.0))
    sd, zd = orc.asym8_scales_zeros(x)
    differ = 0
    for r in range(50):
        lo_f, hi_f = Fraction(float(x[r].min())), Fraction(float(x[r].max()))
        d = Fraction(rn_f32(hi_f - lo_f))
        assert float(s[r, 0]) == rn_f32(d / 127)
        assert float(sd[r, 0]) == rn_f32(d * Fraction(inv))
        assert float(zd[r, 0]) == float(np.rint(rn_f32(-lo_f / Fraction(float(sd[r, 0])))))
        differ += float(s[r, 0]) != float(sd[r, 0])
    assert 0 < differ < 50       # the two forms are not the same function


def test_matmul_s8_brute_force_and_wrap():
    rng = np.random.default_rng(4)
    a = rng.integers(-128, 128, (3, 40)).astype(np.int8)
    b = rng.integers(-128, 128, (5, 40)).astype(np.int8)
    want = [[sum(int(a[m, k]) * int(b[n, k]) for k in range(40)) for n in range(5)] for m in range(3)]
    assert np.array_equal(orc.matmul_s8(a, b), np.array(want))
    a[:] = -128
    b[:] = -128
    assert np.all(orc.matmul_s8(a, b) == 40 * 16384)
    # 2^17 products of 2^14 reach 2^31, which wraps to -2^31 in the int32 accumulator
    big = np.full((1, 1 << 17), -128, np.int8)
    assert int(orc.matmul_s8(big, big)[0, 0]) == -(1 << 31)
    # not symmetric in its operands' shapes: A is [M,K], B is [N,K]
    assert orc.matmul_s8(np.ones((2, 32), np.int8), np.ones((7, 32), np.int8)).shape == (2, 7)


def test_asym_dequant_hprec_exact_rational():
    rng = np.random.default_rng(5)
    rows, cols = 6, 9
    acc = rng.integers(-2 ** 20, 2 ** 20, (rows, cols)).astype(np.int32)
    acc[0, 0] = 2 ** 31 - 1      # float(acc) itself rounds
    acc[1, 1] = -(2 ** 24) - 1
    sr = rng.uniform(0.001, 0.1, rows).astype(F32)
    zr = np.rint(rng.uniform(0, 126, rows)).astype(F32)
    sc = rng.uniform(0.0001, 0.01, cols).astype(F32)
    zc = np.rint(rng.uniform(-50, 50, cols)).astype(F32)
    zr[2] = F32(16777216.0)      # z_r + z_c rounds
    zc[3] = F32(1.0)
    got = orc.asym_dequant_hprec(acc, sr, zr, sc, zc)
    assert got.dtype == F32 and got.shape == (rows, cols)
    for r in range(rows):
        for c in range(cols):
            scales = rn_f32(Fraction(float(sr[r])) * Fraction(float(sc[c])))
            zeros = rn_f32(Fraction(float(zr[r])) + Fraction(float(zc[c])))
            af = rn_f32(Fraction(int(acc[r, c])))
            diff = rn_f32(Fraction(af) - Fraction(zeros))
            assert float(got[r, c]) == rn_f32(Fraction(scales) * Fraction(diff)), (r, c)
    # the operator order matters and is the reference's: s_r * (s_c * t) would differ somewhere
    t = (acc.astype(F32) - (zr[:, None] + zc[None, :]).astype(F32)).astype(F32)
    other = (sr[:, None] * (sc[None, :] * t).astype(F32)).astype(F32)
    assert not np.array_equal(other, got)


def test_weight_asym8_from_linear_hand_and_torch():
    import torch
    q, s, z = orc.weight_asym8_from_linear(np.array([[0.5, -1.0, 2.0, -0.25]], F32))
    # |w|: max 2, min 0.25 -> scale 1.75/127, zero = rint(-18.14) = -18;
    # w/scale = 36.29, -72.57, 145.14, -18.14 -> 36, -73, 145, -18 -> minus 18, clamped to [0, 127]
    assert q.dtype == np.int8 and q.tolist() == [[18, 0, 127, 0]]
    assert float(s[0, 0]) == rn_f32(Fraction(7, 4) / 127) and float(z[0, 0]) == -18.0
    rng = np.random.default_rng(6)
    for dt, tdt in ((np.float32, torch.float32), (np.float16, torch.float16)):
        w = (rng.standard_normal((24, 96)) * 0.05).astype(dt)
        q, s, z = orc.weight_asym8_from_linear(w)
        wt = torch.from_numpy(w)
        w_max = torch.max(torch.abs(wt), dim=-1, keepdim=True)[0]
        w_min = torch.min(torch.abs(wt), dim=-1, keepdim=True)[0]
        w_scale = (w_max - w_min) / 127
        w_zeros = (-w_min / w_scale).round().to(torch.float32)
        codes = torch.clamp(torch.round(wt / w_scale) + w_zeros, 0, 127)
        assert codes.dtype == torch.float32
        assert np.array_equal(q, codes.to(torch.int8).numpy())
        assert np.array_equal(s, w_scale.to(torch.float32).numpy()) and np.array_equal(z, w_zeros.numpy())
        assert tdt == wt.dtype


def test_linear8bit_forward_is_the_composition():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((9, 64)).astype(F32)
    w = (rng.standard_normal((12, 64)) * 0.1).astype(F32)
    bias = rng.standard_normal(12).astype(F32)
    wq, ws, wz = orc.weight_asym8_from_linear(w)
    y, acc, q, s, z = orc.linear8bit_asq_forward(x, wq, ws, wz, bias)
    assert np.array_equal(q, orc.asym_quant_8bit(x, *orc.asym8_scales_zeros(x)))
    assert np.array_equal(acc, orc.matmul_s8(q, wq))
    assert np.array_equal(y, (orc.asym_dequant_hprec(acc, s, z, ws, wz) + bias[None, :]).astype(F32))
    assert y.dtype == F32 and y.shape == (9, 12)


def test_weight_tile_layout_by_plain_loops():
    rng = np.random.default_rng(8)
    n, k = 40, 96
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    got = orc.weight_tile_8bit(w)
    assert got.dtype == np.int8 and got.size == 64 * k
    want = np.zeros(64 * k, np.int8)
    for nt in range(2):
        for ks in range(k // 32):
            for lane in range(64):
                row, k0 = nt * 32 + lane % 32, ks * 32 + (lane // 32) * 16
                if row < n:
                    base = ((nt * (k // 32) + ks) * 64 + lane) * 16
                    want[base:base + 16] = w[row, k0:k0 + 16]
    assert np.array_equal(got, want)


def test_c_oracle_agrees_with_numpy_oracle_8bit():
    """The plain-C restatement (own binary16 conversion, scalar float arithmetic) against the NumPy one."""
    from oracle import duq_oracle_c as orc_c
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((40, 257)) * rng.uniform(0.01, 30, (40, 1))).astype(F32)
    x[3, 5] = np.nan
    x[4, :] = 2.5
    x[5, 7] = np.inf
    x[6, :] = np.abs(x[6, :]) + 1
    for dev_div in (True, False):
        s, z = orc.asym8_scales_zeros(x, device_division=dev_div)
        sc, zc = orc_c.asym8_scales_zeros(x, dev_div)
        assert np.array_equal(s, sc, equal_nan=True) and np.array_equal(z, zc, equal_nan=True)
    s, z = orc.asym8_scales_zeros(x)
    s[7, 0], z[8, 0], z[9, 0] = 3e-39, 2049.0, -70000.0
    assert np.array_equal(orc_c.asym_quant_8bit(x, s, z), orc.asym_quant_8bit(x, s, z))
    a = rng.integers(-128, 128, (17, 96)).astype(np.int8)
    b = rng.integers(-128, 128, (23, 96)).astype(np.int8)
    assert np.array_equal(orc_c.matmul_s8(a, b), orc.matmul_s8(a, b))
    big = np.full((1, 1 << 17), -128, np.int8)
    assert int(orc_c.matmul_s8(big, big)[0, 0]) == -(1 << 31)
    acc = rng.integers(-2 ** 31, 2 ** 31, (17, 23)).astype(np.int32)
    sr, zr = rng.uniform(1e-3, 1, 17).astype(F32), np.rint(rng.uniform(-100, 126, 17)).astype(F32)
    scl, zcl = rng.uniform(1e-4, 0.1, 23).astype(F32), np.rint(rng.uniform(-100, 100, 23)).astype(F32)
    got, want = orc_c.asym_dequant_hprec(acc, sr, zr, scl, zcl), orc.asym_dequant_hprec(acc, sr, zr, scl, zcl)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# ------------------------------------------------------------------ ABI (CPU, no compute)
def test_abi_validation_8bit_entries():
    from duqlinear4bitcuda_amd import _lib
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    P = (ctypes.addressof(buf) + 15) & ~15
    mm = lib.duq_matmul_host_8bit
    assert mm(P, P, 4, 8, 48, P, None) == -3            # K % 32
    assert mm(P, P, 4, 8, 0, P, None) == -3
    assert mm(P, None, 4, 8, 32, P, None) == -1
    assert mm(P, P, 4, 8, 32, None, None) == -1
    assert mm(P + 8, P, 4, 8, 32, P, None) == -5
    assert mm(P, P, 4, (1 << 22) + 1, 32, P, None) == -6
    assert mm(P, P, 4, 8, 131072, P, None) == -6          # an accumulator could overflow
    assert 16384 * 131040 < 2 ** 31
    assert mm(None, None, 0, 8, 32, None, None) == 0
    fwd = lib.duq_linear8bit_forward
    assert fwd(P, P, P, P, P, P, None, 4, 8, 40, P, None) == -3
    assert fwd(P, P, None, P, P, P, None, 4, 8, 32, P, None) == -1
    assert fwd(P, P, P, P, P, P, None, 4, 8, 32, None, None) == -1
    assert fwd(None, None, None, None, None, None, None, 4, 0, 32, None, None) == 0
    tf = lib.duq_linear8bit_forward_tiled
    assert tf(P, P, P, P, P, P, None, 4, 8, 40, P, None) == -3
    assert tf(P, P, P, P + 4, P, P, None, 4, 8, 32, P, None) == -5
    assert tf(P, P, P, P, None, P, None, 4, 8, 32, P, None) == -1
    assert lib.duq_weight_tile_8bit(P, 8, 48, P, None) == -3
    assert lib.duq_weight_tile_8bit(P, 8, 32, None, None) == -1
    assert lib.duq_weight_tile_8bit(None, 0, 32, None, None) == 0
    assert lib.duq_asym_quant_host_8bit(P, P, None, 2, 8, P, None) == -1
    assert lib.duq_asym_quant_host_8bit(None, None, None, 0, 8, None, None) == 0
    assert lib.duq_asym_dequant_host_hprec(P, P, P, P, None, 2, 8, P, None) == -1
    assert lib.duq_quantize_rows_asym_8bit(P, 2, 6, P, P, P, None) == -2      # cols % 4
    assert lib.duq_quantize_rows_asym_8bit(P + 4, 2, 8, P, P, P, None) == -5
    assert lib.duq_quantize_rows_asym_8bit(P, 2, 8, None, P, P, None) == -1
    # quantizer + forward in one call
    ql = lib.duq_quantize_linear8bit_forward
    nb = lib.duq_quantize_linear8bit_workspace_bytes
    assert nb(4, 32) == 128 + 16 + 16 and nb(5, 4096) == 5 * 4096 + 32 + 32
    assert ql(P, P, None, P, P, None, 4, 8, 40, P, P, 1024, None) == -3          # K % 32
    assert ql(P, None, None, P, P, None, 4, 8, 32, P, P, 1024, None) == -1       # no weight at all
    assert ql(P, P, None, P, P, None, 4, 8, 32, P, None, 0, None) == -1          # no workspace
    assert ql(P, P, None, P, P, None, 4, 8, 32, P, P, 100, None) == -2           # too small
    assert ql(P + 4, P, None, P, P, None, 4, 8, 32, P, P, 1024, None) == -5
    assert ql(P, P, None, None, P, None, 4, 8, 32, P, P, 1024, None) == -1
    assert ql(None, None, None, None, None, None, 0, 8, 32, None, None, 0, None) == 0


def test_python_ops_reject_bad_arguments():
    import torch
    from duqlinear4bitcuda_amd import _HIP
    from duqlinear4bitcuda_amd.tools import tensor_utils
    a = torch.zeros((4, 32), dtype=torch.int8)
    with pytest.raises(RuntimeError):
        _HIP.matmul_8bit(a, a)                        # not on a GPU
    with pytest.raises(AssertionError):
        tensor_utils.matmul_8bit(torch.zeros((4, 48), dtype=torch.int8), a)
    with pytest.raises(AssertionError):
        tensor_utils.asym_quant_8bit(torch.zeros((4, 32), dtype=torch.float16), torch.zeros(4), torch.zeros(4))
    with pytest.raises(AssertionError):
        tensor_utils.asym_dequant_hprec(torch.zeros((4, 8), dtype=torch.int32), torch.zeros(4, dtype=torch.float16),
                                        torch.zeros(4), torch.zeros(8), torch.zeros(8))


# ------------------------------------------------------------------ GPU parity
@pytest.fixture(scope="module")
def hip(dev):
    from duqlinear4bitcuda_amd import _HIP
    return _HIP


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _acts(rng, rows, cols):
    x = (rng.standard_normal((rows, cols)) * rng.uniform(0.05, 20, (rows, 1))).astype(F32)
    x += rng.uniform(-3, 3, (rows, 1)).astype(F32)
    return x


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 7), (16, 32), (5, 33), (64, 4096), (33, 1000), (2, 40004)])
def test_gpu_asym_quant_8bit(dev, hip, rows, cols):
    rng = np.random.default_rng(rows * 131 + cols)
    x = _acts(rng, rows, cols)
    s, z = orc.asym8_scales_zeros(x)
    if rows >= 3:
        x[1, 0] = np.nan
        x[2, -1] = np.inf
        x[0, cols // 2] = -3e38
        z[2, 0] = 2049.0            # not representable in binary16
        s[1, 0] = 3e-39             # denormal scale
    want = orc.asym_quant_8bit(x, s, z)
    got = hip.asym_quant_8bit(_t(x, dev), _t(s.reshape(-1), dev), _t(z.reshape(-1), dev)).cpu().numpy()
    assert got.dtype == np.int8 and np.array_equal(got, want)


@pytest.mark.gpu
def test_gpu_asym_quant_8bit_unaligned_rows(dev, hip):
    import torch
    rng = np.random.default_rng(11)
    x = _acts(rng, 8, 36)
    s, z = orc.asym8_scales_zeros(x)
    base = torch.zeros(8 * 36 + 1, dtype=torch.float32, device=dev)
    view = base[1:].view(8, 36)      # 4-byte aligned only
    view.copy_(_t(x, dev))
    got = hip.asym_quant_8bit(view, _t(s.reshape(-1), dev), _t(z.reshape(-1), dev)).cpu().numpy()
    assert np.array_equal(got, orc.asym_quant_8bit(x, s, z))


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols", [(1, 4), (7, 36), (16, 256), (33, 1000), (64, 4096), (5, 8192), (3, 11008),
                                       (2, 32768), (2, 40004)])
def test_gpu_fused_quantizer_8bit(dev, hip, rows, cols):
    rng = np.random.default_rng(rows * 17 + cols)
    x = _acts(rng, rows, cols)
    if rows >= 5:
        x[1, cols // 3] = np.nan     # torch's min / max give NaN for this row
        x[2, :] = 1.25               # constant row: scale 0
        x[3, 1] = np.inf
        x[4, :] = np.abs(x[4, :])    # min > 0: negative zero point
    s, z = orc.asym8_scales_zeros(x)
    q = orc.asym_quant_8bit(x, s, z)
    gq, gs, gz = hip.quantize_rows_asym_8bit(_t(x, dev))
    assert gs.shape == (rows, 1) and gz.shape == (rows, 1) and gq.shape == (rows, cols)
    assert np.array_equal(gs.cpu().numpy(), s, equal_nan=True)
    assert np.array_equal(gz.cpu().numpy(), z, equal_nan=True)
    assert np.array_equal(gq.cpu().numpy(), q)


@pytest.mark.gpu
def test_gpu_fused_quantizer_8bit_matches_torch_ops(dev, hip):
    """scale / zero as torch computes them on the GPU (the reference's own statements)."""
    import torch
    rng = np.random.default_rng(12)
    x = _t(_acts(rng, 300, 4096), dev)
    lo, hi = x.min(dim=-1, keepdim=True)[0], x.max(dim=-1, keepdim=True)[0]
    scale = (hi - lo) / 127
    zeros = (-lo / scale).round().to(torch.float32)
    gq, gs, gz = hip.quantize_rows_asym_8bit(x.view(3, 100, 4096))
    assert gq.shape == (3, 100, 4096) and gs.shape == (3, 100, 1)
    assert torch.equal(gs.view(300, 1), scale) and torch.equal(gz.view(300, 1), zeros)
    assert torch.equal(gq.view(300, 4096), hip.asym_quant_8bit(x, scale.view(-1), zeros.view(-1)))


GEMM_SHAPES = [(1, 1, 32), (5, 7, 64), (32, 64, 96), (16, 16, 32), (9, 40, 96), (17, 250, 416), (32, 1030, 1056),
               (3, 48, 8192), (16, 4096, 8192), (31, 300, 4128),   # skinny kernel: K split over four wavefronts
               # decode kernel: up to 64 rows of at most 4096 elements, one to several column tiles per workgroup
               (16, 4096, 4096), (5, 4100, 4096), (16, 11008, 2048), (33, 5000, 1056), (48, 300, 4096), (64, 4099, 4096),
               (20, 8200, 96), (64, 16384, 32), (64, 17000, 64), (32, 17000, 64),
               (1, 4096, 4096), (2, 300, 8192), (4, 1000, 4096), (2, 35, 2080), (4, 17, 1056), (1, 5, 8192), (3, 21, 32),   # rows kernel
 (33, 250, 128), (100, 256, 160), (128, 260, 416),
               (129, 512, 1024), (300, 100, 32), (64, 1024, 4096), (65, 300, 224),
               (3, 40, 66560), (40, 300, 33280), (70, 260, 65600),   # long rows
               (512, 4096, 256), (300, 3100, 288), (200, 3990, 96),   # 64 x 128 tiles (48..128 tiles of 64 x 256)
               (1024, 3072, 256),   # 64 x 256 tiles
               (1000, 3100, 288), (2048, 4096, 4096),
               (4090, 4088, 4128)]   # 256 x 256 tiles (at least one per CU): ragged rows and columns, a last chunk of 32 k


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_gpu_matmul_8bit(dev, hip, M, N, K):
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    a = rng.integers(-128, 128, (M, K)).astype(np.int8)
    b = rng.integers(-128, 128, (N, K)).astype(np.int8)
    if M > 4 and N > 4:
        a[3, :] = -128
        b[2, :] = -128
        a[M - 1, :] = 127
        b[N - 1, :] = 127
    got = hip.matmul_8bit(_t(a, dev), _t(b, dev)).cpu().numpy()
    assert got.dtype == np.int32 and np.array_equal(got, orc.matmul_s8(a, b))


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols", [(1, 1), (7, 5), (64, 256), (300, 1001)])
def test_gpu_asym_dequant_hprec(dev, hip, rows, cols):
    rng = np.random.default_rng(rows + cols)
    acc = rng.integers(-2 ** 31, 2 ** 31, (rows, cols)).astype(np.int32)
    sr = rng.uniform(1e-4, 0.5, rows).astype(F32)
    zr = np.rint(rng.uniform(-200, 200, rows)).astype(F32)
    sc = rng.uniform(1e-5, 0.1, cols).astype(F32)
    zc = np.rint(rng.uniform(-200, 200, cols)).astype(F32)
    want = orc.asym_dequant_hprec(acc, sr, zr, sc, zc)
    got = hip.asym_dequant_hprec(_t(acc, dev), _t(sr, dev), _t(zr, dev), _t(sc, dev), _t(zc, dev)).cpu().numpy()
    assert got.dtype == F32 and np.array_equal(got.view(np.uint32), want.view(np.uint32))


FWD_SHAPES = [(5, 4100, 4096), (16, 11008, 1056), (33, 5000, 416), (64, 4099, 2080), (48, 260, 4096), (17, 40, 32),
              (1, 4096, 4096), (2, 250, 5120), (3, 33, 1056), (512, 4096, 128), (300, 3102, 288), (1, 16, 32), (7, 33, 64), (16, 48, 96), (17, 250, 416), (32, 1030, 1056), (4, 4096, 4096), (40, 250, 160), (128, 512, 1024), (130, 1030, 416), (1024, 3072, 256),
              (1000, 3102, 288),
              (4090, 4088, 1056)]   # 256 x 256 tiles


@pytest.mark.gpu
@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("M,N,K", FWD_SHAPES)
def test_gpu_linear8bit_forward(dev, hip, M, N, K, with_bias):
    rng = np.random.default_rng(M + N + K + int(with_bias))
    x = _acts(rng, M, K)
    w = (rng.standard_normal((N, K)) * 0.05).astype(F32)
    bias = rng.standard_normal(N).astype(F32) if with_bias else None
    wq, ws, wz = orc.weight_asym8_from_linear(w)
    y, acc, q, s, z = orc.linear8bit_asq_forward(x, wq, ws, wz, bias)
    gq, gs, gz = hip.quantize_rows_asym_8bit(_t(x, dev))
    assert np.array_equal(gq.cpu().numpy(), q)
    got = hip.linear8bit_forward(gq, gs, gz, _t(wq, dev), _t(ws, dev), _t(wz, dev),
                                 None if bias is None else _t(bias, dev)).cpu().numpy()
    assert got.dtype == F32 and got.shape == (M, N)
    assert np.array_equal(got.view(np.uint32), y.view(np.uint32))
    # the same launch on the tiled copy of the weight
    wt = hip.weight_tile_8bit(_t(wq, dev))
    assert np.array_equal(wt.cpu().numpy(), orc.weight_tile_8bit(wq))
    got_t = hip.linear8bit_forward(gq, gs, gz, wt, _t(ws, dev), _t(wz, dev), None if bias is None else _t(bias, dev),
                                   tiled_rows=N).cpu().numpy()
    assert np.array_equal(got_t.view(np.uint32), y.view(np.uint32))
    # and the three separate steps of the reference give the same bits
    acc_g = hip.matmul_8bit(gq, _t(wq, dev))
    assert np.array_equal(acc_g.cpu().numpy(), acc)
    y3 = hip.asym_dequant_hprec(acc_g, gs.view(-1), gz.view(-1), _t(ws.reshape(-1), dev), _t(wz.reshape(-1), dev))
    if bias is not None:
        y3 = y3 + _t(bias, dev)
    assert np.array_equal(y3.cpu().numpy().view(np.uint32), y.view(np.uint32))


@pytest.mark.gpu
def test_gpu_layer_8bit(dev):
    import torch
    from duqlinear4bitcuda_amd.nn import AsymQuantizer8bit, LinearQuant8bitASQ
    from duqlinear4bitcuda_amd.tools import tensor_utils
    rng = np.random.default_rng(21)
    K, N = 512, 384
    lin = torch.nn.Linear(K, N, bias=True)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy((rng.standard_normal((N, K)) * 0.03).astype(F32)))
        lin.bias.copy_(torch.from_numpy(rng.standard_normal(N).astype(F32)))
    layer = LinearQuant8bitASQ.from_linear(lin)
    sd = layer.state_dict()
    assert set(sd) == {"weight_scales", "weight_zeros", "weight", "bias"}
    assert sd["weight"].dtype == torch.int8 and tuple(sd["weight"].shape) == (N, K)
    assert sd["weight_scales"].dtype == torch.float32 and tuple(sd["weight_scales"].shape) == (N, 1)
    assert sd["weight_zeros"].dtype == torch.float32 and sd["bias"].dtype == torch.float32
    wq, ws, wz = orc.weight_asym8_from_linear(lin.weight.detach().numpy())
    assert np.array_equal(sd["weight"].numpy(), wq) and np.array_equal(sd["weight_scales"].numpy(), ws)
    assert np.array_equal(sd["weight_zeros"].numpy(), wz)
    layer = layer.to(dev)
    x = _acts(rng, 2 * 37, K).reshape(2, 37, K)
    want = orc.linear8bit_asq_forward(x.reshape(-1, K), wq, ws, wz, lin.bias.detach().numpy())[0].reshape(2, 37, N)
    xt = _t(x, dev)
    y = layer(xt)
    assert y.dtype == torch.float32 and tuple(y.shape) == (2, 37, N)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert "weight_tiled" not in layer.state_dict() and layer._buffers["weight_tiled"].numel() == N * K
    layer.tiled = False                       # the fused launch on the row-major weight
    assert torch.equal(layer(xt), y)
    layer.fused = False                       # the reference's three steps
    assert torch.equal(layer(xt), y)
    layer.fused = layer.tiled = True
    with torch.no_grad():                     # the tiled copy follows the weight
        layer.weight[5, :] = 1
    y_mod = layer(xt)
    layer.tiled = False
    assert torch.equal(layer(xt), y_mod) and not torch.equal(y_mod, y)
    with torch.no_grad():
        layer.weight.copy_(torch.from_numpy(wq))
    layer.fused = False
    assert torch.equal(layer(xt), y)
    layer.quantizer.fused = False             # torch computes scale and zero, as in the reference
    assert torch.equal(layer(xt), y)
    # a layer without its own quantizer takes the packed tensor
    bare = LinearQuant8bitASQ.from_linear(lin, require_quantizer=False).to(dev)
    assert torch.equal(bare(AsymQuantizer8bit()(xt)), y)
    with pytest.raises(AssertionError):
        bare(xt)
    # reload through the state_dict
    again = LinearQuant8bitASQ(K, N, bias=True).to(dev)
    again.load_state_dict(layer.state_dict())
    assert torch.equal(again(xt), y)
    # wrappers keep leading dimensions
    p = AsymQuantizer8bit()(xt)
    assert tuple(tensor_utils.matmul_8bit(p.quantized_x, layer.weight).shape) == (2, 37, N)


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [1, 4, 5, 16, 74, 256, 1024, 1030])
def test_gpu_layer_8bit_one_call(dev, monkeypatch, rows):
    """LinearQuant8bitASQ with its own quantizer: up to 1024 rows quantizer + GEMM are one library call, the bits of
    the oracle and of the two calls; above, two calls."""
    import torch
    from duqlinear4bitcuda_amd import _lib
    from duqlinear4bitcuda_amd.nn import LinearQuant8bitASQ
    print("8-bit layer, one call", rows, flush=True)
    rng = np.random.default_rng(rows)
    K, N = 1024, 320
    lin = torch.nn.Linear(K, N, bias=True)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy((rng.standard_normal((N, K)) * 0.03).astype(F32)))
        lin.bias.copy_(torch.from_numpy(rng.standard_normal(N).astype(F32)))
    layer = LinearQuant8bitASQ.from_linear(lin).to(dev)
    wq, ws, wz = orc.weight_asym8_from_linear(lin.weight.detach().numpy())
    x = _acts(rng, rows, K)
    want = orc.linear8bit_asq_forward(x, wq, ws, wz, lin.bias.detach().numpy())[0]
    xt = _t(x, dev)
    layer(xt)
    lib = _lib.load()
    calls = []
    for name in ("duq_quantize_linear8bit_forward", "duq_quantize_rows_asym_8bit", "duq_linear8bit_forward",
                 "duq_linear8bit_forward_tiled"):
        real = getattr(lib, name)
        monkeypatch.setattr(lib, name, (lambda *a, _r=real, _n=name: (calls.append(_n), _r(*a))[1]), raising=False)
    y = layer(xt)
    tiled_fwd = "duq_linear8bit_forward" if rows <= 4 else "duq_linear8bit_forward_tiled"
    assert calls == (["duq_quantize_linear8bit_forward"] if rows <= 1024 else ["duq_quantize_rows_asym_8bit", tiled_fwd]), calls
    assert np.array_equal(y.cpu().numpy().view(np.uint32), want.view(np.uint32))
    for tiled, one_call in ((False, 1024), (True, 0)):
        layer.tiled, layer.one_call_rows = tiled, one_call
        assert torch.equal(layer(xt), y), (tiled, one_call)


@pytest.mark.gpu
def test_gpu_8bit_full_size_properties(dev, hip):
    """M=2048, K=N=4096: the fused launch equals the three steps; the GEMM is linear in A."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(5)
    M, N, K = 2048, 4096, 4096
    x = torch.randn((M, K), generator=g).to(dev)
    wq = torch.randint(0, 128, (N, K), dtype=torch.int8, generator=g).to(dev)
    ws = (torch.rand((N, 1), generator=g) * 0.01 + 1e-4).to(dev)
    wz = torch.randint(-20, 1, (N, 1), generator=g).float().to(dev)
    bias = torch.randn(N, generator=g).to(dev)
    q, s, z = hip.quantize_rows_asym_8bit(x)
    assert int(q.min()) == 0 and int(q.max()) == 126
    y = hip.linear8bit_forward(q, s, z, wq, ws, wz, bias)
    assert torch.equal(hip.linear8bit_forward(q, s, z, hip.weight_tile_8bit(wq), ws, wz, bias, tiled_rows=N), y)
    acc = hip.matmul_8bit(q, wq)
    y3 = hip.asym_dequant_hprec(acc, s.view(-1), z.view(-1), ws.view(-1), wz.view(-1)) + bias
    assert torch.equal(y, y3)
    # column sums of C against a GEMV computed by torch in int64: sum_m C[m,n] = sum_k (sum_m A[m,k]) B[n,k]
    colsum = acc.sum(dim=0, dtype=torch.int64)
    a_sum = q.sum(dim=0, dtype=torch.int64)
    assert torch.equal(colsum, (wq.to(torch.int64) * a_sum[None, :]).sum(dim=1))
    # linearity: (A1 + A2) B = A1 B + A2 B with codes halved so that the sum stays int8
    a1 = (q // 2).to(torch.int8)
    a2 = (q - a1).to(torch.int8)
    assert torch.equal(hip.matmul_8bit(a1, wq) + hip.matmul_8bit(a2, wq), acc)
