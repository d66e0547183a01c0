"""Pins for the CPU oracle (oracle/duq_oracle.py, oracle/duq_oracle.c): every function is
checked against something that does not share its code - an exact rational model of
binary16 rounding written with fractions.Fraction, hand-computed answers, brute force,
closed forms, invariants, the torch-CPU operators the reference itself calls, and the two
independently written oracles against each other."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from oracle import duq_oracle_c as orc_c
from oracle import fakequant_torch as fq


# ------------------------------------------------------------------ exact binary16 model
def round_f16_exact(v: Fraction) -> float:
    """Round an exact rational to binary16, nearest-even, with overflow to inf from 65520.
    Independent of NumPy's casts: pure integer arithmetic."""
    if v == 0:
        return 0.0
    sign = -1 if v < 0 else 1
    a = abs(v)
    # exponent e with 2^e <= a < 2^(e+1), clamped to the subnormal exponent
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -14)
    ulp = Fraction(2) ** (e - 10)
    q = a / ulp
    n = q.numerator // q.denominator
    rem = q - n
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
        n += 1
    r = n * ulp
    if r >= 65520:
        return sign * float("inf")
    return sign * float(r)


def F(x):
    return Fraction(float(x))


def test_exact_model_agrees_with_numpy_cast_on_float32_inputs():
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(3000).astype(np.float32) * rng.choice([1e-7, 1e-4, 1e-2, 1, 50, 3e4], 3000).astype(np.float32),
        np.array([65504, 65519.99, 65520, -65520, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25, 2.0 ** -14, 1023.5, 2049, 2051], np.float32)])
    with np.errstate(over="ignore"):
        got = vals.astype(np.float16).astype(np.float64)
    want = np.array([round_f16_exact(F(v)) for v in vals])
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ C conversions
def test_c_half_conversions_all_bit_patterns():
    lib = orc_c.lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([lib.duqo_h2f(int(b)) for b in bits], dtype=np.float32)
    ok = (got == ref) | (np.isnan(got) & np.isnan(ref))
    assert ok.all()
    # float -> half on every half value, on midpoints between neighbours and just off them
    finite = ref[np.isfinite(ref)]
    f = np.unique(np.concatenate([finite, (finite[:-1] + finite[1:]) / 2, np.nextafter(finite, np.float32(np.inf)),
                                  np.nextafter(finite, np.float32(-np.inf))]).astype(np.float32))
    f = f[::7]  # ~37k samples keep the ctypes loop short
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([lib.duqo_f2h(float(v)) for v in f], dtype=np.uint16)
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ A10 pack / unpack
def test_pack_known_bytes():
    assert orc.pack_i4(np.array([[-8, 7]])).tolist() == [[0x78]]
    assert orc.pack_i4(np.array([[1, -1, 0, -8]])).tolist() == [[0xF1, 0x80]]
    assert orc.pack_i4(np.array([[3, 2, 1]])).tolist() == [[0x23, 0x01]]          # odd K: high nibble 0
    assert orc.pack_i4(np.array([[15, 0, 9, 8]]), sym=False).tolist() == [[0x0F, 0x89]]
    with pytest.raises(AssertionError):
        orc.pack_i4(np.array([[8, 0]]))
    with pytest.raises(AssertionError):
        orc.pack_i4(np.array([[-1, 0]]), sym=False)


def test_unpack_exhaustive_bytes():
    allb = np.arange(256, dtype=np.uint8).reshape(1, -1)
    s = orc.unpack_i4(allb, signed=True)[0]
    u = orc.unpack_i4(allb, signed=False)[0]
    for byte in range(256):
        lo, hi = byte & 15, byte >> 4
        assert u[2 * byte] == lo and u[2 * byte + 1] == hi
        assert s[2 * byte] == (lo - 16 if lo >= 8 else lo) and s[2 * byte + 1] == (hi - 16 if hi >= 8 else hi)
    q = np.arange(-8, 8).reshape(1, -1)
    assert np.array_equal(orc.unpack_i4(orc.pack_i4(q)), q)
    # torch implementation of the product package packs the same bytes
    from duqlinear4bitcuda_amd.tools import quantization as tq
    rng = np.random.default_rng(1)
    qq = rng.integers(-8, 8, (5, 16))
    assert np.array_equal(tq.pack_i4(torch.from_numpy(qq)).numpy(), orc.pack_i4(qq))
    assert np.array_equal(tq.unpack_i4(torch.from_numpy(orc.pack_i4(qq))).numpy(), qq)


# ------------------------------------------------------------------ A1 / A3 scales
def test_sym_scale_exhaustive_division_vs_reciprocal_and_exact_model():
    """Every non-negative binary16 maximum: h(m/7) computed (a) as the oracle does, (b) as
    torch-on-GPU does (multiply by float32(1/7)), (c) exactly.  All three agree, so the
    oracle's choice cannot matter."""
    m = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16)  # all finite >= 0
    a = orc.sym_scales(m.reshape(-1, 1))[:, 0]
    inv7 = np.float32(1.0) / np.float32(7.0)
    b = (m.astype(np.float32) * inv7).astype(np.float16)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
    idx = np.arange(0, len(m), 37)
    want = np.array([round_f16_exact(F(m[i]) / 7) for i in idx])
    assert np.array_equal(a[idx].astype(np.float64), want)


def test_asym_scale_division_by_15_vs_reciprocal():
    d = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16)
    a = (d.astype(np.float32) / np.float32(15)).astype(np.float16)
    b = (d.astype(np.float32) * (np.float32(1) / np.float32(15))).astype(np.float16)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16))


def test_scales_against_torch_ops_and_c_oracle():
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(64, 96, generator=g) * 3).half()
    x[3] = 0
    x[4] = x[4].abs()  # a non-negative row for the asym case
    for clip in (1.0, 0.9, 0.5):
        want = (torch.max(torch.abs(x), dim=-1)[0].unsqueeze(1) / 7).to(torch.float16) * clip  # quantizer.py:13
        got = orc.sym_scales(x.numpy(), clip)
        assert np.array_equal(got.view(np.uint16), want.numpy().view(np.uint16))
        assert np.array_equal(orc_c.sym_scales(x.numpy(), clip).view(np.uint16), got.view(np.uint16))
    mn = x.min(dim=-1, keepdim=True)[0]
    mx = x.max(dim=-1, keepdim=True)[0]
    scale = (mx - mn) / 15                                   # quantizer.py:30
    zeros = (-mn / scale).round().to(torch.float16)          # quantizer.py:31
    s, z = orc.asym_scales_zeros(x.numpy())
    assert np.array_equal(s.view(np.uint16), scale.numpy().view(np.uint16))
    ok = (z.view(np.uint16) == zeros.numpy().view(np.uint16)) | (np.isnan(z) & np.isnan(zeros.numpy()))
    assert ok.all()
    sc, zc = orc_c.asym_scales_zeros(x.numpy())
    assert np.array_equal(sc.view(np.uint16), s.view(np.uint16))
    assert ((zc.view(np.uint16) == z.view(np.uint16)) | (np.isnan(zc) & np.isnan(z))).all()


# ------------------------------------------------------------------ A2 / A3 quantize
def test_sym_quant_hand_computed():
    # scale 1: ties go to even, clamp at -8 and at qmax
    x = np.array([[0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 6.5, 7.0, 7.5, 100.0, -7.5, -8.5, -100.0, 0.0, 6.49]], np.float16)
    s = np.array([[1.0]], np.float16)
    assert orc.sym_quant_values(x, s, 7)[0].tolist() == [0, 2, 2, 4, 0, -2, -2, 6, 7, 7, 7, -8, -8, -8, 0, 6]
    assert orc.sym_quant_values(x, s, 6)[0].tolist() == [0, 2, 2, 4, 0, -2, -2, 6, 6, 6, 6, -8, -8, -8, 0, 6]
    # scale 0.5: x/s doubles
    assert orc.sym_quant_values(np.array([[0.25, 0.75, 1.25, -3.9]], np.float16), np.array([[0.5]], np.float16), 7)[0].tolist() == [0, 2, 2, -8]
    # zero scale: 0/0 -> NaN -> 0, x/0 -> +-inf -> clamp
    assert orc.sym_quant_values(np.array([[0.0, 1.0, -1.0]], np.float16), np.array([[0.0]], np.float16), 6)[0].tolist() == [0, 6, -8]


def test_sym_quant_double_rounding_case_found_by_brute_force():
    """The quotient is rounded to binary16 BEFORE the integer rounding.  Search for (x, s)
    where that changes the result against rounding the exact quotient once, and check the
    oracle returns the two-step answer there and everywhere else on the grid."""
    rng = np.random.default_rng(7)
    xs = rng.uniform(0.01, 8, 6000).astype(np.float16)
    ss = rng.uniform(0.2, 1.3, 6000).astype(np.float16)
    found = 0
    for x, s in zip(xs, ss):
        exact = F(x) / F(s)
        two_step = round(Fraction(round_f16_exact(exact)))        # python round: ties to even
        one_step = round(exact)
        got = int(orc.sym_quant_values(np.array([[x]]), np.array([[s]]), 1000)[0, 0])
        assert got == max(-8, two_step)
        found += two_step != one_step
    assert found > 0, "grid too small to contain a double-rounding case"


def test_sym_quant_invariants_and_both_oracles():
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((32, 257)) * 4).astype(np.float16)   # odd K: tail nibble 0
    s = orc.sym_scales(x)
    for qmax in (6, 7):
        q = orc.sym_quant_values(x, s, qmax)
        assert q.min() >= -8 and q.max() <= qmax
        order = np.argsort(x.astype(np.float32), axis=1, kind="stable")
        assert (np.diff(np.take_along_axis(q, order, axis=1), axis=1) >= 0).all()      # monotone in x
        inner = np.abs(q) < qmax
        assert np.array_equal(orc.sym_quant_values(-x, s, qmax)[inner], -q[inner])      # odd away from the clamp
        packed = orc.sym_quant(x, s, qmax)
        assert packed.shape == (32, 129) and (packed[:, -1] >> 4 == 0).all()
        assert np.array_equal(orc_c.sym_quant(x, s, qmax), packed)
    # with clip = 1 the row maximum always quantizes to +-7 under qmax 7 and to 6 / -7 under qmax 6
    q7 = orc.sym_quant_values(x, s, 7)
    assert (np.abs(q7).max(axis=1) == 7).all()


def test_fake_quant_path_is_the_torch_operators():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(16, 128, generator=g).half()
    s = fq.sym_scales(x)
    q_t = torch.clamp(torch.round(x / s), -8, 7)                  # quantization.py:29-32 with maxq 7
    assert np.array_equal(orc.fq_sym_quant(x.numpy(), s.numpy(), 7).view(np.uint16), q_t.numpy().view(np.uint16))
    assert np.array_equal(orc.sym_quant_values(x.numpy(), s.numpy(), 7), q_t.numpy().astype(np.int32))
    z = torch.full((16, 1), 3.0).half()
    qa = torch.clamp(torch.round(x / s) + z, 0, 15)               # quantization.py:17-21
    assert np.array_equal(orc.fq_asym_quant(x.numpy(), s.numpy(), z.numpy(), 15).view(np.uint16), qa.numpy().view(np.uint16))
    assert np.array_equal(orc.fq_asym_dequant(qa.numpy(), s.numpy(), z.numpy()).view(np.uint16),
                          (s * (qa - z)).numpy().view(np.uint16))
    assert np.array_equal(orc.fq_sym_dequant(q_t.numpy(), s.numpy()).view(np.uint16), (s * q_t).numpy().view(np.uint16))


def test_asym_and_dual_quant_hand_cases_and_c_oracle():
    x = np.array([[0.0, 0.4, 0.6, 2.5, 6.0, -1.0, 3.5, 100.0]], np.float16)
    s = np.array([[1.0]], np.float16)
    z = np.array([[2.0]], np.float16)
    # rint(x) + 2 clamped to [0, 15]
    assert orc.asym_quant_values(x, s, z)[0].tolist() == [2, 2, 3, 4, 8, 1, 6, 15]
    assert orc.asym_quant(x, s, z).tolist() == [[0x22, 0x43, 0x18, 0xF6]]
    # dual: zero added BEFORE rounding (quant2.cu:133): 2.5 + 0.5 = 3.0 -> 3, whereas rint(2.5) + rint(0.5) = 2
    zh = np.array([[0.5]], np.float16)
    assert orc.asym_dual_quant_values(x, s, zh, s, zh)[0].tolist() == [0, 1, 1, 3, 6, 0, 4, 15]
    assert orc.asym_quant_values(x, s, zh)[0].tolist()[3] == 2
    # dual split at column 10
    x2 = np.full((1, 24), 3.0, np.float16)
    q = orc.sym_dual_quant_values(x2, np.array([[1.0]], np.float16), np.array([[0.5]], np.float16))
    assert q[0].tolist() == [3] * 10 + [6] * 14
    rng = np.random.default_rng(2)
    xr = rng.uniform(0, 6, (9, 40)).astype(np.float16)
    s1 = rng.uniform(0.1, 1, (9, 1)).astype(np.float16)
    s2 = rng.uniform(0.1, 1, (9, 1)).astype(np.float16)
    z1 = rng.integers(0, 9, (9, 1)).astype(np.float16)
    z2 = (rng.integers(0, 9, (9, 1)) + 0.5).astype(np.float16)
    assert np.array_equal(orc_c.asym_quant(xr, s1, z1), orc.asym_quant(xr, s1, z1))
    assert np.array_equal(orc_c.sym_dual_quant(xr, s1, s2), orc.sym_dual_quant(xr, s1, s2))
    assert np.array_equal(orc_c.asym_dual_quant(xr, s1, z1, s2, z2), orc.asym_dual_quant(xr, s1, z1, s2, z2))
    # degenerate scale 0 rows follow the saturating conversion + wrapping add
    x0 = np.array([[1.5, 0.0, -2.0]], np.float16)
    s0 = np.array([[0.0]], np.float16)
    for zz in (np.inf, -np.inf, 3.0):
        zt = np.array([[zz]], np.float16)
        assert np.array_equal(orc_c.asym_quant(x0, s0, zt), orc.asym_quant(x0, s0, zt))


# ------------------------------------------------------------------ A4 GEMM
def test_matmul_brute_force_and_closed_forms():
    rng = np.random.default_rng(4)
    for (M, N, K) in [(3, 5, 64), (7, 2, 128), (4, 4, 192)]:
        a = rng.integers(0, 256, (M, K // 2), dtype=np.uint8)
        b = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        want = np.zeros((M, N), np.int64)
        for m in range(M):
            for n in range(N):
                acc = 0
                for k in range(K):
                    va = (int(a[m, k // 2]) >> (4 * (k % 2))) & 15
                    vb = (int(b[n, k // 2]) >> (4 * (k % 2))) & 15
                    acc += (va - 16 if va >= 8 else va) * (vb - 16 if vb >= 8 else vb)
                want[m, n] = acc
        assert np.array_equal(orc.matmul_s4(a, b), want)
        assert np.array_equal(orc_c.matmul_s4(a, b), want)
    K = 4096
    assert (orc.matmul_s4(np.full((2, K // 2), 0x88, np.uint8), np.full((3, K // 2), 0x88, np.uint8)) == 64 * K).all()
    assert (orc.matmul_s4(np.full((2, K // 2), 0x88, np.uint8), np.full((3, K // 2), 0x77, np.uint8)) == -56 * K).all()
    # the int64 branch (64*K >= 2^24) agrees with the float32 branch's closed form too
    K = 1 << 18
    assert (orc.matmul_s4(np.full((1, K // 2), 0x88, np.uint8), np.full((1, K // 2), 0x88, np.uint8)) == 64 * K).all()
    # unsigned asym nibbles 8..15 enter the product as -8..-1 (README known issue 1)
    a = orc.pack_i4(np.array([[15] * 64]), sym=False)
    b = orc.pack_i4(np.array([[1] * 64]), sym=True)
    assert orc.matmul_s4(a, b)[0, 0] == -64


# ------------------------------------------------------------------ A5 / A6 / A7 epilogues
def _exact_sym(acc, sr, sc):
    e = round_f16_exact(Fraction(int(acc)))
    ss = round_f16_exact(F(sr) * F(sc))
    if np.isinf(e) or np.isinf(ss):
        return float(np.float16(ss) * np.float16(e))
    return round_f16_exact(Fraction(ss) * Fraction(e))


def test_sym_dequant_exact_model_grid():
    accs = [0, 1, -1, 2047, 2049, 2051, 4097, 65503, 65519, -65519, 12345, -54321, 1000000 // 16]
    srs = np.array([0.5713, 1.0, 0.00731, 3.25], np.float16)
    scs = np.array([0.00201, 0.0099, 1.0, 0.333], np.float16)
    acc = np.array(accs, np.int32).reshape(1, -1)
    for sr in srs:
        for sc in scs:
            got = orc.sym_dequant(np.repeat(acc, 1, 0).T.reshape(-1, 1), np.full((len(accs), 1), sr), np.array([sc]))
            for i, a in enumerate(accs):
                want = _exact_sym(a, sr, sc)
                assert float(got[i, 0]) == want or (np.isnan(got[i, 0]) and np.isnan(want)), (a, sr, sc)
    # the accumulator conversion overflows from 65520
    big = orc.sym_dequant(np.array([[65519, 65520, -65520, 1 << 20]], np.int32), np.array([1.0], np.float16),
                          np.array([1.0] * 4, np.float16))
    assert big[0].tolist() == [65504.0, np.inf, -np.inf, np.inf]
    assert orc.int_to_half(np.array([2049, 2051, 4098, 4102])).tolist() == [2048.0, 2052.0, 4096.0, 4104.0]


def test_asym_dequant_order_of_operations():
    # (h(acc) - z_r) - z_c in that order, each rounded: 2049 -> 2048; 2048 - 1 = 2047; 2047 - 0.5 = 2046.5 -> 2046
    y = orc.asym_dequant(np.array([[2049]], np.int32), np.array([1.0], np.float16), np.array([1.0], np.float16),
                         np.array([1.0], np.float16), np.array([0.5], np.float16))
    assert float(y[0, 0]) == 2046.0
    # not the true zero-point correction: acc 10, z 3 and 4, scales 0.5 * 0.25 -> 0.125 * 3 = 0.375
    y = orc.asym_dequant(np.array([[10]], np.int32), np.array([0.5], np.float16), np.array([3.0], np.float16),
                         np.array([0.25], np.float16), np.array([4.0], np.float16))
    assert float(y[0, 0]) == 0.375


def test_dual_selectors_enumerated():
    n = 140
    s1 = np.arange(n).astype(np.float16)
    s2 = -np.arange(n).astype(np.float16) - 1000
    pick = orc.sym_dual_col_scale(s1, s2)
    assert [float(v) for v in pick[:10]] == [float(i) for i in range(10)]
    assert all(float(pick[i]) == -i - 1000 for i in range(10, n))
    pick = orc.asym_dual_col_select(s1, s2)
    assert float(pick[0]) == 0.0 and all(float(pick[i]) == -i - 1000 for i in range(1, n))
    # QUANT_COL_ST as written in include/quant.h:7: ((ST << col) & 1) is non-zero for col == 0 only
    ST = sum(1 << b for b in (0, 1, 2, 3, 4, 10, 11, 12, 13, 14))
    assert [((ST << col) & 1) != 0 for col in range(128)] == [col == 0 for col in range(128)]


def test_epilogues_both_oracles_agree():
    rng = np.random.default_rng(9)
    M, N = 17, 45
    acc = rng.integers(-70000, 70000, (M, N)).astype(np.int32)
    sr = rng.uniform(0.01, 1, (M, 1)).astype(np.float16)
    zr = rng.integers(0, 16, (M, 1)).astype(np.float16)
    sc1 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    sc2 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    zc1 = rng.integers(0, 16, (N, 1)).astype(np.float16)
    zc2 = rng.integers(0, 16, (N, 1)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)

    def same(a, b):
        return ((a.view(np.uint16) == b.view(np.uint16)) | (np.isnan(a) & np.isnan(b))).all()

    assert same(orc.sym_dequant(acc, sr, sc1), orc_c.sym_dequant(acc, sr, sc1))
    assert same(orc.sym_dual_dequant(acc, sr, sc1, sc2), orc_c.sym_dual_dequant(acc, sr, sc1, sc2))
    assert same(orc.asym_dequant(acc, sr, zr, sc1, zc1), orc_c.asym_dequant(acc, sr, zr, sc1, zc1))
    assert same(orc.asym_dual_dequant(acc, sr, zr, sc1, zc1, sc2, zc2), orc_c.asym_dual_dequant(acc, sr, zr, sc1, zc1, sc2, zc2))
    y = orc.sym_dequant(acc, sr, sc1)
    assert same(orc.add_bias(y, bias), orc_c.add_bias(y, bias))
    assert same(orc.add_bias(y, bias), (torch.from_numpy(y) + torch.from_numpy(bias)).numpy())  # linear.py:53-54


# ------------------------------------------------------------------ A8 / A11 composition
def test_forward_composition_against_torch_fake_quant_path():
    """With qmax 7 the oracle's symmetric forward equals the reference's CPU fake-quant path
    (torch operators) bit for bit: codes, accumulators and fp16 outputs."""
    g = torch.Generator().manual_seed(8)
    M, K, N = 24, 256, 40
    x = torch.randn(M, K, generator=g).half()
    wq = torch.randint(-8, 8, (N, K), generator=g)
    sw = (torch.rand(N, 1, generator=g) * 0.009 + 0.001).half()
    y_t, acc_t, q_t, s_t = fq.linear4bit_forward(x, wq, sw, maxq=7)
    y, acc, qx, sx = orc.linear4bit_sq_forward(x.numpy(), orc.pack_i4(wq.numpy()), sw.numpy(), qmax=7)
    assert np.array_equal(orc.unpack_i4(qx), q_t.numpy().astype(np.int32))
    assert np.array_equal(acc, acc_t.numpy())
    assert np.array_equal(y.view(np.uint16), y_t.numpy().view(np.uint16))
    # the device clamp (qmax 6) differs exactly where the fake-quant code is 7
    _, _, qx6, _ = orc.linear4bit_sq_forward(x.numpy(), orc.pack_i4(wq.numpy()), sw.numpy(), qmax=6)
    u7, u6 = orc.unpack_i4(qx), orc.unpack_i4(qx6)
    assert np.array_equal(u6 != u7, u7 == 7) and (u6[u7 == 7] == 6).all()


def test_weight_prep_matches_torch_arithmetic():
    g = torch.Generator().manual_seed(12)
    w = (torch.randn(12, 64, generator=g) * 0.02).half()
    s = (w.abs().amax(-1, keepdim=True) / 7).half()
    from duqlinear4bitcuda_amd.tools import quantization as tq
    want = tq.pack_i4((w / s).round().to(torch.int8)).numpy()       # linear.py:72-73
    assert np.array_equal(orc.weight_sym_from_float(w.numpy(), s.numpy()), want)
    aw = w.abs()
    mx, mn = aw.amax(-1, keepdim=True), aw.amin(-1, keepdim=True)
    scale = (mx - mn) / 15
    zeros = (-mn / scale).round().to(torch.float16)
    codes = torch.clamp(torch.round(w / scale) + zeros, 0, 15)        # linear.py:129-136
    p, sc, z = orc.weight_asym_from_linear(w.numpy())
    assert np.array_equal(p, tq.pack_i4(codes.to(torch.int8), sym=False).numpy())
    assert np.array_equal(sc.view(np.uint16), scale.numpy().view(np.uint16))
    assert np.array_equal(z.view(np.uint16), zeros.numpy().view(np.uint16))
