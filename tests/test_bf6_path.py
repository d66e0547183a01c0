"""The 6-bit float (E3M2) matrix path: the same Linear4bit forward, computed by the MFMA for
6-bit floats on "shadows" of the packed-int4 operands.  The reference has no such path; what it
must reproduce is the integer GEMM of the reference (oracle ``matmul_s4``) and its epilogues,
bit for bit.  The oracle's description of the shadow format is pinned here by the published
E3M2 table, by decode(encode(v)) == v, by the round trip through the unpacker, and by a
plain-loop restatement of the two layouts; the exactness argument (integer products summed in
float32 in any order) is checked numerically."""
import ctypes

import numpy as np
import pytest

from oracle import duq_oracle as orc
from tests import cases


# ------------------------------------------------------------------ oracle pins (CPU)
def test_e3m2_decode_published_values():
    # OCP Microscaling Formats v1.0, table of FP6 E3M2: bias 3, max normal 28, min normal 0.25,
    # max subnormal 0.1875, min subnormal 0.0625, no inf / NaN
    assert orc.e3m2_decode(0b011111) == 28.0 and orc.e3m2_decode(0b111111) == -28.0
    assert orc.e3m2_decode(0b000100) == 0.25
    assert orc.e3m2_decode(0b000011) == 0.1875 and orc.e3m2_decode(0b000001) == 0.0625
    assert orc.e3m2_decode(0) == 0.0 and orc.e3m2_decode(0b001100) == 1.0 and orc.e3m2_decode(0b010000) == 2.0
    assert np.all(np.isfinite(orc.e3m2_decode(np.arange(64))))
    # one value per code, symmetric in sign
    vals = orc.e3m2_decode(np.arange(64))
    assert len(set(vals[:32].tolist())) == 32 and np.array_equal(vals[32:], -vals[:32])


def test_e3m2_encode_is_exact_for_every_int4_value():
    v = np.arange(-8, 8)
    codes = orc.e3m2_encode_int4(v)
    assert np.array_equal(orc.e3m2_decode(codes), v.astype(np.float64))
    assert codes[8] == 0  # zero is +0
    # the codes listed in csrc/duq_bf6.hip's derivation: 1 -> 0b001100, 7 -> 0b010111, -8 -> 0b111000
    assert codes[9] == 0b001100 and codes[15] == 0b010111 and codes[0] == 0b111000


def test_float32_accumulation_of_int4_products_is_exact():
    """The claim the path rests on: products of int4 values summed in float32, in any order, give
    the integer sum as long as it stays below 2^24; 64 * K < 2^24 for every K the library takes."""
    assert 64 * 131008 < 2 ** 24
    rng = np.random.default_rng(0)
    for K in (128, 4096, 131008):
        a = rng.integers(-8, 8, K)
        b = rng.integers(-8, 8, K)
        if K == 131008:
            a[:] = -8
            b[:] = -8  # the extreme: every product is 64
        want = int((a.astype(np.int64) * b.astype(np.int64)).sum())
        prods = (a * b).astype(np.float32)
        for order in (np.arange(K), rng.permutation(K), np.argsort(prods), np.argsort(-prods)):
            acc = np.float32(0)
            for chunk in np.array_split(prods[order], 64):  # partial sums like a blocked kernel's
                acc = np.float32(acc + np.float32(chunk.sum(dtype=np.float32)))
            assert int(acc) == want and float(acc) == float(want)


def test_shadow_block_round_trip_and_positions():
    rng = np.random.default_rng(1)
    v = rng.integers(-8, 8, (4, 7, 32))
    blk = orc.shadow_block_pack(v)
    assert blk.shape == (4, 7, 24) and blk.dtype == np.uint8
    assert np.array_equal(orc.shadow_block_unpack(blk), v)
    assert sorted(orc._shadow_positions().tolist()) == list(range(32))
    # position p sits in bits 6p..6p+5: a block holding one non-zero element
    one = np.zeros(32, np.int64)
    one[5] = -8                                     # element 5 = word 0, nibble 5 = pair i=1, half 1 -> position 3
    bits = np.unpackbits(orc.shadow_block_pack(one), bitorder="little")
    assert bits[18:24].tolist() == [0, 0, 0, 1, 1, 1] and bits.sum() == 3   # 0b111000 at bits 18..23


def _loop_activation_shadow(q):
    v = orc.unpack_i4(q, signed=True)
    M, K = v.shape
    out = np.zeros((M, K * 3 // 4), np.uint8)
    for m in range(M):
        for b in range(K // 32):
            blk = orc.shadow_block_pack(v[m, 32 * b:32 * b + 32])
            out[m, 16 * b:16 * b + 16] = blk[:16]
            out[m, (K // 32) * 16 + 8 * b:(K // 32) * 16 + 8 * b + 8] = blk[16:]
    return out


def _loop_weight_shadow(q):
    v = orc.unpack_i4(q, signed=True)
    N, K = v.shape
    pairs = (N // 16 + 1) // 2
    out = np.zeros(pairs * 32 * K * 3 // 4, np.uint8)
    ksteps = K // 128
    for pair in range(pairs):
        for step in range(ksteps):
            base = (pair * ksteps + step) * 3072
            for lane in range(64):
                row, kb = lane % 16, lane // 16
                k0 = step * 128 + kb * 32
                both = np.zeros(48, np.uint8)      # the lane's twelve dwords: tile 2*pair, then tile 2*pair + 1
                for half in range(2):
                    n = (2 * pair + half) * 16 + row
                    if n < N:
                        both[24 * half:24 * half + 24] = orc.shadow_block_pack(v[n, k0:k0 + 32])
                for piece in range(3):
                    at = base + piece * 1024 + lane * 16
                    out[at:at + 16] = both[16 * piece:16 * piece + 16]
    return out.reshape(pairs * 32, K * 3 // 4)


def test_shadow_layouts_against_plain_loops():
    rng = np.random.default_rng(2)
    q = rng.integers(0, 256, (5, 128), dtype=np.uint8)       # M = 5, K = 256
    assert np.array_equal(orc.activation_shadow_bf6(q), _loop_activation_shadow(q))
    w = rng.integers(0, 256, (48, 192), dtype=np.uint8)      # N = 48 (an odd number of 16-row tiles), K = 384
    assert np.array_equal(orc.weight_shadow_bf6(w), _loop_weight_shadow(w))
    assert orc.weight_shadow_bf6(w).shape == (64, 288)
    w = rng.integers(0, 256, (64, 64), dtype=np.uint8)       # N = 64, K = 128
    assert np.array_equal(orc.weight_shadow_bf6(w), _loop_weight_shadow(w))


def test_abi_validation_bf6_entries():
    from duqlinear4bitcuda_amd import _lib
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    P = (ctypes.addressof(buf) + 15) & ~15
    assert lib.duq_weight_shadow_bf6(P, 32, 64, P, None) == -3          # K % 128
    assert lib.duq_weight_shadow_bf6(P, 24, 128, P, None) == -2         # N % 16
    assert lib.duq_weight_shadow_bf6(P, 32, 128, None, None) == -1
    assert lib.duq_weight_shadow_bf6(P, 0, 128, None, None) == 0
    assert lib.duq_activation_shadow_bf6(P, 4, 192, P, None) == -3
    assert lib.duq_activation_shadow_bf6(P + 4, 4, 128, P, None) == -5
    assert lib.duq_quantize_rows_sym_bf6(P, 2, 64, 1.0, 6, P, P, P, None) == -2
    assert lib.duq_quantize_rows_sym_bf6(P, 2, 128, 1.0, 6, None, None, P, None) == -1   # the shadow is required
    assert lib.duq_quantize_rows_sym_bf6(P, 2, 128, 1.0, 9, P, P, P, None) == -4
    assert lib.duq_quantize_rows_asym_bf6(P, 2, 128, None, P, P, None, None, None) == -1
    fwd = lib.duq_linear4bit_forward_bf6
    assert fwd(0, P, P, None, None, P, P, None, None, None, None, None, 4, 32, 64, P, None) == -3
    assert fwd(0, P, P, None, None, P, P, None, None, None, None, None, 4, 40, 128, P, None) == -2
    assert fwd(5, P, P, None, None, P, P, None, None, None, None, None, 4, 32, 128, P, None) == -4
    assert fwd(1, P, P, None, None, P, P, None, None, None, None, None, 4, 32, 128, P, None) == -1   # zeros missing
    assert fwd(4, P, P, P, None, P, P, P, None, None, None, None, 4, 32, 128, P, None) == -1          # row sums missing
    assert fwd(0, P, P, None, None, P, P + 2, None, None, None, None, None, 4, 32, 128, P, None) == -5
    assert fwd(0, None, None, None, None, None, None, None, None, None, None, None, 0, 32, 128, None, None) == 0
    assert fwd(0, P, P, None, None, P, P, None, None, None, None, None, 4, (1 << 22) + 16, 128, P, None) == -6
    assert lib.duq_matmul_host_4bit(P, P, 4, (1 << 22) + 1, 64, P, None) == -6


# ------------------------------------------------------------------ GPU parity
@pytest.fixture(scope="module")
def hip(dev):
    from duqlinear4bitcuda_amd import _HIP
    return _HIP


def _rand_packed(rng, rows, K):
    return rng.integers(0, 256, (rows, K // 2), dtype=np.uint8)


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 16, 128), (5, 64, 256), (130, 80, 384), (64, 256, 4096), (33, 1008, 1152)])
def test_gpu_shadow_kernels_match_the_format(hip, dev, M, N, K):
    print("bf6 shadows", M, N, K, flush=True)
    rng = np.random.default_rng(M + N + K)
    a, b = _rand_packed(rng, M, K), _rand_packed(rng, N, K)
    assert np.array_equal(hip.activation_shadow_bf6(cases.t(a, dev)).cpu().numpy(), orc.activation_shadow_bf6(a))
    assert np.array_equal(hip.weight_shadow_bf6(cases.t(b, dev)).cpu().numpy(), orc.weight_shadow_bf6(b))


@pytest.mark.gpu
@pytest.mark.parametrize("M,K", [(1, 128), (16, 4096), (300, 1024), (2048, 4096), (3, 11008), (2, 66048), (5, 130944)])
def test_gpu_quantizers_write_the_shadow_of_their_codes(hip, dev, M, K):
    print("bf6 quantizers", M, K, flush=True)
    x = cases.acts_uniform(M, K, seed=M + K) if K % 3 else cases.acts_outliers(M, K, seed=M + K)
    if M > 2:
        x[1, 7] = np.float16(np.nan)   # a row that takes the element-wise path
        x[2] = 0
    X = cases.t(x, dev)
    s_want = orc.sym_scales(x)
    q_want = orc.sym_quant(x, s_want)
    q, sh, s = hip.quantize_rows_sym_bf6(X)
    assert np.array_equal(q.cpu().numpy(), q_want) and cases.bits_equal(s.cpu().numpy(), s_want)
    assert np.array_equal(sh.cpu().numpy(), orc.activation_shadow_bf6(q_want))
    none, sh2, _ = hip.quantize_rows_sym_bf6(X, with_q=False)
    assert none is None and np.array_equal(sh2.cpu().numpy(), sh.cpu().numpy())

    sa, za = orc.asym_scales_zeros(x)
    qa = orc.asym_quant(x, sa, za)
    q, sh, s, z = hip.quantize_rows_asym_bf6(X)
    assert np.array_equal(q.cpu().numpy(), qa) and cases.bits_equal(z.cpu().numpy(), za)
    assert np.array_equal(sh.cpu().numpy(), orc.activation_shadow_bf6(qa))   # unsigned codes, read as signed nibbles

    wq, ws, wz, wr = orc.asym_quant_shifted(x)
    q, sh, s, z, r = hip.quantize_rows_asym_bf6(X, shifted=True)
    assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(r.cpu().numpy(), wr)
    assert np.array_equal(sh.cpu().numpy(), orc.activation_shadow_bf6(wq))


def _epi_inputs(rng, M, N):
    sr = rng.uniform(0.01, 1.0, (M, 1)).astype(np.float16)
    zr = rng.integers(0, 16, (M, 1)).astype(np.float16)
    sc1 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    sc2 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    zc1 = rng.integers(0, 16, (N, 1)).astype(np.float16)
    zc2 = rng.integers(0, 16, (N, 1)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    return sr, zr, sc1, zc1, sc2, zc2, bias


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(1, 16, 128), (128, 256, 128), (128, 256, 256), (100, 240, 640), (257, 512, 1024),
                                   (130, 80, 384), (300, 1008, 1152), (512, 4096, 4096), (64, 1024, 11008),
                                   # more than 160 tiles of 64 x 256 (the ones above run 64 x 128 tiles): 64 x 256 tiles
                                   (704, 4096, 512), (1000, 4096, 256), (900, 3000 - 8, 384),
                                   # enough tiles for the 128-row variant of the kernel
                                   (2048 + 70, 4096 - 48, 384), (2048, 4096, 128),
                                   # ... and for the 256-row variant: one to seven steps (its loop turns every four), ragged edges
                                   (4096, 4096, 128), (4096 - 37, 4096 - 48, 384), (4096, 4096, 512), (4096, 4096 - 16, 896)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_gpu_forward_bf6_equals_oracle(hip, dev, M, N, K, with_bias):
    """One and several chunks, odd and even numbers of 128-k steps, ragged M, N that ends inside a
    workgroup tile and inside a wavefront's four tiles; every epilogue."""
    print("bf6 forward", M, N, K, with_bias, flush=True)
    rng = np.random.default_rng(M * 11 + N * 5 + K)
    a, b = _rand_packed(rng, M, K), _rand_packed(rng, N, K)
    sr, zr, sc1, zc1, sc2, zc2, bias = _epi_inputs(rng, M, N)
    acc = orc.matmul_s4(a, b)
    T = lambda v: cases.t(v, dev)
    tb = T(bias) if with_bias else None
    fin = (lambda y: orc.add_bias(y, bias)) if with_bias else (lambda y: y)
    xs, ws = hip.activation_shadow_bf6(T(a)), hip.weight_shadow_bf6(T(b))

    got = hip.linear4bit_forward_bf6(hip.EPI_SYM, xs, T(sr), None, ws, T(sc1), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.sym_dequant(acc, sr, sc1)))
    got = hip.linear4bit_forward_bf6(hip.EPI_ASYM, xs, T(sr), T(zr), ws, T(sc1), T(zc1), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.asym_dequant(acc, sr, zr, sc1, zc1)))
    got = hip.linear4bit_forward_bf6(hip.EPI_SYM_DUAL, xs, T(sr), None, ws, T(sc1), None, T(sc2), bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.sym_dual_dequant(acc, sr, sc1, sc2)))
    got = hip.linear4bit_forward_bf6(hip.EPI_ASYM_DUAL, xs, T(sr), T(zr), ws, T(sc1), T(zc1), T(sc2), T(zc2),
                                     bias=tb).cpu().numpy()
    assert cases.bits_equal(got, fin(orc.asym_dual_dequant(acc, sr, zr, sc1, zc1, sc2, zc2)))
    rr = rng.integers(-8 * K, 8 * K, M).astype(np.int32)
    rc = rng.integers(-8 * K, 8 * K, N).astype(np.int32)
    got = hip.linear4bit_forward_bf6(hip.EPI_ASYM_ROWSUM, xs, T(sr), T(zr), ws, T(sc1), T(zc1), bias=tb, rowsum_x=T(rr),
                                     w_rowsum_adj=T(rc)).cpu().numpy()
    assert cases.bits_equal(got, orc.asym_rowsum_dequant(acc, sr, zr, rr, sc1, zc1, rc, bias if with_bias else None))


@pytest.mark.gpu
def test_gpu_forward_bf6_extreme_accumulation(hip, dev):
    """Every product 64 (or -64) over the longest row the library takes: |acc| = 64 * 130944, the largest
    magnitude the float32 accumulator has to hold exactly; plus rows that cancel to small odd sums."""
    K, M, N = 130944, 8, 32
    a = np.full((M, K // 2), 0x88, np.uint8)            # all -8
    b = np.full((N, K // 2), 0x88, np.uint8)
    b[1] = 0x77                                          # all +7: acc = -56 * K
    a[2, :] = 0x78                                       # alternating -8 (low nibble) / +7 (high nibble)
    a[3, :] = 0x00
    a[3, 0] = 0x01                                       # a single 1 in a row of zeros
    # odd products added to an accumulator within 2^14 of 2^23: rows / columns of -8 that share one index holding
    # +1 (x +1) or +7 (x +1), in the middle of the row and in its last element; an addend aligned below 24 bits
    # would lose exactly these
    k1, k2 = 12345, K - 1
    def put(row, k, v):
        byte, hi = k // 2, k % 2
        row[byte] = (row[byte] & (0x0F if hi else 0xF0)) | ((v & 0xF) << (4 if hi else 0))
    put(a[4], k1, 1), put(b[2], k1, 1)
    put(a[5], k2, 7), put(b[3], k2, 1)
    acc = orc.matmul_s4(a, b)
    assert acc[0, 0] == 64 * K and acc[0, 1] == -56 * K and acc[3, 0] == -8
    assert acc[4, 2] == 64 * (K - 1) + 1 and acc[5, 3] == 64 * (K - 1) + 7 and acc[4, 2] > (1 << 23) - (1 << 14)
    one = np.ones((max(M, N), 1), np.float16)
    T = lambda v: cases.t(v, dev)
    # scale 2^-14 per side would underflow; use the asym epilogue with zero points 0 and scales 1 / 2^-10 so that
    # the binary16 result still distinguishes neighbouring integers where it can: compare through the rounding
    sr, sc = one[:M] * np.float16(2.0 ** -10), one[:N] * np.float16(2.0 ** -10)
    got = hip.linear4bit_forward_bf6(hip.EPI_SYM, hip.activation_shadow_bf6(T(a)), T(sr), None,
                                     hip.weight_shadow_bf6(T(b)), T(sc)).cpu().numpy()
    assert cases.bits_equal(got, orc.sym_dequant(acc, sr, sc))
    # and the integers themselves, through the row-sum epilogue with scales 1 and a correction that brings the
    # accumulator back into binary16's exact range: y = acc - 1 * rc  with rc = acc of row 0
    zr = np.ones((M, 1), np.float16)
    zc = np.zeros((N, 1), np.float16)
    rc = acc[0].astype(np.int32)
    got = hip.linear4bit_forward_bf6(hip.EPI_ASYM_ROWSUM, hip.activation_shadow_bf6(T(a)), T(one[:M]), T(zr),
                                     hip.weight_shadow_bf6(T(b)), T(one[:N]), T(zc), rowsum_x=T(np.zeros(M, np.int32)),
                                     w_rowsum_adj=T(rc)).cpu().numpy()
    assert np.array_equal(got[0].astype(np.int64), np.zeros(N, np.int64))       # row 0: acc - acc, exactly 0
    assert int(got[4, 2]) == acc[4, 2] - acc[0, 2] == 9 and int(got[5, 3]) == acc[5, 3] - acc[0, 3] == 15
    assert cases.bits_equal(got, orc.asym_rowsum_dequant(acc, one[:M], zr, np.zeros(M, np.int32), one[:N], zc, rc))


@pytest.mark.gpu
@pytest.mark.parametrize("M,N,K", [(2048, 4096, 4096), (2048, 11008, 4096), (1000, 4096, 11008), (4096, 4096, 4096),
                                   (8192, 4096, 640)])
def test_gpu_forward_bf6_full_size_equals_integer_kernels(hip, dev, M, N, K):
    """At the benchmark sizes the oracle is too slow: the integer kernels (pinned to the oracle at
    small sizes) are the comparison, on quantizer output, for the whole step."""
    print("bf6 full size", M, N, K, flush=True)
    import torch
    x = cases.t(cases.acts_outliers(M, K, seed=3), dev)
    w = cases.t(cases.acts_normal(N, K, seed=4), dev)
    wq, wsc = hip.quantize_rows_sym(w, 1.0, 7)
    q, s = hip.quantize_rows_sym(x)
    want = hip.linear4bit_forward(hip.EPI_SYM, q, s, None, wq, wsc)
    _, sh, s2 = hip.quantize_rows_sym_bf6(x, with_q=False)
    got = hip.linear4bit_forward_bf6(hip.EPI_SYM, sh, s2, None, hip.weight_shadow_bf6(wq), wsc)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
