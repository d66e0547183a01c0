"""GPU parity of the decode kernels (up to 64 activation rows) and of the quantize + GEMM + dequant entry point
that takes binary16 activations, against the oracle, through the C ABI."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def hip(dev):
    from duqlinear4bitcuda_amd import _HIP

    return _HIP


# rows kernel (M <= 4: every K bucket, K and N tails), MFMA decode kernel (5..16 rows: K buckets of 4096 / 8192 /
# 12288, tiles that end inside N, several tiles per workgroup), ring kernel for long rows
SHAPES = [(1, 64, 64), (1, 20, 128), (2, 37, 4096), (3, 100, 2048), (4, 4096, 4096), (1, 4096, 4096), (1, 515, 11008),
          (4, 130, 8192), (2, 64, 16384), (3, 33, 12352), (1, 11008, 4096),
          # three or four rows from binary16 on more than 256 column tiles: several tiles per workgroup
          (4, 11008, 4096), (3, 4500, 8192), (4, 9001, 2048), (4, 16384, 64), (4, 4112, 12288),
          (5, 64, 64), (16, 48, 128), (7, 100, 4096), (16, 4096, 4096), (16, 1000, 11008), (9, 257, 8192),
          (13, 77, 12288), (8, 50, 2112), (16, 32, 6208),
          (16, 11008, 4096), (6, 8200, 8192), (11, 8192, 2048),
          (12, 40, 16384), (16, 24, 12352),
          # five to eight rows: from binary16 the rows kernel with eight rows (one launch), pre-quantized the MFMA kernel
          (5, 4096, 4096), (8, 11008, 4096), (6, 300, 2048), (7, 4100, 8192), (8, 16384, 64), (8, 8200, 8192), (8, 20000, 128),
          # nine to sixteen rows of at most 32768 elements together (40960 on at most 4096 columns): from binary16 the MFMA
          # kernel quantizes them itself
          (16, 4090, 2048), (9, 300, 4096), (8, 11008, 4032), (12, 520, 3072), (16, 100, 2560), (13, 9000, 1984),
          (16, 16384, 1024), (11, 4096, 3712),
          # up to eight rows on more than 16384 columns: one launch from binary16 (rows of at most 8192 elements at
          # two to four rows, of at most 4096 at five to eight)
          (4, 20000, 8192), (2, 17000, 4096), (3, 30000, 256), (8, 20000, 4096), (5, 40000, 1024), (7, 17000, 2112),
          # MFMA decode kernel with two to four row tiles (17..64 rows of at most 4096 elements, 17..32 of at most
          # 8192), one to several column tiles per workgroup, tiles that end inside M and N
          (17, 4096, 4096), (32, 300, 4096), (33, 4099, 2048), (48, 1000, 4096), (64, 11008, 4096), (50, 72, 64),
          (64, 40, 128), (20, 520, 8192), (32, 4100, 8192), (29, 9000, 4160), (64, 5000, 1024),
          # the long-row forms (three and four row tiles of up to 8192 elements, two and three of up to 12288: from
          # 192 column tiles on) and their neighbours on the ring kernel
          (33, 3072, 8192), (64, 3100, 4160), (48, 4096, 11008), (20, 3080, 12288), (40, 6200, 8256),
          (33, 300, 8192), (64, 130, 4160), (49, 3072, 11008),
          # 9..16 rows on 1536 or more column tiles: the skinny kernel
          (9, 24600, 64), (16, 28672, 256),
          # rows longer than 16384 elements: the dot kernel
          (1, 300, 20480), (1, 64, 28672), (1, 130, 16448), (2, 100, 20480), (4, 40, 28672)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_decode_kernels_against_the_oracle(hip, dev, M, N, K):
    """int32 accumulators bit-exact, every fused epilogue bit-equal to the oracle's dequant of them, and the
    binary16-input entry point equal to quantizer + forward (codes and scales included)."""
    _say("decode", M, N, K, "kernel", hip.gemm_kernel_for(M, N, K))
    rng = np.random.default_rng(M * 7 + N + K)
    x = cases.acts_outliers(M, K, seed=M + K)
    wq, sw = cases.weights_random_nibbles(N, K, seed=N + K)
    sw2 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    zw = rng.integers(0, 16, (N, 1)).astype(np.float16)
    zw2 = rng.integers(0, 16, (N, 1)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    sx = orc.sym_scales(x)
    q = orc.sym_quant(x, sx)
    zx = rng.integers(0, 16, (M, 1)).astype(np.float16)
    acc = orc.matmul_s4(q, wq)
    X, W, Q, SX, ZX = (cases.t(a, dev) for a in (x, wq, q, sx, zx))
    SW, SW2, ZW, ZW2, B = (cases.t(a, dev) for a in (sw, sw2, zw, zw2, bias))
    assert np.array_equal(hip.matmul(Q, W).cpu().numpy(), acc)
    want = {
        hip.EPI_SYM: orc.sym_dequant(acc, sx, sw),
        hip.EPI_ASYM: orc.asym_dequant(acc, sx, zx, sw, zw),
        hip.EPI_SYM_DUAL: orc.sym_dual_dequant(acc, sx, sw, sw2),
        hip.EPI_ASYM_DUAL: orc.asym_dual_dequant(acc, sx, zx, sw, zw, sw2, zw2),
    }
    for mode, w in want.items():
        asym, dual = mode in (hip.EPI_ASYM, hip.EPI_ASYM_DUAL), mode in (hip.EPI_SYM_DUAL, hip.EPI_ASYM_DUAL)
        for b in (None, B):
            y = hip.linear4bit_forward(mode, Q, SX, ZX if asym else None, W, SW, ZW if asym else None,
                                       SW2 if dual else None, ZW2 if asym and dual else None, b)
            assert cases.bits_equal(y.cpu().numpy(), w if b is None else orc.add_bias(w, bias)), (mode, b is not None)
    for sw2_t, b, w in ((None, None, want[hip.EPI_SYM]), (SW2, B, orc.add_bias(want[hip.EPI_SYM_DUAL], bias))):
        y, qf, sf = hip.quantize_linear4bit_forward(X, W, SW, sw2_t, b, return_quantized=True)
        assert cases.bits_equal(y.cpu().numpy(), w)
        assert np.array_equal(qf.cpu().numpy(), q) and cases.bits_equal(sf.cpu().numpy(), sx)
        assert cases.bits_equal(hip.quantize_linear4bit_forward(X, W, SW, sw2_t, b).cpu().numpy(), w)


def test_decode_rowsum_epilogue(hip, dev):
    """The row-sum epilogue (mode 4) through both decode kernels."""
    for M, N, K in ((3, 96, 512), (10, 80, 4096)):
        _say("decode rowsum", M, N, K)
        x = cases.acts_uniform(M, K, seed=31 + M)
        w = (torch.randn(N, K, generator=torch.Generator().manual_seed(M)) * 0.02).to(torch.float16).numpy()
        wq, sw, zw, adj = orc.weight_asym_shifted_from_linear(w)
        want, *_ = orc.linear4bit_asq_rowsum_forward(x, wq, sw, zw, adj)
        q, s, z, r = hip.quantize_rows_asym_shifted(cases.t(x, dev))
        y = hip.linear4bit_forward_rowsum(q, s, z, r, cases.t(wq, dev), cases.t(sw, dev), cases.t(zw, dev), cases.t(adj, dev))
        assert cases.bits_equal(y.cpu().numpy(), want)


@pytest.mark.parametrize("M", [1, 2, 4, 7, 12, 16])
def test_fp16_input_special_rows_and_clamps(hip, dev, M):
    """Rows of zeros, with an infinity, with a NaN, with subnormals only, clip 0.9 and both upper clamps: the
    one-launch path gives the stand-alone quantizer's codes and scales and the oracle's outputs."""
    _say("decode special rows", M)
    N, K = 72, 1024
    x = cases.acts_normal(max(M, 4), K, seed=5)
    x[0] = 0
    x[1, 7] = np.inf
    x[2, 100] = np.nan
    x[3] = np.float16(3e-7)
    x = np.ascontiguousarray(x[:M]) if M > 1 else np.ascontiguousarray(x[[1]])
    wq, sw = cases.weights_random_nibbles(N, K, seed=9)
    for clip, qmax in ((1.0, 6), (0.9, 7)):
        sx = orc.sym_scales(x, clip)
        q = orc.sym_quant(x, sx, qmax)
        want = orc.sym_dequant(orc.matmul_s4(q, wq), sx, sw)
        y, qf, sf = hip.quantize_linear4bit_forward(cases.t(x, dev), cases.t(wq, dev), cases.t(sw, dev), clip=clip,
                                                    qmax=qmax, return_quantized=True)
        assert np.array_equal(qf.cpu().numpy(), q) and cases.bits_equal(sf.cpu().numpy(), sx)
        assert cases.bits_equal(y.cpu().numpy(), want)


@pytest.mark.parametrize("kind", ["zeros", "inf", "nan", "subnormal", "normal"])
def test_fp16_input_one_long_row(hip, dev, kind):
    """One row of 20480 elements (quantizer launch + dot kernel): special rows, clip 0.9 and both upper clamps give
    the stand-alone quantizer's codes and scales and the oracle's outputs."""
    _say("long row", kind)
    N, K = 40, 20480
    x = cases.acts_normal(1, K, seed=15)
    if kind == "zeros":
        x[:] = 0
    elif kind == "inf":
        x[0, 20000] = -np.inf
    elif kind == "nan":
        x[0, 17] = np.nan
    elif kind == "subnormal":
        x[:] = np.float16(-2e-7)
    wq, sw = cases.weights_random_nibbles(N, K, seed=19)
    for clip, qmax in ((1.0, 6), (0.9, 7)):
        sx = orc.sym_scales(x, clip)
        q = orc.sym_quant(x, sx, qmax)
        want = orc.sym_dequant(orc.matmul_s4(q, wq), sx, sw)
        y, qf, sf = hip.quantize_linear4bit_forward(cases.t(x, dev), cases.t(wq, dev), cases.t(sw, dev), clip=clip,
                                                    qmax=qmax, return_quantized=True)
        assert np.array_equal(qf.cpu().numpy(), q) and cases.bits_equal(sf.cpu().numpy(), sx)
        assert cases.bits_equal(y.cpu().numpy(), want)


def test_fp16_input_entry_point_workspace_and_errors(dev):
    """The C entry point itself: one-launch shapes take no workspace; others need it (too small / missing /
    misaligned is rejected before any launch) and give the same bits; unknown modes are rejected."""
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    M, N, K = 24, 96, 256
    x = cases.acts_normal(M, K, seed=3)
    wq, sw = cases.weights_random_nibbles(N, K, seed=4)
    want, *_ = orc.linear4bit_sq_forward(x, wq, sw)
    X, W, SW = cases.t(x, dev), cases.t(wq, dev), cases.t(sw, dev)
    y = torch.zeros(M, N, dtype=torch.float16, device=dev)
    need = lib.duq_quantize_linear4bit_workspace_bytes(M, N, K)
    assert need == M * K // 2 + 48 and lib.duq_quantize_linear4bit_workspace_bytes(1, N, K) == 0
    ws = torch.zeros(need + 16, dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    call = lambda mode, wsp, nbytes, m=M: lib.duq_quantize_linear4bit_forward(
        mode, X.data_ptr(), 1.0, 6, W.data_ptr(), SW.data_ptr(), None, None, m, N, K, y.data_ptr(), None, None, wsp,
        nbytes, st)
    assert call(0, None, 0) == -1
    assert call(0, ws.data_ptr(), need - 1) == -2
    assert call(0, ws.data_ptr() + 8, need) == -5
    assert call(1, ws.data_ptr(), need) == -4 and call(2, ws.data_ptr(), need) == -1  # asym unsupported; dual needs scale 2
    assert call(0, ws.data_ptr(), need) == 0
    torch.cuda.synchronize()
    assert cases.bits_equal(y.cpu().numpy(), want)
    # the staged codes and scales are the quantizer's
    assert np.array_equal(ws[:M * K // 2].view(M, K // 2).cpu().numpy(), orc.sym_quant(x, orc.sym_scales(x)))
    y.zero_()
    assert call(0, None, 0, 3) == 0  # three rows: one launch, no workspace
    torch.cuda.synchronize()
    assert cases.bits_equal(y[:3].cpu().numpy(), want[:3]) and not y[3:].any()


def test_config2_all_shapes_one_launch(hip, dev):
    """Benchmark configuration 2 (M in {1, 4, 16}, K = 4096, N in {4096, 11008}; uniform random nibbles, scales
    U[0.001, 0.01], activations ~N(0,1)) from binary16 activations through the single entry point."""
    K = 4096
    for N in (4096, 11008):
        wq, sw = cases.weights_random_nibbles(N, K, seed=22)
        W, SW = cases.t(wq, dev), cases.t(sw, dev)
        for M in (1, 4, 16):
            _say("config 2 fp16-in", M, N)
            x = cases.acts_normal(M, K, seed=2)
            want, *_ = orc.linear4bit_sq_forward(x, wq, sw)
            assert cases.bits_equal(hip.quantize_linear4bit_forward(cases.t(x, dev), W, SW).cpu().numpy(), want)
