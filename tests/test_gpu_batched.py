"""GPU parity of the batched ops: one launch for a whole batch of s4 x s4 products (batched_matmul,
src/export/bindings.cpp:46-86 over src/kernels/gemm.cu:83-117), the batched asymmetric epilogue
(src/kernels/quant.cu:190-239), their fused form, and the two modules of qlinear4bit/nn/matmul.py on 3-D and
4-D inputs.  Every batch entry is compared with the oracle's single-problem functions; integers bit-exact,
binary16 outputs bit-equal."""
import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def _nibbles(n, rows, K, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, 256, (n, rows, K // 2), generator=g, dtype=torch.uint8).numpy()


# (n, M, N, K): one row, B heights off 32, K of one / several / ragged 256-element chunks, shapes on both sides
# of the batched kernel choice (more or fewer than 32 tiles of 32 x 256 over the whole batch), a tile-kernel
# shape with 128-row tiles, short rows (64-row tiles) and a narrow B (128 x 128 tiles)
SHAPES = [(3, 40, 33, 128), (5, 1, 70, 64), (2, 130, 300, 512), (8, 160, 520, 320), (4, 33, 2100, 256),
          (2, 520, 2100, 192), (1, 77, 130, 128), (7, 16, 16, 64), (3, 100, 600, 256), (6, 200, 100, 512),
          (3, 700, 1024, 1024)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_batched_matmul_bit_exact(dev, shape):
    from duqlinear4bitcuda_amd.tools import tensor_utils
    n, M, N, K = shape
    _say("batched_matmul", shape)
    a, b = _nibbles(n, M, K, 1), _nibbles(n, N, K, 2)
    got = tensor_utils.batched_matmul(cases.t(a, dev), cases.t(b, dev))
    assert got.shape == (n, M, N) and got.dtype == torch.int32
    got = got.cpu().numpy()
    for i in range(n):
        assert np.array_equal(got[i], orc.matmul_s4(a[i], b[i])), f"batch entry {i}"


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("mode", ["sym", "asym"])
def test_batched_fused_forward(dev, shape, mode):
    """Fused batched GEMM + dequant (+ bias per batch entry) = oracle GEMM + oracle epilogue per entry =
    the single-problem entry point on the slices."""
    from duqlinear4bitcuda_amd import _HIP as ops
    n, M, N, K = shape
    _say("batch_linear4bit_forward", mode, shape)
    a, b = _nibbles(n, M, K, 3), _nibbles(n, N, K, 4)
    g = np.random.default_rng(5)
    sa = (g.random((n, M, 1)) * 0.05 + 0.01).astype(np.float16)
    sb = (g.random((n, N, 1)) * 0.02 + 0.001).astype(np.float16)
    za = np.rint(g.random((n, M, 1)) * 15).astype(np.float16)
    zb = np.rint(g.random((n, N, 1)) * 15).astype(np.float16)
    bias = g.standard_normal((n, N)).astype(np.float16)
    T = lambda v: cases.t(v, dev)
    for with_bias in (False, True):
        tb = T(bias) if with_bias else None
        if mode == "sym":
            got = ops.batch_linear4bit_forward(ops.EPI_SYM, T(a), T(sa), None, T(b), T(sb), bias=tb)
        else:
            got = ops.batch_linear4bit_forward(ops.EPI_ASYM, T(a), T(sa), T(za), T(b), T(sb), T(zb), bias=tb)
        got = got.cpu().numpy()
        for i in range(n):
            acc = orc.matmul_s4(a[i], b[i])
            want = orc.sym_dequant(acc, sa[i], sb[i]) if mode == "sym" else orc.asym_dequant(acc, sa[i], za[i], sb[i], zb[i])
            if with_bias:
                want = orc.add_bias(want, bias[i])
            assert cases.bits_equal(got[i], want), f"batch entry {i}, bias {with_bias}"
    # against the single-problem entry point on the last slice
    i = n - 1
    if mode == "sym":
        one = ops.linear4bit_forward(ops.EPI_SYM, T(a[i]), T(sa[i]), None, T(b[i]), T(sb[i]), bias=T(bias[i]))
    else:
        one = ops.linear4bit_forward(ops.EPI_ASYM, T(a[i]), T(sa[i]), T(za[i]), T(b[i]), T(sb[i]), T(zb[i]), bias=T(bias[i]))
    assert cases.bits_equal(one.cpu().numpy(), got[i])


@pytest.mark.parametrize("shape", [(6, 40, 33), (3, 17, 64), (70000, 2, 8), (2, 300, 1000)], ids=str)
def test_asym_batch_dequant_one_launch(dev, shape):
    """q [batches, rows, cols] with per-entry parameters; cols that take the 8-wide and the element-wise form;
    more batch entries than one launch holds (65535)."""
    from duqlinear4bitcuda_amd.tools import tensor_utils
    n, rows, cols = shape
    _say("asym_batch_dequant", shape)
    g = np.random.default_rng(9)
    q = g.integers(-70000, 70000, (n, rows, cols), dtype=np.int32)
    sr = (g.random((n, rows, 1)) * 0.05 + 0.01).astype(np.float16)
    sc = (g.random((n, cols, 1)) * 0.02 + 0.001).astype(np.float16)
    zr = np.rint(g.random((n, rows, 1)) * 15).astype(np.float16)
    zc = np.rint(g.random((n, cols, 1)) * 15).astype(np.float16)
    T = lambda v: cases.t(v, dev)
    got = tensor_utils.asym_batch_dequant(T(q), T(sr), T(zr), T(sc), T(zc)).cpu().numpy()
    # the epilogue is element-wise, so one oracle call over the batch-flattened rows with the column parameters
    # broadcast per entry gives every entry's expectation; compare a sample of entries through the
    # single-problem function too
    for i in sorted({0, n // 2, n - 1}):
        assert cases.bits_equal(got[i], orc.asym_dequant(q[i], sr[i], zr[i], sc[i], zc[i])), f"batch entry {i}"
    if n <= 8:
        for i in range(n):
            assert cases.bits_equal(got[i], orc.asym_dequant(q[i], sr[i], zr[i], sc[i], zc[i])), f"batch entry {i}"
    else:  # all entries at once: the oracle's binary16 operators in the epilogue's order, broadcast over the batch
        scr, zcr = sc.reshape(n, 1, cols), zc.reshape(n, 1, cols)
        want = orc.hmul(orc.hmul(sr, scr), orc.hsub(orc.hsub(orc.int_to_half(q), zr), zcr))
        assert cases.bits_equal(got, want)


def test_matmul_modules_issue_one_gemm_launch(dev, monkeypatch):
    """AsymQuantMatMul / SymQuantMatMul on batched inputs: the number of library calls does not grow with the
    batch (two quantizer launches + one fused launch; three steps + two quantizers when fused is off)."""
    from duqlinear4bitcuda_amd import _HIP as ops
    from duqlinear4bitcuda_amd.nn import AsymQuantMatMul, SymQuantMatMul
    calls = []
    real = ops._launch

    def counting(dev_, fn, *args):
        calls.append(getattr(fn, "__name__", str(fn)))
        return real(dev_, fn, *args)

    monkeypatch.setattr(ops, "_launch", counting)
    for n in (2, 24):
        a = cases.t(cases.acts_uniform(n * 48, 128, seed=n).reshape(n, 48, 128), dev)
        b = cases.t(cases.acts_normal(n * 40, 128, seed=n + 1).reshape(n, 40, 128), dev)
        for mod, per_fused, per_steps in ((AsymQuantMatMul(), 3, 4), (SymQuantMatMul(), 3, None)):
            calls.clear()
            mod.fused = True
            mod(a, b)
            assert len(calls) == per_fused, calls
            if per_steps:
                calls.clear()
                mod.fused = False
                mod(a, b)
                assert len(calls) == per_steps, calls


@pytest.mark.parametrize("lead", [(4,), (2, 3)], ids=str)
def test_sym_quant_matmul_batched(dev, lead):
    from duqlinear4bitcuda_amd.nn import SymQuantMatMul
    n = int(np.prod(lead))
    M, N, K = 50, 37, 192
    a = cases.acts_normal(n * M, K, seed=31).reshape(*lead, M, K)
    b = cases.acts_normal(n * N, K, seed=32).reshape(*lead, N, K)
    mod = SymQuantMatMul()
    for fused in (True, False):
        mod.fused = fused
        got = mod(cases.t(a, dev), cases.t(b, dev))
        assert got.shape == (*lead, M, N)
        got = got.cpu().numpy().reshape(n, M, N)
        for i in range(n):
            ai, bi = a.reshape(n, M, K)[i], b.reshape(n, N, K)[i]
            sa, sb = orc.sym_scales(ai), orc.sym_scales(bi)
            want = orc.sym_dequant(orc.matmul_s4(orc.sym_quant(ai, sa), orc.sym_quant(bi, sb)), sa, sb)
            assert cases.bits_equal(got[i], want), f"fused {fused}, batch entry {i}"


def test_attention_like_batch(dev):
    """n = 32 heads, HA = HB = 512 tokens, W = 128: scores Q K^T through AsymQuantMatMul (one launch), sampled
    heads against the oracle; and P V with transpose_B (HB = 128, W = 512)."""
    from duqlinear4bitcuda_amd.nn import AsymQuantMatMul
    n, H, W = 32, 512, 128
    _say("attention-like batch")
    qh = cases.acts_normal(n * H, W, seed=41).reshape(n, H, W)
    kh = cases.acts_normal(n * H, W, seed=42).reshape(n, H, W)
    got = AsymQuantMatMul()(cases.t(qh, dev), cases.t(kh, dev)).cpu().numpy()
    for i in (0, 13, 31):
        sa, za = orc.asym_scales_zeros(qh[i])
        sb, zb = orc.asym_scales_zeros(kh[i])
        acc = orc.matmul_s4(orc.asym_quant(qh[i], sa, za), orc.asym_quant(kh[i], sb, zb))
        assert cases.bits_equal(got[i], orc.asym_dequant(acc, sa, za, sb, zb)), f"head {i}"
    p = cases.acts_uniform(n * H, H, seed=43, hi=1.0).reshape(n, H, H)
    v = cases.acts_normal(n * H, W, seed=44).reshape(n, H, W)       # [n, tokens, W]: B^T of the product P V
    got = AsymQuantMatMul(transpose_B=True)(cases.t(p, dev), cases.t(v, dev)).cpu().numpy()
    assert got.shape == (n, H, W)
    for i in (0, 31):
        vt = np.ascontiguousarray(v[i].T)
        sa, za = orc.asym_scales_zeros(p[i])
        sb, zb = orc.asym_scales_zeros(vt)
        acc = orc.matmul_s4(orc.asym_quant(p[i], sa, za), orc.asym_quant(vt, sb, zb))
        assert cases.bits_equal(got[i], orc.asym_dequant(acc, sa, za, sb, zb)), f"head {i}"


def test_batched_argument_errors(dev):
    from duqlinear4bitcuda_amd import _HIP as ops
    a = torch.zeros((2, 4, 32), dtype=torch.uint8, device=dev)
    with pytest.raises(RuntimeError):
        ops.batched_matmul(a, torch.zeros((3, 4, 32), dtype=torch.uint8, device=dev))
    with pytest.raises(RuntimeError):
        ops.batched_matmul(a, torch.zeros((2, 4, 64), dtype=torch.uint8, device=dev))
    with pytest.raises(RuntimeError):
        ops.batched_matmul(a[0], a[0])
    with pytest.raises(RuntimeError):
        ops.batched_matmul(a.cpu(), a.cpu())
    with pytest.raises(RuntimeError):  # K = 48 is not a multiple of 64
        ops.batched_matmul(torch.zeros((2, 4, 24), dtype=torch.uint8, device=dev),
                           torch.zeros((2, 4, 24), dtype=torch.uint8, device=dev))
    assert ops.batched_matmul(a[:0], a[:0]).shape == (0, 4, 4)


def test_sym_quant_matmul_shapes_of_the_reference_and_mismatch(dev):
    """A with leading dimensions against a 2-D B gives [..., M, N] as the reference's flattening wrappers do
    (qlinear4bit/tools/tensor_utils.py:51-55, nn/matmul.py:76-84); a batched B whose leading dimensions differ from
    A's is rejected with a RuntimeError."""
    from duqlinear4bitcuda_amd.nn import SymQuantMatMul
    a = cases.acts_normal(3 * 20, 128, seed=41).reshape(3, 20, 128)
    b = cases.acts_normal(24, 128, seed=42)
    mod = SymQuantMatMul()
    got = mod(cases.t(a, dev), cases.t(b, dev))
    assert got.shape == (3, 20, 24)
    a2 = a.reshape(60, 128)
    sa, sb = orc.sym_scales(a2), orc.sym_scales(b)
    want = orc.sym_dequant(orc.matmul_s4(orc.sym_quant(a2, sa), orc.sym_quant(b, sb)), sa, sb)
    assert cases.bits_equal(got.cpu().numpy().reshape(60, 24), want)
    with pytest.raises(RuntimeError, match="leading dimensions"):
        mod(cases.t(a[0], dev), cases.t(np.stack([b, b]), dev))
    with pytest.raises(RuntimeError, match="leading dimensions"):
        mod(cases.t(a, dev), cases.t(np.stack([b, b]), dev))
