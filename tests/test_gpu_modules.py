"""GPU tests of the module layer and of the benchmark configurations: module forward ==
oracle composition, leading dimensions, error paths, and size-independent properties at
the full benchmark sizes where the oracle would be too slow."""
import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from oracle import duq_oracle_c as orc_c
from tests import cases

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def qnn(dev):
    from duqlinear4bitcuda_amd import nn

    return nn


def _sq_module(qnn, dev, wq, sw, bias=None):
    N, K = wq.shape[0], wq.shape[1] * 2
    lin = qnn.Linear4bitSQ(K, N, bias=bias is not None).half().to(dev)
    sd = {"weight": cases.t(wq, dev), "weight_scales": cases.t(sw, dev)}
    if bias is not None:
        sd["bias"] = cases.t(bias, dev)
    lin.load_state_dict(sd)
    return lin


def test_config1_cpu_fakequant_parity(qnn, dev):
    """Config 1: M16, K = N = 4096, N(0,1) activations with 0.5 % channels x20, W ~ N(0,0.02)
    quantized per output channel; both clamp conventions; packed codes and accumulators
    bit-exact, fp16 outputs equal."""
    _say("config 1")
    M, K, N = 16, 4096, 4096
    x = cases.acts_outliers(M, K, seed=1)
    wq, sw = cases.weights_from_float_sym(N, K, seed=11)
    lin = _sq_module(qnn, dev, wq, sw)
    from duqlinear4bitcuda_amd.tools import tensor_utils as tu

    for qmax in (6, 7):
        y_want, acc_want, q_want, s_want = orc.linear4bit_sq_forward(x, wq, sw, qmax=qmax)
        p = qnn.SymQuantizer(1.0, qmax=qmax)(cases.t(x, dev))
        assert np.array_equal(p.quantized_x.cpu().numpy(), q_want)
        assert cases.bits_equal(p.scales_x.cpu().numpy(), s_want)
        acc = tu.matmul(p.quantized_x, lin.weight)
        assert np.array_equal(acc.cpu().numpy(), acc_want)
        y = lin(p).cpu().numpy()
        assert cases.bits_equal(y, y_want)
        rel = np.abs(y.astype(np.float32) - y_want.astype(np.float32)) / np.maximum(np.abs(y_want.astype(np.float32)), 1e-3)
        assert rel.max() <= 1e-3  # the stated bar; bit equality above is stronger


@pytest.mark.parametrize("M,N", [(1, 4096), (4, 4096), (16, 4096), (1, 11008), (4, 11008), (16, 11008)])
def test_config2_decode(qnn, dev, M, N):
    _say("config 2", M, N)
    K = 4096
    x = cases.acts_normal(M, K, seed=2)
    wq, sw = cases.weights_random_nibbles(N, K, seed=22)
    y_want, acc_want, q_want, s_want = orc.linear4bit_sq_forward(x, wq, sw)
    lin = _sq_module(qnn, dev, wq, sw)
    y = torch.nn.Sequential(qnn.SymQuantizer(1.0), lin)(cases.t(x, dev)).cpu().numpy()
    assert cases.bits_equal(y, y_want)


def test_config3_prefill_against_c_oracle(qnn, dev):
    """Config 3 at full size for K = N = 4096 (the C oracle does the 34 G multiply-adds on
    the host cores), heavy-tailed activations."""
    _say("config 3 full")
    M, K, N = 2048, 4096, 4096
    x = cases.acts_heavy_tail(M, K, seed=3)
    wq, sw = cases.weights_random_nibbles(N, K, seed=33)
    s_want = orc.sym_scales(x)
    q_want = orc.sym_quant(x, s_want)
    lin = _sq_module(qnn, dev, wq, sw)
    p = qnn.SymQuantizer(1.0)(cases.t(x, dev))
    assert np.array_equal(p.quantized_x.cpu().numpy(), q_want)
    assert cases.bits_equal(p.scales_x.cpu().numpy(), s_want)
    from duqlinear4bitcuda_amd.tools import tensor_utils as tu

    acc_want = orc_c.matmul_s4(q_want, wq)
    acc = tu.matmul(p.quantized_x, lin.weight).cpu().numpy()
    assert np.array_equal(acc, acc_want)
    y_want = orc.sym_dequant(acc_want, s_want, sw)
    y = lin(p).cpu().numpy()
    assert cases.bits_equal(y, y_want)
    # the same forward on the 6-bit float matrix path (the benchmark's headline kernel at its headline shape),
    # from the shadow-writing quantizer: directly against the oracle
    lin.enable_fp6()
    for shadow in ("only", True):
        p6 = qnn.SymQuantizer(1.0, shadow=shadow, shadow_min_rows=1)(cases.t(x, dev))
        assert p6.shadow_x is not None and cases.bits_equal(p6.scales_x.cpu().numpy(), s_want)
        if shadow is True:
            assert np.array_equal(p6.quantized_x.cpu().numpy(), q_want)
        assert lin._use_shadow(p6)
        assert cases.bits_equal(lin(p6).cpu().numpy(), y_want)
    from duqlinear4bitcuda_amd import _HIP as hip

    assert np.array_equal(p6.shadow_x.cpu().numpy(), orc.activation_shadow_bf6(q_want))
    y6 = hip.linear4bit_forward_bf6(hip.EPI_SYM, p6.shadow_x, p6.scales_x, None, lin.weight_shadow, lin.weight_scales)
    assert cases.bits_equal(y6.cpu().numpy(), y_want)


@pytest.mark.parametrize("K,N", [(4096, 11008), (11008, 4096)])
def test_config3_other_shapes_by_properties(qnn, dev, K, N):
    """Full-size prefill shapes checked through properties that need no CPU GEMM:
    (1) a sampled set of rows/columns against the oracle, (2) linearity in the weights:
    acc(A, B1) + acc(A, B2) == acc(A, B1 + B2) when the nibble sums stay in range,
    (3) the fused fp16 output equals the stand-alone dequant of the int32 output."""
    _say("config 3 properties", K, N)
    M = 2048
    from duqlinear4bitcuda_amd import _HIP as hip

    rng = np.random.default_rng(K + N)
    x = cases.acts_heavy_tail(M, K, seed=3)
    q, s = hip.quantize_rows_sym(cases.t(x, dev))
    b1 = rng.integers(-4, 4, (N, K)).astype(np.int8)
    b2 = rng.integers(-4, 4, (N, K)).astype(np.int8)
    B1, B2, B12 = (cases.t(orc.pack_i4(b), dev) for b in (b1, b2, b1 + b2))
    c1, c2, c12 = hip.matmul(q, B1), hip.matmul(q, B2), hip.matmul(q, B12)
    assert torch.equal(c1 + c2, c12)
    rows = rng.choice(M, 24, replace=False)
    cols = rng.choice(N, 40, replace=False)
    a_cpu = orc.unpack_i4(q.cpu().numpy()[rows]).astype(np.int64)
    want = a_cpu @ b1[cols].astype(np.int64).T
    assert np.array_equal(c1.cpu().numpy()[np.ix_(rows, cols)], want)
    sw = cases.t(rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16), dev)
    y_fused = hip.linear4bit_forward(hip.EPI_SYM, q, s, None, B1, sw)
    y_unfused = hip.sym_dequant(c1, s.view(-1), sw, 32)
    assert torch.equal(y_fused.view(torch.int16), y_unfused.view(torch.int16))


def test_config4_asym_dual_uniform(qnn, dev):
    _say("config 4")
    M, K, N = 512, 4096, 4096
    x = cases.acts_uniform(M, K, seed=4)
    wq, sw, zw = cases.weights_from_linear_asym(N, K, seed=44)
    y_want, acc_want, q_want, s_want, z_want = orc.linear4bit_asq_forward(x, wq, sw, zw)
    m = qnn.Linear4bitASQ(K, N).to(dev)
    m.load_state_dict({"weight": cases.t(wq, dev), "weight_scales": cases.t(sw, dev), "weight_zeros": cases.t(zw, dev)})
    p = m.quantizer(cases.t(x, dev))
    assert np.array_equal(p.quantized_x.cpu().numpy(), q_want)
    assert cases.bits_equal(p.scales_x.cpu().numpy(), s_want) and cases.bits_equal(p.zeros_x.cpu().numpy(), z_want)
    from duqlinear4bitcuda_amd.tools import tensor_utils as tu

    assert np.array_equal(tu.matmul(p.quantized_x, m.weight).cpu().numpy(), acc_want)
    assert cases.bits_equal(m(cases.t(x, dev)).cpu().numpy(), y_want)
    # the dual-uniform layer on the same input (from_linear on the device)
    lin = torch.nn.Linear(K, N, bias=False).half()
    with torch.no_grad():
        lin.weight.copy_((torch.randn(N, K, generator=torch.Generator().manual_seed(45)) * 0.02).half())
    du = qnn.LinearQuant4bitDUASQ.from_linear(lin).to(dev)
    sd = {k: v.cpu().numpy() for k, v in du.state_dict().items()}
    y_want, *_ = orc.linear4bit_duasq_forward(x, sd["weight"], sd["weight_scales_1"], sd["weight_zeros_1"],
                                             sd["weight_scales_2"], sd["weight_zeros_2"])
    assert cases.bits_equal(du(cases.t(x, dev)).cpu().numpy(), y_want)


@pytest.mark.parametrize("M,K,N", [(1, 8192, 28672), (1, 28672, 8192)])
def test_config5_decode_70b_shapes(qnn, dev, M, K, N):
    _say("config 5 decode", K, N)
    x = cases.acts_outliers(M, K, seed=5)
    wq, sw = cases.weights_random_nibbles(N, K, seed=55)
    y_want, *_ = orc.linear4bit_sq_forward(x, wq, sw)
    lin = _sq_module(qnn, dev, wq, sw)
    y = lin(qnn.SymQuantizer(1.0)(cases.t(x, dev))).cpu().numpy()
    assert cases.bits_equal(y, y_want)


@pytest.mark.parametrize("K,N", [(8192, 28672), (28672, 8192)])
def test_config5_prefill_70b_shape_by_properties(qnn, dev, K, N):
    """M 4096 at both Llama-2-70B MLP shapes (1.9 T multiply-adds each): quantizer rows and sampled accumulators
    against the oracle, fused == unfused, and the 6-bit float matrix path == the integer path == the oracle on the
    sampled entries."""
    _say("config 5 prefill", K, N)
    from duqlinear4bitcuda_amd import _HIP as hip

    M = 4096
    rng = np.random.default_rng(5)
    x = cases.acts_outliers(M, K, seed=5)
    X = cases.t(x, dev)
    q, s = hip.quantize_rows_sym(X)
    assert np.array_equal(q.cpu().numpy()[::97], orc.sym_quant(x[::97], orc.sym_scales(x[::97])))
    wq, sw = cases.weights_random_nibbles(N, K, seed=56)
    W, SW = cases.t(wq, dev), cases.t(sw, dev)
    c = hip.matmul(q, W)
    rows = rng.choice(M, 16, replace=False)
    cols = rng.choice(N, 32, replace=False)
    want = orc.unpack_i4(q.cpu().numpy()[rows]).astype(np.int64) @ orc.unpack_i4(wq[cols]).astype(np.int64).T
    assert np.array_equal(c.cpu().numpy()[np.ix_(rows, cols)], want)
    y_fused = hip.linear4bit_forward(hip.EPI_SYM, q, s, None, W, SW)
    y_unfused = hip.sym_dequant(c, s.view(-1), SW, 32)
    assert torch.equal(y_fused.view(torch.int16), y_unfused.view(torch.int16))
    del c, y_unfused
    y_want = orc.sym_dequant(want, s.cpu().numpy()[rows], sw[cols])
    assert cases.bits_equal(y_fused.cpu().numpy()[np.ix_(rows, cols)], y_want)
    _, xs, s6 = hip.quantize_rows_sym_bf6(X, with_q=False)
    assert torch.equal(s6, s)
    y6 = hip.linear4bit_forward_bf6(hip.EPI_SYM, xs, s6, None, hip.weight_shadow_bf6(W), SW)
    assert torch.equal(y6.view(torch.int16), y_fused.view(torch.int16))


@pytest.mark.parametrize("K,N", [(5120, 5120), (5120, 13824), (13824, 5120)])
def test_llama13b_shapes_by_properties(qnn, dev, K, N):
    """The Llama-2-13B layer sizes of the reference's own benchmark (test/benchmark.py:8-18: 5120 x 5120 and
    5120 x 13824; 320 / 864 output tiles of 128 x 256 at 2048 tokens, i.e. ragged rounds on 256 CUs) on both matrix
    paths: quantizer rows and sampled accumulators against the oracle, fused == unfused, the 6-bit float path == the
    integer path, and the module forward at 2048, 16 and 1 tokens against the oracle on sampled outputs."""
    _say("13B shape", K, N)
    from duqlinear4bitcuda_amd import _HIP as hip

    M = 2048
    rng = np.random.default_rng(K + 3 * N)
    x = cases.acts_heavy_tail(M, K, seed=13)
    X = cases.t(x, dev)
    q, s = hip.quantize_rows_sym(X)
    assert np.array_equal(q.cpu().numpy()[::131], orc.sym_quant(x[::131], orc.sym_scales(x[::131])))
    wq, sw = cases.weights_random_nibbles(N, K, seed=130)
    W, SW = cases.t(wq, dev), cases.t(sw, dev)
    c = hip.matmul(q, W)
    rows = np.concatenate([rng.choice(M, 14, replace=False), [0, M - 1]])
    cols = np.concatenate([rng.choice(N, 30, replace=False), [0, N - 1]])
    want = orc.unpack_i4(q.cpu().numpy()[rows]).astype(np.int64) @ orc.unpack_i4(wq[cols]).astype(np.int64).T
    assert np.array_equal(c.cpu().numpy()[np.ix_(rows, cols)], want)
    y_fused = hip.linear4bit_forward(hip.EPI_SYM, q, s, None, W, SW)
    assert torch.equal(y_fused.view(torch.int16), hip.sym_dequant(c, s.view(-1), SW, 32).view(torch.int16))
    y_want = orc.sym_dequant(want, s.cpu().numpy()[rows], sw[cols])
    assert cases.bits_equal(y_fused.cpu().numpy()[np.ix_(rows, cols)], y_want)
    lin = _sq_module(qnn, dev, wq, sw)
    lin.enable_fp6()
    p6 = qnn.SymQuantizer(1.0, shadow="only", shadow_min_rows=1)(X)
    assert lin._use_shadow(p6)
    assert torch.equal(lin(p6).view(torch.int16), y_fused.view(torch.int16))
    # decode through the modules at the same layer: 16 tokens (two launches) and 1 token (one launch), full oracle
    for m in (16, 1):
        xm = x[:m]
        y_m = torch.nn.Sequential(qnn.SymQuantizer(1.0), lin)(cases.t(xm, dev).view(1, m, K)).cpu().numpy().reshape(m, N)
        sm = orc.sym_scales(xm)
        acc_cols = orc.unpack_i4(orc.sym_quant(xm, sm)).astype(np.int64) @ orc.unpack_i4(wq[cols]).astype(np.int64).T
        assert cases.bits_equal(y_m[:, cols], orc.sym_dequant(acc_cols, sm, sw[cols]))
        assert cases.bits_equal(y_m, y_fused.cpu().numpy()[:m])


def test_leading_dims_and_odd_widths(qnn, dev):
    """[B, S, K] inputs keep their leading dims; a width that is not a multiple of 32 takes
    the torch-scale + given-scale kernel route and gives the same bits."""
    _say("leading dims")
    B, S, K, N = 2, 5, 128, 64
    x = cases.acts_normal(B * S, K, seed=6).reshape(B, S, K)
    wq, sw = cases.weights_random_nibbles(N, K, seed=66)
    lin = _sq_module(qnn, dev, wq, sw)
    p = qnn.SymQuantizer(1.0)(cases.t(x, dev))
    assert tuple(p.quantized_x.shape) == (B, S, K // 2) and tuple(p.scales_x.shape) == (B, S, 1)
    y = lin(p)
    assert tuple(y.shape) == (B, S, N)
    y_want, *_ = orc.linear4bit_sq_forward(x.reshape(-1, K), wq, sw)
    assert cases.bits_equal(y.cpu().numpy().reshape(-1, N), y_want)
    lin.fused = False
    assert cases.bits_equal(lin(p).cpu().numpy().reshape(-1, N), y_want)
    # odd width for the quantizers only (the GEMM needs K % 64 == 0)
    xo = cases.acts_normal(7, 50, seed=7)
    po = qnn.SymQuantizer(1.0)(cases.t(xo, dev))
    so = orc.sym_scales(xo)
    assert cases.bits_equal(po.scales_x.cpu().numpy(), so)
    assert np.array_equal(po.quantized_x.cpu().numpy(), orc.sym_quant(xo, so))
    pa = qnn.AsymQuantizer()(cases.t(xo, dev))
    sa, za = orc.asym_scales_zeros(xo)
    assert cases.bits_equal(pa.scales_x.cpu().numpy(), sa) and cases.bits_equal(pa.zeros_x.cpu().numpy(), za)
    assert np.array_equal(pa.quantized_x.cpu().numpy(), orc.asym_quant(xo, sa, za))
    # a non-contiguous input is made contiguous first (quantizer.py:11-12)
    xt = cases.t(cases.acts_normal(64, 8, seed=8), dev).t()
    pt = qnn.SymQuantizer(1.0)(xt)
    assert np.array_equal(pt.quantized_x.cpu().numpy(), orc.sym_quant(xt.cpu().numpy(), orc.sym_scales(xt.cpu().numpy())))


def test_error_paths_on_device(dev):
    from duqlinear4bitcuda_amd import _HIP as hip
    from duqlinear4bitcuda_amd.tools import tensor_utils as tu

    a = torch.zeros(4, 32, dtype=torch.uint8, device=dev)
    q = torch.zeros(4, 4, dtype=torch.int32, device=dev)
    s4 = torch.ones(4, dtype=torch.float16, device=dev)
    with pytest.raises(RuntimeError, match="Unsupported data type"):
        hip.sym_dequant(q, s4, s4, 16)                                   # bindings.cpp:159-167
    with pytest.raises(RuntimeError, match="contiguous"):
        hip.matmul(a.t(), a)
    with pytest.raises(RuntimeError, match="size"):
        hip.sym_dequant(q, s4[:3], s4, 32)
    with pytest.raises(RuntimeError, match="size"):
        hip.sym_quant(torch.zeros(4, 64, dtype=torch.float16, device=dev), s4[:2])
    with pytest.raises(RuntimeError):
        hip.matmul(a, torch.zeros(4, 32, dtype=torch.uint8))             # other device
    with pytest.raises(RuntimeError, match="multiple of 64"):
        hip.matmul(torch.zeros(4, 48, dtype=torch.uint8, device=dev), torch.zeros(4, 48, dtype=torch.uint8, device=dev))
    with pytest.raises(AssertionError):
        tu.matmul(torch.zeros(4, 48, dtype=torch.uint8, device=dev), torch.zeros(4, 48, dtype=torch.uint8, device=dev))
    # empty problems are no-ops
    assert tuple(hip.matmul(a[:0], a).shape) == (0, 4)
    assert tuple(hip.sym_quant(torch.zeros(0, 64, dtype=torch.float16, device=dev), s4[:0]).shape) == (0, 32)


def test_runs_on_a_side_stream(qnn, dev):
    """The ops launch on torch's current stream."""
    M, K, N = 64, 256, 128
    x = cases.acts_normal(M, K, seed=9)
    wq, sw = cases.weights_random_nibbles(N, K, seed=99)
    lin = _sq_module(qnn, dev, wq, sw)
    want, *_ = orc.linear4bit_sq_forward(x, wq, sw)
    side = torch.cuda.Stream()
    xt = cases.t(x, dev)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        y = lin(qnn.SymQuantizer(1.0)(xt))
    side.synchronize()
    assert cases.bits_equal(y.cpu().numpy(), want)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(48, 256, 192), (6, 4096, 512), (384, 1024, 1024)])
def test_libtorch_classes_fused_equals_three_step(shape):
    """The C++ classes of include/duq_torch.hpp (twin of the reference's include/linear.h and
    include/quant_tensor.h) run in a stand-alone libtorch program: fused forward == matmul +
    dequant + bias bit for bit, quantizer scale/codes as specified, error paths raise."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "duq_torch_check")
    assert os.path.exists(exe), "tests/cpp/duq_torch_check is not built (run build())"
    r = subprocess.run([exe] + [str(v) for v in shape], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and r.stdout.startswith("OK"), (r.returncode, r.stdout[-2000:], r.stderr[-2000:])


@pytest.mark.gpu
def test_libtorch_classes_against_the_oracle_fixture(tmp_path):
    """The same program fed with the committed fixture (tests/golden/linear4bit_small.npz, every array written out
    as a raw file): Quantizer4bit codes and scales, Linear4bit::from_float / Linear4bitDUQ::from_float weight codes
    prepared on the device, int32 accumulators and both layers' forwards equal the CPU oracle's."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "duq_torch_check")
    assert os.path.exists(exe), "tests/cpp/duq_torch_check is not built (run build())"
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "linear4bit_small.npz"))
    for k in g.files:
        np.ascontiguousarray(g[k]).tofile(str(tmp_path / f"{k}.bin"))
    r = subprocess.run([exe, "--fixture", str(tmp_path)], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and r.stdout.startswith("OK fixture"), (r.returncode, r.stdout[-2000:], r.stderr[-2000:])


@pytest.mark.gpu
def test_sym_quant_matmul_module(dev):
    """SymQuantMatMul (qlinear4bit/nn/matmul.py:69-84): both operands quantized per row, A @ B^T."""
    from duqlinear4bitcuda_amd.nn import SymQuantMatMul
    a = cases.acts_outliers(48, 256, seed=71)
    b = cases.acts_normal(96, 256, seed=72)
    sa, sb = orc.sym_scales(a), orc.sym_scales(b)
    want = orc.sym_dequant(orc.matmul_s4(orc.sym_quant(a, sa), orc.sym_quant(b, sb)), sa, sb)
    mod = SymQuantMatMul()
    for fused in (True, False):
        mod.fused = fused
        got = mod(cases.t(a, dev), cases.t(b, dev)).cpu().numpy()
        assert cases.bits_equal(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("transpose_b", [False, True])
def test_asym_quant_matmul_module(dev, transpose_b):
    """AsymQuantMatMul (qlinear4bit/nn/matmul.py:19-66): batched, per-batch-entry scales and zero
    points, a B height that is not a multiple of 32 (the reference pads and unpads it)."""
    from duqlinear4bitcuda_amd.nn import AsymQuantMatMul
    from duqlinear4bitcuda_amd.tools import tensor_utils
    lead, HA, HB, W = (2, 3), 40, 33, 128
    a = cases.acts_uniform(6 * HA, W, seed=81).reshape(*lead, HA, W)
    b = cases.acts_normal(6 * HB, W, seed=82).reshape(*lead, HB, W)
    want = np.empty((*lead, HA, HB), np.float16)
    accs = np.empty((6, HA, HB), np.int32)
    params = []
    for i in range(2):
        for j in range(3):
            sa, za = orc.asym_scales_zeros(a[i, j])
            sb, zb = orc.asym_scales_zeros(b[i, j])
            acc = orc.matmul_s4(orc.asym_quant(a[i, j], sa, za), orc.asym_quant(b[i, j], sb, zb))
            want[i, j] = orc.asym_dequant(acc, sa, za, sb, zb)
            accs[i * 3 + j] = acc
            params.append((sa, za, sb, zb))
    mod = AsymQuantMatMul(transpose_B=transpose_b)
    tb = cases.t(b, dev)
    if transpose_b:
        tb = tb.transpose(-1, -2).contiguous()
    for fused in (True, False):
        mod.fused = fused
        got = mod(cases.t(a, dev), tb)
        assert got.shape == (*lead, HA, HB)
        assert cases.bits_equal(got.cpu().numpy(), want)
    # the batched dequant op on its own, 4-D accumulators as the reference wrapper accepts them
    st = lambda k: cases.t(np.stack([p[k] for p in params]), dev)
    got = tensor_utils.asym_batch_dequant(cases.t(accs.reshape(*lead, HA, HB), dev), st(0), st(1), st(2), st(3))
    assert cases.bits_equal(got.cpu().numpy(), want)


def _bits(t):
    return t.view(torch.int16)


@pytest.mark.gpu
def test_enable_fp6_over_a_model(qnn, dev, monkeypatch):
    """nn.enable_fp6(model): every 4-bit layer it can take gets its weight shadow, every quantizer writes the
    activation shadow, the model's output keeps its bits and the large input runs the 6-bit float entry point."""
    from duqlinear4bitcuda_amd import _lib
    torch.manual_seed(11)
    K, N = 512, 1024
    lin = torch.nn.Linear(K, N, bias=True).half().to(dev)
    sw = (lin.weight.abs().amax(dim=1, keepdim=True) / 7).half()
    odd = torch.nn.Linear(K, 40, bias=False).half().to(dev)   # 40 columns: not a shape the path takes
    model = torch.nn.ModuleList([
        torch.nn.Sequential(qnn.SymQuantizer(1.0), qnn.Linear4bitSQ.from_float(lin, sw).to(dev)),
        qnn.Linear4bitASQ.from_linear(lin).to(dev),
        torch.nn.Sequential(qnn.SymQuantizer(1.0), qnn.Linear4bitSQ.from_float(odd, (odd.weight.abs().amax(dim=1, keepdim=True) / 7).half()).to(dev)),
    ])
    x = torch.randn(600, K, device=dev).half()
    want = [m(x) for m in model]
    assert qnn.enable_fp6(model) == 2
    assert model[0][0].shadow is True and model[2][0].shadow is True
    lib = _lib.load()
    calls = []
    real = lib.duq_linear4bit_forward_bf6
    monkeypatch.setattr(lib, "duq_linear4bit_forward_bf6", lambda *a: (calls.append(1), real(*a))[1], raising=False)
    got = [m(x) for m in model]
    assert len(calls) == 2
    for g, w in zip(got, want):
        assert torch.equal(_bits(g), _bits(w))
    assert qnn.enable_fp6(torch.nn.Sequential(qnn.SymQuantizer(1.0)), "only") == 0


@pytest.mark.gpu
def test_fp6_matrix_path_in_the_layers(qnn, dev):
    """enable_fp6(): every layer class gives the same bits through the 6-bit float matrix path as through the
    integer kernels; the shadow stays out of the state_dict and follows the weights."""
    _say("fp6 modules")
    M, K, N = 300, 512, 352
    torch.manual_seed(5)
    x = torch.randn(2, M // 2, K, device=dev).half()
    lin = torch.nn.Linear(K, N, bias=True).half().to(dev)
    sw = (lin.weight.abs().amax(dim=1, keepdim=True) / 7).half()
    split = 10
    s1 = (lin.weight[:, :split].abs().amax(dim=1, keepdim=True) / 7).half()
    s2 = (lin.weight[:, split:].abs().amax(dim=1, keepdim=True) / 7).half()
    layers = [
        (qnn.Linear4bitSQ.from_float(lin, sw).to(dev), qnn.SymQuantizer),
        (qnn.Linear4bitDUSQ.from_float(lin, s1, s2).to(dev), qnn.SymQuantizer),
        (qnn.Linear4bitASQ.from_linear(lin).to(dev), None),
        (qnn.LinearQuant4bitDUASQ.from_linear(lin).to(dev), None),
        (qnn.Linear4bitASQRowSum.from_linear(lin), None),
    ]
    for layer, quantizer in layers:
        name = type(layer).__name__
        _say("  ", name)
        feed = (lambda q: q(x)) if quantizer else (lambda q: x)
        want = layer(feed(quantizer() if quantizer else None))
        layer.enable_fp6()
        layer.fp6_min_tiles = 1
        assert "weight_shadow" not in layer.state_dict() and layer.weight_shadow.shape == (N, K * 3 // 4)
        if quantizer:
            for shadow in (True, "only"):
                p = quantizer(shadow=shadow, shadow_min_rows=1)(x)
                assert p.shadow_x is not None and (p.quantized_x is None) == (shadow == "only")
                assert p.size() == torch.Size((2, M // 2, K // 2))
                assert torch.equal(_bits(layer(p)), _bits(want)), name
            # a small input keeps the nibbles only
            assert quantizer(shadow="only", shadow_min_rows=1024)(x).shadow_x is None
        else:
            got = layer(x)
            assert got.shape == want.shape and torch.equal(_bits(got), _bits(want)), name
            layer.fp6_min_tiles = 10 ** 6          # too small for the path: integer kernels, same bits
            assert torch.equal(_bits(layer(x)), _bits(want)), name
            layer.fp6_min_tiles = 1
        # new weights: the shadow is rebuilt
        sd = {k: v.clone() for k, v in layer.state_dict().items()}
        sd["weight"] = sd["weight"].flip(0).contiguous()
        layer.load_state_dict(sd)
        old_shadow = layer.weight_shadow
        layer.fp6_min_tiles = 10 ** 6
        want2 = layer(feed(quantizer() if quantizer else None))
        layer.fp6_min_tiles = 1
        got2 = layer(quantizer(shadow=True, shadow_min_rows=1)(x)) if quantizer else layer(x)
        assert torch.equal(_bits(got2), _bits(want2)) and not torch.equal(_bits(got2), _bits(want)), name
        assert layer.weight_shadow is not old_shadow


@pytest.mark.gpu
def test_step_replays_from_a_hip_graph(qnn, dev):
    """A whole step (quantize + linear) on either matrix path, captured once and replayed several times with the
    program's own eager work and synchronisations in between: every replay equals the eager result (the library
    allocates nothing and records no memset; outputs come from torch's graph-private pool)."""
    _say("graph replay")
    M, K, N = 2304, 512, 512
    torch.manual_seed(11)
    lin = torch.nn.Linear(K, N, bias=True).half().to(dev)
    sw = (lin.weight.abs().amax(dim=1, keepdim=True) / 7).half()
    layer = qnn.Linear4bitSQ.from_float(lin, sw).to(dev)
    for fp6 in (False, True):
        if fp6:
            layer.enable_fp6()
        quant = qnn.SymQuantizer(1.0, shadow="only" if fp6 else False, shadow_min_rows=1)
        x = torch.randn(M, K, device=dev).half()
        want = layer(quant(x)).clone()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            layer(quant(x))
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y = layer(quant(x))
        for rep in range(4):
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(_bits(y), _bits(want)), (fp6, rep)
            # eager work between replays, and new input in the captured buffer for the next one
            noise = layer(quant(torch.randn(M, K, device=dev).half()))
            x.copy_(torch.randn(M, K, device=dev).half())
            want = layer(quant(x)).clone()
            torch.cuda.synchronize()
            assert noise.shape == want.shape


@pytest.mark.gpu
def test_weight_preparation_on_the_device_against_the_oracle(qnn, dev):
    """from_float / from_linear of the four reference-format layers with the float layer ON the device
    (qlinear4bit/nn/linear.py:58-78, 117-145, 178-206, 252-297): packed codes, scales and zero points equal the
    oracle's weight preparation, and equal what the same call gives on the CPU."""
    _say("weight prep on device")
    K, N = 512, 192
    g = torch.Generator().manual_seed(77)
    lin = torch.nn.Linear(K, N, bias=True).half()
    with torch.no_grad():
        lin.weight.copy_((torch.randn(N, K, generator=g) * 0.02).half())
        lin.weight[6, ::2] *= -1
        lin.bias.copy_(torch.randn(N, generator=g).half())
    w = lin.weight.detach().numpy()
    lin_dev = torch.nn.Linear(K, N, bias=True).half().to(dev)
    lin_dev.load_state_dict(lin.state_dict())
    split = 10

    def state(m):
        return {k: v.detach().cpu().numpy() for k, v in m.state_dict().items()}

    def same(a, b):
        assert a.keys() == b.keys()
        for k in a:
            if a[k].dtype == np.float16:
                assert cases.bits_equal(a[k], b[k]), k
            else:
                assert np.array_equal(a[k], b[k]), k

    # Linear4bitSQ.from_float
    sw = orc.sym_scales(w)
    on_dev = state(qnn.Linear4bitSQ.from_float(lin_dev, cases.t(sw, dev)))
    same(on_dev, state(qnn.Linear4bitSQ.from_float(lin, torch.from_numpy(sw))))
    assert np.array_equal(on_dev["weight"], orc.weight_sym_from_float(w, sw)) and cases.bits_equal(on_dev["weight_scales"], sw)
    assert cases.bits_equal(on_dev["bias"], lin.bias.detach().numpy())
    # Linear4bitDUSQ.from_float
    s1, s2 = orc.sym_scales(w[:, :split]), orc.sym_scales(w[:, split:])
    on_dev = state(qnn.Linear4bitDUSQ.from_float(lin_dev, cases.t(s1, dev), cases.t(s2, dev)))
    same(on_dev, state(qnn.Linear4bitDUSQ.from_float(lin, torch.from_numpy(s1), torch.from_numpy(s2))))
    codes = np.concatenate([orc.unpack_i4(orc.weight_sym_from_float(w[:, :split], s1)),
                            orc.unpack_i4(orc.weight_sym_from_float(w[:, split:], s2))], axis=1)
    assert np.array_equal(on_dev["weight"], orc.pack_i4(codes, sym=True))
    assert cases.bits_equal(on_dev["weight_scales_1"], s1) and cases.bits_equal(on_dev["weight_scales_2"], s2)
    # Linear4bitASQ.from_linear
    on_dev = state(qnn.Linear4bitASQ.from_linear(lin_dev))
    same(on_dev, state(qnn.Linear4bitASQ.from_linear(lin)))
    wa, sa, za = orc.weight_asym_from_linear(w)
    assert np.array_equal(on_dev["weight"], wa)
    assert cases.bits_equal(on_dev["weight_scales"], sa) and cases.bits_equal(on_dev["weight_zeros"], za)
    # LinearQuant4bitDUASQ.from_linear
    on_dev = state(qnn.LinearQuant4bitDUASQ.from_linear(lin_dev))
    same(on_dev, state(qnn.LinearQuant4bitDUASQ.from_linear(lin)))
    w1, sa1, za1 = orc.weight_asym_from_linear(w[:, :split])
    w2, sa2, za2 = orc.weight_asym_from_linear(w[:, split:])
    codes = np.concatenate([orc.unpack_i4(w1, signed=False), orc.unpack_i4(w2, signed=False)], axis=1)
    assert np.array_equal(on_dev["weight"], orc.pack_i4(codes, sym=False))
    for k, v in (("weight_scales_1", sa1), ("weight_zeros_1", za1), ("weight_scales_2", sa2), ("weight_zeros_2", za2)):
        assert cases.bits_equal(on_dev[k], v), k
