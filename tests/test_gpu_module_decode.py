"""Decode through the drop-in modules: Sequential(SymQuantizer, Linear4bitSQ / Linear4bitDUSQ) and the layers with
their own AsymQuantizer run quantizer + GEMM + dequant as ONE library call for up to 1024 rows (one launch up to
eight), with the bits of the oracle; and the binary16-input entry point of the asymmetric modes against the oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu

# entry points that launch nothing (queries, set-up)
_QUERIES = {"duq_abi_version", "duq_get_dual_quant_col_k", "duq_gemm_kernel_for", "duq_gemm_stream_tile_for", "duq_quantize_linear4bit_workspace_bytes", "duq_quantize_linear8bit_workspace_bytes",
            "duq_quantize_linear4bit_asym_workspace_bytes", "duq_linear4bit_dual_rowsum_workspace_bytes",
            "duq_static_scratch_init"}


def _say(*a):
    print(*a, flush=True)


@pytest.fixture()
def library_calls(dev, monkeypatch):
    """Names of the launching C entry points called, in order (every route into the library: the ops and the
    modules' prepared calls both fetch their functions from the loaded library object)."""
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    calls = []

    def wrap(name, fn):
        def counted(*args):
            calls.append(name)
            return fn(*args)
        return counted

    for name in _lib.PROTOTYPES:
        if name not in _QUERIES:
            monkeypatch.setattr(lib, name, wrap(name, getattr(lib, name)), raising=False)
    return calls


def _sq_layers(dev, N, K, seed, bias):
    from duqlinear4bitcuda_amd.nn import Linear4bitDUSQ, Linear4bitSQ
    rng = np.random.default_rng(seed)
    wq, sw = cases.weights_random_nibbles(N, K, seed=seed)
    sw2 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    b = rng.standard_normal(N).astype(np.float16) if bias else None
    sq = Linear4bitSQ(K, N, bias=bias).to(dev)
    du = Linear4bitDUSQ(K, N, bias=bias).to(dev)
    for layer in (sq, du):
        layer.weight.copy_(cases.t(wq, dev))
        if bias:
            layer.bias.copy_(cases.t(b, dev))
    sq.weight_scales = cases.t(sw, dev)
    du.weight_scales_1 = cases.t(sw, dev)
    du.weight_scales_2 = cases.t(sw2, dev)
    return sq, du, wq, sw, sw2, b


@pytest.mark.parametrize("M", [1, 4, 8, 16, 64])
@pytest.mark.parametrize("N", [4096, 11008])
def test_sequential_symquantizer_linear_is_one_library_call(dev, library_calls, M, N):
    """Configuration 2 shapes through the reference's own usage (test/benchmark.py:67-70): one library call, the
    oracle's bits, for Linear4bitSQ and Linear4bitDUSQ; reading the quantized tensor afterwards still gives the quantizer's
    codes and scales."""
    from duqlinear4bitcuda_amd.nn import SymQuantizer
    K = 4096
    _say("module decode sym", M, N)
    sq, du, wq, sw, sw2, b = _sq_layers(dev, N, K, seed=N + M, bias=(M == 4))
    x = cases.acts_normal(M, K, seed=2 + M)
    X = cases.t(x, dev).view(1, M, K)   # the reference harness feeds [1, seq, in]
    for layer, want in ((sq, orc.linear4bit_sq_forward(x, wq, sw, b)[0]),
                        (du, orc.linear4bit_dusq_forward(x, wq, sw, sw2, b)[0])):
        model = torch.nn.Sequential(SymQuantizer(1.0), layer)
        model(X)  # first call builds the layer's prepared call
        library_calls.clear()
        y = model(X)
        assert library_calls == ["duq_quantize_linear4bit_forward_layer"], library_calls
        assert y.shape == (1, M, N)
        assert cases.bits_equal(y.cpu().numpy().reshape(M, N), want)
    # what the quantizer hands over still reads as a quantized tensor
    pq = SymQuantizer(1.0)(X)
    library_calls.clear()
    assert pq.size() == (1, M, K // 2) and pq.device == X.device
    assert library_calls == []
    sx = orc.sym_scales(x)
    assert np.array_equal(pq.quantized_x.cpu().numpy().reshape(M, K // 2), orc.sym_quant(x, sx))
    assert cases.bits_equal(pq.scales_x.cpu().numpy().reshape(M, 1), sx)
    assert library_calls == ["duq_quantize_rows_sym"], library_calls
    library_calls.clear()
    y = sq(pq)   # already quantized: the GEMM launch alone
    assert library_calls == ["duq_linear4bit_forward"], library_calls
    assert cases.bits_equal(y.cpu().numpy().reshape(M, N), orc.linear4bit_sq_forward(x, wq, sw, b)[0])


def test_symquantizer_settings_reach_the_one_launch_path(dev, library_calls):
    """clip ratio and upper clamp of the quantizer in front, a quantizer with deferral switched off, a layer with
    fused = False, 9, 130 and 1025 rows, and an input written to between the quantizer and the layer."""
    from duqlinear4bitcuda_amd.nn import SymQuantizer
    M, N, K = 3, 200, 1024
    sq, _, wq, sw, _, _ = _sq_layers(dev, N, K, seed=5, bias=False)
    x = cases.acts_outliers(M, K, seed=6)
    X = cases.t(x, dev)
    for clip, qmax in ((1.0, 6), (0.9, 7), (0.8, 6)):
        want = orc.linear4bit_sq_forward(x, wq, sw, None, clip, qmax)[0]
        library_calls.clear()
        y = torch.nn.Sequential(SymQuantizer(clip, qmax=qmax), sq)(X)
        assert library_calls == ["duq_quantize_linear4bit_forward_layer"], library_calls
        assert cases.bits_equal(y.cpu().numpy(), want), (clip, qmax)
    want = orc.linear4bit_sq_forward(x, wq, sw)[0]
    eager = SymQuantizer(1.0)
    eager.defer_rows = 0
    library_calls.clear()
    assert cases.bits_equal(torch.nn.Sequential(eager, sq)(X).cpu().numpy(), want)
    assert library_calls == ["duq_quantize_rows_sym", "duq_linear4bit_forward"], library_calls
    sq.fused = False
    library_calls.clear()
    assert cases.bits_equal(torch.nn.Sequential(SymQuantizer(1.0), sq)(X).cpu().numpy(), want)
    assert library_calls == ["duq_quantize_rows_sym", "duq_matmul_host_4bit", "duq_sym_dequant_host"], library_calls
    sq.fused = True
    for rows, calls in ((9, ["duq_quantize_linear4bit_forward_layer"]), (130, ["duq_quantize_linear4bit_forward_layer"]),
                        (1025, ["duq_quantize_rows_sym", "duq_linear4bit_forward"])):
        x9 = cases.acts_normal(rows, K, seed=7)
        library_calls.clear()
        y9 = torch.nn.Sequential(SymQuantizer(1.0), sq)(cases.t(x9, dev))
        assert library_calls == calls, (rows, library_calls)
        assert cases.bits_equal(y9.cpu().numpy(), orc.linear4bit_sq_forward(x9, wq, sw)[0])
    pq = SymQuantizer(1.0)(X)
    X.add_(1)
    with pytest.raises(RuntimeError, match="modified in place"):
        sq(pq)


def test_one_launch_follows_the_layer_buffers(dev, library_calls):
    """Weights reloaded in place, replaced by load_state_dict into a moved module, or a changed scale tensor are
    what the next decode step uses."""
    from duqlinear4bitcuda_amd.nn import Linear4bitSQ, SymQuantizer
    M, N, K = 2, 96, 512
    sq, _, wq, sw, _, _ = _sq_layers(dev, N, K, seed=11, bias=True)
    b = sq.bias.cpu().numpy()
    x = cases.acts_normal(M, K, seed=12)
    X = cases.t(x, dev)
    model = torch.nn.Sequential(SymQuantizer(1.0), sq)
    assert cases.bits_equal(model(X).cpu().numpy(), orc.linear4bit_sq_forward(x, wq, sw, b)[0])
    wq2, sw2 = cases.weights_random_nibbles(N, K, seed=13)
    sq.weight.copy_(cases.t(wq2, dev))               # in place: same tensor, same address
    assert cases.bits_equal(model(X).cpu().numpy(), orc.linear4bit_sq_forward(x, wq2, sw, b)[0])
    sq.weight_scales = cases.t(sw2, dev)             # another tensor
    assert cases.bits_equal(model(X).cpu().numpy(), orc.linear4bit_sq_forward(x, wq2, sw2, b)[0])
    fresh = Linear4bitSQ(K, N, bias=True)
    fresh.load_state_dict({k: v.cpu() for k, v in sq.state_dict().items()})
    fresh = fresh.half().to(dev)                     # a new module holds float32 scales until cast (linear.py:32-33); .to() replaces every buffer
    library_calls.clear()
    y = torch.nn.Sequential(SymQuantizer(1.0), fresh)(X)
    assert library_calls == ["duq_quantize_linear4bit_forward_layer"], library_calls
    assert cases.bits_equal(y.cpu().numpy(), orc.linear4bit_sq_forward(x, wq2, sw2, b)[0])


def _asym_weights(N, K, seed):
    w = (torch.randn(N, K, generator=torch.Generator().manual_seed(seed)) * 0.02).to(torch.float16).numpy()
    return w


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (4, 11008, 4096), (8, 4096, 4096), (3, 100, 2048), (2, 64, 8192),
                                    (7, 300, 1024), (4, 16000, 128), (16, 4096, 4096), (40, 1000, 1024), (64, 11008, 4096),
                                    (12, 300, 2048), (16, 4104, 1024), (9, 520, 4096), (10, 8200, 3008),
                                    (6, 20000, 1024), (3, 18000, 2048)])
def test_asymmetric_layers_decode_in_one_library_call(dev, library_calls, M, N, K):
    """Linear4bitASQ, LinearQuant4bitDUASQ (qlinear4bit/nn/linear.py:104-115, 239-250) and the row-sum layer from
    binary16 rows: one library call (one launch up to eight rows and for sixteen short ones), the oracle's bits (activations ~U[0, 6] as in
    configuration 4)."""
    from duqlinear4bitcuda_amd.nn import Linear4bitASQ, Linear4bitASQRowSum, LinearQuant4bitDUASQ
    _say("module decode asym", M, N, K)
    w = _asym_weights(N, K, seed=N + K)
    bias = np.random.default_rng(M).standard_normal(N).astype(np.float16)
    lin = torch.nn.Linear(K, N, bias=True).half()
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(w))
        lin.bias.copy_(torch.from_numpy(bias))
    x = cases.acts_uniform(M, K, seed=40 + M)
    X = cases.t(x, dev)
    with torch.no_grad():
        asq = Linear4bitASQ.from_linear(lin).to(dev)
        duasq = LinearQuant4bitDUASQ.from_linear(lin).to(dev)
        rs = Linear4bitASQRowSum.from_linear(lin.to(dev))
    g = lambda t: t.detach().cpu().numpy()
    wants = (
        (asq, orc.linear4bit_asq_forward(x, g(asq.weight), g(asq.weight_scales), g(asq.weight_zeros), bias)[0]),
        (duasq, orc.linear4bit_duasq_forward(x, g(duasq.weight), g(duasq.weight_scales_1), g(duasq.weight_zeros_1),
                                             g(duasq.weight_scales_2), g(duasq.weight_zeros_2), bias)[0]),
        (rs, orc.linear4bit_asq_rowsum_forward(x, g(rs.weight), g(rs.weight_scales), g(rs.weight_zeros),
                                               g(rs.weight_rowsum), bias)[0]),
    )
    for layer, want in wants:
        layer(X)
        library_calls.clear()
        y = layer(X)
        assert library_calls == ["duq_quantize_linear4bit_forward_layer"], (type(layer).__name__, library_calls)
        assert cases.bits_equal(y.detach().cpu().numpy(), want), type(layer).__name__
        layer.fused = False   # the reference's sequence of steps: same bits
        assert cases.bits_equal(layer(X).cpu().numpy(), want), type(layer).__name__


@pytest.mark.parametrize("M", [1, 2, 4, 6, 10, 16])
def test_asym_fp16_input_entry_point_codes_and_special_rows(dev, M):
    """duq_quantize_linear4bit_forward_asym through the op: codes, scales, zero points (and row sums) equal to the
    stand-alone quantizer's and the oracle's, for rows of zeros, constant rows, rows with inf / NaN, all-negative
    rows; every mode with and without bias."""
    from duqlinear4bitcuda_amd import _HIP as hip
    N, K = 88, 1024
    _say("asym fp16-in special rows", M)
    x = cases.acts_uniform(max(M, 6), K, seed=50 + M)
    x[0] = 0
    x[1, 9] = np.inf
    x[2, 77] = np.nan
    x[3] = np.float16(2.5)
    x[4] = -np.abs(x[4]) - np.float16(1)
    x = np.ascontiguousarray(x[:M]) if M > 1 else np.ascontiguousarray(x[[5]])
    w = _asym_weights(N, K, seed=3)
    wq, sw, zw = orc.weight_asym_from_linear(w)
    wq2, sw2, zw2 = orc.weight_asym_from_linear(_asym_weights(N, K, seed=4))
    wqs, sws, zws, adj = orc.weight_asym_shifted_from_linear(w)
    bias = np.random.default_rng(9).standard_normal(N).astype(np.float16)
    X = cases.t(x, dev)
    T = lambda a: cases.t(a, dev)
    for b in (None, bias):
        B = None if b is None else T(b)
        with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
            want, _, q, s, z = orc.linear4bit_asq_forward(x, wq, sw, zw, b)
            y, qf, sf, zf = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM, X, T(wq), T(sw), T(zw), bias=B, return_quantized=True)
            assert np.array_equal(qf.cpu().numpy(), q) and cases.bits_equal(sf.cpu().numpy(), s) and cases.bits_equal(zf.cpu().numpy(), z)
            assert cases.bits_equal(y.cpu().numpy(), want)
            want, _, q, s, z = orc.linear4bit_duasq_forward(x, wq, sw, zw, sw2, zw2, b)
            y = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM_DUAL, X, T(wq), T(sw), T(zw), T(sw2), T(zw2), bias=B)
            assert cases.bits_equal(y.cpu().numpy(), want)
            want, _, q, s, z, r = orc.linear4bit_asq_rowsum_forward(x, wqs, sws, zws, adj, b)
            y, qf, sf, zf, rf = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM_ROWSUM, X, T(wqs), T(sws), T(zws),
                                                                     w_rowsum_adj=T(adj), bias=B, return_quantized=True)
            assert np.array_equal(qf.cpu().numpy(), q) and cases.bits_equal(sf.cpu().numpy(), s) and cases.bits_equal(zf.cpu().numpy(), z)
            assert np.array_equal(rf.cpu().numpy(), r)
            assert cases.bits_equal(y.cpu().numpy(), want)


def test_asym_fp16_input_two_launch_shapes_and_errors(dev):
    """More than eight rows: quantizer + GEMM with the codes staged in the workspace, same bits; the workspace is
    checked before any launch."""
    from duqlinear4bitcuda_amd import _HIP as hip
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    M, N, K = 24, 96, 256
    x = cases.acts_uniform(M, K, seed=61)
    w = _asym_weights(N, K, seed=62)
    wq, sw, zw = orc.weight_asym_from_linear(w)
    wqs, sws, zws, adj = orc.weight_asym_shifted_from_linear(w)
    T = lambda a: cases.t(a, dev)
    assert cases.bits_equal(hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM, T(x), T(wq), T(sw), T(zw)).cpu().numpy(),
                            orc.linear4bit_asq_forward(x, wq, sw, zw)[0])
    assert cases.bits_equal(hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM_ROWSUM, T(x), T(wqs), T(sws), T(zws),
                                                                 w_rowsum_adj=T(adj)).cpu().numpy(),
                            orc.linear4bit_asq_rowsum_forward(x, wqs, sws, zws, adj)[0])
    assert lib.duq_quantize_linear4bit_asym_workspace_bytes(1, M, N, K) == M * K // 2 + 48 + 48
    assert lib.duq_quantize_linear4bit_asym_workspace_bytes(4, M, N, K) == M * K // 2 + 48 + 48 + 96
    assert lib.duq_quantize_linear4bit_asym_workspace_bytes(1, 8, N, K) == 0
    assert lib.duq_quantize_linear4bit_asym_workspace_bytes(0, M, N, K) == 0   # not an asymmetric mode
    X, W, SW, ZW = T(x), T(wq), T(sw), T(zw)
    y = torch.zeros(M, N, dtype=torch.float16, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    need = lib.duq_quantize_linear4bit_asym_workspace_bytes(1, M, N, K)
    ws = torch.zeros(need + 16, dtype=torch.uint8, device=dev)
    call = lambda mode, wsp, nbytes, zp=ZW.data_ptr(): lib.duq_quantize_linear4bit_forward_asym(
        mode, X.data_ptr(), W.data_ptr(), SW.data_ptr(), zp, None, None, None, None, None, M, N, K, y.data_ptr(), None, None,
        None, None, wsp, nbytes, st)
    assert call(1, None, 0) == -1 and call(1, ws.data_ptr(), need - 1) == -2 and call(1, ws.data_ptr() + 8, need) == -5
    assert call(0, ws.data_ptr(), need) == -4 and call(2, ws.data_ptr(), need) == -4   # symmetric modes: the other entry point
    assert call(1, ws.data_ptr(), need, None) == -1 and call(3, ws.data_ptr(), need) == -1 and call(4, ws.data_ptr(), need) == -1
    assert call(1, ws.data_ptr(), need) == 0
    torch.cuda.synchronize()
    assert cases.bits_equal(y.cpu().numpy(), orc.linear4bit_asq_forward(x, wq, sw, zw)[0])


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (4, 11008, 4096), (8, 512, 2048), (3, 100, 8192), (16, 4096, 4096),
                                    (40, 1000, 1024), (100, 1000, 512), (16, 1000, 2048), (9, 200, 4096), (12, 4500, 2560),
                                    (8, 17000, 512)])
def test_dual_uniform_rowsum_layer_decode(dev, library_calls, M, N, K):
    """LinearQuant4bitDUASQRowSum from binary16 rows: one library call up to 1024 rows (one launch up to eight, the
    quantizer inside the rows kernel; quantizer + GEMM with the epilogue inside for the MFMA decode kernel's shapes;
    three launches on the ring kernel's); the oracle's bits everywhere, and the op's codes / scales / zero points / row sums."""
    from duqlinear4bitcuda_amd import _HIP as hip
    from duqlinear4bitcuda_amd.nn import LinearQuant4bitDUASQRowSum
    _say("dual row-sum decode", M, N, K)
    rng = np.random.default_rng(M + N + K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)
    w[:, :10] *= 6
    bias = rng.standard_normal(N).astype(np.float16)
    lin = torch.nn.Linear(K, N, bias=True).half()
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(w))
        lin.bias.copy_(torch.from_numpy(bias))
        layer = LinearQuant4bitDUASQRowSum.from_linear(lin.to(dev))
    wq, s1, z1, s2, z2, a1, a2 = orc.weight_asym_dual_shifted_from_linear(w)
    assert np.array_equal(layer.weight.cpu().numpy(), wq)
    x = cases.acts_uniform(M, K, seed=70 + M)
    X = cases.t(x, dev)
    want, acc, qx, sx, zx, rx = orc.linear4bit_duasq_rowsum_forward(x, wq, s1, z1, s2, z2, a1, a2, bias)
    layer(X)
    library_calls.clear()
    y = layer(X)
    assert library_calls == ["duq_quantize_linear4bit_forward_layer"], library_calls
    assert cases.bits_equal(y.detach().cpu().numpy(), want)
    layer.fused = False
    assert cases.bits_equal(layer(X).detach().cpu().numpy(), want)
    T = lambda a: cases.t(a, dev)
    y, qf, sf, zf, rf = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM_DUAL_ROWSUM, X, T(wq), T(s1), T(z1), T(s2), T(z2),
                                                             T(a1), T(bias), return_quantized=True, w_rowsum_adj_2=T(a2))
    assert np.array_equal(qf.cpu().numpy(), qx) and cases.bits_equal(sf.cpu().numpy(), sx) and cases.bits_equal(zf.cpu().numpy(), zx)
    assert np.array_equal(rf.cpu().numpy(), rx)
    assert cases.bits_equal(y.cpu().numpy(), want)
    # without the caller's buffers: staged in a workspace allocated by the op (with the accumulators where the GEMM
    # of the shape cannot apply the epilogue itself)
    y = hip.quantize_linear4bit_forward_asym(hip.EPI_ASYM_DUAL_ROWSUM, X, T(wq), T(s1), T(z1), T(s2), T(z2), T(a1), None,
                                             w_rowsum_adj_2=T(a2))
    assert cases.bits_equal(y.cpu().numpy(), orc.linear4bit_duasq_rowsum_forward(x, wq, s1, z1, s2, z2, a1, a2)[0])


def test_deferred_input_meets_a_layer_on_the_6bit_float_path(dev, library_calls):
    """130 rows from a plain SymQuantizer into a layer with enable_fp6(): the layer quantizes them with the shadow
    and takes the 6-bit float kernel; without enable_fp6() the same rows are one library call; same bits."""
    from duqlinear4bitcuda_amd.nn import SymQuantizer
    M, N, K = 130, 4096, 512
    sq, _, wq, sw, _, _ = _sq_layers(dev, N, K, seed=9, bias=False)
    x = cases.acts_normal(M, K, seed=10)
    X = cases.t(x, dev)
    want = orc.linear4bit_sq_forward(x, wq, sw)[0]
    library_calls.clear()
    y = torch.nn.Sequential(SymQuantizer(1.0), sq)(X)
    assert library_calls == ["duq_quantize_linear4bit_forward_layer"], library_calls
    assert cases.bits_equal(y.cpu().numpy(), want)
    sq.enable_fp6()
    assert sq._fp6_wanted(M)
    library_calls.clear()
    pq = SymQuantizer(1.0)(X)
    y = sq(pq)
    assert library_calls == ["duq_quantize_rows_sym_bf6", "duq_linear4bit_forward_bf6"], library_calls
    assert cases.bits_equal(y.cpu().numpy(), want)
    assert pq.shadow_x is not None and np.array_equal(pq.quantized_x.cpu().numpy(), orc.sym_quant(x, orc.sym_scales(x)))
    # a quantizer that is set to write the shadow itself does not hand such rows on
    p2 = SymQuantizer(1.0, shadow="only")(X)
    assert p2._src is None and p2.shadow_x is not None and p2.quantized_x is None
