"""The entry point that allocates nothing (duq_quantize_linear4bit_forward_static: staging buffer in a static device
array of the library) against duq_quantize_linear4bit_forward with a caller workspace, through the C ABI: same bits
on two calls in a row, the second with a smaller input; the size limit; no device memory allocated by the call."""
import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from tests import cases

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def _run_both(lib, dev, M, N, K, seed, dual_bias, slot=0):
    x = cases.acts_outliers(M, K, seed=seed)
    wq, sw = cases.weights_random_nibbles(N, K, seed=seed + 1)
    rng = np.random.default_rng(seed)
    sw2 = rng.uniform(0.001, 0.01, (N, 1)).astype(np.float16)
    bias = rng.standard_normal(N).astype(np.float16)
    X, W, SW, SW2, B = (cases.t(a, dev) for a in (x, wq, sw, sw2, bias))
    mode = 2 if dual_bias else 0
    p2, pb = (SW2.data_ptr(), B.data_ptr()) if dual_bias else (None, None)
    st = torch.cuda.current_stream().cuda_stream
    need = lib.duq_quantize_linear4bit_workspace_bytes(M, N, K)
    ws = torch.zeros(max(need, 16), dtype=torch.uint8, device=dev)
    y_ref = torch.zeros(M, N, dtype=torch.float16, device=dev)
    y_new = torch.zeros(M, N, dtype=torch.float16, device=dev)
    torch.cuda.synchronize()
    assert lib.duq_quantize_linear4bit_forward(mode, X.data_ptr(), 1.0, 6, W.data_ptr(), SW.data_ptr(), p2, pb, M, N, K,
                                               y_ref.data_ptr(), None, None, ws.data_ptr(), need, st) == 0
    before = torch.cuda.mem_get_info()[0]
    assert lib.duq_quantize_linear4bit_forward_static(mode, X.data_ptr(), 1.0, 6, W.data_ptr(), SW.data_ptr(), p2, pb, M,
                                                      N, K, y_new.data_ptr(), None, None, slot, st) == 0
    torch.cuda.synchronize()
    after = torch.cuda.mem_get_info()[0]
    got, ref = y_new.cpu().numpy(), y_ref.cpu().numpy()
    assert cases.bits_equal(got, ref), (M, N, K)
    # and the oracle, so that two equally wrong outputs cannot pass
    sx = orc.sym_scales(x)
    acc = orc.matmul_s4(orc.sym_quant(x, sx), wq)
    want = orc.add_bias(orc.sym_dual_dequant(acc, sx, sw, sw2), bias) if dual_bias else orc.sym_dequant(acc, sx, sw)
    assert cases.bits_equal(got, want), (M, N, K)
    return before, after


def test_static_scratch_entry_point_two_calls_second_smaller(dev):
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    # both shapes run two launches (more than four rows), so both stage codes and scales in the static array; the
    # second is smaller in rows and in row length, so stale codes of the first call lie behind and between its own
    _say("static scratch: call 1, 96 x 4096 -> 320")
    _run_both(lib, dev, 96, 320, 4096, seed=41, dual_bias=False)
    _say("static scratch: call 2, 24 x 1024 -> 200")
    before, after = _run_both(lib, dev, 24, 200, 1024, seed=43, dual_bias=True)
    assert after >= before, "the call took device memory"
    # a one-launch shape (up to four rows) goes through untouched by the scratch
    _say("static scratch: call 3, 3 x 2048 -> 128")
    _run_both(lib, dev, 3, 128, 2048, seed=45, dual_bias=False)
    # another slot of the array: same bits (callers whose work may overlap on one GPU name different slots)
    _say("static scratch: call 4, 40 x 512 -> 96, slot 3")
    _run_both(lib, dev, 40, 96, 512, seed=47, dual_bias=True, slot=3)


def test_static_scratch_limits_and_errors(dev):
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    one = torch.zeros(64, dtype=torch.uint8, device=dev)   # never dereferenced: every call below is rejected first
    p = one.data_ptr()
    call = lambda M, N, K, mode=0, slot=0: lib.duq_quantize_linear4bit_forward_static(mode, p, 1.0, 6, p, p, None, None, M, N,
                                                                                      K, p, None, None, slot, st)
    _say("static scratch: limits")
    assert call(4096, 64, 8192) == -7          # 16 MiB of codes
    assert call(4097, 64, 4096) == -7          # one row too many for 8 MiB
    assert call(32769, 64, 64) == -7           # more rows than scale slots
    assert call(2, 64, 131072) == -6           # fits the scratch, rejected like everywhere else: K too large
    assert call(8, 64, 96) == -3 and call(8, 64, 256, mode=1) == -4
    assert b"scratch" in lib.duq_status_string(-7)
    assert call(8, 64, 64, slot=4) == -7       # slots 0..3
    assert lib.duq_static_scratch_init() == 0  # the address lookup, for callers that capture their first call
    assert call(0, 64, 64) == 0 and call(8, 0, 64) == 0   # nothing to do
    torch.cuda.synchronize()


def test_static_scratch_two_streams_two_slots(dev):
    """Two calls that may overlap in time (two streams, nothing ordering them) on two slots of the array: each gives
    the bits of the workspace form."""
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    assert lib.duq_static_scratch_init() == 0
    M, N, K = 512, 1024, 4096
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    work = []
    for i, s in enumerate(streams):
        x = cases.acts_outliers(M, K, seed=71 + i)
        wq, sw = cases.weights_random_nibbles(N, K, seed=81 + i)
        X, W, SW = (cases.t(a, dev) for a in (x, wq, sw))
        need = lib.duq_quantize_linear4bit_workspace_bytes(M, N, K)
        ws = torch.zeros(need, dtype=torch.uint8, device=dev)
        y_ref = torch.zeros(M, N, dtype=torch.float16, device=dev)
        y_new = torch.zeros(M, N, dtype=torch.float16, device=dev)
        work.append((X, W, SW, ws, need, y_ref, y_new))
    torch.cuda.synchronize()
    _say("static scratch: two streams, slots 1 and 2")
    for rep in range(3):
        for i, s in enumerate(streams):
            X, W, SW, ws, need, y_ref, y_new = work[i]
            assert lib.duq_quantize_linear4bit_forward_static(0, X.data_ptr(), 1.0, 6, W.data_ptr(), SW.data_ptr(), None, None,
                                                              M, N, K, y_new.data_ptr(), None, None, 1 + i, s.cuda_stream) == 0
    torch.cuda.synchronize()
    st = torch.cuda.current_stream().cuda_stream
    for X, W, SW, ws, need, y_ref, y_new in work:
        assert lib.duq_quantize_linear4bit_forward(0, X.data_ptr(), 1.0, 6, W.data_ptr(), SW.data_ptr(), None, None, M, N, K,
                                                   y_ref.data_ptr(), None, None, ws.data_ptr(), need, st) == 0
    torch.cuda.synchronize()
    for X, W, SW, ws, need, y_ref, y_new in work:
        assert cases.bits_equal(y_new.cpu().numpy(), y_ref.cpu().numpy())
