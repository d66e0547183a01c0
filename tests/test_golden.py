"""The committed fixture tests/golden/linear4bit_small.npz against the oracle (CPU) and
against the HIP path through the module interface (GPU)."""
import os

import numpy as np
import pytest
import torch

from oracle import duq_oracle as orc
from tests import cases

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "linear4bit_small.npz"))
G8 = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "linear8bit_small.npz"))


def same16(a, b):
    a = np.asarray(a, np.float16)
    b = np.asarray(b, np.float16)
    return bool(((a.view(np.uint16) == b.view(np.uint16)) | (np.isnan(a) & np.isnan(b))).all())


def test_oracle_reproduces_the_fixture():
    for qmax in (6, 7):
        y, acc, qx, sx = orc.linear4bit_sq_forward(G["sym_x"], G["sym_w"], G["sym_sw"], G["bias"], qmax=qmax)
        assert np.array_equal(qx, G[f"sym_q{qmax}_qx"]) and np.array_equal(acc, G[f"sym_q{qmax}_acc"])
        assert same16(sx, G[f"sym_q{qmax}_sx"]) and same16(y, G[f"sym_q{qmax}_y"])
    y, *_ = orc.linear4bit_dusq_forward(G["sym_x"], G["sym_w"], G["sym_sw"], G["dusq_sw2"], G["bias"])
    assert same16(y, G["dusq_y"])
    y, acc, qx, sx, zx = orc.linear4bit_asq_forward(G["asym_x"], G["asym_w"], G["asym_sw"], G["asym_zw"], G["bias"])
    assert np.array_equal(qx, G["asym_qx"]) and np.array_equal(acc, G["asym_acc"])
    assert same16(sx, G["asym_sx"]) and same16(zx, G["asym_zx"]) and same16(y, G["asym_y"])
    y, *_ = orc.linear4bit_duasq_forward(G["asym_x"], G["duasq_w"], G["duasq_s1"], G["duasq_z1"], G["duasq_s2"],
                                        G["duasq_z2"], G["bias"])
    assert same16(y, G["duasq_y"])
    y, acc, qx, sx, zx, rx = orc.linear4bit_asq_rowsum_forward(G["asym_x"], G["rs_w"], G["rs_sw"], G["rs_zw"], G["rs_adj"],
                                                             G["bias"])
    assert np.array_equal(qx, G["rs_qx"]) and np.array_equal(acc, G["rs_acc"]) and np.array_equal(rx, G["rs_rx"])
    assert same16(sx, G["rs_sx"]) and same16(zx, G["rs_zx"]) and same16(y, G["rs_y"])


def test_fixture_sanity():
    # accumulators of the fixture equal the plain integer product of its own codes
    a = orc.unpack_i4(G["sym_q6_qx"]).astype(np.int64)
    b = orc.unpack_i4(G["sym_w"]).astype(np.int64)
    assert np.array_equal(a @ b.T, G["sym_q6_acc"])
    assert (G["sym_q6_qx"][3] == 0).all() and float(G["sym_q6_sx"][3, 0]) == 0.0   # the all-zero token
    assert orc.unpack_i4(G["sym_q6_qx"]).max() == 6 and orc.unpack_i4(G["sym_q7_qx"]).max() == 7
    # row-sum vectors: shifted codes are the unshifted ones minus 8; sums and accumulators follow from the codes
    assert np.array_equal(G["rs_qx"], G["asym_qx"] ^ 0x88)
    cx = orc.unpack_i4(G["rs_qx"]).astype(np.int64)
    cw = orc.unpack_i4(G["rs_w"]).astype(np.int64)
    assert np.array_equal(cx.sum(1), G["rs_rx"]) and np.array_equal(cx @ cw.T, G["rs_acc"])
    zw = np.rint(G["rs_zw"].astype(np.float64)).astype(np.int64).reshape(-1)
    assert np.array_equal(cw.sum(1) - cw.shape[1] * zw, G["rs_adj"])


@pytest.mark.gpu
def test_modules_reproduce_the_fixture(dev):
    from duqlinear4bitcuda_amd import nn as qnn

    T = lambda k: cases.t(G[k], dev)
    K, N = G["sym_x"].shape[1], G["sym_w"].shape[0]
    for qmax in (6, 7):
        lin = qnn.Linear4bitSQ(K, N, bias=True).half().to(dev)
        lin.load_state_dict({"weight": T("sym_w"), "weight_scales": T("sym_sw"), "bias": T("bias")})
        p = qnn.SymQuantizer(1.0, qmax=qmax)(T("sym_x"))
        assert np.array_equal(p.quantized_x.cpu().numpy(), G[f"sym_q{qmax}_qx"])
        assert same16(p.scales_x.cpu().numpy(), G[f"sym_q{qmax}_sx"])
        for fused in (True, False):
            lin.fused = fused
            assert same16(lin(p).cpu().numpy(), G[f"sym_q{qmax}_y"])
    du = qnn.Linear4bitDUSQ(K, N, bias=True).half().to(dev)
    du.load_state_dict({"weight": T("sym_w"), "weight_scales_1": T("sym_sw"), "weight_scales_2": T("dusq_sw2"), "bias": T("bias")})
    p = qnn.SymQuantizer(1.0)(T("sym_x"))
    for fused in (True, False):
        du.fused = fused
        assert same16(du(p).cpu().numpy(), G["dusq_y"])
    a = qnn.Linear4bitASQ(K, N, bias=True).to(dev)
    a.load_state_dict({"weight": T("asym_w"), "weight_scales": T("asym_sw"), "weight_zeros": T("asym_zw"), "bias": T("bias")})
    for fused in (True, False):
        a.fused = fused
        assert same16(a(T("asym_x")).cpu().numpy(), G["asym_y"])
    p = a.quantizer(T("asym_x"))
    assert np.array_equal(p.quantized_x.cpu().numpy(), G["asym_qx"])
    assert same16(p.scales_x.cpu().numpy(), G["asym_sx"]) and same16(p.zeros_x.cpu().numpy(), G["asym_zx"])
    d = qnn.LinearQuant4bitDUASQ(K, N, bias=True).to(dev)
    d.load_state_dict({"weight": T("duasq_w"), "weight_scales_1": T("duasq_s1"), "weight_zeros_1": T("duasq_z1"),
                       "weight_scales_2": T("duasq_s2"), "weight_zeros_2": T("duasq_z2"), "bias": T("bias")})
    for fused in (True, False):
        d.fused = fused
        assert same16(d(T("asym_x")).cpu().numpy(), G["duasq_y"])
    r = qnn.Linear4bitASQRowSum(K, N, bias=True).to(dev)
    r.load_state_dict({"weight": T("rs_w"), "weight_scales": T("rs_sw"), "weight_zeros": T("rs_zw"),
                       "weight_rowsum": T("rs_adj"), "bias": T("bias")})
    for fused in (True, False):
        r.fused = fused
        assert same16(r(T("asym_x")).cpu().numpy(), G["rs_y"])
    p = r.quantizer(T("asym_x"))
    assert np.array_equal(p.quantized_x.cpu().numpy(), G["rs_qx"]) and np.array_equal(p.rowsum_x.cpu().numpy(), G["rs_rx"])
    assert same16(p.zeros_x.cpu().numpy(), G["rs_zx"])


def same32(a, b):
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    return bool(((a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))).all())


def test_oracle_reproduces_the_8bit_fixture():
    wq, ws, wz = orc.weight_asym8_from_linear(G8["w_float"])
    assert np.array_equal(wq, G8["w"]) and same32(ws, G8["sw"]) and same32(wz, G8["zw"])
    y, acc, q, sx, zx = orc.linear8bit_asq_forward(G8["x"], G8["w"], G8["sw"], G8["zw"], G8["bias"])
    assert np.array_equal(q, G8["qx"]) and np.array_equal(acc, G8["acc"])
    assert same32(sx, G8["sx"]) and same32(zx, G8["zx"]) and same32(y, G8["y"])
    assert np.array_equal(orc.weight_tile_8bit(G8["w"]), G8["w_tiled"])
    # sanity of the data itself: accumulators are the plain integer product of the codes; code ranges; the constant
    # token (-2.25) has scale 0, zero point 2.25 / 0 = +inf and codes INT_MIN + INT_MAX = -1 -> 0; the two forms of
    # the scale differ somewhere
    assert np.array_equal(G8["qx"].astype(np.int64) @ G8["w"].astype(np.int64).T, G8["acc"])
    assert G8["qx"].min() == 0 and G8["qx"].max() == 126 and G8["w"].min() == 0 and G8["w"].max() == 127
    assert float(G8["sx"][2, 0]) == 0.0 and np.isposinf(G8["zx"][2, 0]) and (G8["qx"][2] == 0).all()
    assert float(G8["zx"][5, 0]) < 0                      # all-positive token: negative zero point
    assert not same32(G8["sx"], G8["sx_quotient_form"])
    assert np.allclose(G8["sx"], G8["sx_quotient_form"], rtol=2e-7, atol=0)


@pytest.mark.gpu
def test_8bit_layer_reproduces_the_fixture(dev):
    from duqlinear4bitcuda_amd import _HIP
    from duqlinear4bitcuda_amd import nn as qnn

    T = lambda k: cases.t(G8[k], dev)
    K, N = G8["x"].shape[1], G8["w"].shape[0]
    layer = qnn.LinearQuant8bitASQ(K, N, bias=True).to(dev)
    layer.load_state_dict({"weight": T("w"), "weight_scales": T("sw"), "weight_zeros": T("zw"), "bias": T("bias")})
    p = layer.quantizer(T("x"))
    assert np.array_equal(p.quantized_x.cpu().numpy(), G8["qx"])
    assert same32(p.scales_x.cpu().numpy(), G8["sx"]) and same32(p.zeros_x.cpu().numpy(), G8["zx"])
    assert np.array_equal(_HIP.matmul_8bit(p.quantized_x, layer.weight).cpu().numpy(), G8["acc"])
    assert np.array_equal(_HIP.weight_tile_8bit(layer.weight).cpu().numpy(), G8["w_tiled"])
    for fused, tiled in ((True, True), (True, False), (False, False)):
        layer.fused, layer.tiled = fused, tiled
        assert same32(layer(T("x")).cpu().numpy(), G8["y"])
