"""Writes tests/golden/linear4bit_small.npz: seeded inputs and the expected packed codes,
scales, int32 accumulators and fp16 outputs of the four Linear4bit forwards and of the row-sum
(exact zero-point correction) forward; and tests/golden/linear8bit_small.npz: the same for the
8-bit asymmetric layer (float32 activations, int8 codes, float32 outputs).

The reference ships no golden vectors for this path (its tests only print), so these come
from the pinned CPU oracle; the file freezes them so that a later change of the oracle or
of a kernel shows up as a diff against data, not against code.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import duq_oracle as orc  # noqa: E402


def main():
    g = torch.Generator().manual_seed(20240)
    M, K, N = 24, 256, 48
    out = {}
    # symmetric: N(0,1) activations with two x20 outlier channels, one all-zero token
    x = torch.randn(M, K, generator=g)
    x[:, [5, 77]] *= 20
    x[3] = 0
    x = x.half().numpy()
    w = (torch.randn(N, K, generator=g) * 0.02).half().numpy()
    s_w = orc.sym_scales(w)
    wq = orc.weight_sym_from_float(w, s_w)
    bias = torch.randn(N, generator=g).half().numpy()
    out.update(sym_x=x, sym_w=wq, sym_sw=s_w, bias=bias)
    for qmax in (6, 7):
        y, acc, qx, sx = orc.linear4bit_sq_forward(x, wq, s_w, bias, qmax=qmax)
        out.update({f"sym_q{qmax}_y": y, f"sym_q{qmax}_acc": acc, f"sym_q{qmax}_qx": qx, f"sym_q{qmax}_sx": sx})
    s_w2 = (s_w.astype(np.float32) * 1.5).astype(np.float16)
    y, acc, qx, sx = orc.linear4bit_dusq_forward(x, wq, s_w, s_w2, bias)
    out.update(dusq_sw2=s_w2, dusq_y=y)
    # the float weights themselves, and the dual-uniform layer as its from_float builds it (columns < 10 divided by
    # the scale of those columns, the rest by the scale of the rest): for checks of the weight preparation
    s_w1 = orc.sym_scales(w[:, :10])
    s_w2b = orc.sym_scales(w[:, 10:])
    codes = np.concatenate([orc.unpack_i4(orc.weight_sym_from_float(w[:, :10], s_w1)),
                            orc.unpack_i4(orc.weight_sym_from_float(w[:, 10:], s_w2b))], axis=1)
    wdu = orc.pack_i4(codes, sym=True)
    y, *_ = orc.linear4bit_dusq_forward(x, wdu, s_w1, s_w2b, bias)
    out.update(sym_w_float=w, dusq_ff_s1=s_w1, dusq_ff_s2=s_w2b, dusq_ff_w=wdu, dusq_ff_y=y)
    # asymmetric: U[0,6) activations plus one signed and one constant token
    xa = (torch.rand(M, K, generator=g) * 6)
    xa[1] = torch.randn(K, generator=g)
    xa[2] = 1.5
    xa = xa.half().numpy()
    wa, sa, za = orc.weight_asym_from_linear(w)
    y, acc, qx, sx, zx = orc.linear4bit_asq_forward(xa, wa, sa, za, bias)
    out.update(asym_x=xa, asym_w=wa, asym_sw=sa, asym_zw=za, asym_y=y, asym_acc=acc, asym_qx=qx, asym_sx=sx, asym_zx=zx)
    wa1, sa1, za1 = orc.weight_asym_from_linear(w[:, :10])
    wa2, sa2, za2 = orc.weight_asym_from_linear(w[:, 10:])
    codes = np.concatenate([orc.unpack_i4(wa1, signed=False), orc.unpack_i4(wa2, signed=False)], axis=1)
    wd = orc.pack_i4(codes, sym=False)
    y, *_ = orc.linear4bit_duasq_forward(xa, wd, sa1, za1, sa2, za2, bias)
    out.update(duasq_w=wd, duasq_s1=sa1, duasq_z1=za1, duasq_s2=sa2, duasq_z2=za2, duasq_y=y)
    # asymmetric with exact zero-point correction (row sums): signed-shifted codes, same activations
    wr, sr, zr, adj = orc.weight_asym_shifted_from_linear(w)
    y, acc, qx, sx, zx, rx = orc.linear4bit_asq_rowsum_forward(xa, wr, sr, zr, adj, bias)
    out.update(rs_w=wr, rs_sw=sr, rs_zw=zr, rs_adj=adj, rs_y=y, rs_acc=acc, rs_qx=qx, rs_sx=sx, rs_zx=zx, rs_rx=rx)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "linear4bit_small.npz")
    if "--only-8bit" not in sys.argv:
        np.savez_compressed(path, **out)
        print(path, os.path.getsize(path), "bytes")

    # 8-bit asymmetric layer: float32 activations with an offset, one constant and one all-positive token
    g = torch.Generator().manual_seed(20248)
    M, K, N = 20, 160, 40
    x8 = torch.randn(M, K, generator=g) * 3 + 0.7
    x8[2] = -2.25
    x8[5] = x8[5].abs() + 1
    x8 = x8.numpy()
    w8 = (torch.randn(N, K, generator=g) * 0.05).numpy()
    b8 = torch.randn(N, generator=g).numpy()
    wq, ws, wz = orc.weight_asym8_from_linear(w8)
    y, acc, q, sx, zx = orc.linear8bit_asq_forward(x8, wq, ws, wz, b8)
    sx_cpu, zx_cpu = orc.asym8_scales_zeros(x8, device_division=False)
    out8 = dict(x=x8, w_float=w8, bias=b8, w=wq, sw=ws, zw=wz, y=y, acc=acc.astype(np.int32), qx=q, sx=sx, zx=zx,
                sx_quotient_form=sx_cpu, zx_quotient_form=zx_cpu, w_tiled=orc.weight_tile_8bit(wq))
    path8 = os.path.join(os.path.dirname(os.path.abspath(__file__)), "linear8bit_small.npz")
    np.savez_compressed(path8, **out8)
    print(path8, os.path.getsize(path8), "bytes")


if __name__ == "__main__":
    main()
