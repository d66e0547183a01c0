"""Seeded synthetic inputs for the benchmark configurations (generated on the CPU in
float32, cast to float16, so the oracle and the GPU see the same bits)."""
from __future__ import annotations

import numpy as np
import torch

from oracle import duq_oracle as orc


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def acts_outliers(M, K, seed, frac=0.005, factor=20.0):
    """~N(0,1) with a fraction of channels scaled (configs 1 and 5)."""
    g = _gen(seed)
    x = torch.randn(M, K, generator=g)
    n = max(1, round(frac * K))
    ch = torch.randperm(K, generator=g)[:n]
    x[:, ch] *= factor
    return x.to(torch.float16).numpy()


def acts_normal(M, K, seed):
    return torch.randn(M, K, generator=_gen(seed)).to(torch.float16).numpy()


def acts_heavy_tail(M, K, seed, frac=0.01):
    """~N(0,1) with 1% of channels drawn from Student-t(3) (config 3)."""
    g = _gen(seed)
    x = torch.randn(M, K, generator=g)
    n = max(1, round(frac * K))
    ch = torch.randperm(K, generator=g)[:n]
    # Student-t(3) = N(0,1) / sqrt(chi2(3)/3)
    z = torch.randn(M, n, generator=g)
    chi = (torch.randn(M, n, 3, generator=g) ** 2).sum(-1) / 3.0
    x[:, ch] = z / chi.sqrt()
    return x.to(torch.float16).numpy()


def acts_uniform(M, K, seed, hi=6.0):
    return (torch.rand(M, K, generator=_gen(seed)) * hi).to(torch.float16).numpy()


def weights_random_nibbles(N, K, seed):
    """Pre-packed s4 weights, uniform in [-8, 7], per-channel scales U[0.001, 0.01]
    (config 2)."""
    g = _gen(seed)
    wq = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int8).numpy()
    s = (torch.rand(N, 1, generator=g) * 0.009 + 0.001).to(torch.float16).numpy()
    return orc.pack_i4(wq, sym=True), s


def weights_from_float_sym(N, K, seed, std=0.02):
    """W ~ N(0, std), s_w = fp16(rowmax|W|/7), Wq = round(W/s_w) as Linear4bitSQ.from_float
    (config 1)."""
    g = _gen(seed)
    w = (torch.randn(N, K, generator=g) * std).to(torch.float16).numpy()
    s = orc.sym_scales(w)
    return orc.weight_sym_from_float(w, s), s


def weights_from_linear_asym(N, K, seed, std=0.02):
    g = _gen(seed)
    w = (torch.randn(N, K, generator=g) * std).to(torch.float16).numpy()
    return orc.weight_asym_from_linear(w)


def t(a, dev):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def bits_equal(a, b):
    """Exact equality of two float16 arrays, NaNs equal to NaNs."""
    a = np.asarray(a, np.float16)
    b = np.asarray(b, np.float16)
    both_nan = np.isnan(a) & np.isnan(b)
    return bool(np.all((a.view(np.uint16) == b.view(np.uint16)) | both_nan))
