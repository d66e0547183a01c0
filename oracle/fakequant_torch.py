"""The reference's CPU fake-quant path, restated with torch-CPU ops.

TEST / BASELINE INFRASTRUCTURE ONLY (imported by tests and by bench.py's cpu_baseline
leg; never by the product package).

The reference has no CPU linear layer; its CPU-runnable pieces are the fake-quant
primitives of qlinear4bit/tools/quantization.py:17-37.  A Linear4bit forward on that
path is: per-token scale (qlinear4bit/nn/quantizer.py:13) -> sym_quant with the Python
clamp [-8, 7] (quantization.py:29-32) -> integer matmul -> (s_x * s_w^T) * acc as fp16
(operator order of src/kernels/quant.cu:79-80).  The integer matmul is done in float32,
which is exact while 64*K < 2**24.
"""
from __future__ import annotations

import torch


def sym_scales(x: torch.Tensor, clip: float = 1.0) -> torch.Tensor:
    return (torch.max(torch.abs(x), dim=-1)[0].unsqueeze(1) / 7).to(torch.float16) * clip


def sym_quant(x: torch.Tensor, scale: torch.Tensor, maxq: int = 7) -> torch.Tensor:
    return torch.clamp(torch.round(x / scale), -(maxq + 1), maxq)


def linear4bit_forward(x: torch.Tensor, wq: torch.Tensor, w_scales: torch.Tensor, maxq: int = 7, clip: float = 1.0):
    """x fp16 [M,K]; wq integer-valued weights [N,K] (any dtype); w_scales fp16 [N,1].
    Returns (y fp16 [M,N], acc int32 [M,N], q_x fp16 [M,K], s_x fp16 [M,1])."""
    assert 64 * x.shape[-1] < (1 << 24)
    s_x = sym_scales(x, clip)
    q_x = sym_quant(x, s_x, maxq)
    acc = torch.matmul(q_x.float(), wq.float().t())
    y = (s_x * w_scales.view(1, -1)) * acc.half()
    return y, acc.to(torch.int32), q_x, s_x
