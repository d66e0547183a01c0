"""Quantized activation x activation products with the class names of the reference's
``qlinear4bit/nn/matmul.py``: both operands are quantized per row on the fly, multiplied as
int4 x int4 and dequantized.  Rows of ``B`` play the part of weight rows: the result is
``A @ B^T`` over the last dimension.

Each batch entry runs one fused GEMM + dequant launch (the reference runs a GEMM per batch
entry into a zero-filled int32 tensor, pads B's rows to a multiple of 32, then one batched
dequant: matmul.py:46-63); the bits are the same.
"""
from __future__ import annotations

import math

import torch

from .. import _HIP as _ops
from ..tools import tensor_utils
from .quantizer import AsymQuantizer, SymQuantizer


class SymQuantMatMul(torch.nn.Module):
    """sym_dequant(matmul(q(A), q(B)), s_A, s_B) (matmul.py:69-84); A [M, K], B [N, K]."""

    fused = True

    def __init__(self):
        super().__init__()
        self.quantizer_A = SymQuantizer()
        self.quantizer_B = SymQuantizer()

    def forward(self, A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
        A = self.quantizer_A(A)
        B = self.quantizer_B(B)
        if self.fused and B.quantized_x.dim() == 2:
            return tensor_utils.linear_forward(_ops.EPI_SYM, A.quantized_x, A.scales_x, None, B.quantized_x, B.scales_x)
        out = tensor_utils.matmul(A.quantized_x, B.quantized_x)
        return tensor_utils.sym_dequant(out, A.scales_x, B.scales_x)


class AsymQuantMatMul(torch.nn.Module):
    """Batched asymmetric product (matmul.py:19-66): A [..., HA, W], B [..., HB, W] (or [..., W, HB] with
    ``transpose_B``), leading dimensions equal; returns fp16 [..., HA, HB] with the reference's asymmetric
    epilogue applied per batch entry."""

    fused = True

    def __init__(self, transpose_B=False):
        super().__init__()
        self.quantizer_A = AsymQuantizer()
        self.quantizer_B = AsymQuantizer()
        self.transpose_B = transpose_B

    def forward(self, A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
        if self.transpose_B:
            B = B.transpose(-1, -2)
        ext_a, HA, WA = A.shape[:-2], A.shape[-2], A.shape[-1]
        ext_b, HB, WB = B.shape[:-2], B.shape[-2], B.shape[-1]
        for da, db in zip(ext_a, ext_b):
            assert da == db, "Batch dimensions must match"
        n = math.prod(ext_a)
        qa = self.quantizer_A(A.reshape(n, HA, WA))
        qb = self.quantizer_B(B.reshape(n, HB, WB))
        if self.fused:
            out = torch.empty((n, HA, HB), dtype=torch.float16, device=A.device)
            for b in range(n):
                out[b] = tensor_utils.linear_forward(_ops.EPI_ASYM, qa.quantized_x[b], qa.scales_x[b], qa.zeros_x[b],
                                                     qb.quantized_x[b], qb.scales_x[b], qb.zeros_x[b])
        else:
            acc = torch.stack([tensor_utils.matmul(qa.quantized_x[b], qb.quantized_x[b]) for b in range(n)])
            out = tensor_utils.asym_batch_dequant(acc, qa.scales_x, qa.zeros_x, qb.scales_x, qb.zeros_x)
        return out.view(list(ext_a) + [HA, HB])
