"""Quantized activation x activation products with the class names of the reference's
``qlinear4bit/nn/matmul.py``: both operands are quantized per row on the fly, multiplied as
int4 x int4 and dequantized.  Rows of ``B`` play the part of weight rows: the result is
``A @ B^T`` over the last dimension.

A whole batch runs as ONE fused GEMM + dequant launch, whatever the number of batch entries
(the reference runs a GEMM per batch entry into a zero-filled int32 tensor, pads B's rows to a
multiple of 32, then one batched dequant: matmul.py:46-63); the bits are the same.  With
``fused = False`` the steps are the reference's: one batched GEMM launch into int32, one
batched dequant launch.
"""
from __future__ import annotations

import math

import torch

from .. import _HIP as _ops
from ..tools import tensor_utils
from .quantizer import AsymQuantizer, SymQuantizer


class SymQuantMatMul(torch.nn.Module):
    """sym_dequant(matmul(q(A), q(B)), s_A, s_B) (matmul.py:69-84): A [..., M, K] against a 2-D B [N, K] gives
    [..., M, N], as in the reference (its wrappers flatten the leading dimensions of A).

    Extension: a B of more than two dimensions, [..., N, K] with the leading dimensions of A, is one product per
    batch entry (per-entry scales, one launch), result [..., M, N].  The reference has no such case: its
    ``tensor_utils.matmul`` would form the cross product of all rows of A with all rows of B and its
    ``sym_dequant`` then rejects the scale sizes (src/export/bindings.cpp:152-155).  Leading dimensions that differ
    raise ``RuntimeError``."""

    fused = True

    def __init__(self):
        super().__init__()
        self.quantizer_A = SymQuantizer()
        self.quantizer_B = SymQuantizer()

    def forward(self, A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
        A = self.quantizer_A(A)
        B = self.quantizer_B(B)
        qa, qb = A.quantized_x, B.quantized_x
        if qb.dim() > 2:
            lead = tuple(qb.shape[:-2])
            if tuple(qa.shape[:-2]) != lead:
                raise RuntimeError(f"SymQuantMatMul: a batched B {tuple(qb.shape[:-2])} x [N, K] needs an A with the same "
                                   f"leading dimensions, got {tuple(qa.shape[:-2])} x [M, K]")
            qa3, qb3 = qa.reshape(-1, *qa.shape[-2:]), qb.reshape(-1, *qb.shape[-2:])
            if self.fused:
                out = _ops.batch_linear4bit_forward(_ops.EPI_SYM, qa3, A.scales_x, None, qb3, B.scales_x)
            else:
                acc = tensor_utils.batched_matmul(qa3, qb3)
                n, M, N = acc.shape
                sa, sb = A.scales_x.reshape(n, M), B.scales_x.reshape(n, N)
                out = torch.stack([tensor_utils.sym_dequant(acc[b], sa[b], sb[b]) for b in range(n)])
            return out.view(*lead, qa.shape[-2], qb.shape[-2])
        if self.fused:
            return tensor_utils.linear_forward(_ops.EPI_SYM, qa, A.scales_x, None, qb, B.scales_x)
        out = tensor_utils.matmul(qa, qb)
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
            out = _ops.batch_linear4bit_forward(_ops.EPI_ASYM, qa.quantized_x, qa.scales_x, qa.zeros_x,
                                                qb.quantized_x, qb.scales_x, qb.zeros_x)
        else:
            acc = tensor_utils.batched_matmul(qa.quantized_x, qb.quantized_x)
            out = tensor_utils.asym_batch_dequant(acc, qa.scales_x, qa.zeros_x, qb.scales_x, qb.zeros_x)
        return out.view(list(ext_a) + [HA, HB])
