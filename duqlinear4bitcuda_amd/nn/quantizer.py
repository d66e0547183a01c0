"""Per-token activation quantizers with the interface of the reference's
``qlinear4bit/nn/quantizer.py``; the scale (and zero) computation and the packing run
as one HIP kernel instead of ~5 torch ops plus a kernel."""
from __future__ import annotations

import torch

from ..tools import tensor_utils


class SymQuantizer(torch.nn.Module):
    """x fp16 [..., K] -> PackedQuantizedTensor(q u8 [..., K/2], scales fp16 [..., 1]).

    scale = fp16(max|x| / 7) * input_clip_ratio (quantizer.py:13).  ``qmax`` is the upper
    clamp of the codes: 6 is what the reference's device kernel applies
    (include/common.h:53-54), 7 what its Python fake-quant path applies."""

    def __init__(self, input_clip_ratio=1.0, qmax: int = 6):
        super().__init__()
        self.input_clip_ratio = input_clip_ratio
        self.qmax = qmax

    def forward(self, x) -> tensor_utils.PackedQuantizedTensor:
        if not x.is_contiguous():
            x = x.contiguous()
        if x.shape[-1] % 32 == 0 and x.data_ptr() % 16 == 0:
            q, scales = tensor_utils.quantize_sym(x, self.input_clip_ratio, self.qmax)
        else:  # odd widths: scale with torch ops, quantize with the given-scale kernel
            scales = (x.abs().amax(dim=-1, keepdim=True) / 7).to(torch.float16) * self.input_clip_ratio
            q = tensor_utils.sym_quant(x, scales, self.qmax)
        return tensor_utils.PackedQuantizedTensor(q, scales)


class AsymQuantizer(torch.nn.Module):
    """scale = (max - min) / 15, zero = round(-min / scale), unsigned codes 0..15
    (quantizer.py:24-35).  ``input_clip_ratio`` is accepted and unused, as in the
    reference."""

    def __init__(self, input_clip_ratio: float = 1.0, shifted: bool = False):
        super().__init__()
        self.n_levels = 2 ** 4
        self.input_clip_ratio = input_clip_ratio
        # shifted=True (not in the reference): codes and zero points are stored minus 8, so that the signed
        # GEMM reads them exactly, and the per-token sums of the codes come along for the row-sum epilogue
        self.shifted = shifted

    def forward(self, x) -> tensor_utils.PackedQuantizedTensor:
        if not x.is_contiguous():
            x = x.contiguous()
        if self.shifted:
            assert x.shape[-1] % 32 == 0 and x.data_ptr() % 16 == 0, "shifted quantization needs K % 32 == 0"
            return tensor_utils.PackedQuantizedTensor(*tensor_utils.quantize_asym_shifted(x))
        if x.shape[-1] % 32 == 0 and x.data_ptr() % 16 == 0:
            q, scale, zeros = tensor_utils.quantize_asym(x)
        else:
            lo = x.amin(dim=-1, keepdim=True)
            hi = x.amax(dim=-1, keepdim=True)
            scale = (hi - lo) / (self.n_levels - 1)
            zeros = (-lo / scale).round().to(torch.float16)
            q = tensor_utils.asym_quant(x, scale, zeros)
        return tensor_utils.PackedQuantizedTensor(q, scale, zeros)
