"""Per-token activation quantizers with the interface of the reference's
``qlinear4bit/nn/quantizer.py``; the scale (and zero) computation and the packing run
as one HIP kernel instead of ~5 torch ops plus a kernel."""
from __future__ import annotations

import torch

from ..tools import tensor_utils


def _shadow_choice(quantizer, x, override):
    """False, True or "only": the per-call override if given, else the module's setting when the input is
    large enough; never for widths the matrix path does not take."""
    if x.shape[-1] % 128 or x.data_ptr() % 16 or not x.is_cuda:
        return False
    if override is not None:
        return override
    if quantizer.shadow and x.numel() // x.shape[-1] >= quantizer.shadow_min_rows:
        return quantizer.shadow
    return False


class SymQuantizer(torch.nn.Module):
    """x fp16 [..., K] -> PackedQuantizedTensor(q u8 [..., K/2], scales fp16 [..., 1]).

    scale = fp16(max|x| / 7) * input_clip_ratio (quantizer.py:13).  ``qmax`` is the upper
    clamp of the codes: 6 is what the reference's device kernel applies
    (include/common.h:53-54), 7 what its Python fake-quant path applies."""

    # Inputs of at most this many rows (decode) are handed on unquantized inside the PackedQuantizedTensor: a
    # Linear4bitSQ / Linear4bitDUSQ that follows quantizes them inside its own library call (up to eight rows, sixteen short ones,
    # quantizer + GEMM + dequant are ONE launch; above, the quantizer launch and the GEMM launch of one call: at
    # these sizes a step costs more on the host than on the GPU, and a call less is most of it), and anything
    # else that reads quantized_x / scales_x triggers this quantizer's launch then, with the same bits.  Not for
    # inputs this quantizer is set to write the 6-bit float shadow for.  0 switches that off.
    defer_rows = 1024

    def __init__(self, input_clip_ratio=1.0, qmax: int = 6, shadow=False, shadow_min_rows: int = 96):
        super().__init__()
        self.input_clip_ratio = input_clip_ratio
        self.qmax = qmax
        # shadow (not in the reference): True also writes the codes as 6-bit floats for the 6-bit float
        # matrix path of the linear layers, "only" writes nothing else (quantized_x is None); applies to
        # inputs of at least shadow_min_rows tokens whose width is a multiple of 128
        self.shadow = shadow
        self.shadow_min_rows = shadow_min_rows

    def forward(self, x, shadow=None) -> tensor_utils.PackedQuantizedTensor:
        if not x.is_contiguous():
            x = x.contiguous()
        cols = x.shape[-1]
        if shadow is None and self.defer_rows and cols % 64 == 0 and 0 < x.numel() <= self.defer_rows * cols and \
                x.is_cuda and x.dtype is torch.float16 and x.data_ptr() % 16 == 0 and \
                not (self.shadow and x.numel() >= self.shadow_min_rows * cols and cols % 128 == 0):
            return tensor_utils.PackedQuantizedTensor.deferred(x, self.input_clip_ratio, self.qmax)
        shadow = _shadow_choice(self, x, shadow)
        if shadow:
            q, sh, scales = tensor_utils.quantize_sym_shadow(x, self.input_clip_ratio, self.qmax, shadow != "only")
            return tensor_utils.PackedQuantizedTensor(q, scales, shadow_x=sh)
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

    def __init__(self, input_clip_ratio: float = 1.0, shifted: bool = False, shadow=False, shadow_min_rows: int = 96):
        super().__init__()
        self.shadow = shadow                  # see SymQuantizer
        self.shadow_min_rows = shadow_min_rows
        self.n_levels = 2 ** 4
        self.input_clip_ratio = input_clip_ratio
        # shifted=True (not in the reference): codes and zero points are stored minus 8, so that the signed
        # GEMM reads them exactly, and the per-token sums of the codes come along for the row-sum epilogue
        self.shifted = shifted

    def forward(self, x, shadow=None) -> tensor_utils.PackedQuantizedTensor:
        if not x.is_contiguous():
            x = x.contiguous()
        shadow = _shadow_choice(self, x, shadow)
        if shadow:
            out = tensor_utils.quantize_asym_shadow(x, self.shifted, shadow != "only")
            return tensor_utils.PackedQuantizedTensor(out[0], out[2], out[3], out[4] if self.shifted else None, shadow_x=out[1])
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


class AsymQuantizer8bit(torch.nn.Module):
    """float32 activations -> int8 codes 0..126 with per-token float32 scale = (max - min) / 127 and
    zero = round(-min / scale) (quantizer.py:38-55).  One launch when the row length is a multiple of 4;
    otherwise torch computes scale and zero and the given-scale kernel quantizes, as in the reference."""

    def __init__(self, input_clip_ratio: float = 1.0):
        super().__init__()
        self.n_levels = 2 ** 7
        self.input_clip_ratio = input_clip_ratio
        self.fused = True

    def forward(self, x) -> tensor_utils.PackedQuantizedTensor:
        if not x.is_contiguous():
            x = x.contiguous()
        if self.fused and x.shape[-1] % 4 == 0 and x.data_ptr() % 16 == 0 and x.dtype == torch.float32:
            return tensor_utils.PackedQuantizedTensor(*tensor_utils.quantize_asym_8bit(x))
        min_val, _ = x.min(dim=-1, keepdim=True)
        max_val, _ = x.max(dim=-1, keepdim=True)
        scale = (max_val - min_val) / (self.n_levels - 1)
        zeros = (-min_val / scale).round().to(torch.float32)
        q = tensor_utils.asym_quant_8bit(x, scale, zeros)
        return tensor_utils.PackedQuantizedTensor(q, scale, zeros)
