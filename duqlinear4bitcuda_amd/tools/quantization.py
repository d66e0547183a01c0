"""Pure-torch int4 packing helpers and the fake-quant primitives, any device.

Same names and results as the reference's ``qlinear4bit/tools/quantization.py``:
pack_i4 / unpack_i4 define the weight storage format ([N, K/2] uint8, element 2j in the
low nibble of byte j), the ``*_quant`` / ``*_dequant`` functions are the CPU-runnable
fake-quant path.
"""
from __future__ import annotations

import torch


def get_minq_maxq(bits: int, sym: bool):
    """(minq, maxq) as 0-dim tensors: [-2^(b-1), 2^(b-1)-1] or [0, 2^b-1]
    (quantization.py:7-15)."""
    if sym:
        hi = (1 << (bits - 1)) - 1
        lo = -(hi + 1)
    else:
        hi = (1 << bits) - 1
        lo = 0
    return torch.tensor(lo), torch.tensor(hi)


def two_compl(x: torch.Tensor, bits: int) -> torch.Tensor:
    """Map negative values to their unsigned two's-complement code (quantization.py:4-5)."""
    return torch.where(x < 0, x + (1 << bits), x)


def pack_i4(q: torch.Tensor, sym: bool = True) -> torch.Tensor:
    """[rows, K] signed integer tensor -> [rows, K/2] uint8 (quantization.py:40-47).
    Values outside the int4 range raise AssertionError, like the reference."""
    assert torch.is_signed(q), "The tensor to be packed should be signed int"
    lo, hi = get_minq_maxq(4, sym)
    assert bool(torch.all((q >= lo.to(q.device)) & (q <= hi.to(q.device)))), "value outside the int4 range"
    codes = two_compl(q.to(torch.int8), 4).to(torch.uint8)
    return codes[:, 0::2] | (codes[:, 1::2] << 4)


def unpack_i4(x: torch.Tensor) -> torch.Tensor:
    """uint8 [..., Kb] -> int32 [..., 2*Kb] of sign-extended nibbles (quantization.py:49-72)."""
    assert x.dtype == torch.uint8, "The tensor to be unpacked should be stored in uint8"
    lo = (x & 0x0F).to(torch.int32)
    hi = (x >> 4).to(torch.int32)
    lo = torch.where(lo >= 8, lo - 16, lo)
    hi = torch.where(hi >= 8, hi - 16, hi)
    return torch.stack((lo, hi), dim=-1).reshape(*x.shape[:-1], x.shape[-1] * 2)


def sym_quant(x, scale, maxq):
    """q = clamp(round(x / scale), -(maxq+1), maxq) (quantization.py:29-32)."""
    scale = scale.to(x.device)
    return torch.clamp(torch.round(x / scale), -(maxq + 1), maxq), scale


def sym_dequant(q, scale):
    return scale * q


def sym_quant_dequant(x, scale, maxq):
    return sym_dequant(*sym_quant(x, scale, maxq))


def asym_quant(x, scale, zero, maxq):
    """q = clamp(round(x / scale) + zero, 0, maxq) (quantization.py:17-21)."""
    scale = scale.to(x.device)
    zero = zero.to(x.device)
    return torch.clamp(torch.round(x / scale) + zero, 0, maxq), scale, zero


def asym_dequant(q, scale, zero):
    return scale * (q - zero)


def asym_quant_dequant(x, scale, zero, maxq):
    return asym_dequant(*asym_quant(x, scale, zero, maxq))
