"""Shape-handling wrappers over the device ops, with the names, argument order and
asserts of the reference's ``qlinear4bit/tools/tensor_utils.py`` (which calls
``qlinear4bit._CUDA``; this one calls ``duqlinear4bitcuda_amd._HIP``).

Leading dimensions are flattened for the kernels and restored on the result.
"""
from __future__ import annotations

import torch

from .. import _HIP as _ops


class PackedQuantizedTensor:
    """A quantized activation: packed nibbles plus per-token scale (and zero point)
    (tensor_utils.py:20-38).

    A few rows (decode) may arrive *deferred* from ``SymQuantizer``: the object then holds the binary16 rows and
    the quantizer's settings, a ``Linear4bitSQ`` / ``Linear4bitDUSQ`` that can run quantize + GEMM + dequant as one
    launch consumes those directly, and ``quantized_x`` / ``scales_x`` are computed (one quantizer launch, the same
    bits) the first time anything reads them."""

    __slots__ = ("_q", "_s", "zeros_x", "rowsum_x", "shadow_x", "_src", "_src_version", "_clip", "_qmax")

    def __init__(self, quantized_x: torch.Tensor, scales_x: torch.Tensor, zeros_x: torch.Tensor = None,
                 rowsum_x: torch.Tensor = None, shadow_x: torch.Tensor = None):
        self._q = quantized_x
        self._s = scales_x
        self.zeros_x = zeros_x
        # set only by the signed-shifted asymmetric quantizer (codes - 8, zeros - 8): per-token sums of the codes
        self.rowsum_x = rowsum_x
        # set by a quantizer with shadow=True / "only": the same codes as 6-bit floats [..., 3K/4] for the
        # 6-bit float matrix path; with "only", quantized_x is None
        self.shadow_x = shadow_x
        self._src = None

    @classmethod
    def deferred(cls, x: torch.Tensor, clip: float, qmax: int):
        """The symmetric quantization of ``x`` (contiguous binary16 [..., K], K % 32 == 0, 16-byte aligned), not
        yet computed."""
        self = cls.__new__(cls)
        self._q = self._s = self.zeros_x = self.rowsum_x = self.shadow_x = None
        self._src = x
        self._src_version = x._version
        self._clip = clip
        self._qmax = qmax
        return self

    def source(self):
        """The binary16 rows of a deferred tensor (None once quantized, or when it never was deferred).  Raises
        when they were written to since the quantizer saw them: the codes would be those of the new values."""
        x = self._src
        if x is not None and x._version != self._src_version:
            raise RuntimeError("PackedQuantizedTensor: the activations were modified in place between the quantizer "
                               "and the first use of its result")
        return x

    def _materialize(self, shadow=False):
        x = self.source()
        if shadow:
            self._q, self.shadow_x, self._s = quantize_sym_shadow(x, self._clip, self._qmax, shadow != "only")
        else:
            self._q, self._s = _ops.quantize_rows_sym(x, self._clip, self._qmax)
        self._src = None

    def materialize(self, shadow=False):
        """Quantize a deferred tensor now (no effect on one that is quantized already).  ``shadow``: True also
        writes the 6-bit float shadow of the codes (inputs whose width is a multiple of 128), "only" nothing else."""
        if self._src is not None:
            self._materialize(shadow)
        return self

    @property
    def quantized_x(self):
        if self._src is not None:
            self._materialize()
        return self._q

    @quantized_x.setter
    def quantized_x(self, v):
        if self._src is not None:
            self._materialize()
        self._q = v

    @property
    def scales_x(self):
        if self._src is not None:
            self._materialize()
        return self._s

    @scales_x.setter
    def scales_x(self, v):
        if self._src is not None:
            self._materialize()
        self._s = v

    def size(self):
        if self._src is not None:
            return torch.Size(self._src.shape[:-1] + (self._src.shape[-1] // 2,))
        if self._q is not None:
            return self._q.size()
        return torch.Size(self.shadow_x.shape[:-1] + (self.shadow_x.shape[-1] * 2 // 3,))

    @property
    def device(self):
        return self._src.device if self._src is not None else self._s.device

    @property
    def dtype(self):
        return torch.uint8


def flatten_last_dim_and_return_shape(x: torch.Tensor):
    lead = x.shape[:-1]
    return x.view(-1, x.shape[-1]), lead


def _flat(x):
    return x.view(-1, x.shape[-1]), tuple(x.shape[:-1])


def matmul(A, B):
    """Packed s4 x packed s4 -> int32; the packed last dim must be a multiple of 32 bytes
    (tensor_utils.py:51-55)."""
    assert A.shape[-1] % 32 == 0, "A.shape[-1]: {} must be multiplication of 32".format(A.shape[-1])
    A2, a_lead = _flat(A)
    B2, b_lead = _flat(B)
    return _ops.matmul(A2, B2).view(*a_lead, *b_lead)


def batched_matmul(A, B):
    """A [n, M, K/2] x B [n, N, K/2] -> int32 [n, M, N] in one launch (tensor_utils.py:63-68, whose body stops
    in an interactive ``IPython.embed()`` before the call; that line is not reproduced)."""
    assert A.shape[-1] % 32 == 0, "A.shape[-1]: {} must be multiplication of 32".format(A.shape[-1])
    return _ops.batched_matmul(A, B)


def matmul_8bit(A, B):
    """int8 x int8 -> int32 (tensor_utils.py:57-61)."""
    assert A.shape[-1] % 32 == 0, "A.shape[-1]: {} must be multiplication of 32".format(A.shape[-1])
    A2, a_lead = _flat(A)
    B2, b_lead = _flat(B)
    return _ops.matmul_8bit(A2, B2).view(*a_lead, *b_lead)


def sym_quant(x, scale, qmax: int = 6):
    assert x.dtype == scale.dtype == torch.float16
    x2, lead = _flat(x)
    return _ops.sym_quant(x2, scale.view(-1), qmax).view(*lead, -1)


def sym_dual_quant(x, scale_1, scale_2):
    assert x.dtype == scale_1.dtype == scale_2.dtype == torch.float16
    x2, lead = _flat(x)
    return _ops.sym_dual_quant(x2, scale_1.view(-1), scale_2.view(-1)).view(*lead, -1)


def sym_dequant(q, scale_row, scale_col, bits=32):
    assert q.dtype == torch.int32
    assert scale_row.dtype == scale_col.dtype == torch.float16
    q2, lead = _flat(q)
    return _ops.sym_dequant(q2, scale_row.view(-1), scale_col, bits).view(*lead, -1)


def sym_dual_dequant(q, scale_row, scale_col_1, scale_col_2, bits=32):
    assert q.dtype == torch.int32
    assert scale_row.dtype == scale_col_1.dtype == scale_col_2.dtype == torch.float16
    q2, lead = _flat(q)
    return _ops.sym_dual_dequant(q2, scale_row.view(-1), scale_col_1, scale_col_2, bits).view(*lead, -1)


def asym_quant(q, scale, zero):
    assert q.dtype == torch.float16
    assert scale.dtype == zero.dtype == torch.float16
    x2, lead = _flat(q)
    return _ops.asym_quant(x2, scale.view(-1), zero.view(-1)).view(*lead, -1)


def asym_quant_8bit(q, scale, zero):
    """tensor_utils.py:98-102."""
    assert q.dtype == torch.float32
    assert scale.dtype == zero.dtype == torch.float32
    x2, lead = _flat(q)
    return _ops.asym_quant_8bit(x2, scale.view(-1), zero.view(-1)).view(*lead, -1)


def asym_dequant_hprec(q, scale_row, zeros_row, scale_col, zeros_col, bits=32):
    """tensor_utils.py:110-114."""
    assert q.dtype == torch.int32
    assert scale_row.dtype == zeros_row.dtype == scale_col.dtype == zeros_col.dtype == torch.float32
    q2, lead = _flat(q)
    return _ops.asym_dequant_hprec(q2, scale_row.view(-1), zeros_row.view(-1), scale_col.view(-1), zeros_col.view(-1),
                                   bits).view(*lead, -1)


def asym_dequant(q, scale_row, zeros_row, scale_col, zeros_col, bits=32):
    assert q.dtype == torch.int32
    assert scale_row.dtype == zeros_row.dtype == scale_col.dtype == zeros_col.dtype == torch.float16
    q2, lead = _flat(q)
    return _ops.asym_dequant(q2, scale_row.view(-1), zeros_row.view(-1), scale_col.view(-1), zeros_col.view(-1),
                             bits).view(*lead, -1)


def flatten_last_two_dim_and_return_shape(x: torch.Tensor):
    return x.reshape(-1, x.shape[-2], x.shape[-1]), x.shape[:-2], x.shape[-2:]


def asym_batch_dequant(q, scale_row, zeros_row, scale_col, zeros_col, bits=32):
    """tensor_utils.py:116-123."""
    assert q.dtype == torch.int32
    assert scale_row.dtype == zeros_row.dtype == scale_col.dtype == zeros_col.dtype == torch.float16
    q3, lead, last2 = flatten_last_two_dim_and_return_shape(q)
    return _ops.asym_batch_dequant(q3, scale_row, zeros_row, scale_col, zeros_col, bits).view(*lead, last2[0], last2[1])


def asym_dual_quant(q, scale_1, zeros1, scale_2, zeros2):
    """The reference wrapper asserts ``q.dtype == int32`` here (tensor_utils.py:126), which
    can never hold for the fp16 input the kernel takes; fp16 is what is checked."""
    assert q.dtype == torch.float16
    assert scale_1.dtype == scale_2.dtype == torch.float16
    assert zeros1.dtype == zeros2.dtype == torch.float16
    x2, lead = _flat(q)
    return _ops.asym_dual_quant(x2, scale_1.view(-1), zeros1.view(-1), scale_2.view(-1),
                                zeros2.view(-1)).view(*lead, -1)


def asym_dual_dequant(q, scale_row, zeros_row, scale_col_1, zeros_col_1, scale_col_2, zeros_col_2, bits=32):
    assert q.dtype == torch.int32
    assert scale_row.dtype == scale_col_1.dtype == scale_col_2.dtype == torch.float16
    assert zeros_row.dtype == zeros_col_1.dtype == zeros_col_2.dtype == torch.float16
    q2, lead = _flat(q)
    return _ops.asym_dual_dequant(q2, scale_row.view(-1), zeros_row.view(-1), scale_col_1.view(-1),
                                  zeros_col_1.view(-1), scale_col_2.view(-1), zeros_col_2.view(-1),
                                  bits).view(*lead, -1)


def get_dual_quant_col():
    return _ops.get_dual_quant_col_k()


# ---- fused additions (no counterpart in the reference wrappers) ------------------------

def quantize_sym(x, clip: float = 1.0, qmax: int = 6):
    """One launch for scale + quantize; returns (q [..., K/2], scales [..., 1])."""
    assert x.dtype == torch.float16
    return _ops.quantize_rows_sym(x, clip, qmax)


def quantize_asym(x):
    assert x.dtype == torch.float16
    return _ops.quantize_rows_asym(x)


def quantize_asym_shifted(x):
    """Signed-shifted asymmetric quantization for the row-sum epilogue:
    (q [..., K/2], scales [..., 1], zeros - 8 [..., 1], rowsum int32 [...])."""
    assert x.dtype == torch.float16
    return _ops.quantize_rows_asym_shifted(x)


def linear_forward_rowsum(xq, scales_x, zeros_x, rowsum_x, weight, w_scale, w_zeros, w_rowsum_adj, bias=None):
    """GEMM + exact zero-point correction (+ bias) in one launch on signed-shifted operands."""
    assert xq.shape[-1] % 32 == 0, "A.shape[-1]: {} must be multiplication of 32".format(xq.shape[-1])
    return _ops.linear4bit_forward_rowsum(xq, scales_x, zeros_x, rowsum_x, weight, w_scale, w_zeros, w_rowsum_adj, bias)


def linear_forward(mode, xq, scales_x, zeros_x, weight, w_scale_1, w_zeros_1=None, w_scale_2=None, w_zeros_2=None,
                   bias=None):
    """GEMM + dequant (+ bias) in one launch; result has xq's leading dims and N columns."""
    assert xq.shape[-1] % 32 == 0, "A.shape[-1]: {} must be multiplication of 32".format(xq.shape[-1])
    return _ops.linear4bit_forward(mode, xq, scales_x, zeros_x, weight, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2, bias)


# ---- 6-bit float matrix path (no counterpart in the reference) ---------------------------

def quantize_sym_shadow(x, clip: float = 1.0, qmax: int = 6, with_q: bool = True):
    """(q or None, shadow [..., 3K/4], scales): quantize_sym that also (or only) writes the E3M2 shadow."""
    assert x.dtype == torch.float16
    return _ops.quantize_rows_sym_bf6(x, clip, qmax, with_q)


def quantize_asym_shadow(x, shifted: bool = False, with_q: bool = True):
    """(q or None, shadow, scales, zeros[, rowsum])."""
    assert x.dtype == torch.float16
    return _ops.quantize_rows_asym_bf6(x, shifted, with_q)


def weight_shadow(weight):
    return _ops.weight_shadow_bf6(weight)


def linear_forward_shadow(mode, x_shadow, scales_x, zeros_x, weight_shadow, w_scale_1, w_zeros_1=None, w_scale_2=None,
                          w_zeros_2=None, bias=None, rowsum_x=None, w_rowsum_adj=None):
    """linear_forward / linear_forward_rowsum on shadows; bit-identical results."""
    return _ops.linear4bit_forward_bf6(mode, x_shadow, scales_x, zeros_x, weight_shadow, w_scale_1, w_zeros_1, w_scale_2,
                                       w_zeros_2, bias, rowsum_x, w_rowsum_adj)


# ---- 8-bit asymmetric layer, fused (no counterpart in the reference wrappers) --------------

def quantize_asym_8bit(x):
    """(q int8 [..., K], scales [..., 1], zeros [..., 1]) in one launch."""
    assert x.dtype == torch.float32
    return _ops.quantize_rows_asym_8bit(x)


def weight_tile_8bit(weight):
    return _ops.weight_tile_8bit(weight)


def linear8bit_forward(xq, scales_x, zeros_x, weight, w_scale, w_zeros, bias=None, tiled_rows=None):
    """int8 GEMM + float32 dequant (+ bias) in one launch; with ``tiled_rows`` = N, ``weight`` is the tiled copy."""
    assert xq.shape[-1] % 32 == 0, "A.shape[-1]: {} must be multiplication of 32".format(xq.shape[-1])
    return _ops.linear8bit_forward(xq, scales_x, zeros_x, weight, w_scale, w_zeros, bias, tiled_rows)
