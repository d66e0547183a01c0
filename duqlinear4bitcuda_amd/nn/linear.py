"""4-bit linear layers with the class names, buffer names/shapes and forward semantics
of the reference's ``qlinear4bit/nn/linear.py``.  The forward is one fused launch
(GEMM + dequant + bias) instead of matmul + dequant + a torch add; ``fused = False`` on
a module switches back to the reference's three-step sequence (same bits).

Buffers (the state_dict contract): ``weight`` uint8 [N, K/2]; ``weight_scales`` [N, 1]
(``weight_scales_1/_2`` for the dual layers); ``weight_zeros*`` fp16 [N, 1] for the
asymmetric layers; optional ``bias`` [N].
"""
from __future__ import annotations

import torch

from .. import _HIP as _ops
from ..tools import quantization as quant_utils
from ..tools import tensor_utils
from .quantizer import AsymQuantizer, AsymQuantizer8bit, SymQuantizer  # noqa: F401  (re-exported like the reference)

_INT4_LEVELS = 2 ** 4


def _placeholder_weight(out_features, in_features):
    return torch.randint(1, 7, (out_features, in_features // 2), dtype=torch.uint8, requires_grad=False)


def _asym_params(w: torch.Tensor):
    """Per-row scale / zero / codes the way the reference's ``from_linear`` computes them:
    max and min are taken over |W| (linear.py:129-136)."""
    aw = w.abs()
    w_max = aw.amax(dim=-1, keepdim=True)
    w_min = aw.amin(dim=-1, keepdim=True)
    scale = (w_max - w_min) / (_INT4_LEVELS - 1)
    zeros = (-w_min / scale).round().to(torch.float16)
    codes = torch.clamp(torch.round(w / scale) + zeros, 0, _INT4_LEVELS - 1)
    return scale, zeros, codes


class _Linear4bitBase(torch.nn.Module):
    fused = True
    # 6-bit float matrix path (not in the reference): taken when the layer holds a weight shadow
    # (enable_fp6) and the input brings one, for more rows than the integer decode kernel takes (64 of up to 8192
    # elements, 48 of up to 12288, 32 beyond) and at least fp6_min_tiles output tiles of 64 x 256, or more than 256
    # rows and 5/8 of that (below, the integer kernels' smaller tiles and the decode kernels do better; measured
    # crossover on an MI355X)
    fp6_min_tiles = 32
    _shadow_key = None

    def _finish(self, y):
        return y if self.bias is None else y + self.bias

    # ---- decode: quantizer + GEMM + dequant as ONE launch (up to eight rows of binary16 activations, sixteen short ones) ----
    # _decode_spec: (epilogue mode, ((argument of _HIP.FusedDecode, buffer name), ...)) of a layer class that has a
    # one-launch form; the weight comes first.
    _decode_spec = None
    _decode = None
    _decode_held = ()

    def _decode_call(self):
        """The layer's prepared one-launch call (``_HIP.FusedDecode``), rebuilt when a buffer was replaced (moved,
        cast, reloaded into a new tensor); None for a layer that has none or is not on a GPU."""
        d = self._decode
        b = self._buffers
        if d is not None:
            for name, t in self._decode_held:
                if b.get(name) is not t:
                    break
            else:
                if d.w_ptr == self._decode_held[0][1].data_ptr():
                    return d
        spec = self._decode_spec
        if spec is None:
            return None
        names = spec[1] + (("bias", "bias"),)
        held = tuple((buf, b.get(buf)) for _, buf in names)
        if not held[0][1].is_cuda:
            return None
        d = self._decode = _ops.FusedDecode(spec[0], **{arg: t for (arg, _), (_, t) in zip(names, held)})
        self._decode_held = held
        return d

    def _decode_forward(self, x, clip=1.0, qmax=6, checked=False):
        """y for binary16 rows ``x`` when the layer takes them in one library call (up to eight rows, or nine to sixteen
        that hold at most 32768 elements together: one launch, quantizer inside; up to 1024: quantizer launch + GEMM launch), else None."""
        if not self.fused:
            return None
        d = self._decode_call()
        if d is None:
            return None
        K = d.K
        if K % 64 or x.shape[-1] != K:
            return None
        M = x.numel() // K
        if d._one.get(M, -1) < 0 and not d.admits(M):
            return None
        if M > 64 and self._fp6_wanted(M):  # large enough for the 6-bit float path, and the layer holds a shadow
            return None
        return d.run(x, M, clip, qmax, checked)

    def _take_deferred(self, x):
        """A PackedQuantizedTensor that SymQuantizer handed on unquantized: the result of the one-call path, or None
        after quantizing it now (with the 6-bit float shadow when this layer will take that path)."""
        y = self._decode_forward(x.source(), x._clip, x._qmax, True)
        if y is None:
            src = x._src
            rows = src.numel() // src.shape[-1]
            x.materialize(shadow=bool(self.fused and src.shape[-1] % 128 == 0 and self._fp6_wanted(rows)))
        return y

    def enable_fp6(self):
        """Build the E3M2 shadow of ``weight`` (3/4 byte per element next to the 1/2 byte of the packed
        nibbles; not part of the state_dict; rebuilt when ``weight`` changes).  Results are bit-identical;
        large inputs run 20-25 % faster.  Needs out_features % 16 == 0 and in_features % 128 == 0."""
        assert self.weight.is_cuda, "the shadow is built on the GPU: move the layer there first"
        assert self.out_features % 16 == 0 and self.in_features % 128 == 0, \
            "the 6-bit float path needs out_features % 16 == 0 and in_features % 128 == 0"
        self.register_buffer("weight_shadow", tensor_utils.weight_shadow(self.weight), persistent=False)
        self._shadow_key = (self.weight._version, self.weight.data_ptr())
        return self

    def _fp6_ready(self):
        if self._buffers.get("weight_shadow") is None:
            return False
        if self._shadow_key != (self.weight._version, self.weight.data_ptr()) or \
                self.weight_shadow.device != self.weight.device:
            self.enable_fp6()  # weights were loaded or moved since
        return True

    def _fp6_wanted(self, rows):
        tiles = -(-rows // 64) * -(-self.out_features // 256)
        decode_rows = 64 if self.in_features <= 8192 else (48 if self.in_features <= 12288 else 32)
        return self._fp6_ready() and rows > decode_rows and \
            (tiles >= self.fp6_min_tiles or (rows > 256 and 8 * tiles >= 5 * self.fp6_min_tiles))

    def _use_shadow(self, x):
        """The input's shadow is used when the layer is ready for it and the problem is large enough, or
        when the input brings nothing else."""
        if x.shadow_x is None:
            return False
        if x.quantized_x is None:
            assert self._fp6_ready(), "the input holds only a 6-bit float shadow: call enable_fp6() on the layer"
            return True
        return self._fp6_wanted(x.shadow_x.numel() // x.shadow_x.shape[-1])

    def _own_quantizer_decode(self, x):
        """Layers with their own AsymQuantizer: a few contiguous binary16 rows on the GPU run quantizer + GEMM +
        dequant as one launch (the quantizer inside the GEMM kernel, same bits); None for anything else."""
        if type(x) is not torch.Tensor or x.dtype is not torch.float16 or not x.is_cuda or not x.is_contiguous() or \
                x.data_ptr() % 16:
            return None
        return self._decode_forward(x)

    def _quantize(self, x):
        """Own quantizer of the asymmetric layers: shadow only when this call will take the 6-bit float path."""
        rows = x.numel() // x.shape[-1]
        return self.quantizer(x, shadow="only" if self._fp6_wanted(rows) else False)


class Linear4bitSQ(_Linear4bitBase):
    """Symmetric 4-bit linear layer; takes a PackedQuantizedTensor (linear.py:24-78)."""

    def __init__(self, in_features, out_features, bias=False, dtype=torch.float16):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer("weight_scales", torch.zeros((out_features, 1), requires_grad=False))
        self.register_buffer("weight", _placeholder_weight(out_features, in_features))
        if bias:
            self.register_buffer("bias", torch.zeros((out_features), dtype=dtype))
        else:
            self.bias = None

    _decode_spec = (_ops.EPI_SYM, (("w", "weight"), ("w_scale_1", "weight_scales")))

    def forward(self, x):
        assert type(x) == tensor_utils.PackedQuantizedTensor  # quantized input is required
        if x._src is not None:  # up to 1024 rows straight from SymQuantizer: quantizer and GEMM in one library call
            y = self._take_deferred(x)
            if y is not None:
                return y
        xq, scales_x = x.quantized_x, x.scales_x
        if self.fused and self._use_shadow(x):
            return tensor_utils.linear_forward_shadow(_ops.EPI_SYM, x.shadow_x, scales_x, None, self.weight_shadow,
                                                      self.weight_scales, bias=self.bias)
        if self.fused:
            return tensor_utils.linear_forward(_ops.EPI_SYM, xq, scales_x, None, self.weight, self.weight_scales,
                                               bias=self.bias)
        acc = tensor_utils.matmul(xq, self.weight)
        return self._finish(tensor_utils.sym_dequant(acc, scales_x, self.weight_scales))

    @staticmethod
    def from_float(module: torch.nn.Linear, weight_scales=None):
        """Quantize ``module.weight`` with the given per-row scales: round(W / s), no clamp
        (pack_i4 rejects values outside [-8, 7]) (linear.py:58-78)."""
        w = module.weight.data
        new = Linear4bitSQ(module.in_features, module.out_features, bias=module.bias is not None,
                           dtype=w.dtype).to(w.dtype)
        if weight_scales is not None:
            assert weight_scales.shape == (module.out_features, 1), "weight_scales should have shape (out_features, 1)"
            new.weight_scales.copy_(weight_scales.to(w.dtype))
            codes = (w / weight_scales.to(w.device)).round()
            new.weight.copy_(quant_utils.pack_i4(codes.to(torch.int8)))
            if module.bias is not None:
                new.bias.copy_(module.bias)
        return new


class Linear4bitASQ(_Linear4bitBase):
    """Asymmetric 4-bit linear layer with its own AsymQuantizer (linear.py:80-145)."""

    def __init__(self, in_features, out_features, bias=False, require_quantizer=True):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.require_quantizer = require_quantizer
        self.register_buffer("weight_scales", torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float16))
        self.register_buffer("weight_zeros", torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float16))
        self.register_buffer("weight", _placeholder_weight(out_features, in_features))
        if bias:
            self.register_buffer("bias", torch.zeros((out_features), dtype=torch.float16))
        else:
            self.bias = None
        if require_quantizer:
            self.quantizer = AsymQuantizer()

    _decode_spec = (_ops.EPI_ASYM, (("w", "weight"), ("w_scale_1", "weight_scales"), ("w_zeros_1", "weight_zeros")))

    def forward(self, x):
        if self.require_quantizer:
            y = self._own_quantizer_decode(x)
            if y is not None:
                return y
            x = self._quantize(x) if self.fused else self.quantizer(x)
        assert type(x) == tensor_utils.PackedQuantizedTensor, \
            "Input should be quantized tensor, or require_quantizer should be passed as initial argument"
        xq, scales_x, zeros_x = x.quantized_x, x.scales_x, x.zeros_x
        if self.fused and self._use_shadow(x):
            return tensor_utils.linear_forward_shadow(_ops.EPI_ASYM, x.shadow_x, scales_x, zeros_x, self.weight_shadow,
                                                      self.weight_scales, self.weight_zeros, bias=self.bias)
        if self.fused:
            return tensor_utils.linear_forward(_ops.EPI_ASYM, xq, scales_x, zeros_x, self.weight, self.weight_scales,
                                               self.weight_zeros, bias=self.bias)
        acc = tensor_utils.matmul(xq, self.weight)
        return self._finish(tensor_utils.asym_dequant(acc, scales_x, zeros_x, self.weight_scales, self.weight_zeros))

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, require_quantizer: bool = True):
        new = cls(module.in_features, module.out_features, bias=module.bias is not None,
                  require_quantizer=require_quantizer)
        scale, zeros, codes = _asym_params(module.weight.data)
        new.weight.copy_(quant_utils.pack_i4(codes.to(torch.int8), sym=False))
        new.weight_scales.copy_(scale.to(torch.float16))
        new.weight_zeros.copy_(zeros.to(torch.float16))
        if module.bias is not None:
            new.bias.copy_(module.bias)
        return new


class Linear4bitASQRowSum(_Linear4bitBase):
    """Asymmetric 4-bit linear layer with the exact zero-point correction.  Not in the
    reference: its Linear4bitASQ stores unsigned codes that the signed GEMM misreads
    (README.md:31-32) and its epilogue subtracts the zero points from the accumulator
    (src/kernels/quant.cu:167-168).  Here codes and zero points are stored minus 8, the signed
    GEMM is exact for them, and the epilogue applies
        y = s_x * s_w * (acc - z_x * (R_w - K * z_w) - z_w * R_x)
    with R_w - K * z_w precomputed per output channel (``weight_rowsum``) and R_x delivered by
    the activation quantizer."""

    def __init__(self, in_features, out_features, bias=False, require_quantizer=True):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.require_quantizer = require_quantizer
        self.register_buffer("weight_scales", torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float16))
        self.register_buffer("weight_zeros", torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float16))
        self.register_buffer("weight_rowsum", torch.zeros((out_features,), requires_grad=False, dtype=torch.int32))
        self.register_buffer("weight", _placeholder_weight(out_features, in_features))
        if bias:
            self.register_buffer("bias", torch.zeros((out_features), dtype=torch.float16))
        else:
            self.bias = None
        if require_quantizer:
            self.quantizer = AsymQuantizer(shifted=True)

    _decode_spec = (_ops.EPI_ASYM_ROWSUM, (("w", "weight"), ("w_scale_1", "weight_scales"), ("w_zeros_1", "weight_zeros"),
                                           ("w_rowsum_adj", "weight_rowsum")))

    def forward(self, x):
        if self.require_quantizer:
            y = self._own_quantizer_decode(x)
            if y is not None:
                return y
            x = self._quantize(x) if self.fused else self.quantizer(x)
        assert type(x) == tensor_utils.PackedQuantizedTensor and x.rowsum_x is not None, \
            "Input should come from AsymQuantizer(shifted=True), or require_quantizer should be set"
        if self.fused and self._use_shadow(x):
            return tensor_utils.linear_forward_shadow(_ops.EPI_ASYM_ROWSUM, x.shadow_x, x.scales_x, x.zeros_x,
                                                      self.weight_shadow, self.weight_scales, self.weight_zeros,
                                                      bias=self.bias, rowsum_x=x.rowsum_x, w_rowsum_adj=self.weight_rowsum)
        if self.fused:
            return tensor_utils.linear_forward_rowsum(x.quantized_x, x.scales_x, x.zeros_x, x.rowsum_x, self.weight,
                                                      self.weight_scales, self.weight_zeros, self.weight_rowsum,
                                                      bias=self.bias)
        acc = tensor_utils.matmul(x.quantized_x, self.weight)
        lead = acc.shape[:-1]
        y = _ops.asym_rowsum_dequant(acc.view(-1, acc.shape[-1]), x.scales_x, x.zeros_x, x.rowsum_x, self.weight_scales,
                                     self.weight_zeros, self.weight_rowsum, self.bias)
        return y.view(*lead, -1)

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, require_quantizer: bool = True):
        """Per-output-channel min/max quantization of ``module.weight`` on the device it lives on
        (the activation quantizer kernel, applied to the weight rows)."""
        w = module.weight.data
        assert w.is_cuda, "weight preparation runs on the GPU: move the layer there first"
        new = cls(module.in_features, module.out_features, bias=module.bias is not None,
                  require_quantizer=require_quantizer).to(w.device)
        q, scale, zeros, rowsum = tensor_utils.quantize_asym_shifted(w.to(torch.float16).contiguous())
        new.weight.copy_(q)
        new.weight_scales.copy_(scale)
        new.weight_zeros.copy_(zeros)
        new.weight_rowsum.copy_(rowsum - module.in_features * zeros.view(-1).to(torch.int32))
        if module.bias is not None:
            new.bias.copy_(module.bias)
        return new


class LinearQuant4bitDUASQRowSum(_Linear4bitBase):
    """Dual-uniform asymmetric layer with the exact zero-point correction.  Not in the reference: its
    LinearQuant4bitDUASQ (linear.py:209-297) quantizes input columns 0..9 of every weight row with one
    (scale, zero) pair and the others with a second pair, and its epilogue (src/kernels/quant2.cu:158-186) then
    applies ONE pair per output column to the whole accumulator.  Here the accumulator is split at input column 10
    and each part gets the row-sum correction with its own pair:
        y = s_x * ( s_1 * corr(k < 10) + s_2 * corr(k >= 10) ),  corr = acc - z_x * (R_w - n_k * z_w) - z_w * R_x
    Codes and zero points are stored minus 8 (the signed GEMM reads them exactly), ``weight_rowsum_1/2`` hold
    ``R_w - n_k * z_w`` of the two ranges.  The forward is one launch for up to eight rows (sixteen short ones), quantizer + GEMM with the
    epilogue inside for the shapes of the decode and prefill kernels, else quantizer, GEMM into int32, epilogue."""

    def __init__(self, in_features, out_features, bias=False, require_quantizer=True):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.require_quantizer = require_quantizer
        for k in (1, 2):
            self.register_buffer(f"weight_scales_{k}", torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float16))
            self.register_buffer(f"weight_zeros_{k}", torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float16))
            self.register_buffer(f"weight_rowsum_{k}", torch.zeros((out_features,), requires_grad=False, dtype=torch.int32))
        self.register_buffer("weight", _placeholder_weight(out_features, in_features))
        if bias:
            self.register_buffer("bias", torch.zeros((out_features), dtype=torch.float16))
        else:
            self.bias = None
        if require_quantizer:
            self.quantizer = AsymQuantizer(shifted=True)

    _decode_spec = (_ops.EPI_ASYM_DUAL_ROWSUM, (("w", "weight"), ("w_scale_1", "weight_scales_1"), ("w_zeros_1", "weight_zeros_1"),
                                                ("w_scale_2", "weight_scales_2"), ("w_zeros_2", "weight_zeros_2"),
                                                ("w_rowsum_adj", "weight_rowsum_1"), ("w_rowsum_adj_2", "weight_rowsum_2")))

    def forward(self, x):
        if self.require_quantizer:
            y = self._own_quantizer_decode(x)
            if y is not None:
                return y
            # (the 6-bit float path of this layer reads the packed codes too: shadow and codes)
            rows = x.numel() // x.shape[-1]
            x = self.quantizer(x, shadow=True if self.fused and self._fp6_wanted(rows) else False)
        assert type(x) == tensor_utils.PackedQuantizedTensor and x.rowsum_x is not None, \
            "Input should come from AsymQuantizer(shifted=True), or require_quantizer should be set"
        xq = x.quantized_x
        lead = xq.shape[:-1]
        xq2 = xq.reshape(-1, xq.shape[-1])
        if self.fused and x.shadow_x is not None and self._fp6_wanted(xq2.shape[0]):
            y = _ops.linear4bit_forward_dual_rowsum_bf6(x.shadow_x.reshape(xq2.shape[0], -1), xq2, x.scales_x, x.zeros_x,
                                                        x.rowsum_x, self.weight_shadow, self.weight,
                                                        self.weight_scales_1, self.weight_zeros_1, self.weight_scales_2,
                                                        self.weight_zeros_2, self.weight_rowsum_1, self.weight_rowsum_2,
                                                        self.bias)
        elif self.fused:
            y = _ops.linear4bit_forward_dual_rowsum(xq2, x.scales_x, x.zeros_x, x.rowsum_x, self.weight,
                                                    self.weight_scales_1, self.weight_zeros_1, self.weight_scales_2,
                                                    self.weight_zeros_2, self.weight_rowsum_1, self.weight_rowsum_2,
                                                    self.bias)
        else:
            acc = _ops.matmul(xq2, self.weight)
            y = _ops.asym_dual_rowsum_dequant(acc, xq2, x.scales_x, x.zeros_x, x.rowsum_x, self.weight,
                                              self.weight_scales_1, self.weight_zeros_1, self.weight_scales_2,
                                              self.weight_zeros_2, self.weight_rowsum_1, self.weight_rowsum_2, self.bias)
        return y.view(*lead, -1)

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, require_quantizer: bool = True):
        """Per-output-channel min/max quantization of input columns 0..9 and of the others, each range on its own,
        on the device the weight lives on (the activation quantizer kernel applied to the two column ranges,
        each padded with copies of its last column to a width the kernel takes: a copy changes neither the
        minimum nor the maximum)."""
        w = module.weight.data
        assert w.is_cuda, "weight preparation runs on the GPU: move the layer there first"
        K, split = module.in_features, tensor_utils.get_dual_quant_col()
        assert K > split and K % 2 == 0
        new = cls(K, module.out_features, bias=module.bias is not None, require_quantizer=require_quantizer).to(w.device)
        w = w.to(torch.float16)
        codes = []
        for k, (lo, hi) in enumerate(((0, split), (split, K)), start=1):
            part = w[:, lo:hi]
            pad = (-(hi - lo)) % 32
            if pad:
                part = torch.cat([part, part[:, -1:].expand(-1, pad)], dim=1)
            q, scale, zeros, _ = tensor_utils.quantize_asym_shifted(part.contiguous())
            c = quant_utils.unpack_i4(q)[:, :hi - lo]          # signed codes
            codes.append(c)
            getattr(new, f"weight_scales_{k}").copy_(scale)
            getattr(new, f"weight_zeros_{k}").copy_(zeros)
            getattr(new, f"weight_rowsum_{k}").copy_(c.sum(dim=1, dtype=torch.int32) - (hi - lo) * zeros.view(-1).to(torch.int32))
        new.weight.copy_(quant_utils.pack_i4(torch.cat(codes, dim=1).to(torch.int8), sym=True))
        if module.bias is not None:
            new.bias.copy_(module.bias)
        return new


class Linear4bitDUSQ(_Linear4bitBase):
    """Symmetric layer with two per-row weight scales: input columns < 10 were quantized
    with scale 1, the rest with scale 2; the epilogue picks per OUTPUT column < 10
    (linear.py:147-206, quant2.cu:81)."""

    def __init__(self, in_features, out_features, bias=False, dtype=torch.float16):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer("weight_scales_1", torch.zeros((out_features, 1), requires_grad=False))
        self.register_buffer("weight_scales_2", torch.zeros((out_features, 1), requires_grad=False))
        self.register_buffer("weight", _placeholder_weight(out_features, in_features))
        if bias:
            self.register_buffer("bias", torch.zeros((out_features), dtype=dtype))
        else:
            self.bias = None

    _decode_spec = (_ops.EPI_SYM_DUAL, (("w", "weight"), ("w_scale_1", "weight_scales_1"), ("w_scale_2", "weight_scales_2")))

    def forward(self, x):
        assert type(x) == tensor_utils.PackedQuantizedTensor
        if x._src is not None:  # up to 1024 rows straight from SymQuantizer: quantizer and GEMM in one library call
            y = self._take_deferred(x)
            if y is not None:
                return y
        xq, scales_x = x.quantized_x, x.scales_x
        if self.fused and self._use_shadow(x):
            return tensor_utils.linear_forward_shadow(_ops.EPI_SYM_DUAL, x.shadow_x, scales_x, None, self.weight_shadow,
                                                      self.weight_scales_1, None, self.weight_scales_2, bias=self.bias)
        if self.fused:
            return tensor_utils.linear_forward(_ops.EPI_SYM_DUAL, xq, scales_x, None, self.weight,
                                               self.weight_scales_1, None, self.weight_scales_2, bias=self.bias)
        acc = tensor_utils.matmul(xq, self.weight)
        return self._finish(tensor_utils.sym_dual_dequant(acc, scales_x, self.weight_scales_1, self.weight_scales_2))

    @staticmethod
    def from_float(module: torch.nn.Linear, weight_scales_1=None, weight_scales_2=None):
        w = module.weight.data
        new = Linear4bitDUSQ(module.in_features, module.out_features, bias=module.bias is not None,
                             dtype=w.dtype).to(w.dtype)
        if weight_scales_1 is not None and weight_scales_2 is not None:
            shape = (module.out_features, 1)
            assert weight_scales_1.shape == shape, "weight_scales_1 should have shape (out_features, 1)"
            assert weight_scales_2.shape == shape, "weight_scales_2 should have shape (out_features, 1)"
            new.weight_scales_1.copy_(weight_scales_1.to(w.dtype))
            new.weight_scales_2.copy_(weight_scales_2.to(w.dtype))
            split = tensor_utils.get_dual_quant_col()
            left = (w[:, :split] / weight_scales_1.to(w.device)).round()
            right = (w[:, split:] / weight_scales_2.to(w.device)).round()
            codes = torch.cat([left, right], dim=-1)
            new.weight.copy_(quant_utils.pack_i4(codes.to(torch.int8)))
            if module.bias is not None:
                new.bias.copy_(module.bias)
        return new


class LinearQuant4bitDUASQ(_Linear4bitBase):
    """Asymmetric dual-uniform layer (linear.py:209-297)."""

    def __init__(self, in_features, out_features, bias=False, require_quantizer=True):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.require_quantizer = require_quantizer
        for name in ("weight_scales_1", "weight_zeros_1", "weight_scales_2", "weight_zeros_2"):
            self.register_buffer(name, torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float16))
        self.register_buffer("weight", _placeholder_weight(out_features, in_features))
        if bias:
            self.register_buffer("bias", torch.zeros((out_features), dtype=torch.float16))
        else:
            self.bias = None
        if self.require_quantizer:
            self.quantizer = AsymQuantizer()

    _decode_spec = (_ops.EPI_ASYM_DUAL, (("w", "weight"), ("w_scale_1", "weight_scales_1"), ("w_zeros_1", "weight_zeros_1"),
                                         ("w_scale_2", "weight_scales_2"), ("w_zeros_2", "weight_zeros_2")))

    def forward(self, x):
        if self.require_quantizer:
            y = self._own_quantizer_decode(x)
            if y is not None:
                return y
            x = self._quantize(x) if self.fused else self.quantizer(x)
        assert type(x) == tensor_utils.PackedQuantizedTensor, \
            "Input should be quantized tensor, or require_quantizer should be passed as initial argument"
        xq, scales_x, zeros_x = x.quantized_x, x.scales_x, x.zeros_x
        if self.fused and self._use_shadow(x):
            return tensor_utils.linear_forward_shadow(_ops.EPI_ASYM_DUAL, x.shadow_x, scales_x, zeros_x,
                                                      self.weight_shadow, self.weight_scales_1, self.weight_zeros_1,
                                                      self.weight_scales_2, self.weight_zeros_2, bias=self.bias)
        if self.fused:
            return tensor_utils.linear_forward(_ops.EPI_ASYM_DUAL, xq, scales_x, zeros_x, self.weight,
                                               self.weight_scales_1, self.weight_zeros_1, self.weight_scales_2,
                                               self.weight_zeros_2, bias=self.bias)
        acc = tensor_utils.matmul(xq, self.weight)
        return self._finish(tensor_utils.asym_dual_dequant(acc, scales_x, zeros_x, self.weight_scales_1,
                                                           self.weight_zeros_1, self.weight_scales_2,
                                                           self.weight_zeros_2))

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, require_quantizer=True):
        new = cls(module.in_features, module.out_features, bias=module.bias is not None,
                  require_quantizer=require_quantizer)
        w = module.weight.data
        split = tensor_utils.get_dual_quant_col()
        s1, z1, c1 = _asym_params(w[:, :split])
        s2, z2, c2 = _asym_params(w[:, split:])
        codes = torch.cat([c1, c2], dim=-1)
        new.weight.copy_(quant_utils.pack_i4(codes.to(torch.int8), sym=False))
        new.weight_scales_1.copy_(s1.to(torch.float16))
        new.weight_zeros_1.copy_(z1.to(torch.float16))
        new.weight_scales_2.copy_(s2.to(torch.float16))
        new.weight_zeros_2.copy_(z2.to(torch.float16))
        if module.bias is not None:
            new.bias.copy_(module.bias)
        return new


class LinearQuant8bitASQ(torch.nn.Module):
    """Asymmetric 8-bit linear layer on float32 activations (linear.py:300-368): buffers ``weight`` int8
    [N, K] (codes 0..127), ``weight_scales`` / ``weight_zeros`` float32 [N, 1], optional ``bias``
    float32 [N]; float32 result.  ``fused = False`` runs the reference's three steps (same bits)."""

    fused = True
    # the fused forward reads a copy of ``weight`` arranged for the MFMA operand layout (as many bytes again; not
    # part of the state_dict; rebuilt when ``weight`` changes).  tiled = False reads ``weight`` itself: same bits,
    # about half the speed on large inputs
    tiled = True
    _tiled_key = None

    def _tiled_weight(self):
        key = (self.weight._version, self.weight.data_ptr(), self.weight.device)
        if self._tiled_key != key or self._buffers.get("weight_tiled") is None:
            self.register_buffer("weight_tiled", tensor_utils.weight_tile_8bit(self.weight), persistent=False)
            self._tiled_key = key
        return self.weight_tiled

    def __init__(self, in_features, out_features, bias=False, require_quantizer=True):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.require_quantizer = require_quantizer
        self.register_buffer("weight_scales", torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float32))
        self.register_buffer("weight_zeros", torch.zeros((out_features, 1), requires_grad=False, dtype=torch.float32))
        self.register_buffer("weight", torch.randint(1, 7, (out_features, in_features), dtype=torch.int8,
                                                     requires_grad=False))
        if bias:
            self.register_buffer("bias", torch.zeros((out_features), dtype=torch.float32))
        else:
            self.bias = None
        if require_quantizer:
            self.quantizer = AsymQuantizer8bit()

    # rows up to which the layer's own quantizer and the GEMM go through one library call (a step of a few rows
    # costs more on the host than on the GPU; larger inputs hide the second call behind the first launch)
    one_call_rows = 1024

    def forward(self, x):
        if self.require_quantizer:
            if self.fused and type(x) is torch.Tensor and x.dtype is torch.float32 and x.is_cuda and x.is_contiguous() \
                    and x.shape[-1] == self.in_features and self.in_features % 32 == 0 and x.data_ptr() % 16 == 0 \
                    and 0 < x.numel() <= self.one_call_rows * self.in_features and type(self.quantizer) is AsymQuantizer8bit \
                    and self.quantizer.fused:
                return _ops.quantize_linear8bit_forward(x, self.weight, self._tiled_weight() if self.tiled else None,
                                                        self.weight_scales, self.weight_zeros, self.bias)
            x = self.quantizer(x)
        assert type(x) == tensor_utils.PackedQuantizedTensor, \
            "Input should be quantized tensor, or require_quantizer should be passed as initial argument"
        xq, scales_x, zeros_x = x.quantized_x, x.scales_x, x.zeros_x
        rows = xq.numel() // xq.shape[-1] if xq.shape[-1] else 0
        # up to four rows (two for rows longer than 4096 elements) run a kernel that reads `weight` itself
        few_rows = rows <= 4 and self.in_features <= (8192 if rows <= 2 else 4096)
        if self.fused and self.tiled and not few_rows:
            return tensor_utils.linear8bit_forward(xq, scales_x, zeros_x, self._tiled_weight(), self.weight_scales,
                                                   self.weight_zeros, self.bias, tiled_rows=self.out_features)
        if self.fused:
            return tensor_utils.linear8bit_forward(xq, scales_x, zeros_x, self.weight, self.weight_scales,
                                                   self.weight_zeros, self.bias)
        acc = tensor_utils.matmul_8bit(xq, self.weight)
        y = tensor_utils.asym_dequant_hprec(acc, scales_x, zeros_x, self.weight_scales, self.weight_zeros)
        return y if self.bias is None else y + self.bias

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, require_quantizer: bool = True):
        """Per-row scale / zero over |W| with 127 steps, codes clamp(round(W / s) + z, 0, 127)
        (linear.py:338-368)."""
        new = cls(module.in_features, module.out_features, bias=module.bias is not None,
                  require_quantizer=require_quantizer)
        w = module.weight.data
        levels = 2 ** 7
        aw = w.abs()
        w_max = aw.amax(dim=-1, keepdim=True)
        w_min = aw.amin(dim=-1, keepdim=True)
        scale = (w_max - w_min) / (levels - 1)
        zeros = (-w_min / scale).round().to(torch.float32)
        codes = torch.clamp(torch.round(w / scale) + zeros, 0, levels - 1)
        new.weight.copy_(codes.to(torch.int8))
        new.weight_scales.copy_(scale.to(torch.float32))
        new.weight_zeros.copy_(zeros.to(torch.float32))
        if module.bias is not None:
            new.bias.copy_(module.bias)
        return new
