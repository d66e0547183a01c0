"""CPU oracle for the Linear4bit forward path (quantize -> s4 x s4 GEMM -> dequant).

TEST INFRASTRUCTURE ONLY.  This module is the checker the HIP kernels are compared
against.  Nothing in the product package may import it; only tests, the smoke entry
and the benchmark's cpu_baseline leg do.

Every function restates, in NumPy, what one piece of the reference computes, and
cites the reference lines it follows (paths relative to the reference checkout).

Conventions
-----------
* ``h(v)``: round-to-nearest-even to IEEE binary16.  Every fp16 operator of the
  reference rounds after each operation; here each operation is computed in float32
  and rounded to float16, which is identical for +, -, *, / on binary16 operands
  (float32 carries 24 >= 2*11+2 significand bits).
* Packed int4: element ``i`` of a row lives in byte ``i // 2``, low nibble first
  (include/int4.h:86-98, qlinear4bit/tools/quantization.py:45-46).
* ``QMAX_SYM_DEVICE = 6``: the device quantizer clamps to [-8, 6] because
  ``constexpr int qmax_sym = (7 - 1e-8)`` truncates (include/common.h:53-54).
  The Python fake-quant path clamps to [-8, 7]
  (qlinear4bit/tools/quantization.py:29-32).

Pinning status (which independent check fixes each function) is listed next to each
function; the checks themselves live in tests/test_oracle_*.py.

Behaviour that only the reference's own hardware could settle, and that this oracle
fixes by definition instead ("parity unpinned" for exactly these corners):
  * ``__hdiv`` is taken to be the IEEE binary16 quotient (CUDA's is a reciprocal
    based approximation with a fix-up and may differ in the last bit in rare cases).
  * the undefined shift in src/kernels/quant2.cu:182-183 for column >= 128 is taken
    as "false" (the second scale/zero set), the same value it has for 1 <= col < 128.
  * float->int conversion of +-inf / NaN follows the PTX ``cvt.rni.s32.f16`` rule
    (saturate, NaN -> 0) and the following int add wraps modulo 2**32.
The row-sum functions (``asym_quant_shifted`` ... ``linear4bit_asq_rowsum_forward``) restate a
mode the reference does not have; there is nothing of the reference to be in parity with, and
they are pinned by the integer identity and the float64 product of the dequantized operands.
The 8-bit functions (``asym8_scales_zeros`` ... ``linear8bit_asq_forward``) restate the reference's
LinearQuant8bitASQ path (float32 arithmetic, one rounding per operator); pinned by hand-computed
cases, float64 evaluation where float64 is exact, a brute-force GEMM and torch-CPU operators.
The E3M2 shadow functions (``e3m2_decode`` ... ``weight_shadow_bf6``) describe a storage format
of the library, not of the reference: they are pinned by the published OCP Microscaling
formula for E3M2 (decode), by decode(encode(v)) == v for every int4 value, and by the round
trip through ``shadow_block_unpack``; what the GEMM computes from them stays ``matmul_s4``.
"""
from __future__ import annotations

import numpy as np

QMIN_SYM = -8
QMAX_SYM_DEVICE = 6      # include/common.h:53-54
QMAX_SYM_FAKEQUANT = 7   # qlinear4bit/tools/quantization.py:7-8,29-32
QMIN_ASYM = 0
QMAX_ASYM = 15           # include/common.h:56-57
QUANT_COL_K = 10         # include/quant.h:5

_F32 = np.float32
_F16 = np.float16


# ----------------------------------------------------------------------------------
# fp16 helpers
# ----------------------------------------------------------------------------------
def h(v):
    """Round to binary16 (nearest-even)."""
    with np.errstate(over="ignore", invalid="ignore"):
        return np.asarray(v, dtype=_F32).astype(_F16)


def _f32(v):
    return np.asarray(v).astype(_F32)


def hmul(a, b):
    with np.errstate(over="ignore", invalid="ignore"):
        return h(_f32(a) * _f32(b))


def hsub(a, b):
    with np.errstate(over="ignore", invalid="ignore"):
        return h(_f32(a) - _f32(b))


def hadd(a, b):
    with np.errstate(over="ignore", invalid="ignore"):
        return h(_f32(a) + _f32(b))


def hdiv(a, b):
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        return h(_f32(a) / _f32(b))


def int_to_half(acc):
    """``__int2half_rn`` (src/kernels/quant.cu:4-8): one rounding int32 -> binary16,
    overflow to +-inf from |v| >= 65520."""
    with np.errstate(over="ignore"):
        return np.asarray(acc, dtype=np.int64).astype(np.float64).astype(_F16)


def half_to_int_rn(v):
    """``__half2int_rn``: nearest-even to int32, saturating, NaN -> 0."""
    x = np.asarray(v, dtype=_F16).astype(np.float64)
    with np.errstate(invalid="ignore"):
        r = np.rint(x)
    r = np.where(np.isnan(r), 0.0, r)
    r = np.clip(r, -2147483648.0, 2147483647.0)
    return r.astype(np.int64).astype(np.int32)


# ----------------------------------------------------------------------------------
# A10  pack / unpack  (qlinear4bit/tools/quantization.py:4-15,40-72; int4.h:86-98)
# pinned by: exhaustive enumeration of all 256 byte values + hand-written bytes.
# ----------------------------------------------------------------------------------
def pack_i4(q, sym: bool = True):
    """[rows, K] integer array -> [rows, ceil(K/2)] uint8.  Range is asserted like the
    reference (quantization.py:41-43).  Odd K leaves the last high nibble 0, as the
    device kernels do (src/kernels/quant.cu:27-35)."""
    q = np.asarray(q)
    assert q.ndim == 2
    lo, hi = (-8, 7) if sym else (0, 15)
    assert q.size == 0 or (q.min() >= lo and q.max() <= hi), "value out of int4 range"
    nib = (q.astype(np.int64) & 0xF).astype(np.uint8)
    rows, k = nib.shape
    if k % 2:
        nib = np.concatenate([nib, np.zeros((rows, 1), np.uint8)], axis=1)
    return (nib[:, 0::2] | (nib[:, 1::2] << 4)).astype(np.uint8)


def unpack_i4(b, signed: bool = True):
    """uint8 [..., Kb] -> int32 [..., 2*Kb]; sign-extends when ``signed``
    (quantization.py:49-72)."""
    b = np.asarray(b, dtype=np.uint8)
    lo = (b & 0x0F).astype(np.int32)
    hi = (b >> 4).astype(np.int32)
    if signed:
        lo = np.where(lo >= 8, lo - 16, lo)
        hi = np.where(hi >= 8, hi - 16, hi)
    out = np.empty(b.shape[:-1] + (b.shape[-1] * 2,), np.int32)
    out[..., 0::2] = lo
    out[..., 1::2] = hi
    return out


# ----------------------------------------------------------------------------------
# A1  symmetric per-token scale  (qlinear4bit/nn/quantizer.py:13;
#     src/module/quant_tensor.cu:151-156)
# pinned by: exact rational model over all non-negative binary16 maxima; torch-CPU.
# ----------------------------------------------------------------------------------
def sym_scales(x, clip: float = 1.0):
    """scale[m] = h( h(max_k|x[m,k]| / 7) * clip ), shape [M, 1] float16.

    torch evaluates fp16-tensor <op> python-scalar in float32 and rounds once.  On a
    GPU torch multiplies by float32(1/7) instead of dividing; both give the same
    binary16 for every binary16 maximum (checked exhaustively in the tests)."""
    x = np.asarray(x, dtype=_F16)
    amax = np.max(np.abs(x), axis=-1, keepdims=True)
    with np.errstate(invalid="ignore"):
        s = h(_f32(amax) / _F32(7.0))
        s = h(_f32(s) * _F32(clip))
    return s


# ----------------------------------------------------------------------------------
# A2  symmetric quantize  (src/kernels/quant.cu:11-45)
# pinned by: hand-computed tie cases; exact rational model on a brute-force grid;
#            invariants (range, monotone, odd symmetry away from the clamp).
# ----------------------------------------------------------------------------------
def sym_quant_values(x, scale, qmax: int = QMAX_SYM_DEVICE):
    """Unpacked integer codes, int32 [M, K]."""
    x = np.asarray(x, dtype=_F16)
    s = np.asarray(scale, dtype=_F16).reshape(-1, 1)
    q = half_to_int_rn(hdiv(x, s))
    return np.clip(q, QMIN_SYM, qmax).astype(np.int32)


def sym_quant(x, scale, qmax: int = QMAX_SYM_DEVICE):
    """Packed uint8 [M, ceil(K/2)]."""
    return pack_i4(sym_quant_values(x, scale, qmax), sym=True)


def sym_dual_quant_values(x, scale_1, scale_2, qmax: int = QMAX_SYM_DEVICE):
    """src/kernels/quant2.cu:9-45: column < 10 uses scale_1[row], else scale_2[row]."""
    x = np.asarray(x, dtype=_F16)
    s1 = np.asarray(scale_1, dtype=_F16).reshape(-1, 1)
    s2 = np.asarray(scale_2, dtype=_F16).reshape(-1, 1)
    col = np.arange(x.shape[1])[None, :]
    s = np.where(col < QUANT_COL_K, s1, s2)
    q = half_to_int_rn(hdiv(x, s))
    return np.clip(q, QMIN_SYM, qmax).astype(np.int32)


def sym_dual_quant(x, scale_1, scale_2, qmax: int = QMAX_SYM_DEVICE):
    return pack_i4(sym_dual_quant_values(x, scale_1, scale_2, qmax), sym=True)


# ----------------------------------------------------------------------------------
# A3  asymmetric per-token scale/zero + quantize
#     (qlinear4bit/nn/quantizer.py:24-35; src/kernels/quant.cu:99-132)
# ----------------------------------------------------------------------------------
def asym_scales_zeros(x):
    """scale = h(h(max-min)/15); zero = h(rint(h(h(-min)/scale))); both [M,1] fp16."""
    x = np.asarray(x, dtype=_F16)
    mn = np.min(x, axis=-1, keepdims=True)
    mx = np.max(x, axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        scale = h(_f32(hsub(mx, mn)) / _F32(15.0))
        neg = h(-_f32(mn))
        zero = h(np.rint(_f32(hdiv(neg, scale))))
    return scale, zero


def _wrap_i32(v):
    return ((np.asarray(v, dtype=np.int64) + 2**31) % 2**32 - 2**31).astype(np.int64)


def asym_quant_values(x, scale, zero):
    """u = clamp( rint(h(x/s)) + rint(z), 0, 15 ) (src/kernels/quant.cu:125-126)."""
    x = np.asarray(x, dtype=_F16)
    s = np.asarray(scale, dtype=_F16).reshape(-1, 1)
    z = np.asarray(zero, dtype=_F16).reshape(-1, 1)
    q = half_to_int_rn(hdiv(x, s)).astype(np.int64)
    zi = half_to_int_rn(z).astype(np.int64)
    return np.clip(_wrap_i32(q + zi), QMIN_ASYM, QMAX_ASYM).astype(np.int32)


def asym_quant(x, scale, zero):
    return pack_i4(asym_quant_values(x, scale, zero), sym=False)


def asym_dual_quant_values(x, scale_1, zeros_1, scale_2, zeros_2):
    """src/kernels/quant2.cu:101-139: the zero is added in binary16 BEFORE rounding
    (``__half2int_rn(data + zero_val)``), unlike quant.cu:126."""
    x = np.asarray(x, dtype=_F16)
    col = np.arange(x.shape[1])[None, :]
    pick = col < QUANT_COL_K
    s = np.where(pick, np.asarray(scale_1, _F16).reshape(-1, 1), np.asarray(scale_2, _F16).reshape(-1, 1))
    z = np.where(pick, np.asarray(zeros_1, _F16).reshape(-1, 1), np.asarray(zeros_2, _F16).reshape(-1, 1))
    q = half_to_int_rn(hadd(hdiv(x, s), z))
    return np.clip(q, QMIN_ASYM, QMAX_ASYM).astype(np.int32)


def asym_dual_quant(x, scale_1, zeros_1, scale_2, zeros_2):
    return pack_i4(asym_dual_quant_values(x, scale_1, zeros_1, scale_2, zeros_2), sym=False)


# ----------------------------------------------------------------------------------
# A4  s4 x s4 -> s32 GEMM  (src/kernels/gemm.cu:8-43)
# pinned by: closed form (exact integers), brute-force Python loops on tiny shapes,
#            special cases (all -8, one-hot rows).
# ----------------------------------------------------------------------------------
def matmul_s4(a_packed, b_packed):
    """C[m,n] = sum_k s4(A[m,k]) * s4(B[n,k]); both operands are read as SIGNED nibbles
    whatever produced them (src/kernels/gemm.cu:18-20).  int32 [M, N]."""
    a = unpack_i4(a_packed, signed=True)
    b = unpack_i4(b_packed, signed=True)
    assert a.shape[1] == b.shape[1]
    # float32 GEMM of small integers is exact while |acc| < 2**24 (64*K); use it for
    # speed when that holds, int64 otherwise.
    k = a.shape[1]
    if 64 * k < (1 << 24):
        c = a.astype(np.float32) @ b.astype(np.float32).T
        return c.astype(np.int32)
    return (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)


# ----------------------------------------------------------------------------------
# A5/A6/A7  dequant epilogues  (src/kernels/quant.cu:64-81,149-169;
#                               src/kernels/quant2.cu:62-83,158-186)
# pinned by: exact rational model of each rounding on a grid incl. the 65504/65520
#            boundary; selector enumeration for the dual variants.
# ----------------------------------------------------------------------------------
def sym_dequant(acc, scale_row, scale_col):
    """y = h( h(s_row*s_col) * h_rn(acc) ), float16 [M, N]."""
    sr = np.asarray(scale_row, _F16).reshape(-1, 1)
    sc = np.asarray(scale_col, _F16).reshape(1, -1)
    return hmul(hmul(sr, sc), int_to_half(acc))


def asym_dequant(acc, scale_row, zeros_row, scale_col, zeros_col):
    """y = h( h(s_r*s_c) * h( h( h_rn(acc) - z_r ) - z_c ) )  (quant.cu:167-168)."""
    sr = np.asarray(scale_row, _F16).reshape(-1, 1)
    zr = np.asarray(zeros_row, _F16).reshape(-1, 1)
    sc = np.asarray(scale_col, _F16).reshape(1, -1)
    zc = np.asarray(zeros_col, _F16).reshape(1, -1)
    inner = hsub(hsub(int_to_half(acc), zr), zc)
    return hmul(hmul(sr, sc), inner)


def sym_dual_col_scale(scale_col_1, scale_col_2):
    """col < 10 ? s1[col] : s2[col]  (quant2.cu:81)."""
    s1 = np.asarray(scale_col_1, _F16).reshape(-1)
    s2 = np.asarray(scale_col_2, _F16).reshape(-1)
    col = np.arange(s1.shape[0])
    return np.where(col < QUANT_COL_K, s1, s2)


def sym_dual_dequant(acc, scale_row, scale_col_1, scale_col_2):
    return sym_dequant(acc, scale_row, sym_dual_col_scale(scale_col_1, scale_col_2))


def asym_dual_col_select(v1, v2):
    """``(QUANT_COL_ST << col & 1)`` parses as ``(ST << col) & 1`` and is non-zero only
    for col == 0 (quant2.cu:182-183; bit 0 of ST is set, include/quant.h:7)."""
    v1 = np.asarray(v1, _F16).reshape(-1)
    v2 = np.asarray(v2, _F16).reshape(-1)
    col = np.arange(v1.shape[0])
    return np.where(col == 0, v1, v2)


def asym_dual_dequant(acc, scale_row, zeros_row, scale_col_1, zeros_col_1, scale_col_2, zeros_col_2):
    sc = asym_dual_col_select(scale_col_1, scale_col_2)
    zc = asym_dual_col_select(zeros_col_1, zeros_col_2)
    return asym_dequant(acc, scale_row, zeros_row, sc, zc)


def add_bias(y, bias):
    """y + bias as one fp16 torch op (qlinear4bit/nn/linear.py:53-54)."""
    return hadd(y, np.asarray(bias, _F16).reshape(1, -1))


# ----------------------------------------------------------------------------------
# Row-sum mode: asymmetric forward with the exact zero-point correction.  The reference has
# no such path (its epilogue, src/kernels/quant.cu:167-168, subtracts the zero points from
# the accumulator; README.md:31-32 notes the signed/unsigned mismatch); this restates the
# definition the library documents in include/duq_hip.h.  Pinned by the integer identity
# corr == sum_k (c_x - z_x)(c_w - z_w) (brute force) and by dequantize-then-matmul in float64.
# ----------------------------------------------------------------------------------
def asym_quant_shifted(x):
    """Codes of asym_quant stored as u - 8 (signed nibble), zeros as h(z - 8), and the row sums
    of the shifted codes.  Returns (packed u8, scale [M,1], zeros_shifted [M,1], rowsum int32 [M])."""
    x = np.asarray(x, _F16)
    s, z = asym_scales_zeros(x)
    c = asym_quant_values(x, s, z).astype(np.int32) - 8
    zs = hsub(z, _F16(8.0))
    return pack_i4(c, sym=True), s, zs, c.sum(axis=-1, dtype=np.int64).astype(np.int32)


def weight_rowsum_adj(w_packed_shifted, zeros_shifted):
    """R_w[n] - K * z_w[n] in wrapping int32, from shifted weight codes and shifted zero points."""
    c = unpack_i4(w_packed_shifted, signed=True).astype(np.int64)
    K = c.shape[1]
    z = half_to_int_rn(np.asarray(zeros_shifted, _F16).reshape(-1)).astype(np.int64)
    return _wrap_i32(c.sum(axis=1) - K * z).astype(np.int32)


def asym_rowsum_dequant(acc, scale_row, zeros_row, rowsum_row, scale_col, zeros_col, rowsum_adj_col, bias=None):
    """corr = acc - z_row * adj_col - z_col * rowsum_row (wrapping int32);
    y = h(f32(f32(corr) * (f32(s_row) * f32(s_col)))); with bias y = h(y + bias)."""
    acc = np.asarray(acc, np.int64)
    zr = half_to_int_rn(np.asarray(zeros_row, _F16).reshape(-1)).astype(np.int64)[:, None]
    zc = half_to_int_rn(np.asarray(zeros_col, _F16).reshape(-1)).astype(np.int64)[None, :]
    rr = np.asarray(rowsum_row, np.int64).reshape(-1, 1)
    ac = np.asarray(rowsum_adj_col, np.int64).reshape(1, -1)
    corr = _wrap_i32(_wrap_i32(acc - _wrap_i32(zr * ac)) - _wrap_i32(zc * rr)).astype(np.int32)
    ss = _f32(np.asarray(scale_row, _F16).reshape(-1, 1)) * _f32(np.asarray(scale_col, _F16).reshape(1, -1))
    with np.errstate(invalid="ignore", over="ignore"):
        y = (corr.astype(_F32) * ss).astype(_F16)
    if bias is not None:
        y = add_bias(y, bias)
    return y


def weight_asym_shifted_from_linear(w):
    """Weight preparation for the row-sum mode: per-row true min/max quantization
    scale = h(h(max-min)/15), zero = h(rint(h(h(-min)/scale))), u = clamp(rint(h(w/scale)) + zero, 0, 15),
    stored shifted.  Returns (packed u8, scale [N,1], zeros_shifted [N,1], rowsum_adj int32 [N])."""
    q, s, zs, _ = asym_quant_shifted(w)
    return q, s, zs, weight_rowsum_adj(q, zs)


def linear4bit_asq_rowsum_forward(x, w_packed_shifted, w_scales, w_zeros_shifted, w_rowsum_adj, bias=None):
    """AsymQuantizer(shifted) + row-sum epilogue.  Returns (y, acc, q_x, s_x, z_x, rowsum_x)."""
    q_x, s_x, z_x, r_x = asym_quant_shifted(x)
    acc = matmul_s4(q_x, w_packed_shifted)
    y = asym_rowsum_dequant(acc, s_x, z_x, r_x, w_scales, w_zeros_shifted, w_rowsum_adj, bias)
    return y, acc, q_x, s_x, z_x, r_x


# ----------------------------------------------------------------------------------
# Row-sum mode of the dual-uniform layer.  LinearQuant4bitDUASQ (qlinear4bit/nn/linear.py:252-297) quantizes the
# first QUANT_COL_K = 10 INPUT columns of every weight row with (scale_1, zero_1) and the rest with
# (scale_2, zero_2); its epilogue (src/kernels/quant2.cu:158-186) then applies one pair per OUTPUT column,
# chosen by a selector that is non-zero for column 0 only, to a single accumulator.  The product of the
# dequantized operands needs the accumulator split at input column 10 instead:
#   accL = sum_{k<10} c_x c_w,  accR = acc - accL,  R_xL = sum_{k<10} c_x,  R_xR = R_x - R_xL
#   corrL = accL - z_x * adjL[n] - z_1[n] * R_xL,   adjL[n] = sum_{k<10} c_w[n,k] - 10 * z_1[n]
#   corrR = accR - z_x * adjR[n] - z_2[n] * R_xR,   adjR[n] = sum_{k>=10} c_w[n,k] - (K-10) * z_2[n]
#   y = h( f32(corrL) * (f32(s_x) * f32(s_1)) + f32(corrR) * (f32(s_x) * f32(s_2)) ), every float32 operator
#   rounded; with bias y = h(y + bias).
# This restates the definition in include/duq_hip.h (no counterpart in the reference); pinned by the integer
# identities corrL/R == sum (c_x - z_x)(c_w - z_{1,2}) over their k ranges (brute force) and by the float64
# product of the dequantized operands.
# ----------------------------------------------------------------------------------
def weight_asym_dual_shifted_from_linear(w):
    """Per-row true min/max quantization of the two column ranges, stored shifted.  Returns (packed u8 [N, K/2],
    scale_1, zeros_1_shifted, scale_2, zeros_2_shifted [N,1] each, adjL int32 [N], adjR int32 [N])."""
    w = np.asarray(w, _F16)
    K = w.shape[1]
    parts = []
    for lo, hi in ((0, QUANT_COL_K), (QUANT_COL_K, K)):
        q, s, zs, _ = asym_quant_shifted(np.ascontiguousarray(w[:, lo:hi]) if (hi - lo) % 2 == 0 else
                                         np.concatenate([w[:, lo:hi], w[:, hi - 1:hi]], axis=1))
        c = unpack_i4(q, signed=True)[:, :hi - lo].astype(np.int64)
        z = half_to_int_rn(zs.reshape(-1)).astype(np.int64)
        parts.append((c, s, zs, _wrap_i32(c.sum(axis=1) - (hi - lo) * z).astype(np.int32)))
    codes = np.concatenate([parts[0][0], parts[1][0]], axis=1).astype(np.int8)
    return pack_i4(codes, sym=True), parts[0][1], parts[0][2], parts[1][1], parts[1][2], parts[0][3], parts[1][3]


def asym_dual_rowsum_dequant(acc, x_packed_shifted, scale_row, zeros_row, rowsum_row, w_packed_shifted, scale_col_1,
                             zeros_col_1, scale_col_2, zeros_col_2, adj_col_1, adj_col_2, bias=None):
    """The epilogue defined above on int32 accumulators; the first 10 codes of every activation and weight row
    supply accL and R_xL."""
    cx = unpack_i4(np.asarray(x_packed_shifted)[:, :8], signed=True)[:, :QUANT_COL_K].astype(np.int64)
    cw = unpack_i4(np.asarray(w_packed_shifted)[:, :8], signed=True)[:, :QUANT_COL_K].astype(np.int64)
    accL = cx @ cw.T
    rxL = cx.sum(axis=1)[:, None]
    acc = np.asarray(acc, np.int64)
    zr = half_to_int_rn(np.asarray(zeros_row, _F16).reshape(-1)).astype(np.int64)[:, None]
    z1 = half_to_int_rn(np.asarray(zeros_col_1, _F16).reshape(-1)).astype(np.int64)[None, :]
    z2 = half_to_int_rn(np.asarray(zeros_col_2, _F16).reshape(-1)).astype(np.int64)[None, :]
    rx = np.asarray(rowsum_row, np.int64).reshape(-1, 1)
    a1 = np.asarray(adj_col_1, np.int64).reshape(1, -1)
    a2 = np.asarray(adj_col_2, np.int64).reshape(1, -1)
    corrL = _wrap_i32(accL - zr * a1 - z1 * rxL).astype(np.int32)
    corrR = _wrap_i32((acc - accL) - zr * a2 - z2 * (rx - rxL)).astype(np.int32)
    sr = _f32(np.asarray(scale_row, _F16).reshape(-1, 1))
    ss1 = sr * _f32(np.asarray(scale_col_1, _F16).reshape(1, -1))   # exact in float32 (11-bit significands)
    ss2 = sr * _f32(np.asarray(scale_col_2, _F16).reshape(1, -1))
    with np.errstate(invalid="ignore", over="ignore"):
        t = (corrL.astype(_F32) * ss1).astype(_F32) + (corrR.astype(_F32) * ss2).astype(_F32)
        y = t.astype(_F32).astype(_F16)
    if bias is not None:
        y = add_bias(y, bias)
    return y


def linear4bit_duasq_rowsum_forward(x, w_packed_shifted, ws1, wz1, ws2, wz2, adj1, adj2, bias=None):
    """AsymQuantizer(shifted) + GEMM + dual row-sum epilogue.  Returns (y, acc, q_x, s_x, z_x, rowsum_x)."""
    q_x, s_x, z_x, r_x = asym_quant_shifted(x)
    acc = matmul_s4(q_x, w_packed_shifted)
    y = asym_dual_rowsum_dequant(acc, q_x, s_x, z_x, r_x, w_packed_shifted, ws1, wz1, ws2, wz2, adj1, adj2, bias)
    return y, acc, q_x, s_x, z_x, r_x


# ----------------------------------------------------------------------------------
# A8  module forwards as compositions (qlinear4bit/nn/linear.py:42-56,104-115,
#     167-176,239-250)
# ----------------------------------------------------------------------------------
def linear4bit_sq_forward(x, w_packed, w_scales, bias=None, clip=1.0, qmax=QMAX_SYM_DEVICE):
    """Sequential(SymQuantizer, Linear4bitSQ)(x).  Returns (y, acc, q_x, s_x)."""
    x = np.asarray(x, _F16)
    s_x = sym_scales(x, clip)
    q_x = sym_quant(x, s_x, qmax)
    acc = matmul_s4(q_x, w_packed)
    y = sym_dequant(acc, s_x, w_scales)
    if bias is not None:
        y = add_bias(y, bias)
    return y, acc, q_x, s_x


def linear4bit_asq_forward(x, w_packed, w_scales, w_zeros, bias=None):
    """Linear4bitASQ(x) with its own AsymQuantizer.  Returns (y, acc, q_x, s_x, z_x)."""
    x = np.asarray(x, _F16)
    s_x, z_x = asym_scales_zeros(x)
    q_x = asym_quant(x, s_x, z_x)
    acc = matmul_s4(q_x, w_packed)
    y = asym_dequant(acc, s_x, z_x, w_scales, w_zeros)
    if bias is not None:
        y = add_bias(y, bias)
    return y, acc, q_x, s_x, z_x


def linear4bit_dusq_forward(x, w_packed, w_scales_1, w_scales_2, bias=None, clip=1.0, qmax=QMAX_SYM_DEVICE):
    x = np.asarray(x, _F16)
    s_x = sym_scales(x, clip)
    q_x = sym_quant(x, s_x, qmax)
    acc = matmul_s4(q_x, w_packed)
    y = sym_dual_dequant(acc, s_x, w_scales_1, w_scales_2)
    if bias is not None:
        y = add_bias(y, bias)
    return y, acc, q_x, s_x


def linear4bit_duasq_forward(x, w_packed, ws1, wz1, ws2, wz2, bias=None):
    x = np.asarray(x, _F16)
    s_x, z_x = asym_scales_zeros(x)
    q_x = asym_quant(x, s_x, z_x)
    acc = matmul_s4(q_x, w_packed)
    y = asym_dual_dequant(acc, s_x, z_x, ws1, wz1, ws2, wz2)
    if bias is not None:
        y = add_bias(y, bias)
    return y, acc, q_x, s_x, z_x


# ----------------------------------------------------------------------------------
# A11  CPU fake-quant primitives (qlinear4bit/tools/quantization.py:17-37), for fp16
#      inputs (torch-CPU computes each op in float32 and stores binary16).
# pinned by: the torch-CPU ops themselves (the library routine the reference calls).
# ----------------------------------------------------------------------------------
def fq_sym_quant(x, scale, maxq=QMAX_SYM_FAKEQUANT):
    """q = clamp(round(x / scale), -(maxq+1), maxq), as float16 values."""
    x = np.asarray(x, _F16)
    s = np.asarray(scale, _F16)
    with np.errstate(invalid="ignore"):
        q = h(np.rint(_f32(hdiv(x, s))))
        return h(np.clip(_f32(q), -(maxq + 1), maxq))


def fq_sym_dequant(q, scale):
    return hmul(scale, q)


def fq_asym_quant(x, scale, zero, maxq=QMAX_ASYM):
    x = np.asarray(x, _F16)
    with np.errstate(invalid="ignore"):
        r = h(np.rint(_f32(hdiv(x, scale))))
        return h(np.clip(_f32(hadd(r, zero)), 0, maxq))


def fq_asym_dequant(q, scale, zero):
    return hmul(scale, hsub(q, zero))


# ----------------------------------------------------------------------------------
# Weight preparation (qlinear4bit/nn/linear.py:58-78,117-145) - used to build the
# benchmark / parity inputs the way the reference builds its buffers.
# ----------------------------------------------------------------------------------
def weight_sym_from_float(w, w_scales):
    """int_w = round(W / s_w) in fp16, no clamp; pack_i4 asserts the range
    (linear.py:72-73)."""
    w = np.asarray(w, _F16)
    s = np.asarray(w_scales, _F16).reshape(-1, 1)
    q = np.rint(_f32(hdiv(w, s))).astype(np.int32)
    return pack_i4(q, sym=True)


def weight_asym_from_linear(w):
    """Linear4bitASQ.from_linear (linear.py:126-140): max|W| and min|W| (abs on both),
    scale = (max-min)/15, zero = round(-min/scale), q = clamp(round(W/scale)+zero,0,15).
    Returns (packed u8 [N,K/2], scale fp16 [N,1], zero fp16 [N,1])."""
    w = np.asarray(w, _F16)
    aw = np.abs(w)
    mx = np.max(aw, axis=-1, keepdims=True)
    mn = np.min(aw, axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        scale = h(_f32(hsub(mx, mn)) / _F32(15.0))
        zero = h(np.rint(_f32(hdiv(h(-_f32(mn)), scale))))
        r = h(np.rint(_f32(hdiv(w, scale))))
        q = np.clip(_f32(hadd(r, zero)), 0, 15)
    return pack_i4(q.astype(np.int32), sym=False), scale, zero


# ----------------------------------------------------------------------------------
# E3M2 ("bf6") shadows of packed-int4 tensors: the operand format of the library's 6-bit
# float matrix path (no counterpart in the reference; results stay those of matmul_s4)
# ----------------------------------------------------------------------------------
def e3m2_decode(code):
    """Value of a 6-bit E3M2 code (OCP Microscaling Formats v1.0, FP6 E3M2: 1 sign, 3 exponent
    bits with bias 3, 2 mantissa bits, subnormals at exponent 0, no inf / NaN)."""
    code = np.asarray(code, dtype=np.int64)
    sign = np.where((code >> 5) & 1, -1.0, 1.0)
    e = (code >> 2) & 7
    m = code & 3
    mag = np.where(e == 0, (m / 4.0) * 2.0 ** (1 - 3), (1.0 + m / 4.0) * 2.0 ** (e.astype(np.float64) - 3))
    return sign * mag


def e3m2_encode_int4(v):
    """The E3M2 code of an integer in [-8, 7] (exact: every such integer has at most three
    significant bits).  Zero is +0."""
    v = np.asarray(v, dtype=np.int64)
    table = np.zeros(16, dtype=np.uint8)
    values = e3m2_decode(np.arange(64))
    for x in range(-8, 8):
        hits = [c for c in range(64) if values[c] == x and not (x == 0 and c >= 32)]
        assert len(hits) == 1
        table[x & 15] = hits[0]
    return table[v & 15]


def _shadow_positions():
    """Element index (inside a block of 32 consecutive k) stored at each of the 32 positions:
    position 8d + 2i + hh holds element 8d + i + 4hh (the pairing the quantizer kernels get
    with one shift and one mask per two nibbles)."""
    pos = np.arange(32)
    d, i, hh = pos >> 3, (pos & 7) >> 1, pos & 1
    return 8 * d + i + 4 * hh


def shadow_block_pack(values):
    """values int [..., 32] in [-8, 7] -> uint8 [..., 24]: 32 six-bit codes, position p in bits
    6p .. 6p+5 of the 192-bit little-endian block."""
    values = np.asarray(values)
    codes = e3m2_encode_int4(values[..., _shadow_positions()]).astype(np.uint64)
    bits = np.zeros(values.shape[:-1] + (192,), dtype=np.uint8)
    for b in range(6):
        bits[..., b::6] = ((codes >> np.uint64(b)) & np.uint64(1)).astype(np.uint8)
    out = np.packbits(bits, axis=-1, bitorder="little")
    return out


def shadow_block_unpack(block):
    """Inverse of shadow_block_pack: uint8 [..., 24] -> int [..., 32]."""
    bits = np.unpackbits(np.asarray(block, dtype=np.uint8), axis=-1, bitorder="little")
    codes = np.zeros(bits.shape[:-1] + (32,), dtype=np.int64)
    for b in range(6):
        codes |= bits[..., b::6].astype(np.int64) << b
    vals = e3m2_decode(codes).astype(np.int64)
    out = np.zeros_like(vals)
    out[..., _shadow_positions()] = vals
    return out


def activation_shadow_bf6(q_packed):
    """uint8 [M, K/2] packed nibbles (read as signed, like the GEMM reads them) -> uint8
    [M, 3K/4]: per row the first 16 bytes of each of its K/32 blocks, then the last 8 bytes of
    each.  K % 32 == 0."""
    v = unpack_i4(q_packed, signed=True)
    M, K = v.shape
    blocks = shadow_block_pack(v.reshape(M, K // 32, 32))  # [M, K/32, 24]
    return np.concatenate([blocks[..., :16].reshape(M, -1), blocks[..., 16:].reshape(M, -1)], axis=1)


def weight_shadow_bf6(w_packed):
    """uint8 [N, K/2] -> uint8 [ceil(N/32)*32, 3K/4] in tile-pair order.  For every pair of 16-row tiles and every
    128-k step, lane l = (row l % 16, k-block l // 16) owns one 24-byte block of either tile; the lane's 48 bytes
    [tile 2p | tile 2p+1] are cut into three 16-byte pieces and the 3072 bytes of the (pair, step) are piece 0 of
    the 64 lanes, then piece 1, then piece 2.  An odd last tile is paired with zeros.  N % 16 == 0, K % 128 == 0."""
    v = unpack_i4(w_packed, signed=True)
    N, K = v.shape
    tiles = N // 16
    pairs = (tiles + 1) // 2
    blocks = shadow_block_pack(v.reshape(N, K // 32, 32))  # [N, K/32, 24]
    padded = np.zeros((pairs * 32, K // 32, 24), np.uint8)
    padded[:N] = blocks
    b = padded.reshape(pairs, 2, 16, K // 128, 4, 24)       # pair, half, row, step, kb, byte
    b = b.transpose(0, 3, 4, 2, 1, 5).reshape(pairs, K // 128, 64, 48)  # pair, step, lane = kb*16 + row, [half 0 | half 1]
    out = b.reshape(pairs, K // 128, 64, 3, 16).transpose(0, 1, 3, 2, 4)  # pair, step, piece, lane, byte
    return np.ascontiguousarray(out).reshape(pairs * 32, K * 3 // 4)


# ----------------------------------------------------------------------------------
# 8-bit asymmetric path: AsymQuantizer8bit -> matmul_8bit -> asym_dequant_hprec
# (qlinear4bit/nn/quantizer.py:38-55, src/kernels/quant.cu:241-323, src/kernels/gemm.cu:46-81,
#  qlinear4bit/nn/linear.py:300-368).  Everything is float32 with one rounding per operator.
# ----------------------------------------------------------------------------------
QMAX_ASYM_8BIT = 126     # src/kernels/quant.cu:242
LEVELS_8BIT = 2 ** 7     # quantizer.py:41, linear.py:350


def asym8_scales_zeros(x, device_division: bool = True):
    """AsymQuantizer8bit.forward (quantizer.py:47-51): scale = (max - min) / 127,
    zeros = round(-min / scale), all float32 [rows, 1].

    The reference runs these torch statements on its GPU, where torch evaluates
    tensor / python-scalar as tensor * float32(1 / scalar) (one bit may differ from the
    quotient); ``device_division=False`` gives the true quotient torch computes on a CPU.
    tensor / tensor is the IEEE quotient on both."""
    x = np.asarray(x, _F32)
    lo = x.min(axis=-1, keepdims=True)
    hi = x.max(axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        d = (hi - lo).astype(_F32)
        if device_division:
            scale = (d * (_F32(1.0) / _F32(LEVELS_8BIT - 1))).astype(_F32)
        else:
            scale = (d / _F32(LEVELS_8BIT - 1)).astype(_F32)
        zeros = np.rint(((-lo).astype(_F32) / scale).astype(_F32)).astype(_F32)
    return scale, zeros


def asym_quant_8bit(x, scale, zeros):
    """asym_quantize_f16_i8_kernel (quant.cu:244-264): data = x / scale in float32; both
    ``__half2int_rn`` calls take a float argument, which C++ converts to binary16 first
    (round to nearest even, overflow to inf), then round to the nearest-even integer; the
    int add wraps; clamp to [0, 126]; stored as int8."""
    x = np.asarray(x, _F32)
    s = np.asarray(scale, _F32).reshape(-1, 1)
    z = np.asarray(zeros, _F32).reshape(-1, 1)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        data = (x / s).astype(_F32)
        qi = half_to_int_rn(data.astype(_F16))
        zi = half_to_int_rn(z.astype(_F16))
    total = _wrap_i32(qi.astype(np.int64) + zi.astype(np.int64))
    return np.clip(total, 0, QMAX_ASYM_8BIT).astype(np.int8)


def matmul_s8(a, b):
    """matmul_host_8bit (gemm.cu:46-81): C[m,n] = sum_k A[m,k] * B[n,k], int8 operands,
    int32 accumulation.  The sum is taken modulo 2**32 here; the library accepts K <= 131040 only, where no
    accumulator can overflow (|sum| <= 2**14 * K < 2**31) and wrapping and saturating units agree."""
    # float64 BLAS is exact here: |sum| <= 2^14 * K, far below 2^53
    a = np.asarray(a, np.int8).astype(np.float64)
    b = np.asarray(b, np.int8).astype(np.float64)
    return _wrap_i32((a @ b.T).astype(np.int64))


def asym_dequant_hprec(acc, scale_row, zeros_row, scale_col, zeros_col):
    """asym_dequantize_i32_f16_hp_kernel (quant.cu:283-299), float32 throughout:
    x = (s_r * s_c) * (float(acc) - (z_r + z_c))."""
    acc = np.asarray(acc, np.int32)
    sr = np.asarray(scale_row, _F32).reshape(-1, 1)
    zr = np.asarray(zeros_row, _F32).reshape(-1, 1)
    sc = np.asarray(scale_col, _F32).reshape(1, -1)
    zc = np.asarray(zeros_col, _F32).reshape(1, -1)
    with np.errstate(invalid="ignore", over="ignore"):
        scales = (sr * sc).astype(_F32)
        zeros = (zr + zc).astype(_F32)
        return (scales * (acc.astype(_F32) - zeros).astype(_F32)).astype(_F32)


def weight_asym8_from_linear(w):
    """LinearQuant8bitASQ.from_linear (linear.py:346-360): max|W| and min|W| per row,
    scale = (max - min) / 127, zero = round(-min / scale) as float32,
    q = clamp(round(W / scale) + zero, 0, 127) as int8; the arithmetic runs in the dtype of
    the layer's weight (binary16 in the reference's use).  The division by 127 is the true
    quotient, as torch computes it for a module on the CPU (on a GPU see asym8_scales_zeros)."""
    w = np.asarray(w)
    dt = w.dtype.type
    aw = np.abs(w)
    mx = aw.max(axis=-1, keepdims=True)
    mn = aw.min(axis=-1, keepdims=True)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        scale = ((mx - mn).astype(dt) / dt(LEVELS_8BIT - 1)).astype(dt)
        zero = np.rint(((-mn).astype(dt) / scale).astype(dt)).astype(_F32)
        # the sum of the binary16 quotient and the float32 zero point is float32 (torch's type promotion)
        q = np.clip(np.rint((w / scale).astype(dt)).astype(_F32) + zero, 0, LEVELS_8BIT - 1)
    return q.astype(np.int8), scale.astype(_F32), zero


def weight_tile_8bit(w):
    """The library's tiled copy of an int8 weight [N, K] (K % 32 == 0; a storage format of the library, not of the
    reference): [ceil(N/32)][K/32][h = 0..1][r = 0..31][16 bytes] holding W[32*nt + r][32*ks + 16*h + (0..15)],
    rows past N zero; flat int8."""
    w = np.asarray(w, np.int8)
    n, k = w.shape
    nt = -(-n // 32)
    padded = np.zeros((nt * 32, k), np.int8)
    padded[:n] = w
    return padded.reshape(nt, 32, k // 32, 2, 16).transpose(0, 2, 3, 1, 4).reshape(-1).copy()


def linear8bit_asq_forward(x, w_q, w_scales, w_zeros, bias=None):
    """LinearQuant8bitASQ.forward (linear.py:326-337) for float32 x [M,K]:
    returns (y float32, acc int32, q int8, scale, zeros)."""
    s, z = asym8_scales_zeros(x)
    q = asym_quant_8bit(x, s, z)
    acc = matmul_s8(q, w_q)
    y = asym_dequant_hprec(acc, s, z, w_scales, w_zeros)
    if bias is not None:
        y = (y + np.asarray(bias, _F32).reshape(1, -1)).astype(_F32)
    return y, acc, q, s, z
