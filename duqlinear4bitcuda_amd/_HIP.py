"""Tensor-level ops with the names and signatures of the reference's pybind11 module
``qlinear4bit._CUDA`` (src/export/bindings.cpp:768-932), for the Linear4bit path.

Each op checks its tensors the way the reference binding does (contiguous, on a GPU,
same device, matching sizes), allocates its output with ``torch.empty`` on the input's
device, and calls the C ABI on the current torch stream.  Argument errors raise
``RuntimeError`` as ``torch::check*`` does in the reference.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib

_QUANT_COL_K = 10


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


_raw_stream = torch._C._cuda_getCurrentRawStream  # (device index) -> hipStream_t as int; no Stream object built
_current_device = torch._C._cuda_getDevice
_F16, _U8 = torch.float16, torch.uint8


def _launch(dev: torch.device, fn, *args):
    """Call ``fn(*args, stream)`` with ``dev`` current, on its current torch stream.  The
    device guard is only entered when another device is current."""
    idx = dev.index
    if idx == torch._C._cuda_getDevice():
        return fn(*args, _raw_stream(idx))
    with torch.cuda.device(idx):
        return fn(*args, _raw_stream(idx))


def _fast_check(name, what, t, dtype, dev):
    """Contiguity / device / dtype check of one tensor of a fused op."""
    if t.dtype is not dtype or not t.is_cuda or not t.is_contiguous() or (dev is not None and t.device != dev):
        _check(name, t)
        _check_dtype(name, t, what, dtype)
        raise RuntimeError(f"{name}: expected all tensors on {dev}, {what} is on {t.device}")


def _check(name, *tensors):
    dev = None
    for i, t in enumerate(tensors):
        if not isinstance(t, torch.Tensor):
            raise RuntimeError(f"{name}: argument #{i} is not a tensor")
        if not t.is_contiguous():
            raise RuntimeError(f"{name}: expected argument #{i} to be contiguous")
        if not t.is_cuda:
            raise RuntimeError(f"{name}: expected argument #{i} to be on a GPU device, got {t.device}")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"{name}: expected all tensors on {dev}, argument #{i} is on {t.device}")


def _check_size0(name, t, what, n):
    if t.dim() < 1 or t.size(0) != n:
        raise RuntimeError(f"{name}: expected {what} to have size {n} at dimension 0, got {tuple(t.shape)}")


def _check_dtype(name, t, what, dtype):
    if t.dtype != dtype:
        raise RuntimeError(f"{name}: expected {what} to have dtype {dtype}, got {t.dtype}")


def _ptr(t):
    return t.data_ptr() if t is not None else None


def matmul(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """int4Unpack(A) @ int4Unpack(B)^T -> int32 [M, N] (bindings.cpp:10-26)."""
    _check("matmul", A, B)
    _check_dtype("matmul", A, "A", torch.uint8)
    _check_dtype("matmul", B, "B", torch.uint8)
    M, N, K = A.size(0), B.size(0), A.size(1) * 2
    if B.size(1) != A.size(1):
        raise RuntimeError(f"matmul: packed K differs: A {tuple(A.shape)} vs B {tuple(B.shape)}")
    C = torch.empty((M, N), dtype=torch.int32, device=A.device)
    with torch.cuda.device(A.device):
        st = _lib.load().duq_matmul_host_4bit(_ptr(A), _ptr(B), M, N, K, _ptr(C), _stream(A))
    _lib.check(st, "matmul")
    return C


def batched_matmul(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """A [n, M, K/2], B [n, N, K/2] packed -> int32 [n, M, N], entry i = matmul(A[i], B[i]), in one launch
    (bindings.cpp:46-86; the reference hands CUTLASS pointer arrays built from the same strides and prints two
    lines to stdout, which is left out)."""
    _check("batched_matmul", A, B)
    _check_dtype("batched_matmul", A, "A", torch.uint8)
    _check_dtype("batched_matmul", B, "B", torch.uint8)
    if A.dim() != 3 or B.dim() != 3:
        raise RuntimeError(f"batched_matmul: expected A [n, M, K/2] and B [n, N, K/2], got {tuple(A.shape)} and {tuple(B.shape)}")
    n, M, kb = A.shape
    N = B.size(1)
    if B.size(0) != n or B.size(2) != kb:
        raise RuntimeError(f"batched_matmul: batch or packed K differs: A {tuple(A.shape)} vs B {tuple(B.shape)}")
    C = torch.empty((n, M, N), dtype=torch.int32, device=A.device)
    st = _launch(A.device, _lib.load().duq_batch_matmul_host_4bit, _ptr(A), _ptr(B), M, N, kb * 2, _ptr(C), n)
    _lib.check(st, "batched_matmul")
    return C


def sym_quant(x: torch.Tensor, scale: torch.Tensor, qmax: int = 6) -> torch.Tensor:
    """int4Pack(clamp(rint(x / scale), -8, qmax)) -> uint8 [M, ceil(K/2)] (bindings.cpp:88-105).
    ``qmax`` defaults to 6, the bound the reference device kernel really applies
    (include/common.h:53-54)."""
    _check("sym_quant", x, scale)
    _check_dtype("sym_quant", x, "x", torch.float16)
    _check_dtype("sym_quant", scale, "scale", torch.float16)
    _check_size0("sym_quant", scale, "scale", x.size(0))
    rows, cols = x.size(0), x.size(1)
    cd = (cols + 1) // 2
    q = torch.empty((rows, cd), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        st = _lib.load().duq_sym_quant_host_qmax(_ptr(x), _ptr(scale), rows, cols, cd, qmax, _ptr(q), _stream(x))
    _lib.check(st, "sym_quant")
    return q


def sym_dual_quant(x, scale_1, scale_2):
    """bindings.cpp:107-127."""
    _check("sym_dual_quant", x, scale_1, scale_2)
    for t, n in ((x, "x"), (scale_1, "scale_1"), (scale_2, "scale_2")):
        _check_dtype("sym_dual_quant", t, n, torch.float16)
    _check_size0("sym_dual_quant", scale_1, "scale_1", x.size(0))
    _check_size0("sym_dual_quant", scale_2, "scale_2", x.size(0))
    rows, cols = x.size(0), x.size(1)
    cd = (cols + 1) // 2
    q = torch.empty((rows, cd), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        st = _lib.load().duq_sym_dual_quant_host(_ptr(x), _ptr(scale_1), _ptr(scale_2), rows, cols, cd, _ptr(q),
                                                 _stream(x))
    _lib.check(st, "sym_dual_quant")
    return q


def asym_quant(x, scale, zeros):
    """bindings.cpp:221-243."""
    _check("asym_quant", x, scale, zeros)
    for t, n in ((x, "x"), (scale, "scale"), (zeros, "zeros")):
        _check_dtype("asym_quant", t, n, torch.float16)
    _check_size0("asym_quant", scale, "scale", x.size(0))
    _check_size0("asym_quant", zeros, "zeros", x.size(0))
    rows, cols = x.size(0), x.size(1)
    cd = (cols + 1) // 2
    q = torch.empty((rows, cd), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        st = _lib.load().duq_asym_quant_host(_ptr(x), _ptr(scale), _ptr(zeros), rows, cols, cd, _ptr(q), _stream(x))
    _lib.check(st, "asym_quant")
    return q


def asym_dual_quant(x, scale_1, zeros_1, scale_2, zeros_2):
    """bindings.cpp:393-421 (whose body forgets to return q; this one returns it)."""
    ts = (x, scale_1, zeros_1, scale_2, zeros_2)
    _check("asym_dual_quant", *ts)
    for t, n in zip(ts, ("x", "scale_1", "zeros_1", "scale_2", "zeros_2")):
        _check_dtype("asym_dual_quant", t, n, torch.float16)
        if t is not x:
            _check_size0("asym_dual_quant", t, n, x.size(0))
    rows, cols = x.size(0), x.size(1)
    cd = (cols + 1) // 2
    q = torch.empty((rows, cd), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        st = _lib.load().duq_asym_dual_quant_host(_ptr(x), _ptr(scale_1), _ptr(zeros_1), _ptr(scale_2),
                                                  _ptr(zeros_2), rows, cols, cd, _ptr(q), _stream(x))
    _lib.check(st, "asym_dual_quant")
    return q


def _check_bits(name, bits):
    if bits != 32:
        raise RuntimeError(f"{name}: Unsupported data type")  # bindings.cpp:159-167


def sym_dequant(q, scale_row, scale_col, bits: int = 32):
    """bindings.cpp:130-170."""
    _check("sym_dequant", q, scale_row, scale_col)
    _check_dtype("sym_dequant", q, "q", torch.int32)
    _check_dtype("sym_dequant", scale_row, "scale_row", torch.float16)
    _check_dtype("sym_dequant", scale_col, "scale_col", torch.float16)
    rows, cols = q.size(0), q.size(1)
    _check_size0("sym_dequant", scale_row, "scale_row", rows)
    _check_size0("sym_dequant", scale_col, "scale_col", cols)
    _check_bits("sym_dequant", bits)
    x = torch.empty(q.shape, dtype=torch.float16, device=q.device)
    with torch.cuda.device(q.device):
        st = _lib.load().duq_sym_dequant_host(_ptr(q), _ptr(scale_row), _ptr(scale_col), rows, cols, _ptr(x),
                                              _stream(q))
    _lib.check(st, "sym_dequant")
    return x


def sym_dual_dequant(q, scale_row, scale_col_1, scale_col_2, bits: int = 32):
    """bindings.cpp:172-217."""
    ts = (q, scale_row, scale_col_1, scale_col_2)
    _check("sym_dual_dequant", *ts)
    _check_dtype("sym_dual_dequant", q, "q", torch.int32)
    for t, n in zip(ts[1:], ("scale_row", "scale_col_1", "scale_col_2")):
        _check_dtype("sym_dual_dequant", t, n, torch.float16)
    rows, cols = q.size(0), q.size(1)
    _check_size0("sym_dual_dequant", scale_row, "scale_row", rows)
    _check_size0("sym_dual_dequant", scale_col_1, "scale_col_1", cols)
    _check_size0("sym_dual_dequant", scale_col_2, "scale_col_2", cols)
    _check_bits("sym_dual_dequant", bits)
    x = torch.empty(q.shape, dtype=torch.float16, device=q.device)
    with torch.cuda.device(q.device):
        st = _lib.load().duq_sym_dual_dequant_host(_ptr(q), _ptr(scale_row), _ptr(scale_col_1), _ptr(scale_col_2),
                                                   rows, cols, _ptr(x), _stream(q))
    _lib.check(st, "sym_dual_dequant")
    return x


def asym_dequant(q, scale_row, zeros_row, scale_col, zeros_col, bits: int = 32):
    """bindings.cpp:268-307."""
    ts = (q, scale_row, zeros_row, scale_col, zeros_col)
    _check("asym_dequant", *ts)
    _check_dtype("asym_dequant", q, "q", torch.int32)
    for t, n in zip(ts[1:], ("scale_row", "zeros_row", "scale_col", "zeros_col")):
        _check_dtype("asym_dequant", t, n, torch.float16)
    rows, cols = q.size(0), q.size(1)
    _check_size0("asym_dequant", scale_row, "scale_row", rows)
    _check_size0("asym_dequant", zeros_row, "zeros_row", rows)
    _check_size0("asym_dequant", scale_col, "scale_col", cols)
    _check_size0("asym_dequant", zeros_col, "zeros_col", cols)
    _check_bits("asym_dequant", bits)
    x = torch.empty(q.shape, dtype=torch.float16, device=q.device)
    with torch.cuda.device(q.device):
        st = _lib.load().duq_asym_dequant_host(_ptr(q), _ptr(scale_row), _ptr(zeros_row), _ptr(scale_col),
                                               _ptr(zeros_col), rows, cols, _ptr(x), _stream(q))
    _lib.check(st, "asym_dequant")
    return x


def asym_batch_dequant(q, scale_row, zeros_row, scale_col, zeros_col, bits: int = 32):
    """bindings.cpp:351-391 (kernel src/kernels/quant.cu:190-239): the asymmetric epilogue on a batch
    of accumulator matrices q [batches, rows, cols], every batch with its own row / column
    parameters (scale_row, zeros_row [batches, rows(,1)]; scale_col, zeros_col [batches, cols(,1)])."""
    ts = (q, scale_row, zeros_row, scale_col, zeros_col)
    _check("asym_batch_dequant", *ts)
    _check_dtype("asym_batch_dequant", q, "q", torch.int32)
    if q.dim() != 3:
        raise RuntimeError(f"asym_batch_dequant: expected q [batches, rows, cols], got {tuple(q.shape)}")
    batches, rows, cols = q.shape
    for t, n, want in zip(ts[1:], ("scale_row", "zeros_row", "scale_col", "zeros_col"), (rows, rows, cols, cols)):
        _check_dtype("asym_batch_dequant", t, n, torch.float16)
        if t.dim() < 2 or t.size(1) != want or t.numel() != batches * want:
            raise RuntimeError(f"asym_batch_dequant: expected {n} to have size {want} at dimension 1, got {tuple(t.shape)}")
    _check_bits("asym_batch_dequant", bits)
    x = torch.empty(q.shape, dtype=torch.float16, device=q.device)
    st = _launch(q.device, _lib.load().duq_asym_batch_dequant_host, _ptr(q), _ptr(scale_row), _ptr(zeros_row),
                 _ptr(scale_col), _ptr(zeros_col), batches, rows, cols, _ptr(x))
    _lib.check(st, "asym_batch_dequant")
    return x


def asym_dual_dequant(q, scale_row, zeros_row, scale_col_1, zeros_col_1, scale_col_2, zeros_col_2, bits: int = 32):
    """bindings.cpp:423-467."""
    ts = (q, scale_row, zeros_row, scale_col_1, zeros_col_1, scale_col_2, zeros_col_2)
    _check("asym_dual_dequant", *ts)
    _check_dtype("asym_dual_dequant", q, "q", torch.int32)
    names = ("scale_row", "zeros_row", "scale_col_1", "zeros_col_1", "scale_col_2", "zeros_col_2")
    for t, n in zip(ts[1:], names):
        _check_dtype("asym_dual_dequant", t, n, torch.float16)
    rows, cols = q.size(0), q.size(1)
    for t, n in zip(ts[1:3], names[:2]):
        _check_size0("asym_dual_dequant", t, n, rows)
    for t, n in zip(ts[3:], names[2:]):
        _check_size0("asym_dual_dequant", t, n, cols)
    _check_bits("asym_dual_dequant", bits)
    x = torch.empty(q.shape, dtype=torch.float16, device=q.device)
    with torch.cuda.device(q.device):
        st = _lib.load().duq_asym_dual_dequant_host(_ptr(q), _ptr(scale_row), _ptr(zeros_row), _ptr(scale_col_1),
                                                    _ptr(zeros_col_1), _ptr(scale_col_2), _ptr(zeros_col_2), rows,
                                                    cols, _ptr(x), _stream(q))
    _lib.check(st, "asym_dual_dequant")
    return x


def get_dual_quant_col_k() -> int:
    """bindings.cpp:471-473."""
    return _QUANT_COL_K


# ---- additions over the reference module: fused ops -----------------------------------

def quantize_rows_sym(x: torch.Tensor, clip: float = 1.0, qmax: int = 6):
    """One-pass SymQuantizer (qlinear4bit/nn/quantizer.py:10-16) over the last dimension of a
    contiguous fp16 tensor [..., K]: returns (q uint8 [..., K/2], scales fp16 [..., 1]).
    Requires K % 32 == 0."""
    if not isinstance(x, torch.Tensor):
        raise RuntimeError("quantize_rows_sym: argument #0 is not a tensor")
    _fast_check("quantize_rows_sym", "x", x, _F16, None)
    shape = x.shape
    cols = shape[-1]
    rows = x.numel() // cols if cols else 0
    lead = shape[:-1]
    dev = x.device
    q = torch.empty(lead + (cols // 2,), dtype=_U8, device=dev)
    s = torch.empty(lead + (1,), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_quantize_rows_sym, x.data_ptr(), rows, cols, float(clip), qmax, q.data_ptr(),
                 s.data_ptr())
    if st:
        _lib.check(st, "quantize_rows_sym")
    return q, s


def quantize_rows_asym(x: torch.Tensor):
    """One-pass AsymQuantizer (qlinear4bit/nn/quantizer.py:24-35) over the last dimension:
    returns (q, scale [..., 1], zeros [..., 1]).  Requires K % 32 == 0."""
    if not isinstance(x, torch.Tensor):
        raise RuntimeError("quantize_rows_asym: argument #0 is not a tensor")
    _fast_check("quantize_rows_asym", "x", x, _F16, None)
    shape = x.shape
    cols = shape[-1]
    rows = x.numel() // cols if cols else 0
    lead = shape[:-1]
    dev = x.device
    q = torch.empty(lead + (cols // 2,), dtype=_U8, device=dev)
    s = torch.empty(lead + (1,), dtype=_F16, device=dev)
    z = torch.empty(lead + (1,), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_quantize_rows_asym, x.data_ptr(), rows, cols, q.data_ptr(), s.data_ptr(),
                 z.data_ptr())
    if st:
        _lib.check(st, "quantize_rows_asym")
    return q, s, z


EPI_SYM, EPI_ASYM, EPI_SYM_DUAL, EPI_ASYM_DUAL = 0, 1, 2, 3
EPI_ASYM_ROWSUM = 4        # exact zero-point correction with row sums; not in the reference
EPI_ASYM_DUAL_ROWSUM = 5   # the same for the dual-uniform layer (one-launch decode entry point only)


def linear4bit_forward(mode, xq, scale_x, zeros_x, w, w_scale_1, w_zeros_1=None, w_scale_2=None, w_zeros_2=None,
                       bias=None):
    """matmul + dequant (+ bias) in one launch; bit-identical to the separate ops.
    ``xq`` is uint8 [..., K/2] (leading dimensions are flattened to M rows), ``w`` uint8
    [N, K/2]; per-row tensors hold M, per-column tensors N fp16 values in any contiguous
    shape.  Returns fp16 [..., N]."""
    name = "linear4bit_forward"
    if not isinstance(xq, torch.Tensor) or not isinstance(w, torch.Tensor):
        raise RuntimeError(f"{name}: xq and w must be tensors")
    dev = xq.device
    _fast_check(name, "xq", xq, _U8, None)
    _fast_check(name, "w", w, _U8, dev)
    kb = xq.shape[-1]
    if w.dim() != 2 or w.shape[1] != kb:
        raise RuntimeError(f"{name}: packed K differs: x {tuple(xq.shape)} vs w {tuple(w.shape)}")
    M = xq.numel() // kb if kb else 0
    N = w.shape[0]
    _fast_check(name, "scale_x", scale_x, _F16, dev)
    if scale_x.numel() != M:
        _check_size0(name, scale_x.reshape(-1), "scale_x", M)
    pz = 0
    if zeros_x is not None:
        _fast_check(name, "zeros_x", zeros_x, _F16, dev)
        if zeros_x.numel() != M:
            _check_size0(name, zeros_x.reshape(-1), "zeros_x", M)
        pz = zeros_x.data_ptr()
    _fast_check(name, "w_scale_1", w_scale_1, _F16, dev)
    if w_scale_1.numel() != N:
        _check_size0(name, w_scale_1.reshape(-1), "w_scale_1", N)
    ptrs = [0, 0, 0, 0]
    if w_zeros_1 is not None or w_scale_2 is not None or w_zeros_2 is not None or bias is not None:
        for k, (t, what) in enumerate(((w_zeros_1, "w_zeros_1"), (w_scale_2, "w_scale_2"), (w_zeros_2, "w_zeros_2"),
                                       (bias, "bias"))):
            if t is not None:
                _fast_check(name, what, t, _F16, dev)
                if t.numel() != N:
                    _check_size0(name, t.reshape(-1), what, N)
                ptrs[k] = t.data_ptr()
    y = torch.empty(xq.shape[:-1] + (N,), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_linear4bit_forward, mode, xq.data_ptr(), scale_x.data_ptr(), pz or None,
                 w.data_ptr(), w_scale_1.data_ptr(), ptrs[0] or None, ptrs[1] or None, ptrs[2] or None,
                 ptrs[3] or None, M, N, kb * 2, y.data_ptr())
    if st:
        _lib.check(st, name)
    return y


def batch_linear4bit_forward(mode, xq, scale_x, zeros_x, w, w_scale_1, w_zeros_1=None, w_scale_2=None, w_zeros_2=None,
                             bias=None):
    """``linear4bit_forward`` over a batch in one launch: ``xq`` uint8 [n, M, K/2], ``w`` uint8 [n, N, K/2],
    per-row tensors n * M and per-column tensors (and bias) n * N fp16 values, contiguous over the batch.
    Returns fp16 [n, M, N], entry i bit-identical to ``linear4bit_forward`` on the i-th slices."""
    name = "batch_linear4bit_forward"
    if not isinstance(xq, torch.Tensor) or not isinstance(w, torch.Tensor):
        raise RuntimeError(f"{name}: xq and w must be tensors")
    dev = xq.device
    _fast_check(name, "xq", xq, _U8, None)
    _fast_check(name, "w", w, _U8, dev)
    if xq.dim() != 3 or w.dim() != 3 or w.shape[0] != xq.shape[0] or w.shape[2] != xq.shape[2]:
        raise RuntimeError(f"{name}: expected xq [n, M, K/2] and w [n, N, K/2], got {tuple(xq.shape)} and {tuple(w.shape)}")
    n, M, kb = xq.shape
    N = w.shape[1]
    ptrs = []
    for t, what, cnt, need in ((scale_x, "scale_x", n * M, True), (zeros_x, "zeros_x", n * M, False),
                               (w_scale_1, "w_scale_1", n * N, True), (w_zeros_1, "w_zeros_1", n * N, False),
                               (w_scale_2, "w_scale_2", n * N, False), (w_zeros_2, "w_zeros_2", n * N, False),
                               (bias, "bias", n * N, False)):
        if t is None:
            if need:
                raise RuntimeError(f"{name}: {what} is required")
            ptrs.append(None)
            continue
        _fast_check(name, what, t, _F16, dev)
        if t.numel() != cnt:
            raise RuntimeError(f"{name}: expected {what} to hold {cnt} values, got {tuple(t.shape)}")
        ptrs.append(t.data_ptr())
    y = torch.empty((n, M, N), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_batch_linear4bit_forward, mode, xq.data_ptr(), ptrs[0], ptrs[1], w.data_ptr(),
                 ptrs[2], ptrs[3], ptrs[4], ptrs[5], ptrs[6], n, M, N, kb * 2, y.data_ptr())
    if st:
        _lib.check(st, name)
    return y


def gemm_stream_tile_for(M: int, N: int, K: int) -> int:
    """Tile of the stream kernel for a shape (rows * 1000 + columns), 0 for shapes other kernels run; see
    ``duq_gemm_stream_tile_for`` in include/duq_hip.h."""
    return _lib.load().duq_gemm_stream_tile_for(M, N, K)


def gemm_kernel_for(M: int, N: int, K: int) -> int:
    """Which kernel family the int4 GEMM runs for a shape (host arithmetic, no GPU work): see
    ``duq_gemm_kernel_for`` in include/duq_hip.h."""
    return _lib.load().duq_gemm_kernel_for(M, N, K)


def quantize_linear4bit_one_launch(M: int, N: int, K: int) -> bool:
    """True when ``quantize_linear4bit_forward`` runs the shape as one launch (no staging buffer)."""
    return M > 0 and N > 0 and K > 0 and _lib.load().duq_quantize_linear4bit_workspace_bytes(M, N, K) == 0


def probe_read(t: torch.Tensor):
    """Measurement aid: read every byte of ``t`` with the decode kernels' access pattern and discard them (the
    floor of a decode launch over weights of that size)."""
    _check("probe_read", t)
    st = _launch(t.device, _lib.load().duq_probe_read, t.data_ptr(), t.numel() * t.element_size(), None)
    if st:
        _lib.check(st, "probe_read")


def quantize_linear4bit_forward(x, w, w_scale_1, w_scale_2=None, bias=None, clip: float = 1.0, qmax: int = 6,
                                return_quantized: bool = False, static: bool = False, slot: int = 0):
    """SymQuantizer + Linear4bitSQ / Linear4bitDUSQ forward (qlinear4bit/nn/quantizer.py:10-16,
    qlinear4bit/nn/linear.py:42-56, 167-176) from binary16 activations ``x`` [..., K]: bit-identical to
    ``quantize_rows_sym`` followed by ``linear4bit_forward``.  Up to eight rows (and nine to sixteen that hold at
    most 32768 elements together) are ONE launch; larger inputs run the two launches with the codes staged in a buffer allocated here.  With
    ``return_quantized`` also returns (codes uint8 [..., K/2], scales [..., 1]).  ``static=True`` stages in the
    library's static device array instead (``duq_quantize_linear4bit_forward_static``: nothing but the outputs is
    allocated; M * K / 2 <= 8 MiB; calls that may overlap on one GPU must name different ``slot``s, 0..3)."""
    name = "quantize_linear4bit_forward"
    if not isinstance(x, torch.Tensor) or not isinstance(w, torch.Tensor):
        raise RuntimeError(f"{name}: x and w must be tensors")
    dev = x.device
    _fast_check(name, "x", x, _F16, None)
    _fast_check(name, "w", w, _U8, dev)
    K = x.shape[-1]
    if w.dim() != 2 or w.shape[1] * 2 != K:
        raise RuntimeError(f"{name}: K differs: x {tuple(x.shape)} vs packed w {tuple(w.shape)}")
    M = x.numel() // K if K else 0
    N = w.shape[0]
    ptrs = [0, 0, 0]
    for k, (t, what) in enumerate(((w_scale_1, "w_scale_1"), (w_scale_2, "w_scale_2"), (bias, "bias"))):
        if t is None:
            continue
        _fast_check(name, what, t, _F16, dev)
        if t.numel() != N:
            _check_size0(name, t.reshape(-1), what, N)
        ptrs[k] = t.data_ptr()
    lead = x.shape[:-1]
    y = torch.empty(lead + (N,), dtype=_F16, device=dev)
    q = s = None
    if return_quantized:
        q = torch.empty(lead + (K // 2,), dtype=_U8, device=dev)
        s = torch.empty(lead + (1,), dtype=_F16, device=dev)
    lib = _lib.load()
    ws, ws_bytes = None, 0
    mode = EPI_SYM if w_scale_2 is None else EPI_SYM_DUAL
    if static:
        st = _launch(dev, lib.duq_quantize_linear4bit_forward_static, mode, x.data_ptr(), float(clip), qmax, w.data_ptr(),
                     ptrs[0] or None, ptrs[1] or None, ptrs[2] or None, M, N, K, y.data_ptr(), _ptr(q), _ptr(s), slot)
        if st:
            _lib.check(st, name)
        return (y, q, s) if return_quantized else y
    if not return_quantized:
        ws_bytes = lib.duq_quantize_linear4bit_workspace_bytes(M, N, K)
        if ws_bytes:
            ws = torch.empty(ws_bytes, dtype=_U8, device=dev)
    st = _launch(dev, lib.duq_quantize_linear4bit_forward, mode,
                 x.data_ptr(), float(clip), qmax, w.data_ptr(), ptrs[0] or None, ptrs[1] or None, ptrs[2] or None, M, N, K,
                 y.data_ptr(), _ptr(q), _ptr(s), _ptr(ws), ws_bytes)
    if st:
        _lib.check(st, name)
    return (y, q, s) if return_quantized else y


def quantize_linear4bit_forward_asym(mode, x, w, w_scale_1, w_zeros_1, w_scale_2=None, w_zeros_2=None,
                                     w_rowsum_adj=None, bias=None, return_quantized: bool = False, w_rowsum_adj_2=None):
    """AsymQuantizer + Linear4bitASQ / LinearQuant4bitDUASQ forward (qlinear4bit/nn/quantizer.py:24-35,
    qlinear4bit/nn/linear.py:104-115, 239-250) from binary16 activations ``x`` [..., K], and the row-sum layer's
    (``mode`` EPI_ASYM_ROWSUM with ``w_rowsum_adj``, or EPI_ASYM_DUAL_ROWSUM with ``w_rowsum_adj`` /
    ``w_rowsum_adj_2`` for the dual-uniform layer: the signed-shifted quantizer): bit-identical to
    ``quantize_rows_asym`` (``quantize_rows_asym_shifted``) followed by ``linear4bit_forward``
    (``linear4bit_forward_rowsum`` / ``linear4bit_forward_dual_rowsum``).  Up to eight rows (sixteen short ones) are
    ONE launch; larger inputs run the two launches with the
    codes staged in a buffer allocated here.  With ``return_quantized`` also returns (codes, scales [..., 1],
    zeros [..., 1][, rowsum [...]])."""
    name = "quantize_linear4bit_forward_asym"
    if mode not in (EPI_ASYM, EPI_ASYM_DUAL, EPI_ASYM_ROWSUM, EPI_ASYM_DUAL_ROWSUM):
        raise RuntimeError(f"{name}: mode must be EPI_ASYM, EPI_ASYM_DUAL, EPI_ASYM_ROWSUM or EPI_ASYM_DUAL_ROWSUM")
    if not isinstance(x, torch.Tensor) or not isinstance(w, torch.Tensor):
        raise RuntimeError(f"{name}: x and w must be tensors")
    dev = x.device
    _fast_check(name, "x", x, _F16, None)
    _fast_check(name, "w", w, _U8, dev)
    K = x.shape[-1]
    if w.dim() != 2 or w.shape[1] * 2 != K:
        raise RuntimeError(f"{name}: K differs: x {tuple(x.shape)} vs packed w {tuple(w.shape)}")
    M = x.numel() // K if K else 0
    N = w.shape[0]
    ptrs = []
    for t, what, dt in ((w_scale_1, "w_scale_1", _F16), (w_zeros_1, "w_zeros_1", _F16), (w_scale_2, "w_scale_2", _F16),
                        (w_zeros_2, "w_zeros_2", _F16), (w_rowsum_adj, "w_rowsum_adj", _I32),
                        (w_rowsum_adj_2, "w_rowsum_adj_2", _I32), (bias, "bias", _F16)):
        if t is None:
            ptrs.append(None)
            continue
        _fast_check(name, what, t, dt, dev)
        if t.numel() != N:
            _check_size0(name, t.reshape(-1), what, N)
        ptrs.append(t.data_ptr())
    lead = x.shape[:-1]
    y = torch.empty(lead + (N,), dtype=_F16, device=dev)
    q = s = z = r = None
    rowsum = mode in (EPI_ASYM_ROWSUM, EPI_ASYM_DUAL_ROWSUM)
    if return_quantized:
        q = torch.empty(lead + (K // 2,), dtype=_U8, device=dev)
        s = torch.empty(lead + (1,), dtype=_F16, device=dev)
        z = torch.empty(lead + (1,), dtype=_F16, device=dev)
        r = torch.empty(lead, dtype=_I32, device=dev) if rowsum else None
    lib = _lib.load()
    ws, ws_bytes = None, 0
    if not return_quantized or mode == EPI_ASYM_DUAL_ROWSUM:  # (that mode may also stage its accumulators)
        ws_bytes = lib.duq_quantize_linear4bit_asym_workspace_bytes(mode, M, N, K)
        if ws_bytes:
            ws = torch.empty(ws_bytes, dtype=_U8, device=dev)
    st = _launch(dev, lib.duq_quantize_linear4bit_forward_asym, mode, x.data_ptr(), w.data_ptr(), *ptrs, M, N, K,
                 y.data_ptr(), _ptr(q), _ptr(s), _ptr(z), _ptr(r), _ptr(ws), ws_bytes)
    if st:
        _lib.check(st, name)
    if not return_quantized:
        return y
    return (y, q, s, z, r) if rowsum else (y, q, s, z)


class FusedDecode:
    """One layer's side of the one-launch decode (what ``duq_quantize_linear4bit_forward`` takes for the symmetric
    modes and ``duq_quantize_linear4bit_forward_asym`` for the asymmetric and row-sum modes), checked once and kept
    as a ``duq_fused_layer`` struct for ``duq_quantize_linear4bit_forward_layer``: a decode step of a module then
    costs one ``torch.empty`` (two for the shapes of two launches: the staging buffer) and one foreign call with seven
    arguments.  The tensors are held (``tensors``) so that
    a caller can tell when the layer's buffers were replaced; a change of their contents in place needs no new
    object."""

    __slots__ = ("mode", "N", "K", "device", "index", "tensors", "w_ptr", "_fn", "_ptrs", "_structs", "_one", "_lib")

    def __init__(self, mode, w, w_scale_1, w_zeros_1=None, w_scale_2=None, w_zeros_2=None, w_rowsum_adj=None,
                 w_rowsum_adj_2=None, bias=None):
        name = "FusedDecode"
        if not isinstance(w, torch.Tensor):
            raise RuntimeError(f"{name}: w must be a tensor")
        _fast_check(name, "w", w, _U8, None)
        if w.dim() != 2:
            raise RuntimeError(f"{name}: expected w [N, K/2], got {tuple(w.shape)}")
        dev = w.device
        N, K = w.shape[0], w.shape[1] * 2
        asym = mode in (EPI_ASYM, EPI_ASYM_DUAL, EPI_ASYM_ROWSUM, EPI_ASYM_DUAL_ROWSUM)
        dual = mode in (EPI_SYM_DUAL, EPI_ASYM_DUAL, EPI_ASYM_DUAL_ROWSUM)
        if mode not in (EPI_SYM, EPI_SYM_DUAL) and not asym:
            raise RuntimeError(f"{name}: unknown mode {mode}")
        need = {"w_scale_1": True, "w_zeros_1": asym, "w_scale_2": dual, "w_zeros_2": asym and dual,
                "w_rowsum_adj": mode in (EPI_ASYM_ROWSUM, EPI_ASYM_DUAL_ROWSUM),
                "w_rowsum_adj_2": mode == EPI_ASYM_DUAL_ROWSUM, "bias": False}
        ptrs = {}
        for t, what, dt in ((w_scale_1, "w_scale_1", _F16), (w_zeros_1, "w_zeros_1", _F16), (w_scale_2, "w_scale_2", _F16),
                            (w_zeros_2, "w_zeros_2", _F16), (w_rowsum_adj, "w_rowsum_adj", _I32),
                            (w_rowsum_adj_2, "w_rowsum_adj_2", _I32), (bias, "bias", _F16)):
            if t is None:
                if need[what]:
                    raise RuntimeError(f"{name}: {what} is required for mode {mode}")
                ptrs[what] = None
                continue
            _fast_check(name, what, t, dt, dev)
            if t.numel() != N:
                _check_size0(name, t.reshape(-1), what, N)
            ptrs[what] = t.data_ptr()
        self.mode, self.N, self.K, self.device, self.index = mode, N, K, dev, dev.index
        self.tensors = (w, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2, w_rowsum_adj, w_rowsum_adj_2, bias)
        self.w_ptr = w.data_ptr()
        lib = self._lib = _lib.load()
        self._fn = lib.duq_quantize_linear4bit_forward_layer
        # one struct per quantizer setting (clip, qmax), built on first use
        self._ptrs = ptrs
        self._structs = {}
        self._one = {}

    def _layer(self, clip, qmax):
        key = (clip, qmax)
        ref = self._structs.get(key)
        if ref is None:
            p = self._ptrs
            st = _lib.FusedLayer(self.mode, float(clip), int(qmax), self.N, self.K, self.w_ptr, p["w_scale_1"], p["w_zeros_1"],
                                 p["w_scale_2"], p["w_zeros_2"], p["w_rowsum_adj"], p["w_rowsum_adj_2"], p["bias"])
            ref = self._structs[key] = (ctypes.addressof(st), st)   # (the struct is kept alive beside its address)
        return ref[0]

    # Rows up to which a module hands binary16 activations to this call.  Up to eight rows, sixteen short ones, it is one
    # launch; above, the quantizer launch and the GEMM launch of one library call: up to about 700 rows (N = K = 4096)
    # the two kernels take less time than two calls cost on the host (23 us).
    max_rows = 1024

    def _staging(self, M: int) -> int:
        """Bytes the library stages between its two launches at M rows (0: one launch); -1 when M is out of range."""
        b = self._one.get(M)
        if b is None:
            if not 0 < M <= self.max_rows:
                b = -1
            elif self.mode in (EPI_SYM, EPI_SYM_DUAL):
                b = self._lib.duq_quantize_linear4bit_workspace_bytes(M, self.N, self.K)
            else:
                b = self._lib.duq_quantize_linear4bit_asym_workspace_bytes(self.mode, M, self.N, self.K)
            self._one[M] = b
        return b

    def admits(self, M: int) -> bool:
        """True when M rows of this layer run through one library call from binary16 rows."""
        return self._staging(M) >= 0

    def one_launch(self, M: int) -> bool:
        """True when M rows run as ONE launch with nothing staged."""
        return self._staging(M) == 0

    def run(self, x: torch.Tensor, M: int, clip: float = 1.0, qmax: int = 6, checked: bool = False) -> torch.Tensor:
        """x: contiguous binary16 [..., K] on the layer's device, 16-byte aligned, M = its rows with admits(M);
        clip / qmax: the symmetric quantizer's settings (unused by the asymmetric modes).  ``checked``: the caller
        has verified dtype and contiguity already.  Returns binary16 [..., N]."""
        idx = self.index
        shape = x.shape
        if x.get_device() != idx or shape[-1] != self.K or not (checked or (x.dtype is _F16 and x.is_contiguous())):
            raise RuntimeError(f"FusedDecode: expected a contiguous float16 tensor [..., {self.K}] on {self.device}, got "
                               f"{x.dtype} {tuple(x.shape)} on {x.device}")
        nbytes = self._one.get(M)
        if nbytes is None:
            nbytes = self._staging(M)
        if nbytes < 0:
            raise RuntimeError(f"FusedDecode: {M} rows (at most {self.max_rows})")
        y = x.new_empty((*shape[:-1], self.N))
        ref = self._structs.get((clip, qmax))
        layer = ref[0] if ref is not None else self._layer(clip, qmax)
        if nbytes:
            ws = torch.empty(nbytes, dtype=_U8, device=self.device)
            ws_ptr = ws.data_ptr()
        else:
            ws_ptr = None
        if idx == _current_device():
            st = self._fn(layer, x.data_ptr(), M, y.data_ptr(), ws_ptr, nbytes, _raw_stream(idx))
        else:
            with torch.cuda.device(idx):
                st = self._fn(layer, x.data_ptr(), M, y.data_ptr(), ws_ptr, nbytes, _raw_stream(idx))
        if st:
            _lib.check(st, "quantize_linear4bit_forward")
        return y


# ---- asymmetric path with exact zero-point correction (row sums); not in the reference ----

_I32 = torch.int32


def quantize_rows_asym_shifted(x: torch.Tensor):
    """AsymQuantizer with signed-shifted storage: the codes of ``quantize_rows_asym`` minus 8
    (signed nibbles), zero points minus 8, and the per-row sums of the shifted codes.
    Returns (q uint8 [..., K/2], scale [..., 1], zeros [..., 1], rowsum int32 [...])."""
    if not isinstance(x, torch.Tensor):
        raise RuntimeError("quantize_rows_asym_shifted: argument #0 is not a tensor")
    _fast_check("quantize_rows_asym_shifted", "x", x, _F16, None)
    shape = x.shape
    cols = shape[-1]
    rows = x.numel() // cols if cols else 0
    lead = shape[:-1]
    dev = x.device
    q = torch.empty(lead + (cols // 2,), dtype=_U8, device=dev)
    s = torch.empty(lead + (1,), dtype=_F16, device=dev)
    z = torch.empty(lead + (1,), dtype=_F16, device=dev)
    r = torch.empty(lead, dtype=_I32, device=dev)
    st = _launch(dev, _lib.load().duq_quantize_rows_asym_shifted, x.data_ptr(), rows, cols, q.data_ptr(), s.data_ptr(),
                 z.data_ptr(), r.data_ptr())
    if st:
        _lib.check(st, "quantize_rows_asym_shifted")
    return q, s, z, r


def _rowsum_args(name, M, N, dev, scale_x, zeros_x, rowsum_x, w_scale, w_zeros, w_rowsum_adj, bias):
    for t, what, dt, n in ((scale_x, "scale_x", _F16, M), (zeros_x, "zeros_x", _F16, M), (rowsum_x, "rowsum_x", _I32, M),
                           (w_scale, "w_scale", _F16, N), (w_zeros, "w_zeros", _F16, N),
                           (w_rowsum_adj, "w_rowsum_adj", _I32, N)):
        if not isinstance(t, torch.Tensor):
            raise RuntimeError(f"{name}: {what} must be a tensor")
        _fast_check(name, what, t, dt, dev)
        if t.numel() != n:
            _check_size0(name, t.reshape(-1), what, n)
    pb = None
    if bias is not None:
        _fast_check(name, "bias", bias, _F16, dev)
        if bias.numel() != N:
            _check_size0(name, bias.reshape(-1), "bias", N)
        pb = bias.data_ptr()
    return pb


def linear4bit_forward_rowsum(xq, scale_x, zeros_x, rowsum_x, w, w_scale, w_zeros, w_rowsum_adj, bias=None):
    """GEMM + exact asymmetric dequant (+ bias) in one launch on signed-shifted operands:
    y = s_x*s_w * (acc - z_x*w_rowsum_adj - z_w*rowsum_x), w_rowsum_adj = sum_k c_w - K*z_w.
    ``xq`` uint8 [..., K/2]; returns fp16 [..., N]."""
    name = "linear4bit_forward_rowsum"
    if not isinstance(xq, torch.Tensor) or not isinstance(w, torch.Tensor):
        raise RuntimeError(f"{name}: xq and w must be tensors")
    dev = xq.device
    _fast_check(name, "xq", xq, _U8, None)
    _fast_check(name, "w", w, _U8, dev)
    kb = xq.shape[-1]
    if w.dim() != 2 or w.shape[1] != kb:
        raise RuntimeError(f"{name}: packed K differs: x {tuple(xq.shape)} vs w {tuple(w.shape)}")
    M = xq.numel() // kb if kb else 0
    N = w.shape[0]
    pb = _rowsum_args(name, M, N, dev, scale_x, zeros_x, rowsum_x, w_scale, w_zeros, w_rowsum_adj, bias)
    y = torch.empty(xq.shape[:-1] + (N,), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_linear4bit_forward_rowsum, xq.data_ptr(), scale_x.data_ptr(), zeros_x.data_ptr(),
                 rowsum_x.data_ptr(), w.data_ptr(), w_scale.data_ptr(), w_zeros.data_ptr(), w_rowsum_adj.data_ptr(), pb,
                 M, N, kb * 2, y.data_ptr())
    if st:
        _lib.check(st, name)
    return y


def asym_rowsum_dequant(q, scale_row, zeros_row, rowsum_row, scale_col, zeros_col, rowsum_adj_col, bias=None):
    """The row-sum epilogue on int32 accumulators [rows, cols] already in memory."""
    name = "asym_rowsum_dequant"
    _check(name, q)
    _check_dtype(name, q, "q", _I32)
    rows, cols = q.size(0), q.size(1)
    pb = _rowsum_args(name, rows, cols, q.device, scale_row, zeros_row, rowsum_row, scale_col, zeros_col,
                      rowsum_adj_col, bias)
    x = torch.empty((rows, cols), dtype=_F16, device=q.device)
    st = _launch(q.device, _lib.load().duq_asym_rowsum_dequant_host, q.data_ptr(), scale_row.data_ptr(),
                 zeros_row.data_ptr(), rowsum_row.data_ptr(), scale_col.data_ptr(), zeros_col.data_ptr(),
                 rowsum_adj_col.data_ptr(), pb, rows, cols, x.data_ptr())
    if st:
        _lib.check(st, name)
    return x


def asym_dual_rowsum_dequant(q, xq, scale_row, zeros_row, rowsum_row, w, scale_col_1, zeros_col_1, scale_col_2,
                             zeros_col_2, adj_col_1, adj_col_2, bias=None):
    """Row-sum epilogue of the dual-uniform layer on int32 accumulators ``q`` [rows, cols] = matmul(xq, w): input
    columns 0..9 dequantized with (scale_col_1, zeros_col_1), the others with (scale_col_2, zeros_col_2); the
    codes of columns 0..9 are read from the packed operands ``xq`` [rows, K/2] and ``w`` [cols, K/2]."""
    name = "asym_dual_rowsum_dequant"
    _check(name, q, xq, w)
    _check_dtype(name, q, "q", _I32)
    _check_dtype(name, xq, "xq", _U8)
    _check_dtype(name, w, "w", _U8)
    if q.dim() != 2 or xq.dim() != 2 or w.dim() != 2:
        raise RuntimeError(f"{name}: expected 2-D q, xq and w")
    rows, cols = q.shape
    kb = xq.shape[1]
    if xq.shape[0] != rows or w.shape[0] != cols or w.shape[1] != kb:
        raise RuntimeError(f"{name}: q {tuple(q.shape)} does not match xq {tuple(xq.shape)} and w {tuple(w.shape)}")
    dev = q.device
    for t, what, dt, cnt in ((scale_row, "scale_row", _F16, rows), (zeros_row, "zeros_row", _F16, rows),
                             (rowsum_row, "rowsum_row", _I32, rows), (scale_col_1, "scale_col_1", _F16, cols),
                             (zeros_col_1, "zeros_col_1", _F16, cols), (scale_col_2, "scale_col_2", _F16, cols),
                             (zeros_col_2, "zeros_col_2", _F16, cols), (adj_col_1, "adj_col_1", _I32, cols),
                             (adj_col_2, "adj_col_2", _I32, cols)) + (((bias, "bias", _F16, cols),) if bias is not None else ()):
        _fast_check(name, what, t, dt, dev)
        if t.numel() != cnt:
            _check_size0(name, t.reshape(-1), what, cnt)
    x = torch.empty((rows, cols), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_asym_dual_rowsum_dequant_host, q.data_ptr(), xq.data_ptr(), scale_row.data_ptr(),
                 zeros_row.data_ptr(), rowsum_row.data_ptr(), w.data_ptr(), scale_col_1.data_ptr(), zeros_col_1.data_ptr(),
                 scale_col_2.data_ptr(), zeros_col_2.data_ptr(), adj_col_1.data_ptr(), adj_col_2.data_ptr(), _ptr(bias),
                 rows, cols, kb * 2, x.data_ptr())
    if st:
        _lib.check(st, name)
    return x


def linear4bit_forward_dual_rowsum(xq, scale_x, zeros_x, rowsum_x, w, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2,
                                   w_adj_1, w_adj_2, bias=None):
    """``asym_dual_rowsum_dequant(matmul(xq, w), ...)`` as the library runs it best: one launch where the GEMM
    kernel of the shape applies the epilogue itself, else the GEMM into a scratch int32 tensor and the stand-alone
    epilogue.  Same bits either way.  ``xq`` uint8 [M, K/2], ``w`` uint8 [N, K/2]; returns fp16 [M, N]."""
    name = "linear4bit_forward_dual_rowsum"
    _check(name, xq, w)
    _check_dtype(name, xq, "xq", _U8)
    _check_dtype(name, w, "w", _U8)
    if xq.dim() != 2 or w.dim() != 2 or xq.shape[1] != w.shape[1]:
        raise RuntimeError(f"{name}: expected xq [M, K/2] and w [N, K/2], got {tuple(xq.shape)} and {tuple(w.shape)}")
    M, kb = xq.shape
    N = w.shape[0]
    dev = xq.device
    for t, what, dt, cnt in ((scale_x, "scale_x", _F16, M), (zeros_x, "zeros_x", _F16, M), (rowsum_x, "rowsum_x", _I32, M),
                             (w_scale_1, "w_scale_1", _F16, N), (w_zeros_1, "w_zeros_1", _F16, N),
                             (w_scale_2, "w_scale_2", _F16, N), (w_zeros_2, "w_zeros_2", _F16, N),
                             (w_adj_1, "w_adj_1", _I32, N), (w_adj_2, "w_adj_2", _I32, N)) + \
            (((bias, "bias", _F16, N),) if bias is not None else ()):
        _fast_check(name, what, t, dt, dev)
        if t.numel() != cnt:
            _check_size0(name, t.reshape(-1), what, cnt)
    lib = _lib.load()
    y = torch.empty((M, N), dtype=_F16, device=dev)
    need = int(lib.duq_linear4bit_dual_rowsum_workspace_bytes(M, N, kb * 2))
    ws = torch.empty(need // 4, dtype=_I32, device=dev) if need else None
    st = _launch(dev, lib.duq_linear4bit_forward_dual_rowsum, xq.data_ptr(), scale_x.data_ptr(), zeros_x.data_ptr(),
                 rowsum_x.data_ptr(), w.data_ptr(), w_scale_1.data_ptr(), w_zeros_1.data_ptr(), w_scale_2.data_ptr(),
                 w_zeros_2.data_ptr(), w_adj_1.data_ptr(), w_adj_2.data_ptr(), _ptr(bias), M, N, kb * 2, y.data_ptr(),
                 ws.data_ptr() if ws is not None else None, need)
    if st:
        _lib.check(st, name)
    return y


# ---- the forward on the 6-bit float matrix path (exact; not in the reference) --------------


def weight_shadow_bf6(w: torch.Tensor) -> torch.Tensor:
    """E3M2 shadow of packed-int4 weights ``w`` uint8 [N, K/2]: uint8 [ceil(N/32)*32, 3K/4] in the
    library's tile order.  Made once per weight tensor.  N % 16 == 0, K % 128 == 0."""
    name = "weight_shadow_bf6"
    if not isinstance(w, torch.Tensor):
        raise RuntimeError(f"{name}: argument #0 is not a tensor")
    _fast_check(name, "w", w, _U8, None)
    if w.dim() != 2:
        raise RuntimeError(f"{name}: expected a 2-D tensor, got {tuple(w.shape)}")
    N, kb = w.shape
    out = torch.empty(((N + 31) // 32 * 32, kb * 3 // 2), dtype=_U8, device=w.device)
    st = _launch(w.device, _lib.load().duq_weight_shadow_bf6, w.data_ptr(), N, kb * 2, out.data_ptr())
    if st:
        _lib.check(st, name)
    return out


def activation_shadow_bf6(xq: torch.Tensor) -> torch.Tensor:
    """E3M2 shadow of packed-int4 activations uint8 [..., K/2]: uint8 [..., 3K/4] (per row:
    the 16-byte parts of its K/32 blocks, then the 8-byte parts).  K % 128 == 0."""
    name = "activation_shadow_bf6"
    if not isinstance(xq, torch.Tensor):
        raise RuntimeError(f"{name}: argument #0 is not a tensor")
    _fast_check(name, "xq", xq, _U8, None)
    kb = xq.shape[-1]
    M = xq.numel() // kb if kb else 0
    out = torch.empty(xq.shape[:-1] + (kb * 3 // 2,), dtype=_U8, device=xq.device)
    st = _launch(xq.device, _lib.load().duq_activation_shadow_bf6, xq.data_ptr(), M, kb * 2, out.data_ptr())
    if st:
        _lib.check(st, name)
    return out


def linear4bit_forward_bf6(mode, x_bf6, scale_x, zeros_x, w_bf6, w_scale_1, w_zeros_1=None, w_scale_2=None,
                           w_zeros_2=None, bias=None, rowsum_x=None, w_rowsum_adj=None):
    """``linear4bit_forward`` (modes 0-3) or ``linear4bit_forward_rowsum`` (mode 4) on E3M2
    shadows: ``x_bf6`` uint8 [..., 3K/4], ``w_bf6`` uint8 [ceil(N/32)*32, 3K/4] from weight_shadow_bf6, N taken
    from ``w_scale_1``.  Bit-identical results."""
    name = "linear4bit_forward_bf6"
    if not isinstance(x_bf6, torch.Tensor) or not isinstance(w_bf6, torch.Tensor):
        raise RuntimeError(f"{name}: x_bf6 and w_bf6 must be tensors")
    dev = x_bf6.device
    _fast_check(name, "x_bf6", x_bf6, _U8, None)
    _fast_check(name, "w_bf6", w_bf6, _U8, dev)
    kb = x_bf6.shape[-1]
    if w_bf6.dim() != 2 or w_bf6.shape[1] != kb:
        raise RuntimeError(f"{name}: shadow row length differs: x {tuple(x_bf6.shape)} vs w {tuple(w_bf6.shape)}")
    if kb % 96:
        raise RuntimeError(f"{name}: shadow rows must hold a multiple of 128 elements (96 bytes), got {kb} bytes")
    M = x_bf6.numel() // kb if kb else 0
    if not isinstance(w_scale_1, torch.Tensor):
        raise RuntimeError(f"{name}: w_scale_1 is not a tensor")
    N = w_scale_1.numel()
    if w_bf6.shape[0] != (N + 31) // 32 * 32:
        raise RuntimeError(f"{name}: the weight shadow has {w_bf6.shape[0]} rows, expected {(N + 31) // 32 * 32} for "
                           f"{N} output channels")
    ptrs = []
    for t, what, dt, n in ((scale_x, "scale_x", _F16, M), (zeros_x, "zeros_x", _F16, M), (rowsum_x, "rowsum_x", _I32, M),
                           (w_scale_1, "w_scale_1", _F16, N), (w_zeros_1, "w_zeros_1", _F16, N),
                           (w_scale_2, "w_scale_2", _F16, N), (w_zeros_2, "w_zeros_2", _F16, N),
                           (w_rowsum_adj, "w_rowsum_adj", _I32, N), (bias, "bias", _F16, N)):
        if t is None:
            ptrs.append(None)
            continue
        _fast_check(name, what, t, dt, dev)
        if t.numel() != n:
            _check_size0(name, t.reshape(-1), what, n)
        ptrs.append(t.data_ptr())
    y = torch.empty(x_bf6.shape[:-1] + (N,), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_linear4bit_forward_bf6, mode, x_bf6.data_ptr(), ptrs[0], ptrs[1], ptrs[2],
                 w_bf6.data_ptr(), ptrs[3], ptrs[4], ptrs[5], ptrs[6], ptrs[7], ptrs[8], M, N, kb * 4 // 3, y.data_ptr())
    if st:
        _lib.check(st, name)
    return y


def linear4bit_forward_dual_rowsum_bf6(x_bf6, xq, scale_x, zeros_x, rowsum_x, w_bf6, w, w_scale_1, w_zeros_1, w_scale_2, w_zeros_2,
                                       w_adj_1, w_adj_2, bias=None):
    """``linear4bit_forward_dual_rowsum`` on the 6-bit float matrix path: the GEMM on the shadows ``x_bf6``
    [M, 3K/4] and ``w_bf6``, the epilogue (same launch) with the first ten codes of every row of the packed
    operands ``xq`` [M, K/2] and ``w`` [N, K/2].  Bit-identical results."""
    name = "linear4bit_forward_dual_rowsum_bf6"
    _check(name, x_bf6, xq, w_bf6, w)
    for t, what in ((x_bf6, "x_bf6"), (xq, "xq"), (w_bf6, "w_bf6"), (w, "w")):
        _check_dtype(name, t, what, _U8)
    if xq.dim() != 2 or w.dim() != 2 or x_bf6.dim() != 2 or w_bf6.dim() != 2 or xq.shape[1] != w.shape[1] or \
            x_bf6.shape != (xq.shape[0], xq.shape[1] * 3 // 2) or \
            w_bf6.shape != ((w.shape[0] + 31) // 32 * 32, w.shape[1] * 3 // 2):
        raise RuntimeError(f"{name}: operands and shadows do not match: xq {tuple(xq.shape)}, x_bf6 {tuple(x_bf6.shape)}, "
                           f"w {tuple(w.shape)}, w_bf6 {tuple(w_bf6.shape)}")
    M, kb = xq.shape
    N = w.shape[0]
    dev = xq.device
    for t, what, dt, cnt in ((scale_x, "scale_x", _F16, M), (zeros_x, "zeros_x", _F16, M), (rowsum_x, "rowsum_x", _I32, M),
                             (w_scale_1, "w_scale_1", _F16, N), (w_zeros_1, "w_zeros_1", _F16, N),
                             (w_scale_2, "w_scale_2", _F16, N), (w_zeros_2, "w_zeros_2", _F16, N),
                             (w_adj_1, "w_adj_1", _I32, N), (w_adj_2, "w_adj_2", _I32, N)) + \
            (((bias, "bias", _F16, N),) if bias is not None else ()):
        _fast_check(name, what, t, dt, dev)
        if t.numel() != cnt:
            _check_size0(name, t.reshape(-1), what, cnt)
    y = torch.empty((M, N), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_linear4bit_forward_dual_rowsum_bf6, x_bf6.data_ptr(), xq.data_ptr(), scale_x.data_ptr(),
                 zeros_x.data_ptr(), rowsum_x.data_ptr(), w_bf6.data_ptr(), w.data_ptr(), w_scale_1.data_ptr(),
                 w_zeros_1.data_ptr(), w_scale_2.data_ptr(), w_zeros_2.data_ptr(), w_adj_1.data_ptr(), w_adj_2.data_ptr(),
                 _ptr(bias), M, N, kb * 2, y.data_ptr())
    if st:
        _lib.check(st, name)
    return y


def quantize_rows_sym_bf6(x: torch.Tensor, clip: float = 1.0, qmax: int = 6, with_q: bool = True):
    """``quantize_rows_sym`` that also writes the E3M2 shadow of the codes: returns
    (q or None, x_bf6 uint8 [..., 3K/4], scales).  K % 128 == 0."""
    name = "quantize_rows_sym_bf6"
    if not isinstance(x, torch.Tensor):
        raise RuntimeError(f"{name}: argument #0 is not a tensor")
    _fast_check(name, "x", x, _F16, None)
    shape = x.shape
    cols = shape[-1]
    rows = x.numel() // cols if cols else 0
    lead = shape[:-1]
    dev = x.device
    q = torch.empty(lead + (cols // 2,), dtype=_U8, device=dev) if with_q else None
    b = torch.empty(lead + (cols * 3 // 4,), dtype=_U8, device=dev)
    s = torch.empty(lead + (1,), dtype=_F16, device=dev)
    st = _launch(dev, _lib.load().duq_quantize_rows_sym_bf6, x.data_ptr(), rows, cols, float(clip), qmax,
                 q.data_ptr() if with_q else None, b.data_ptr(), s.data_ptr())
    if st:
        _lib.check(st, name)
    return q, b, s


def quantize_rows_asym_bf6(x: torch.Tensor, shifted: bool = False, with_q: bool = True):
    """``quantize_rows_asym`` (or ``quantize_rows_asym_shifted``) that also writes the E3M2
    shadow: returns (q or None, x_bf6, scale, zeros[, rowsum])."""
    name = "quantize_rows_asym_bf6"
    if not isinstance(x, torch.Tensor):
        raise RuntimeError(f"{name}: argument #0 is not a tensor")
    _fast_check(name, "x", x, _F16, None)
    shape = x.shape
    cols = shape[-1]
    rows = x.numel() // cols if cols else 0
    lead = shape[:-1]
    dev = x.device
    q = torch.empty(lead + (cols // 2,), dtype=_U8, device=dev) if with_q else None
    b = torch.empty(lead + (cols * 3 // 4,), dtype=_U8, device=dev)
    s = torch.empty(lead + (1,), dtype=_F16, device=dev)
    z = torch.empty(lead + (1,), dtype=_F16, device=dev)
    r = torch.empty(lead, dtype=_I32, device=dev) if shifted else None
    st = _launch(dev, _lib.load().duq_quantize_rows_asym_bf6, x.data_ptr(), rows, cols,
                 q.data_ptr() if with_q else None, b.data_ptr(), s.data_ptr(), z.data_ptr(),
                 r.data_ptr() if shifted else None)
    if st:
        _lib.check(st, name)
    return (q, b, s, z, r) if shifted else (q, b, s, z)


# ---- 8-bit asymmetric layer (LinearQuant8bitASQ) --------------------------------------------

_F32, _I8 = torch.float32, torch.int8


def matmul_8bit(A: torch.Tensor, B: torch.Tensor) -> torch.Tensor:
    """A [M, K] int8 @ B [N, K]^T int8 -> int32 [M, N] (bindings.cpp:28-45)."""
    _check("matmul_8bit", A, B)
    _check_dtype("matmul_8bit", A, "A", _I8)
    _check_dtype("matmul_8bit", B, "B", _I8)
    M, N, K = A.size(0), B.size(0), A.size(1)
    if B.size(1) != K:
        raise RuntimeError(f"matmul_8bit: K differs: A {tuple(A.shape)} vs B {tuple(B.shape)}")
    C = torch.empty((M, N), dtype=torch.int32, device=A.device)
    st = _launch(A.device, _lib.load().duq_matmul_host_8bit, _ptr(A), _ptr(B), M, N, K, _ptr(C))
    _lib.check(st, "matmul_8bit")
    return C


def asym_quant_8bit(x, scale, zeros):
    """float32 x [rows, cols], per-row float32 scale / zero -> int8 codes 0..126 (bindings.cpp:245-266)."""
    _check("asym_quant_8bit", x, scale, zeros)
    for t, n in ((x, "x"), (scale, "scale"), (zeros, "zeros")):
        _check_dtype("asym_quant_8bit", t, n, _F32)
    _check_size0("asym_quant_8bit", scale, "scale", x.size(0))
    _check_size0("asym_quant_8bit", zeros, "zeros", x.size(0))
    rows, cols = x.size(0), x.size(1)
    q = torch.empty((rows, cols), dtype=_I8, device=x.device)
    st = _launch(x.device, _lib.load().duq_asym_quant_host_8bit, _ptr(x), _ptr(scale), _ptr(zeros), rows, cols, _ptr(q))
    _lib.check(st, "asym_quant_8bit")
    return q


def asym_dequant_hprec(q, scale_row, zeros_row, scale_col, zeros_col, bits: int = 32):
    """(s_r * s_c) * (float(q) - (z_r + z_c)) in float32 (bindings.cpp:309-350)."""
    _check("asym_dequant_hprec", q, scale_row, zeros_row, scale_col, zeros_col)
    _check_bits("asym_dequant_hprec", bits)
    _check_dtype("asym_dequant_hprec", q, "q", torch.int32)
    for t, n in ((scale_row, "scale_row"), (zeros_row, "zeros_row"), (scale_col, "scale_col"), (zeros_col, "zeros_col")):
        _check_dtype("asym_dequant_hprec", t, n, _F32)
    rows, cols = q.size(0), q.size(1)
    _check_size0("asym_dequant_hprec", scale_row, "scale_row", rows)
    _check_size0("asym_dequant_hprec", zeros_row, "zeros_row", rows)
    _check_size0("asym_dequant_hprec", scale_col, "scale_col", cols)
    _check_size0("asym_dequant_hprec", zeros_col, "zeros_col", cols)
    x = torch.empty((rows, cols), dtype=_F32, device=q.device)
    st = _launch(q.device, _lib.load().duq_asym_dequant_host_hprec, _ptr(q), _ptr(scale_row), _ptr(zeros_row),
                 _ptr(scale_col), _ptr(zeros_col), rows, cols, _ptr(x))
    _lib.check(st, "asym_dequant_hprec")
    return x


def quantize_rows_asym_8bit(x: torch.Tensor):
    """One-pass AsymQuantizer8bit (qlinear4bit/nn/quantizer.py:38-55) over the last dimension:
    (q int8 [..., K], scale [..., 1], zeros [..., 1]) float32.  Requires K % 4 == 0."""
    if not isinstance(x, torch.Tensor):
        raise RuntimeError("quantize_rows_asym_8bit: argument #0 is not a tensor")
    _fast_check("quantize_rows_asym_8bit", "x", x, _F32, None)
    shape = x.shape
    cols = shape[-1]
    rows = x.numel() // cols if cols else 0
    lead = shape[:-1]
    dev = x.device
    q = torch.empty(shape, dtype=_I8, device=dev)
    s = torch.empty(lead + (1,), dtype=_F32, device=dev)
    z = torch.empty(lead + (1,), dtype=_F32, device=dev)
    st = _launch(dev, _lib.load().duq_quantize_rows_asym_8bit, x.data_ptr(), rows, cols, q.data_ptr(), s.data_ptr(),
                 z.data_ptr())
    if st:
        _lib.check(st, "quantize_rows_asym_8bit")
    return q, s, z


def weight_tile_8bit(w: torch.Tensor) -> torch.Tensor:
    """int8 weight [N, K] -> the tiled copy [ceil(N/32)*32*K] that linear8bit_forward(..., tiled_rows=N) takes."""
    _check("weight_tile_8bit", w)
    _check_dtype("weight_tile_8bit", w, "w", _I8)
    N, K = w.size(0), w.size(1)
    out = torch.empty(((N + 31) // 32 * 32 * K,), dtype=_I8, device=w.device)
    st = _launch(w.device, _lib.load().duq_weight_tile_8bit, _ptr(w), N, K, _ptr(out))
    _lib.check(st, "weight_tile_8bit")
    return out


def linear8bit_forward(xq, scale_x, zeros_x, w, w_scale, w_zeros, bias=None, tiled_rows=None):
    """matmul_8bit + asym_dequant_hprec (+ bias) in one launch; xq [..., K] int8 -> float32 [..., N].
    ``w`` is the weight [N, K], or with ``tiled_rows=N`` its tiled copy from weight_tile_8bit (same bits)."""
    name = "linear8bit_forward"
    if not isinstance(xq, torch.Tensor):
        raise RuntimeError(f"{name}: argument #0 is not a tensor")
    dev = xq.device
    _fast_check(name, "xq", xq, _I8, None)
    _fast_check(name, "w", w, _I8, dev)
    K = xq.shape[-1]
    M = xq.numel() // K if K else 0
    if tiled_rows is not None:
        N = int(tiled_rows)
        if w.numel() != (N + 31) // 32 * 32 * K:
            raise RuntimeError(f"{name}: the tiled weight has {w.numel()} bytes, expected {(N + 31) // 32 * 32 * K}")
        entry = _lib.load().duq_linear8bit_forward_tiled
    else:
        N = w.size(0)
        if w.dim() != 2 or w.size(1) != K:
            raise RuntimeError(f"{name}: K differs: xq {tuple(xq.shape)} vs w {tuple(w.shape)}")
        entry = _lib.load().duq_linear8bit_forward
    for t, what, n in ((scale_x, "scale_x", M), (zeros_x, "zeros_x", M), (w_scale, "w_scale", N),
                       (w_zeros, "w_zeros", N), (bias, "bias", N)):
        if t is None and what == "bias":
            continue
        if not isinstance(t, torch.Tensor):
            raise RuntimeError(f"{name}: {what} is not a tensor")
        _fast_check(name, what, t, _F32, dev)
        if t.numel() != n:
            raise RuntimeError(f"{name}: expected {what} to have {n} elements, got {tuple(t.shape)}")
    y = torch.empty(xq.shape[:-1] + (N,), dtype=_F32, device=dev)
    st = _launch(dev, entry, xq.data_ptr(), scale_x.data_ptr(), zeros_x.data_ptr(),
                 w.data_ptr(), w_scale.data_ptr(), w_zeros.data_ptr(), _ptr(bias), M, N, K, y.data_ptr())
    if st:
        _lib.check(st, name)
    return y


def quantize_linear8bit_forward(x, w, w_tiled, w_scale, w_zeros, bias=None):
    """AsymQuantizer8bit + linear8bit_forward in one library call (two launches, the codes staged in a workspace
    allocated here): x float32 [..., K] -> float32 [..., N], the bits of the two calls.  ``w`` the weight [N, K]
    int8, ``w_tiled`` its tiled copy from weight_tile_8bit or None."""
    name = "quantize_linear8bit_forward"
    if not isinstance(x, torch.Tensor) or not isinstance(w, torch.Tensor):
        raise RuntimeError(f"{name}: x and w must be tensors")
    dev = x.device
    _fast_check(name, "x", x, _F32, None)
    _fast_check(name, "w", w, _I8, dev)
    K = x.shape[-1]
    M = x.numel() // K if K else 0
    if w.dim() != 2 or w.size(1) != K:
        raise RuntimeError(f"{name}: K differs: x {tuple(x.shape)} vs w {tuple(w.shape)}")
    N = w.size(0)
    if w_tiled is not None:
        _fast_check(name, "w_tiled", w_tiled, _I8, dev)
        if w_tiled.numel() != (N + 31) // 32 * 32 * K:
            raise RuntimeError(f"{name}: the tiled weight has {w_tiled.numel()} bytes, expected {(N + 31) // 32 * 32 * K}")
    for t, what in ((w_scale, "w_scale"), (w_zeros, "w_zeros"), (bias, "bias")):
        if t is None and what == "bias":
            continue
        if not isinstance(t, torch.Tensor):
            raise RuntimeError(f"{name}: {what} is not a tensor")
        _fast_check(name, what, t, _F32, dev)
        if t.numel() != N:
            raise RuntimeError(f"{name}: expected {what} to have {N} elements, got {tuple(t.shape)}")
    lib = _lib.load()
    y = x.new_empty((*x.shape[:-1], N))
    if M == 0 or N == 0:
        return y
    nbytes = lib.duq_quantize_linear8bit_workspace_bytes(M, K)
    ws = torch.empty(nbytes, dtype=_U8, device=dev)
    st = _launch(dev, lib.duq_quantize_linear8bit_forward, x.data_ptr(), w.data_ptr(), _ptr(w_tiled), w_scale.data_ptr(),
                 w_zeros.data_ptr(), _ptr(bias), M, N, K, y.data_ptr(), ws.data_ptr(), nbytes)
    if st:
        _lib.check(st, name)
    return y
