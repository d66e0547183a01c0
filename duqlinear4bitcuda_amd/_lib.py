"""ctypes binding of libduq_hip.so (the C ABI declared in include/duq_hip.h).

The shared library is built in-tree by ``duqlinear4bitcuda_amd/csrc/Makefile`` (see
``duqlinear4bitcuda_amd.build``).  There is no fallback: if the library is missing,
loading raises and every op of this package fails.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libduq_hip.so")

_c_u32 = ctypes.c_uint32
_c_i32 = ctypes.c_int32
_c_p = ctypes.c_void_p

# name -> argtypes; every function returns int status except where noted
PROTOTYPES = {
    "duq_abi_version": [],
    "duq_get_dual_quant_col_k": [],
    "duq_sym_quant_host": [_c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_sym_quant_host_qmax": [_c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_i32, _c_p, _c_p],
    "duq_sym_dual_quant_host": [_c_p, _c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_asym_quant_host": [_c_p, _c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_asym_dual_quant_host": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_quantize_rows_sym": [_c_p, _c_u32, _c_u32, ctypes.c_float, _c_i32, _c_p, _c_p, _c_p],
    "duq_quantize_rows_asym": [_c_p, _c_u32, _c_u32, _c_p, _c_p, _c_p, _c_p],
    "duq_matmul_host_4bit": [_c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_batch_matmul_host_4bit": [_c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_u32, _c_p],
    "duq_asym_batch_dequant_host": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_batch_linear4bit_forward": [_c_i32, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32,
                                     _c_u32, _c_u32, _c_p, _c_p],
    "duq_sym_dequant_host": [_c_p, _c_p, _c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_sym_dual_dequant_host": [_c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_asym_dequant_host": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_asym_dual_dequant_host": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_linear4bit_forward": [_c_i32, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32,
                               _c_u32, _c_p, _c_p],
    "duq_gemm_kernel_for": [_c_u32, _c_u32, _c_u32],
    "duq_gemm_stream_tile_for": [_c_u32, _c_u32, _c_u32],
    "duq_probe_read": [_c_p, ctypes.c_uint64, _c_p, _c_p],
    "duq_quantize_linear4bit_workspace_bytes": [_c_u32, _c_u32, _c_u32],  # returns uint64_t (restype set in load())
    "duq_quantize_linear4bit_forward": [_c_i32, _c_p, ctypes.c_float, _c_i32, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32,
                                        _c_u32, _c_p, _c_p, _c_p, _c_p, ctypes.c_uint64, _c_p],
    "duq_quantize_linear4bit_forward_static": [_c_i32, _c_p, ctypes.c_float, _c_i32, _c_p, _c_p, _c_p, _c_p, _c_u32,
                                               _c_u32, _c_u32, _c_p, _c_p, _c_p, _c_u32, _c_p],
    "duq_static_scratch_init": [],
    "duq_quantize_linear8bit_workspace_bytes": [_c_u32, _c_u32],  # returns uint64_t
    "duq_quantize_linear8bit_forward": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p,
                                        ctypes.c_uint64, _c_p],
    "duq_quantize_linear4bit_forward_layer": [_c_p, _c_p, _c_u32, _c_p, _c_p, ctypes.c_uint64, _c_p],
    "duq_quantize_linear4bit_asym_workspace_bytes": [_c_i32, _c_u32, _c_u32, _c_u32],  # returns uint64_t
    "duq_quantize_linear4bit_forward_asym": [_c_i32, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32,
                                             _c_u32, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, ctypes.c_uint64, _c_p],
    "duq_quantize_rows_asym_shifted": [_c_p, _c_u32, _c_u32, _c_p, _c_p, _c_p, _c_p, _c_p],
    "duq_linear4bit_forward_rowsum": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_u32,
                                      _c_p, _c_p],
    "duq_asym_rowsum_dequant_host": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_asym_dual_rowsum_dequant_host": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
                                          _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_linear4bit_dual_rowsum_workspace_bytes": [_c_u32, _c_u32, _c_u32],  # returns uint64_t (restype set in load())
    "duq_linear4bit_forward_dual_rowsum": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
                                           _c_u32, _c_u32, _c_u32, _c_p, _c_p, ctypes.c_uint64, _c_p],
    "duq_weight_shadow_bf6": [_c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_quantize_rows_sym_bf6": [_c_p, _c_u32, _c_u32, ctypes.c_float, _c_i32, _c_p, _c_p, _c_p, _c_p],
    "duq_quantize_rows_asym_bf6": [_c_p, _c_u32, _c_u32, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p],
    "duq_activation_shadow_bf6": [_c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_linear4bit_forward_bf6": [_c_i32, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32,
                                   _c_u32, _c_u32, _c_p, _c_p],
    "duq_linear4bit_forward_dual_rowsum_bf6": [_c_p] * 14 + [_c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_asym_quant_host_8bit": [_c_p, _c_p, _c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_matmul_host_8bit": [_c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_asym_dequant_host_hprec": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_quantize_rows_asym_8bit": [_c_p, _c_u32, _c_u32, _c_p, _c_p, _c_p, _c_p],
    "duq_weight_tile_8bit": [_c_p, _c_u32, _c_u32, _c_p, _c_p],
    "duq_linear8bit_forward_tiled": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
    "duq_linear8bit_forward": [_c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_u32, _c_u32, _c_u32, _c_p, _c_p],
}



class FusedLayer(ctypes.Structure):
    """``duq_fused_layer`` of include/duq_hip.h."""
    _fields_ = [("mode", _c_i32), ("clip", ctypes.c_float), ("qmax", _c_i32), ("N", _c_u32), ("K", _c_u32),
                ("w", _c_p), ("w_scale_1", _c_p), ("w_zeros_1", _c_p), ("w_scale_2", _c_p), ("w_zeros_2", _c_p),
                ("w_rowsum_adj", _c_p), ("w_rowsum_adj_2", _c_p), ("bias", _c_p)]


_lib = None


class DuqError(RuntimeError):
    """A non-zero status from the C ABI (the reference raises RuntimeError from its
    torch checks, src/export/bindings.cpp:12-17)."""


def load():
    """Load the shared library once and attach prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m duqlinear4bitcuda_amd.build` "
            "(hipcc --offload-arch=gfx950); there is no CPU or PyTorch fallback")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    lib.duq_quantize_linear4bit_workspace_bytes.restype = ctypes.c_uint64
    lib.duq_linear4bit_dual_rowsum_workspace_bytes.restype = ctypes.c_uint64
    lib.duq_quantize_linear4bit_asym_workspace_bytes.restype = ctypes.c_uint64
    lib.duq_quantize_linear8bit_workspace_bytes.restype = ctypes.c_uint64
    lib.duq_status_string.argtypes = [ctypes.c_int]
    lib.duq_status_string.restype = ctypes.c_char_p
    _lib = lib
    return lib


def check(status: int, what: str):
    if status != 0:
        msg = load().duq_status_string(status).decode()
        raise DuqError(f"{what}: {msg} (status {status})")
