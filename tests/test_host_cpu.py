"""CPU-side checks: the C ABI library loads and exports what include/duq_hip.h declares,
argument validation returns the documented codes before anything is launched, and the
Python host layer keeps the reference's interface (names, buffers, asserts, errors)."""
import ctypes
import os
import re
import subprocess
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_functions():
    text = open(os.path.join(ROOT, "include", "duq_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(duq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    names = _header_functions()
    assert len(names) >= 16
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/duq_hip.h but not exported"
    # and the binding table covers the header
    assert set(_lib.PROTOTYPES) | {"duq_status_string"} == set(names)
    assert lib.duq_abi_version() == 1
    assert lib.duq_get_dual_quant_col_k() == 10


def test_status_strings():
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    assert lib.duq_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6):
        assert len(lib.duq_status_string(code)) > 3
    assert b"64" in lib.duq_status_string(-3)


def test_argument_validation_without_launch():
    """Rejected calls return before touching the device (fake non-null pointers are never
    dereferenced on the host)."""
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    P = 0x1000  # aligned, never dereferenced
    assert lib.duq_matmul_host_4bit(P, P, 4, 4, 100, P, None) == -3          # K % 64
    assert lib.duq_matmul_host_4bit(P, P, 4, 4, 131072, P, None) == -6       # K too large for the scaled accumulators
    assert lib.duq_matmul_host_4bit(None, P, 4, 4, 64, P, None) == -1
    assert lib.duq_matmul_host_4bit(P + 4, P, 4, 4, 64, P, None) == -5       # alignment
    assert lib.duq_matmul_host_4bit(P, P, 4, 4, 64, None, None) == -1
    assert lib.duq_matmul_host_4bit(None, None, 0, 4, 64, None, None) == 0   # empty problem is a no-op
    assert lib.duq_sym_quant_host(P, P, 2, 10, 4, P, None) == -2             # colsDst != ceil(colsSrc/2)
    assert lib.duq_sym_quant_host_qmax(P, P, 2, 10, 5, 9, P, None) == -4     # qmax
    assert lib.duq_sym_quant_host(None, P, 2, 10, 5, P, None) == -1
    assert lib.duq_sym_quant_host(None, None, 0, 10, 5, None, None) == 0
    assert lib.duq_asym_quant_host(P, P, None, 2, 10, 5, P, None) == -1
    assert lib.duq_quantize_rows_sym(P, 2, 48, 1.0, 6, P, P, None) == -2     # cols % 32
    assert lib.duq_quantize_rows_sym(P + 2, 2, 64, 1.0, 6, P, P, None) == -5
    assert lib.duq_quantize_rows_asym(P, 2, 64, P, P, None, None) == -1
    assert lib.duq_sym_dequant_host(P, None, P, 2, 2, P, None) == -1
    assert lib.duq_linear4bit_forward(7, P, P, None, P, P, None, None, None, None, 4, 4, 64, P, None) == -4
    assert lib.duq_linear4bit_forward(1, P, P, None, P, P, None, None, None, None, 4, 4, 64, P, None) == -1  # asym needs zeros
    assert lib.duq_linear4bit_forward(2, P, P, None, P, P, None, None, None, None, 4, 4, 64, P, None) == -1  # dual needs scale 2
    assert lib.duq_linear4bit_forward(0, P, P, None, P, P, None, None, None, None, 4, 4, 96, P, None) == -3


def test_check_raises_runtime_error():
    from duqlinear4bitcuda_amd import _lib

    with pytest.raises(RuntimeError, match="multiple of 64"):
        _lib.check(-3, "matmul")
    _lib.check(0, "ok")


def test_ops_reject_cpu_tensors_like_the_reference_binding():
    from duqlinear4bitcuda_amd import _HIP as hip

    a = torch.zeros(4, 32, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="GPU"):
        hip.matmul(a, a)
    x = torch.zeros(4, 64, dtype=torch.float16)
    with pytest.raises(RuntimeError):
        hip.sym_quant(x, torch.ones(4, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="contiguous"):
        hip.matmul(a.t(), a)
    assert hip.get_dual_quant_col_k() == 10


def test_tensor_utils_asserts():
    from duqlinear4bitcuda_amd.tools import tensor_utils as tu

    with pytest.raises(AssertionError, match="multiplication of 32"):
        tu.matmul(torch.zeros(2, 48, dtype=torch.uint8), torch.zeros(2, 48, dtype=torch.uint8))
    with pytest.raises(AssertionError):
        tu.sym_quant(torch.zeros(2, 64), torch.ones(2, 1, dtype=torch.float16))      # fp32 input
    with pytest.raises(AssertionError):
        tu.sym_dequant(torch.zeros(2, 2, dtype=torch.int64), torch.ones(2, dtype=torch.float16), torch.ones(2, dtype=torch.float16))
    p = tu.PackedQuantizedTensor(torch.zeros(3, 8, dtype=torch.uint8), torch.ones(3, 1))
    assert tuple(p.size()) == (3, 8) and p.dtype == torch.uint8 and p.device.type == "cpu" and p.zeros_x is None
    assert tu.get_dual_quant_col() == 10


def test_module_buffers_and_weight_prep_contract():
    from duqlinear4bitcuda_amd import nn as qnn
    from duqlinear4bitcuda_amd.tools import unpack_i4
    from oracle import duq_oracle as orc

    torch.manual_seed(0)
    lin = torch.nn.Linear(64, 24, bias=True).half()
    w = lin.weight.detach()
    s = (w.abs().amax(-1, keepdim=True) / 7).half()

    m = qnn.Linear4bitSQ.from_float(lin, s)
    sd = m.state_dict()
    assert list(sd) == ["weight_scales", "weight", "bias"]
    assert sd["weight"].dtype == torch.uint8 and tuple(sd["weight"].shape) == (24, 32)
    assert sd["weight_scales"].dtype == torch.float16 and tuple(sd["weight_scales"].shape) == (24, 1)
    assert sd["bias"].dtype == torch.float16 and tuple(sd["bias"].shape) == (24,)
    assert np.array_equal(sd["weight"].numpy(), orc.weight_sym_from_float(w.numpy(), s.numpy()))
    assert torch.equal(unpack_i4(sd["weight"]), (w / s).round().to(torch.int32))
    # a freshly constructed module has fp32 scales until it is cast, like the reference (linear.py:32-33)
    assert qnn.Linear4bitSQ(64, 24).weight_scales.dtype == torch.float32
    assert qnn.Linear4bitSQ(64, 24, bias=False).bias is None
    with pytest.raises(AssertionError, match="out_features"):
        qnn.Linear4bitSQ.from_float(lin, s.view(-1))
    # round trip through state_dict
    m2 = qnn.Linear4bitSQ(64, 24, bias=True).half()
    m2.load_state_dict(sd)
    assert all(torch.equal(a, b) for a, b in zip(m2.state_dict().values(), sd.values()))

    a = qnn.Linear4bitASQ.from_linear(lin)
    assert list(a.state_dict()) == ["weight_scales", "weight_zeros", "weight", "bias"]
    pk, sc, z = orc.weight_asym_from_linear(w.numpy())
    assert np.array_equal(a.weight.numpy(), pk)
    assert np.array_equal(a.weight_scales.numpy().view(np.uint16), sc.view(np.uint16))
    assert np.array_equal(a.weight_zeros.numpy().view(np.uint16), z.view(np.uint16))
    assert isinstance(a.quantizer, qnn.AsymQuantizer)
    assert not hasattr(qnn.Linear4bitASQ.from_linear(lin, require_quantizer=False), "quantizer")

    d = qnn.Linear4bitDUSQ.from_float(lin, s, s * 2)
    assert list(d.state_dict()) == ["weight_scales_1", "weight_scales_2", "weight", "bias"]
    codes = unpack_i4(d.weight)
    assert torch.equal(codes[:, :10], (w[:, :10] / s).round().to(torch.int32))
    assert torch.equal(codes[:, 10:], (w[:, 10:] / (s * 2)).round().to(torch.int32))

    u = qnn.LinearQuant4bitDUASQ.from_linear(lin)
    assert list(u.state_dict()) == ["weight_scales_1", "weight_zeros_1", "weight_scales_2", "weight_zeros_2", "weight", "bias"]
    assert all(v.dtype == torch.float16 and tuple(v.shape) == (24, 1) for k, v in u.state_dict().items() if "scales" in k or "zeros" in k)

    with pytest.raises(AssertionError):
        m(torch.zeros(2, 64).half())  # Linear4bitSQ wants a PackedQuantizedTensor (linear.py:46)


def test_quantizer_attributes():
    from duqlinear4bitcuda_amd import nn as qnn

    q = qnn.SymQuantizer(0.9)
    assert q.input_clip_ratio == 0.9 and q.qmax == 6
    a = qnn.AsymQuantizer()
    assert a.n_levels == 16 and a.input_clip_ratio == 1.0


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr


def test_bench_finds_its_traffic_figures_in_the_profiles():
    """bench.py reads the HBM traffic of its roofline kernels from the committed rocprofv3 summaries by kernel
    name: the names it looks for must be the ones the summaries hold."""
    import re

    sys.path.insert(0, ROOT)
    import bench

    src = open(os.path.join(ROOT, "bench.py")).read()
    calls = re.findall(r'profile_traffic_bytes\(\s*"([^"]+)",\s*"([^"]+)"\)', src)
    shaped = re.findall(r'profile_shape_traffic_bytes\(\s*"([^"]+)",\s*"([^"]+)",\s*(\d+)\)', src)
    assert len(calls) >= 2 and len(shaped) >= 1
    for name, kernel in calls:
        assert bench.profile_traffic_bytes(name, kernel), (name, kernel)
    for name, kernel, wgs in shaped:
        assert bench.profile_shape_traffic_bytes(name, kernel, int(wgs)), (name, kernel, wgs)


def test_reference_package_name_is_importable():
    import qlinear4bit._CUDA as ops
    import qlinear4bit.nn as rnn
    import qlinear4bit.tools.tensor_utils as tu
    from duqlinear4bitcuda_amd import nn as impl
    from qlinear4bit.tools.quantization import pack_i4, unpack_i4  # noqa: F401

    assert rnn.Linear4bitSQ is impl.Linear4bitSQ and rnn.SymQuantizer is impl.SymQuantizer
    assert tu.get_dual_quant_col() == ops.get_dual_quant_col_k() == 10
    for name in ("matmul", "sym_quant", "sym_dual_quant", "sym_dequant", "sym_dual_dequant", "asym_quant",
                 "asym_dequant", "asym_dual_quant", "asym_dual_dequant", "get_dual_quant_col_k"):
        assert callable(getattr(ops, name)), name       # the op names of src/export/bindings.cpp:772-923


def test_libtorch_header_compiles_against_the_c_abi(tmp_path):
    """include/duq_torch.hpp (the C++ twin of include/linear.h / include/quant_tensor.h of the
    reference) must parse and type-check against libtorch's headers and duq_hip.h."""
    import shutil
    if shutil.which("g++") is None:
        pytest.skip("no host C++ compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    tinc = os.path.join(os.path.dirname(torch.__file__), "include")
    if not os.path.exists(os.path.join(tinc, "c10", "hip", "HIPStream.h")):
        pytest.skip("libtorch was built without ROCm headers")
    src = tmp_path / "use_duq_torch.cpp"
    src.write_text(
        '#include "duq_torch.hpp"\n'
        "torch::Tensor run(torch::Tensor x, duq::Linear4bit &l, duq::Linear4bitDUQ &d) {\n"
        "    duq::Quantizer4bit q(1.0f);\n"
        "    auto p = q.forward(x);\n"
        "    return l.forward(p) + d.forward(p) + duq::sym_dequant(duq::matmul(p.quantized_x, l.weight),\n"
        "        p.scale.view(-1), l.weight_scale.view(-1), 32);\n"
        "}\n")
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(root, "include"), "-I", tinc,
           "-I", os.path.join(tinc, "torch", "csrc", "api", "include"), "-I", "/opt/rocm/include", str(src)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]


def test_gemm_kernel_selection_keeps_32_bit_offsets_in_range():
    """The dispatch rule (host arithmetic, exported as duq_gemm_kernel_for): every kernel family that addresses the
    weight tensor with 32-bit byte offsets (decode rows 1, decode MFMA 2, dot 3, ring 4, skinny 5) is only picked
    while the packed weights stay below 2^32 - 256 bytes; anything larger goes to the stream / tile kernels
    (64-bit per-tile bases).  Also pins the shape buckets."""
    from duqlinear4bitcuda_amd import _lib

    f = _lib.load().duq_gemm_kernel_for
    small = {1, 2, 3, 4, 5}
    limit = 0xFFFFFF00
    rng = np.random.default_rng(0)
    ks = [64, 128, 4096, 8192, 11008, 12288, 12352, 16384, 16448, 28672, 131008]
    for M in (1, 2, 3, 4, 5, 8, 16, 17, 32, 64, 65, 128, 256, 257, 2048):
        for K in ks:
            kb = K // 2
            edge = limit // kb
            for N in {1, 16, 4096, 11008, edge - 1, edge, edge + 1, edge + 4096, 1 << 22} | set(rng.integers(1, 1 << 22, 6).tolist()):
                if N < 1 or N > (1 << 22):
                    continue
                k = f(M, int(N), K)
                assert k in (1, 2, 3, 4, 5, 6, 7)
                if int(N) * kb >= limit:
                    assert k not in small, (M, N, K, k)
    # buckets at the benchmark shapes
    assert [f(m, 4096, 4096) for m in (1, 4, 5, 16, 17, 64, 65, 2048)] == [1, 1, 2, 2, 2, 2, 6, 6]
    assert f(100, 1000, 4096) == 4 and f(200, 520, 8192) == 4 and f(128, 11008, 4096) == 6 and f(128, 28672, 8192) == 6
    assert f(16, 11008, 4096) == 2 and f(16, 4096, 11008) == 2 and f(16, 28672, 8192) == 2
    assert f(16, 28672, 4096) == 5 and f(8, 28672, 4096) == 2 and f(64, 28672, 4096) == 2
    assert f(32, 4096, 8192) == 2 and f(33, 4096, 8192) == 2 and f(17, 4096, 11008) == 2 and f(48, 4096, 12288) == 2
    assert f(33, 1024, 8192) == 4 and f(32, 1024, 8192) == 2 and f(49, 4096, 11008) != 2 and f(17, 2048, 11008) == 4
    assert f(1, 28672, 8192) == 1 and f(1, 8192, 28672) == 3 and f(16, 8192, 28672) == 7
    assert f(16, 64, 16384) == 4 and f(4, 64, 16384) == 1 and f(16, 4096, 12288) == 2
    assert f(16, 1 << 22, 4096) == 7 and f(1, 1 << 22, 4096) == 7 and f(64, 1 << 22, 4096) in (6, 7)


def test_fp16_input_entry_point_validation_without_launch():
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    P = 0x1000
    f = lib.duq_quantize_linear4bit_forward
    assert f(0, P, 1.0, 6, P, P, None, None, 4, 4, 100, P, None, None, None, 0, None) == -3      # K % 64
    assert f(5, P, 1.0, 6, P, P, None, None, 4, 4, 64, P, None, None, None, 0, None) == -4       # mode
    assert f(0, P, 1.0, 9, P, P, None, None, 4, 4, 64, P, None, None, None, 0, None) == -4       # qmax
    assert f(0, None, 1.0, 6, P, P, None, None, 4, 4, 64, P, None, None, None, 0, None) == -1
    assert f(0, P, 1.0, 6, P, None, None, None, 4, 4, 64, P, None, None, None, 0, None) == -1
    assert f(2, P, 1.0, 6, P, P, None, None, 4, 4, 64, P, None, None, None, 0, None) == -1       # dual needs scale 2
    assert f(0, P, 1.0, 6, P, P, None, None, 64, 4, 64, P, None, None, None, 0, None) == -1      # needs a workspace
    assert f(0, P, 1.0, 6, P, P, None, None, 64, 4, 64, P, None, None, P, 100, None) == -2       # too small
    assert f(0, None, 1.0, 6, None, None, None, None, 0, 4, 64, None, None, None, None, 0, None) == 0
    assert lib.duq_quantize_linear4bit_workspace_bytes(64, 4, 64) == 64 * 32 + 128
    assert lib.duq_quantize_linear4bit_workspace_bytes(4, 4096, 4096) == 0
    # two to four rows: one launch on any width up to 8192 elements, up to 16384 columns beyond
    assert lib.duq_quantize_linear4bit_workspace_bytes(4, 28672, 8192) == 0
    assert lib.duq_quantize_linear4bit_workspace_bytes(4, 20000, 16384) == 4 * 8192 + 16
    assert lib.duq_quantize_linear4bit_workspace_bytes(1, 20000, 16384) == 0
    # five to eight rows: any width up to 4096 elements, 8192 on at most 4096 columns
    assert lib.duq_quantize_linear4bit_workspace_bytes(8, 28672, 4096) == 0
    assert lib.duq_quantize_linear4bit_workspace_bytes(8, 4112, 8192) == 8 * 4096 + 16


def test_asym_fp16_input_entry_point_validation_without_launch():
    from duqlinear4bitcuda_amd import _lib

    lib = _lib.load()
    P = 0x1000
    f = lib.duq_quantize_linear4bit_forward_asym
    tail = (None, None, None, None, None, 0, None)
    assert f(0, P, P, P, P, None, None, None, None, None, 4, 4, 64, P, *tail) == -4      # symmetric modes: the other entry point
    assert f(6, P, P, P, P, None, None, None, None, None, 4, 4, 64, P, *tail) == -4
    assert f(1, P, P, P, P, None, None, None, None, None, 4, 4, 100, P, *tail) == -3     # K % 64
    assert f(1, None, P, P, P, None, None, None, None, None, 4, 4, 64, P, *tail) == -1
    assert f(1, P, P, P, None, None, None, None, None, None, 4, 4, 64, P, *tail) == -1   # asym needs weight zeros
    assert f(3, P, P, P, P, P, None, None, None, None, 4, 4, 64, P, *tail) == -1         # dual needs the second pair
    assert f(4, P, P, P, P, None, None, None, None, None, 4, 4, 64, P, *tail) == -1      # row-sum needs the weight term
    assert f(5, P, P, P, P, P, P, P, None, None, 4, 4, 64, P, *tail) == -1               # dual row-sum needs both terms
    assert f(1, P, P, P, P, None, None, None, None, None, 64, 4, 64, P, *tail) == -1     # needs a workspace
    assert f(1, P, P, P, P, None, None, None, None, None, 64, 4, 64, P, None, None, None, None, P, 100, None) == -2
    assert f(1, None, None, None, None, None, None, None, None, None, 0, 4, 64, None, *tail) == 0
    g = lib.duq_quantize_linear4bit_asym_workspace_bytes
    assert g(1, 64, 4, 64) == 64 * 32 + 128 + 128 and g(4, 64, 4, 64) == 64 * 32 + 128 + 128 + 256
    assert g(5, 64, 4, 64) == 64 * 32 + 128 + 128 + 256 and g(5, 100, 8, 128) == 100 * 64 + 208 + 208 + 400 + 3200
    assert g(1, 8, 4096, 4096) == 0 and g(5, 8, 4096, 4096) == 0 and g(2, 64, 4, 64) == 0
    # nine to sixteen rows are one launch while they hold at most 32768 elements together (40960 on at most 4096 columns)
    assert g(1, 16, 4096, 2048) == 0 and g(4, 10, 4096, 4096) == 0 and g(1, 11, 4096, 4096) > 0 and g(1, 16, 20000, 2048) > 0
    assert g(1, 16, 16384, 2048) == 0 and g(1, 10, 11008, 4096) > 0
    # the entry point that allocates nothing: slot and size limits are checked before anything else
    s = lib.duq_quantize_linear4bit_forward_static
    assert s(0, P, 1.0, 6, P, P, None, None, 8, 64, 64, P, None, None, 4, None) == -7   # no such slot
    assert s(0, P, 1.0, 6, P, P, None, None, 4097, 64, 4096, P, None, None, 0, None) == -7
    assert s(1, P, 1.0, 6, P, P, None, None, 8, 64, 64, P, None, None, 0, None) == -4
    for code in (-7, -8, -9):
        assert len(lib.duq_status_string(code)) > 10
    # the prepared-layer form: a shape of two launches needs its workspace, checked before anything else is touched
    layer = _lib.FusedLayer(0, 1.0, 6, 4096, 4096, P, P, None, None, None, None, None, None)
    g = lib.duq_quantize_linear4bit_forward_layer
    assert g(ctypes.addressof(layer), P, 12, P, None, 0, None) == -1 and g(None, P, 1, P, None, 0, None) == -1
    assert g(ctypes.addressof(layer), P, 12, P, P, 100, None) == -2
    assert g(ctypes.addressof(layer), P, 12, P, ctypes.c_void_p(4104), 1 << 20, None) == -5
    assert g(ctypes.addressof(layer), P, 0, P, None, 0, None) == 0
    layer.mode = 9
    assert g(ctypes.addressof(layer), P, 1, P, None, 0, None) == -4
    layer.mode, layer.w_scale_1 = 0, None
    assert g(ctypes.addressof(layer), P, 1, P, None, 0, None) == -1


def test_stream_tile_rule():
    """Tile of the stream kernel per shape (host arithmetic, duq_gemm_stream_tile_for): 256-row tiles only with at
    least one per CU and when their rounds come out cheaper."""
    from duqlinear4bitcuda_amd import _lib
    f = _lib.load().duq_gemm_stream_tile_for
    assert f(2048, 4096, 4096) == 128256          # the headline shape: 256 tiles of 128 rows
    assert f(4096, 4096, 4096) == 256256 and f(4096, 11008, 4096) == 256256 and f(2048, 22016, 4096) == 256256
    assert f(4096, 28672, 8192) == 256256 and f(4096, 8192, 28672) == 256256
    assert f(4000, 8200, 4160) == 128256          # three ragged rounds of 256-row tiles against five of 128-row ones
    assert f(2048, 11008, 4096) == 128256         # 344 tiles of 256 rows: two rounds, the second a third full
    assert f(512, 4096, 4096) == 64128 and f(1024, 4096, 4096) == 128128
    assert f(16, 4096, 4096) == 0 and f(1, 4096, 4096) == 0   # decode kernels


def test_deferred_quantized_tensor_host_side():
    """What SymQuantizer hands over for a few rows: shape, device and the check that the rows were not written to,
    without anything being computed (quantizing needs the GPU)."""
    from duqlinear4bitcuda_amd import nn as qnn
    from duqlinear4bitcuda_amd.tools import tensor_utils as tu

    x = torch.zeros(2, 3, 128, dtype=torch.float16)
    p = tu.PackedQuantizedTensor.deferred(x, 0.9, 7)
    assert type(p) is tu.PackedQuantizedTensor
    assert tuple(p.size()) == (2, 3, 64) and p.device.type == "cpu" and p.dtype == torch.uint8
    assert p.source() is x and p.zeros_x is None and p.shadow_x is None and p.rowsum_x is None
    x.add_(1)
    with pytest.raises(RuntimeError, match="modified in place"):
        p.source()
    # CPU inputs are never deferred (the quantizer then fails in the op, like the reference binding)
    with pytest.raises(RuntimeError):
        qnn.SymQuantizer(1.0)(torch.zeros(2, 128, dtype=torch.float16))
    # explicit fields behave like the reference's plain attributes
    q = tu.PackedQuantizedTensor(torch.zeros(3, 8, dtype=torch.uint8), torch.ones(3, 1))
    q.scales_x = torch.full((3, 1), 2.0)
    q.quantized_x = torch.ones(3, 8, dtype=torch.uint8)
    assert q.scales_x[0, 0] == 2 and q.quantized_x[0, 0] == 1 and q.source() is None
