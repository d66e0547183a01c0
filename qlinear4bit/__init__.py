"""Import alias: code written against the reference package (``import qlinear4bit.nn``,
``qlinear4bit.tools.tensor_utils``, ...) runs unchanged on the MI355X implementation.
``qlinear4bit._CUDA`` resolves to the HIP op module with the same function names."""
import importlib
import sys

_IMPL = "duqlinear4bitcuda_amd"
_ALIASES = {
    "nn": "nn",
    "nn.linear": "nn.linear",
    "nn.quantizer": "nn.quantizer",
    "nn.matmul": "nn.matmul",
    "tools": "tools",
    "tools.tensor_utils": "tools.tensor_utils",
    "tools.quantization": "tools.quantization",
    "tools.graphs": "tools.graphs",
    "_CUDA": "_HIP",
}
for _alias, _target in _ALIASES.items():
    _mod = importlib.import_module(f"{_IMPL}.{_target}")
    sys.modules[f"{__name__}.{_alias}"] = _mod
    if "." not in _alias:
        globals()[_alias] = _mod
