"""MI355X (gfx950) implementation of the Linear4bit forward path of DUQLinear4bitCUDA.

``duqlinear4bitcuda_amd.nn`` and ``duqlinear4bitcuda_amd.tools`` keep the module and
function names of the reference's ``qlinear4bit`` package; ``duqlinear4bitcuda_amd._HIP``
takes the place of its ``qlinear4bit._CUDA`` extension and calls hand-written HIP
kernels through the C ABI in ``include/duq_hip.h``.
"""
__version__ = "0.1.0"
