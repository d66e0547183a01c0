from .linear import Linear4bitSQ, Linear4bitASQ, Linear4bitDUSQ, LinearQuant4bitDUASQ, Linear4bitASQRowSum, LinearQuant4bitDUASQRowSum, LinearQuant8bitASQ
from .quantizer import SymQuantizer, AsymQuantizer, AsymQuantizer8bit
from .matmul import SymQuantMatMul, AsymQuantMatMul


def enable_fp6(model, quantizer_shadow=True):
    """Switch every 4-bit layer of ``model`` that the 6-bit float matrix path can take (on a GPU, out_features % 16 ==
    0, in_features % 128 == 0) to it (``layer.enable_fp6()``: + 3/4 byte per weight element, same bits, large inputs
    20-30 % faster) and let every ``SymQuantizer`` / ``AsymQuantizer`` in it write the activation shadow for inputs
    of at least its ``shadow_min_rows`` tokens.  ``quantizer_shadow``: True (codes and shadow: safe for every
    consumer of the quantized tensor) or "only" (the shadow alone, for quantizers that feed such layers only: a
    little faster).  Not in the reference.  Returns the number of layers switched."""
    import torch
    from .linear import _Linear4bitBase
    assert quantizer_shadow in (True, "only")
    n = 0
    for m in model.modules():
        if isinstance(m, _Linear4bitBase) and hasattr(m, "weight") and isinstance(m.weight, torch.Tensor) and m.weight.is_cuda \
                and m.weight.dtype is torch.uint8 and m.out_features % 16 == 0 and m.in_features % 128 == 0:
            m.enable_fp6()
            n += 1
        elif isinstance(m, (SymQuantizer, AsymQuantizer)):
            m.shadow = quantizer_shadow
    return n
