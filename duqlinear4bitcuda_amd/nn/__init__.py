from .linear import Linear4bitSQ, Linear4bitASQ, Linear4bitDUSQ, LinearQuant4bitDUASQ, Linear4bitASQRowSum
from .quantizer import SymQuantizer, AsymQuantizer
from .matmul import SymQuantMatMul, AsymQuantMatMul
