from .linear import Linear4bitSQ, Linear4bitASQ, Linear4bitDUSQ, LinearQuant4bitDUASQ, Linear4bitASQRowSum, LinearQuant4bitDUASQRowSum, LinearQuant8bitASQ
from .quantizer import SymQuantizer, AsymQuantizer, AsymQuantizer8bit
from .matmul import SymQuantMatMul, AsymQuantMatMul
