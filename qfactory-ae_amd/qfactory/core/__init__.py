from .matmul import QMatmul, Matmul
from .qfunc import QFunc
