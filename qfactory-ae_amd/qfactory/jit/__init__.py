from .compiler import jit
