"""ctypes loader for one compiled specialisation.

Counterpart of the reference's ``qfactory/jit/runtime.py``: a runtime directory holds the source,
the argument specification and the shared object (``kernel.hip``, ``kernel.args``, ``kernel.so``);
``Runtime.run(*args)`` marshals tensors / streams / ints to C and calls ``launch`` (runtime.py:37-49),
returning the kernel's return code.  The argument specification is stored as JSON rather than a
pickle so that loading a cache directory never executes anything from it.
"""
import ctypes
import json
import os

import torch

_TYPE_NAMES = {
    "float16": torch.float16,
    "bfloat16": torch.bfloat16,
    "int8": torch.int8,
    "stream": torch.cuda.streams.Stream,
    "int": int,
}
_NAME_OF_TYPE = {v: k for k, v in _TYPE_NAMES.items()}

Python2CTypes = {
    torch.float16: ctypes.c_void_p,
    torch.bfloat16: ctypes.c_void_p,
    torch.int8: ctypes.c_void_p,
    torch.cuda.streams.Stream: ctypes.c_void_p,
    int: ctypes.c_int,
}

RUNTIME_FILES = ("kernel.hip", "kernel.args", "kernel.so")


def dump_args(args_name_type, path):
    with open(path, "w") as f:
        json.dump([[name, _NAME_OF_TYPE[t]] for name, t in args_name_type], f)


def load_args(path):
    with open(path) as f:
        return [(name, _TYPE_NAMES[t]) for name, t in json.load(f)]


def map_ctype(arg, dtype):
    ctype = Python2CTypes[dtype]
    if isinstance(arg, torch.Tensor):
        return ctype(arg.data_ptr())
    if isinstance(arg, torch.cuda.Stream):
        return ctype(arg.cuda_stream)
    return ctype(arg)


class Runtime:
    def __init__(self, path: str):
        self.lib, self.args = None, None
        assert self.is_path_valid(path), f"Invalid Runtime Path {path}"
        self.path = path
        self.lib = ctypes.CDLL(os.path.join(path, "kernel.so"))
        self.args = load_args(os.path.join(path, "kernel.args"))
        sig = [Python2CTypes[t] for _, t in self.args]
        rc_type = ctypes.POINTER(ctypes.c_int)          # `int&` is passed as an address
        self.lib.launch.restype = None
        self.lib.launch.argtypes = sig + [rc_type]
        self._launch_m = getattr(self.lib, "launch_m", None)
        if self._launch_m is not None:
            self._launch_m.restype = None
            self._launch_m.argtypes = [ctypes.c_int] + sig + [rc_type]
        self._launch_m_static = getattr(self.lib, "launch_m_static", None)    # objects that use scratch memory: the same launch on a static array
        if self._launch_m_static is not None:
            self._launch_m_static.restype = None
            self._launch_m_static.argtypes = [ctypes.c_int] + sig + [rc_type]
        self._launch_norm = getattr(self.lib, "launch_norm", None)      # objects with the residual-add + RMSNorm prologue
        if self._launch_norm is not None:
            self._launch_norm.restype = None
            ptr = ctypes.c_void_p
            self._launch_norm.argtypes = [ctypes.c_int, ptr, ptr, ptr, ptr, ctypes.c_float, ptr, ptr, ptr, ptr, ptr, rc_type]
        describe = getattr(self.lib, "qf_describe", None)
        if describe is not None:
            describe.restype = ctypes.c_char_p
            self.description = describe().decode()
        else:
            self.description = ""
        self._rc = ctypes.c_int(0)
        self._rc_ref = ctypes.byref(self._rc)

    @staticmethod
    def is_path_valid(path: str) -> bool:
        if not os.path.isdir(path):
            return False
        return all(os.path.exists(os.path.join(path, f)) for f in RUNTIME_FILES)

    def _marshal(self, args):
        assert len(args) == len(self.args), f"Expected {len(self.args)} arguments, got {len(args)}"
        cargs = []
        for arg, (name, dtype) in zip(args, self.args):
            if isinstance(arg, torch.Tensor):
                assert arg.dtype == dtype, f"Expected tensor dtype {dtype} for {name}, got {arg.dtype}"
            else:
                assert isinstance(arg, dtype), f"Expected built-in type {dtype} for {name}, got {type(arg)}"
            cargs.append(map_ctype(arg, dtype))
        return cargs

    def run(self, *args) -> int:
        """Call ``launch`` with the arguments of ``kernel.args``; returns its return code."""
        return_code = ctypes.c_int(0)
        self.lib.launch(*self._marshal(args), ctypes.byref(return_code))
        return return_code.value

    def run_m(self, m: int, *args) -> int:
        """Call ``launch_m``: like ``run`` but for ``m`` activation rows instead of the built-in M."""
        assert self._launch_m is not None, "this specialisation takes m through launch()"
        return_code = ctypes.c_int(0)
        self._launch_m(ctypes.c_int(m), *self._marshal(args), ctypes.byref(return_code))
        return return_code.value

    def run_m_static(self, m: int, *args) -> int:
        """Call ``launch_m_static``: ``launch_m`` of an object that uses scratch memory, on the object's static device
        array instead of memory allocated at the first call (nothing is allocated, by the call or by this wrapper's
        marshalling of its arguments)."""
        assert self._launch_m_static is not None, "this specialisation uses no scratch memory: launch_m allocates nothing"
        return_code = ctypes.c_int(0)
        self._launch_m_static(ctypes.c_int(m), *self._marshal(args), ctypes.byref(return_code))
        return return_code.value

    def run_raw(self, m, ptrs, stream_handle) -> int:
        """Hot path without per-argument checks: raw device addresses and a raw stream handle.

        The caller has validated shapes, dtypes and contiguity once.  Not re-entrant (shares one
        return-code cell), which matches the single-threaded enqueue of a module's forward.
        """
        fn = self._launch_m if self._launch_m is not None else self.lib.launch
        fn(m, *ptrs, stream_handle, self._rc_ref)
        return self._rc.value


class RuntimeCache:
    def __init__(self):
        self.cache = {}

    def __getitem__(self, path: str):
        if path in self.cache:
            return self.cache[path]
        if Runtime.is_path_valid(path):
            runtime = Runtime(path)
            self.cache[path] = runtime
            return runtime
        return None

    def __setitem__(self, path, runtime):
        self.cache[path] = runtime
