"""The allocate-and-launch extension behind ``forward(x)`` without ``out=`` (csrc/qf_fastpath.cpp).

One native call checks the activation, takes the output from torch's caching allocator and calls the
specialisation's ``launch`` through its address, instead of a dozen tensor attribute reads, ``torch.empty``
and a ctypes call made from Python.  It is host glue: it computes nothing, needs no GPU to build or import,
and a layer without it runs the same launch through the ctypes closure (``QFACTORY_NO_FASTPATH=1`` forces that).

Built in-tree with the host compiler against the installed torch (``build()``); ``load()`` returns the
module, or None when it has not been built or does not match the installed torch.
"""
import importlib.util
import os
import subprocess
import sysconfig
import threading
import warnings

from .native import CSRC_DIR

SOURCE = os.path.join(CSRC_DIR, "qf_fastpath.cpp")
MODULE_NAME = "_qf_fastpath"
LIBRARY = os.path.join(CSRC_DIR, MODULE_NAME + ".so")

_lock = threading.Lock()
_module = None
_tried = False


def source_digest():
    """md5 of csrc/qf_fastpath.cpp: what a built extension must carry to be used."""
    import hashlib
    with open(SOURCE, "rb") as f:
        return hashlib.md5(f.read()).hexdigest()


def build_command(out_path):
    import torch
    from torch.utils import cpp_extension
    cxx = os.environ.get("CXX", "g++")
    cmd = [cxx, "-O2", "-shared", "-fPIC", "-std=c++17", "-fvisibility=hidden", f"-DTORCH_EXTENSION_NAME={MODULE_NAME}",
           f'-DQF_FASTPATH_SOURCE_DIGEST="{source_digest()}"',
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           SOURCE, "-o", out_path]
    for path in cpp_extension.include_paths() + [sysconfig.get_paths()["include"]]:
        cmd += ["-isystem", path]
    lib_dir = cpp_extension.TORCH_LIB_PATH
    cmd += ["-L", lib_dir, "-lc10", "-ltorch", "-ltorch_cpu", "-ltorch_python", f"-Wl,-rpath,{lib_dir}"]
    return cmd


def build(force=False):
    """Compile csrc/qf_fastpath.cpp into csrc/_qf_fastpath.so (host compiler only)."""
    if not force and os.path.exists(LIBRARY):
        with open(LIBRARY, "rb") as f:
            if source_digest().encode() in f.read():       # built from this very source
                return LIBRARY
    tmp = f"{LIBRARY}.tmp.{os.getpid()}"
    proc = subprocess.run(build_command(tmp), capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"building {SOURCE} failed:\n{proc.stderr}")
    os.replace(tmp, LIBRARY)
    global _tried
    with _lock:
        if _module is None:
            _tried = False              # a first (or repaired) build: the next load() looks again
    return LIBRARY


def load():
    """The extension module, or None (not built, built for another torch, or switched off)."""
    global _module, _tried
    if os.environ.get("QFACTORY_NO_FASTPATH") == "1":
        return None
    with _lock:
        if not _tried:
            _tried = True
            if os.path.exists(LIBRARY):
                try:
                    import torch  # noqa: F401  its libraries must be loaded before the extension's
                    spec = importlib.util.spec_from_file_location(MODULE_NAME, LIBRARY)
                    module = importlib.util.module_from_spec(spec)
                    spec.loader.exec_module(module)
                    # a build of another version of the source calls launch with another argument list: never use it
                    if os.path.exists(SOURCE) and getattr(module, "source_digest", None) != source_digest():
                        warnings.warn(f"{LIBRARY} was built from another version of {os.path.basename(SOURCE)}; rebuild it "
                                      "with qfactory.fastpath.build(force=True).  forward() keeps its ctypes path.")
                    else:
                        _module = module
                except ImportError as err:
                    warnings.warn(f"{LIBRARY} does not load against this torch ({err}); rebuild it with "
                                  "qfactory.fastpath.build(force=True).  forward() keeps its ctypes path.")
    return _module


def bound_launch(fn, weight, scale, zero, grouped, n, k, dtype, device_index):
    """``BoundLaunch`` for the ctypes function ``fn`` and a layer's packed tensors, or None without the extension."""
    import ctypes
    module = load()
    if module is None or fn is None:
        return None
    address = ctypes.cast(fn, ctypes.c_void_p).value
    return module.BoundLaunch(address, weight.data_ptr(), scale.data_ptr() if scale is not None else 0,
                              zero.data_ptr() if zero is not None else 0, grouped, n, k, dtype, device_index)
