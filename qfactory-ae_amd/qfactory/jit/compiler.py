"""hipcc JIT: one shared object per emitted translation unit, cached by content hash.

Counterpart of the reference's ``qfactory/jit/compiler.py`` (nvcc JIT, compiler.py:56-116) with the
same cache contract: directory ``$QFACTORY_CACHE_DIR`` or ``~/.qfactory``; key = md5[:12] of
``code $$ compiler(path, version) $$ md5 of the headers $$ flags $$ arch``; files
``runtimes/kernel.<arch>.<hash>/kernel.{hip,args,so}``; compile into a unique temporary name and
publish with an atomic rename, so concurrent compiles of the same key from a thread pool or from
several processes are safe.  ``QFACTORY_ARCH`` selects the offload architecture (default gfx950).
"""
import hashlib
import logging
import os
import re
import shutil
import subprocess
import threading
import uuid

from .runtime import Runtime, RuntimeCache, dump_args

logger = logging.getLogger(__name__)

runtime_cache = RuntimeCache()

DEFAULT_ARCH = "gfx950"
_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE_DIR = os.path.join(_PKG_DIR, "include")
# C-ABI declarations live at <checkout>/include; present in a source checkout, optional otherwise.
ABI_INCLUDE_DIR = os.path.normpath(os.path.join(_PKG_DIR, "..", "..", "include"))

_lock = threading.Lock()
_memo = {}


def hash_to_hex(s: str) -> str:
    return hashlib.md5(s.encode("utf-8")).hexdigest()[0:12]


def include_dirs():
    dirs = [INCLUDE_DIR]
    if os.path.exists(os.path.join(ABI_INCLUDE_DIR, "qfactory_launch.h")):
        dirs.append(ABI_INCLUDE_DIR)
    return dirs


def get_qfactory_version() -> str:
    """md5 over every header the generated code can include."""
    with _lock:
        if "version" in _memo:
            return _memo["version"]
    md5 = hashlib.md5()
    for d in include_dirs():
        for root, _, files in sorted(os.walk(d)):
            for filename in sorted(f for f in files if f.endswith(".h")):
                with open(os.path.join(root, filename), "rb") as f:
                    md5.update(f.read())
    with _lock:
        _memo["version"] = md5.hexdigest()[0:12]
        return _memo["version"]


def get_hipcc_compiler():
    """(path, version) of hipcc; raises if there is none -- there is no other backend."""
    with _lock:
        if "hipcc" in _memo:
            return _memo["hipcc"]
    rocm = os.environ.get("ROCM_PATH") or os.environ.get("ROCM_HOME") or "/opt/rocm"
    path = shutil.which("hipcc") or os.path.join(rocm, "bin", "hipcc")
    try:
        text = subprocess.run([path, "--version"], capture_output=True, text=True, check=True).stdout
        version = re.search(r"HIP version:\s*(\S+)", text).group(1)
    except Exception as exc:
        raise RuntimeError(f"Cannot get the version of the hipcc compiler at {path}") from exc
    with _lock:
        _memo["hipcc"] = (path, version)
        return _memo["hipcc"]


def get_cache_dir():
    if "QFACTORY_CACHE_DIR" in os.environ:
        path = os.getenv("QFACTORY_CACHE_DIR")
        os.makedirs(path, exist_ok=True)
        return path
    return os.path.join(os.path.expanduser("~"), ".qfactory")


def write_file(tmp_dir: str, path: str, content: str):
    tmp_file_path = os.path.join(tmp_dir, f"file.tmp.{uuid.uuid4()}.{hash_to_hex(path)}")
    with open(tmp_file_path, "w") as f:
        f.write(content)
    os.replace(tmp_file_path, path)


def compile_flags(arch):
    return [
        f"--offload-arch={arch}", "-std=c++20", "-shared", "-fPIC", "-O3",
        # never let the compiler form packed-fp32 VALU ops from scalar float code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wno-unused-command-line-argument",
    ]


class JITCompiler:
    def runtime_path_of(self, qfunc):
        """(runtime directory, source) the given QFunc compiles to, without compiling."""
        code = qfunc.emit()
        arch = os.getenv("QFACTORY_ARCH", DEFAULT_ARCH)
        flags = compile_flags(arch)
        signature = f"{code}$${get_hipcc_compiler()}$${get_qfactory_version()}$${flags}$${arch}"
        runtime_name = f"kernel.{arch}.{hash_to_hex(signature)}"
        return os.path.join(get_cache_dir(), "runtimes", runtime_name), code

    def compile(self, qfunc, force: bool = False) -> Runtime:
        runtime_path, code = self.runtime_path_of(qfunc)
        arch = os.getenv("QFACTORY_ARCH", DEFAULT_ARCH)
        flags = compile_flags(arch)

        if not force:
            cached = runtime_cache[runtime_path]
            if cached is not None:
                logger.debug(f"Using cached runtime {runtime_path}")
                return cached

        tmp_dir = os.path.join(get_cache_dir(), "tmp")
        os.makedirs(runtime_path, exist_ok=True)
        os.makedirs(tmp_dir, exist_ok=True)
        src_path = os.path.join(runtime_path, "kernel.hip")
        so_path = os.path.join(runtime_path, "kernel.so")
        args_path = os.path.join(runtime_path, "kernel.args")
        tmp_so_path = os.path.join(tmp_dir, f"hipcc.tmp.{uuid.uuid4()}.{hash_to_hex(so_path)}.so")
        tmp_args_path = os.path.join(tmp_dir, f"args.tmp.{uuid.uuid4()}.{hash_to_hex(args_path)}")

        write_file(tmp_dir, src_path, code)
        command = [get_hipcc_compiler()[0], "-x", "hip", src_path, "-o", tmp_so_path, *flags,
                   *[f"-I{d}" for d in include_dirs()]]
        logger.info(f"Compiling kernel with command: {' '.join(command)}")
        proc = subprocess.run(command, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src_path} (exit {proc.returncode}):\n{proc.stderr[-4000:]}")

        dump_args(qfunc.arg_name_type(), tmp_args_path)
        os.replace(tmp_args_path, args_path)
        os.replace(tmp_so_path, so_path)  # atomic publish; the .so is the last file to appear

        runtime_cache[runtime_path] = Runtime(runtime_path)
        return runtime_cache[runtime_path]


jit = JITCompiler()
