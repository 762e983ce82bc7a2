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
from .verify import gemm_waits_hold

logger = logging.getLogger(__name__)

runtime_cache = RuntimeCache()

DEFAULT_ARCH = "gfx950"
_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE_DIR = os.path.join(_PKG_DIR, "include")
# C-ABI declarations: qfactory/abi in a built distribution (setup.py copies them there), <checkout>/include in a
# source checkout; optional either way (the generated code includes them under __has_include).
ABI_INCLUDE_DIR = (os.path.join(_PKG_DIR, "abi") if os.path.isdir(os.path.join(_PKG_DIR, "abi"))
                   else os.path.normpath(os.path.join(_PKG_DIR, "..", "..", "include")))

_lock = threading.Lock()
_memo = {}


def hash_to_hex(s: str) -> str:
    return hashlib.md5(s.encode("utf-8")).hexdigest()[0:12]


def include_dirs():
    dirs = [INCLUDE_DIR]
    if os.path.exists(os.path.join(ABI_INCLUDE_DIR, "qfactory_launch.h")):
        dirs.append(ABI_INCLUDE_DIR)
    return dirs


_INCLUDE_RE = re.compile(r'^[ \t]*#[ \t]*include[ \t]*"([^"]+)"', re.MULTILINE)


def _read_header(name):
    """(path, text) of a quoted include found in the include directories, or None (a system header)."""
    for d in include_dirs():
        path = os.path.join(d, name)
        if os.path.exists(path):
            with _lock:
                hit = _memo.get(("header", path))
            if hit is None:
                with open(path) as f:
                    hit = f.read()
                with _lock:
                    _memo[("header", path)] = hit
            return path, hit
    return None


def get_qfactory_version(code: str = None) -> str:
    """md5 over the package headers a translation unit includes, directly or through other headers (the
    reference hashes its whole include directory, compiler.py:16-28; hashing what a unit can see keeps the
    objects of the other kernel families valid when one header changes).  Without ``code``: every header."""
    if code is None:
        code = "".join(f'#include "{f}"\n' for d in include_dirs() for f in sorted(os.listdir(d)) if f.endswith(".h"))
    seen, queue = {}, [code]
    while queue:
        for name in _INCLUDE_RE.findall(queue.pop()):
            found = _read_header(name)
            if found is not None and found[0] not in seen:
                seen[found[0]] = found[1]
                queue.append(found[1])
    md5 = hashlib.md5()
    for path in sorted(seen):
        md5.update(os.path.basename(path).encode())
        md5.update(seen[path].encode())
    return md5.hexdigest()[0:12]


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
    check_gemm_waits = staticmethod(gemm_waits_hold)

    def runtime_path_of(self, qfunc):
        """(runtime directory, source) the given QFunc compiles to, without compiling."""
        code = qfunc.emit()
        arch = os.getenv("QFACTORY_ARCH", DEFAULT_ARCH)
        flags = compile_flags(arch)
        signature = f"{code}$${get_hipcc_compiler()}$${get_qfactory_version(code)}$${flags}$${arch}"
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
        # GEMM objects wait on counted loads: keep the device ISA of this compile and re-count (verify.py)
        counted_waits = getattr(qfunc, "regime", None) == "gemm" and "QF_GEMM_FULL_DRAIN 1" not in code
        work_dir = None
        if counted_waits:
            work_dir = os.path.join(tmp_dir, f"temps.{uuid.uuid4()}")
            os.makedirs(work_dir)
            command.append("-save-temps")
        logger.info(f"Compiling kernel with command: {' '.join(command)}")
        try:
            proc = subprocess.run(command, capture_output=True, text=True, cwd=work_dir)
            if proc.returncode != 0:
                raise RuntimeError(f"hipcc failed for {src_path} (exit {proc.returncode}):\n{proc.stderr[-4000:]}")
            if counted_waits:
                isa = "".join(open(os.path.join(work_dir, f)).read() for f in sorted(os.listdir(work_dir))
                              if f.endswith(".s") and "amdgcn" in f)
                ok, detail = self.check_gemm_waits(isa, qfunc.tiling_configs["PA"])
                if not ok:
                    logger.warning(f"GEMM object {runtime_path}: {detail}; rebuilding with a full drain per K-iteration")
                    command = [c for c in command if c != "-save-temps"] + ["-DQF_GEMM_FULL_DRAIN=1"]
                    proc = subprocess.run(command, capture_output=True, text=True)
                    if proc.returncode != 0:
                        raise RuntimeError(f"hipcc failed for {src_path} (exit {proc.returncode}):\n{proc.stderr[-4000:]}")
        finally:
            if work_dir is not None:
                shutil.rmtree(work_dir, ignore_errors=True)

        dump_args(qfunc.arg_name_type(), tmp_args_path)
        os.replace(tmp_args_path, args_path)
        os.replace(tmp_so_path, so_path)  # atomic publish; the .so is the last file to appear

        runtime_cache[runtime_path] = Runtime(runtime_path)
        return runtime_cache[runtime_path]


jit = JITCompiler()
