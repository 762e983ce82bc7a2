"""The C-ABI shared objects load without a GPU and export every symbol the headers in include/
declare.  No compute call is made here."""
import ctypes
import os
import re

import pytest
import torch

from conftest import ROOT

INCLUDE = os.path.join(ROOT, "include")


def _declared_functions(header, guard=None):
    """Names of the function prototypes in a header (optionally only those under `#if defined(guard)`)."""
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    if guard is not None:
        m = re.search(r"#(?:el)?if defined\(%s\)(.*?)#(?:elif|endif)" % guard, text, flags=re.S)
        assert m, f"{guard} block not found in {header}"
        text = m.group(1)
    else:
        text = re.sub(r"#if defined\(.*?#endif", "", text, flags=re.S)
    text = "\n".join(l for l in text.splitlines() if not l.lstrip().startswith(("#", "typedef")))
    return sorted(set(re.findall(r"\b([A-Za-z_]\w*)\s*\([^;{]*\)\s*;", text)))


def test_header_parsers_see_the_expected_prototypes():
    assert _declared_functions("qfactory_hip.h") == sorted(
        ["qf_version", "qf_pack_weight", "qf_pack_zero", "qf_transpose_scale", "qf_bf16_to_f16", "qf_stream_read", "qf_stream_copy", "qf_empty_launch",
         "qf_add_rmsnorm", "qf_rope_kv_store", "qf_rope_kv_store_rows", "qf_decode_attention", "qf_rope_decode_attention", "qf_silu_mul",
         "qf_greedy_next"])
    assert _declared_functions("qfactory_launch.h", "QF_LAUNCH_GROUPED") == ["launch", "launch_m", "qf_describe"]
    assert _declared_functions("qfactory_launch.h", "QF_LAUNCH_PLAIN") == ["launch", "qf_describe"]


def test_aot_library_exports_every_declared_symbol():
    from qfactory import native
    native.build()
    lib = ctypes.CDLL(native.LIBRARY)
    for name in _declared_functions("qfactory_hip.h"):
        assert hasattr(lib, name), f"{name} missing from {native.LIBRARY}"
    assert sorted(native.SIGNATURES) == _declared_functions("qfactory_hip.h")
    lib.qf_version.restype = ctypes.c_int
    assert lib.qf_version() == 102          # host-only call: no device work


@pytest.mark.parametrize("gs,guard", [(128, "QF_LAUNCH_GROUPED"), (-1, "QF_LAUNCH_PLAIN")])
def test_jit_object_exports_the_launch_abi(gs, guard):
    from qfactory.core.qfunc import MatmulQFunc, QMatmulQFunc
    from qfactory.core.qtile import AsymQTile, QTile
    from qfactory.jit import jit
    a = QTile((1, 512), torch.float16, 16)
    if gs == -1:
        qfunc = MatmulQFunc(a, QTile((64, 512), torch.int8, 4), "nt")
    else:
        qfunc = QMatmulQFunc(a, AsymQTile((64, 512), torch.int8, 4, (1, gs)), "nt")
    runtime = jit.compile(qfunc)
    lib = ctypes.CDLL(os.path.join(runtime.path, "kernel.so"))
    for name in _declared_functions("qfactory_launch.h", guard):
        assert hasattr(lib, name), f"{name} missing from {runtime.path}"
    lib.qf_describe.restype = ctypes.c_char_p
    text = lib.qf_describe().decode()
    assert "N=64" in text and "K=512" in text and "NBITS=4" in text
    # the generated translation unit includes the ABI header and implements the matching variant
    src = open(os.path.join(runtime.path, "kernel.hip")).read()
    assert f"#define {guard}" in src and '#include "qfactory_launch.h"' in src


def test_jit_object_with_the_norm_prologue_exports_launch_norm():
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import AsymQTile, QTile
    from qfactory.jit import jit
    assert _declared_functions("qfactory_launch.h", "QF_LAUNCH_NORM") == ["launch_norm"]
    qfunc = QMatmulQFunc(QTile((1, 512), torch.float16, 16), AsymQTile((64, 512), torch.int8, 4, (1, 128)), "nt")
    qfunc.input_prologue = "add_rmsnorm"
    runtime = jit.compile(qfunc)
    lib = ctypes.CDLL(os.path.join(runtime.path, "kernel.so"))
    for name in _declared_functions("qfactory_launch.h", "QF_LAUNCH_GROUPED") + ["launch_norm"]:
        assert hasattr(lib, name), f"{name} missing from {runtime.path}"
    assert runtime._launch_norm is not None and "prologue=add_rmsnorm" in runtime.description
    src = open(os.path.join(runtime.path, "kernel.hip")).read()
    assert "#define QF_LAUNCH_NORM" in src and "#define QF_GEMV_NORM_PROLOGUE 1" in src
    # the prologue is the dot2 GEMV kernel's: a matrix-core problem refuses it
    wide = QMatmulQFunc(QTile((64, 512), torch.float16, 16), AsymQTile((64, 512), torch.int8, 4, (1, 128)), "nt")
    wide.input_prologue = "add_rmsnorm"
    with pytest.raises(AssertionError):
        wide.emit()


def test_jit_object_that_uses_scratch_memory_exports_the_entry_point_that_allocates_nothing():
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import AsymQTile, QTile
    from qfactory.jit import jit
    assert _declared_functions("qfactory_launch.h", "QF_LAUNCH_STATIC") == ["launch_m_static"]
    split = QMatmulQFunc(QTile((16, 8192), torch.float16, 16), AsymQTile((64, 8192), torch.int8, 4, (1, 128)), "nt")
    assert split.tiling_configs["KS"] == 2
    runtime = jit.compile(split)
    lib = ctypes.CDLL(os.path.join(runtime.path, "kernel.so"))
    for name in _declared_functions("qfactory_launch.h", "QF_LAUNCH_GROUPED") + ["launch_m_static"]:
        assert hasattr(lib, name), f"{name} missing from {runtime.path}"
    assert runtime._launch_m_static is not None and "KS=2" in runtime.description
    src = open(os.path.join(runtime.path, "kernel.hip")).read()
    assert "#define QF_LAUNCH_STATIC" in src and "static __device__ __align__(256) unsigned char scratch[" in src
    assert "hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch))" in src
    # ... and only such an object: the others use no device memory of their own, their launch_m allocates nothing
    plain = jit.compile(QMatmulQFunc(QTile((16, 512), torch.float16, 16), AsymQTile((64, 512), torch.int8, 4, (1, 128)), "nt"))
    assert plain._launch_m_static is None and "scratch" not in open(os.path.join(plain.path, "kernel.hip")).read()


def test_add_to_output_epilogue_is_a_header_switch_of_four_kernels():
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import AsymQTile, QTile
    for m, k, regime, split in ((1, 512, "gemv", True), (16, 1024, "mgemv", True), (16, 11008, "skinny", False),
                                (16, 11008, "mgemv", True), (64, 512, "gemm", True)):
        q = QMatmulQFunc(QTile((m, k), torch.float16, 16), AsymQTile((64, k), torch.int8, 4, (1, 128)), "nt", ksplit=split)
        assert q.regime == regime
        q.output_epilogue = "accumulate"
        src = q.emit()
        assert "#define QF_OUT_ACCUMULATE 1" in src and "epilogue=accumulate" in src
        assert ("KS=" in src) == (k == 11008 and split)          # long rows split over blocks keep the epilogue
    bf = QMatmulQFunc(QTile((1, 512), torch.bfloat16, 16), AsymQTile((64, 512), torch.int8, 4, (1, 128)), "nt")
    bf.output_epilogue = "accumulate"
    with pytest.raises(AssertionError):
        bf.emit()


def test_swiglu_epilogue_is_a_header_switch_of_three_kernels():
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import AsymQTile, QTile
    for m, k, regime, define in ((1, 512, "gemv", "QF_GEMV_GATE_UP_SILU"), (16, 1024, "mgemv", "QF_MGEMV_GATE_UP_SILU"),
                                 (64, 512, "gemm", "QF_GEMM_GATE_UP_SILU")):
        q = QMatmulQFunc(QTile((m, k), torch.float16, 16), AsymQTile((64, k), torch.int8, 4, (1, 128)), "nt")
        assert q.regime == regime
        q.output_epilogue = "silu_mul"
        src = q.emit()
        assert f"#define {define} 1" in src and "epilogue=silu_mul" in src
    # neither the streaming kernel nor the A-stationary kernel with its rows split over blocks pairs gate with up
    for split in (False, True):
        long_rows = QMatmulQFunc(QTile((16, 11008), torch.float16, 16), AsymQTile((64, 11008), torch.int8, 4, (1, 128)), "nt",
                                 ksplit=split)
        assert long_rows.regime == ("mgemv" if split else "skinny")
        long_rows.output_epilogue = "silu_mul"
        with pytest.raises(AssertionError):
            long_rows.emit()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from qfactory import native
    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "LIBRARY", str(tmp_path / "absent.so"))
    with pytest.raises(RuntimeError, match="missing"):
        native.load()


def test_built_distribution_carries_headers_and_native_sources(tmp_path):
    """setup.py (the reference ships include/**/* as package data, setup.py:11-23): a built copy of the package holds
    the kernel headers, the sources of libqfactory_hip.so and the C-ABI headers, where the package looks for them."""
    import subprocess
    import sys
    pkg_parent = os.path.join(ROOT, "qfactory-ae_amd")
    build = tmp_path / "build"
    subprocess.run([sys.executable, "setup.py", "-q", "build", "--build-base", str(build)], cwd=pkg_parent, check=True,
                   capture_output=True)
    lib = build / "lib" / "qfactory"
    for rel in ("include/qf_gemv.hip.h", "include/qf_gemm.hip.h", "include/qf_common.hip.h", "csrc/qfactory_hip.hip",
                "csrc/qfactory_decode.hip", "csrc/qf_fastpath.cpp", "abi/qfactory_launch.h", "abi/qfactory_hip.h", "jit/compiler.py", "core/tiling.py",
                "core/gemm_tuned_gfx950.json", "core/gemv_tuned_gfx950.json", "integrations/vllm_qfactory.py"):
        assert (lib / rel).exists(), rel
    probe = ("import qfactory.native as n, qfactory.jit.compiler as c; "
             "print(n.CSRC_DIR); print(n.REPO_INCLUDE); print(c.ABI_INCLUDE_DIR)")
    out = subprocess.run([sys.executable, "-c", probe], cwd=str(tmp_path), check=True, capture_output=True, text=True,
                         env=dict(os.environ, PYTHONPATH=str(build / "lib"))).stdout.split()
    assert out == [str(lib / "csrc"), str(lib / "abi"), str(lib / "abi")]
    import shutil
    shutil.rmtree(os.path.join(pkg_parent, "qfactory.egg-info"), ignore_errors=True)
