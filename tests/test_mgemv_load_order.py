"""The A-stationary kernel requests its activations and its first weight tile together, before it waits for anything:
the activations first, then the tile's packed words, scales and zero-points.  Left to itself the compiler moves the
scale and zero-point loads of the first tile behind the whole activation phase (they are needed last, and the block
that used them was conditional), which puts a second trip to memory in front of the first MFMA; scheduling barriers in
the header hold the order.  Checked here on the compiled ISA, without a GPU."""
import re
import subprocess

import pytest
import torch


def _isa_of(qfunc, tmp_path):
    from qfactory.jit.compiler import compile_flags, get_hipcc_compiler, include_dirs
    src = tmp_path / "kernel.hip"
    src.write_text(qfunc.emit())
    flags = [f for f in compile_flags("gfx950") if f not in ("-shared", "-fPIC")]
    out = tmp_path / "kernel.s"
    subprocess.run([get_hipcc_compiler()[0], *flags, *[f"-I{d}" for d in include_dirs()], "--cuda-device-only", "-S",
                    str(src), "-o", str(out)], check=True, capture_output=True)
    return out.read_text()


def _events(isa):
    """global loads, vector-memory waits and MFMAs of the kernel, in program order."""
    body = isa[isa.index("mgemv_kernel"):]
    out = []
    for line in body.splitlines():
        m = re.match(r"\s+(global_load_\w+|v_mfma_\w+|s_waitcnt)\s*(.*)", line)
        if not m:
            continue
        if m.group(1) == "s_waitcnt":
            if "vmcnt" in m.group(2):
                out.append("wait")
        else:
            out.append("load" if m.group(1).startswith("global_load") else "mfma")
    return out


@pytest.mark.parametrize("M,N,K,sym", [(16, 22016, 4096, False), (16, 4096, 11008, False), (16, 8192, 8192, True)])
def test_first_tile_is_requested_with_the_activations(M, N, K, sym, tmp_path):
    from qfactory.core import QMatmul
    op = QMatmul(M, N, K, 4, sym, torch.float16, torch.int8, 128)
    op.init_qfuncs()
    q = op.qfuncs[0]
    assert q.regime == "mgemv" and q.tiling_configs["PF"] == 1 and q.tiling_configs["CH"] == 2 and q.tiling_configs["MT16"] == 1
    ev = _events(_isa_of(q, tmp_path))
    first_wait, first_mfma = ev.index("wait"), ev.index("mfma")
    # 16 rows x 2 chunks of 256 bytes = 8 activation loads; 2 loads of packed words, one scale, one zero-point (none when symmetric)
    tile = 2 + 1 + (0 if sym else 1)
    assert ev[:first_wait].count("load") == 8 + tile, ev[:first_wait + 1]
    # ... and what is requested between the first wait and the first MFMA is exactly the second tile
    assert ev[first_wait:first_mfma].count("load") == tile, ev[:first_mfma + 1]
