"""The GEMM kernel waits for its activation tiles with explicit counts of the vector-memory loads that may
stay in flight.  The counts are computed from how many loads every K-iteration issues, so the compiled code
must really issue them -- also in the last iterations, whose loads (for 128-byte windows past the end of K)
are never used and which a compiler may drop or merge when the K loop has a single trip.  Checked here on
the generated ISA of such a specialisation, without a GPU."""
import os
import re
import subprocess

import pytest
import torch


def _isa_of(qfunc, tmp_path):
    from qfactory.jit.compiler import compile_flags, get_hipcc_compiler
    src = tmp_path / "kernel.hip"
    src.write_text(qfunc.emit())
    flags = compile_flags("gfx950")
    flags = flags.split() if isinstance(flags, str) else list(flags)
    flags = [f for f in flags if f not in ("-shared", "-fPIC")]
    out = tmp_path / "kernel.s"
    from qfactory.jit import compiler
    include = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(compiler.__file__))), "include")
    abi = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    subprocess.run([get_hipcc_compiler()[0], *flags, f"-I{include}", f"-I{abi}", "--cuda-device-only", "-S", str(src), "-o", str(out)],
                   check=True, capture_output=True)
    return out.read_text()


@pytest.mark.parametrize("M,N,K,nbits,gs", [(70, 96, 4096, 4, 32), (70, 96, 4224, 4, 32), (64, 80, 2816, 2, 128), (48, 64, 2816, 3, 64),
                                           (256, 57344, 8192, 4, 128), (64, 22016, 4096, 4, 128), (128, 8192, 28672, 4, 128),
                                           (33, 100, 512, 4, 128), (300, 256, 2048, 4, 128), (40, 96, 2048, 8, 32)])
def test_every_counted_load_is_issued(M, N, K, nbits, gs, tmp_path):
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import QTile, SymQTile
    q = QMatmulQFunc(QTile((M, K), torch.float16, 16), SymQTile((N, K), torch.int8, nbits, (1, gs)), "nt")
    assert q.regime == "gemm"
    pa = q.tiling_configs["PA"]
    isa = _isa_of(q, tmp_path)
    loads_in_segment, segments, checked = 0, [], 0
    for line in isa.splitlines():
        line = line.strip()
        if line.startswith(("global_load", "buffer_load")):
            loads_in_segment += 1
        m = re.match(r"s_waitcnt vmcnt\((\d+)\) lgkmcnt\(0\)", line)
        if m:                                        # the kernel's explicit wait (with or without a block barrier behind it)
            allowed = int(m.group(1))
            segments.append(loads_in_segment)
            loads_in_segment = 0
            if allowed == 0:
                segments = []                        # a full drain (end of the prologue): nothing older is in flight
            elif len(segments) >= pa - 2:
                # the loads of the last PA - 2 iterations may stay in flight: they must all exist
                assert sum(segments[-(pa - 2):]) == allowed, (segments, allowed)
                checked += 1
    assert checked >= 2
