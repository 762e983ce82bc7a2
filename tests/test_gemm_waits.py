"""The GEMM kernel waits for its activation tiles with explicit counts of the vector-memory loads that may
stay in flight.  The counts are computed from how many loads every K-iteration issues, so the compiled code
must really issue them -- also in the last iterations, whose loads (for 128-byte windows past the end of K)
are never used and which a compiler may drop or merge when the K loop has a single trip.  The JIT re-counts
the loads on the ISA of every GEMM object it builds (qfactory/jit/verify.py) and rebuilds with a full drain
when the count does not hold; checked here without a GPU."""
import ctypes
import os
import subprocess

import pytest
import torch


def _gemm_qfunc(M, N, K, nbits, gs):
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import QTile, SymQTile
    q = QMatmulQFunc(QTile((M, K), torch.float16, 16), SymQTile((N, K), torch.int8, nbits, (1, gs)), "nt")
    assert q.regime == "gemm"
    return q


def _isa_of(qfunc, tmp_path):
    from qfactory.jit.compiler import compile_flags, get_hipcc_compiler, include_dirs
    src = tmp_path / "kernel.hip"
    src.write_text(qfunc.emit())
    flags = [f for f in compile_flags("gfx950") if f not in ("-shared", "-fPIC")]
    out = tmp_path / "kernel.s"
    subprocess.run([get_hipcc_compiler()[0], *flags, *[f"-I{d}" for d in include_dirs()], "--cuda-device-only", "-S",
                    str(src), "-o", str(out)], check=True, capture_output=True)
    return out.read_text()


@pytest.mark.parametrize("M,N,K,nbits,gs", [(70, 96, 4096, 4, 32), (70, 96, 4224, 4, 32), (64, 80, 2816, 2, 128), (48, 64, 2816, 3, 64),
                                           (256, 57344, 8192, 4, 128), (64, 22016, 4096, 4, 128), (128, 8192, 28672, 4, 128),
                                           (33, 100, 512, 4, 128), (300, 256, 2048, 4, 128), (40, 96, 2048, 8, 32)])
def test_every_counted_load_is_issued(M, N, K, nbits, gs, tmp_path):
    from qfactory.jit.verify import gemm_waits_hold
    q = _gemm_qfunc(M, N, K, nbits, gs)
    ok, detail = gemm_waits_hold(_isa_of(q, tmp_path), q.tiling_configs["PA"])
    assert ok, detail


@pytest.mark.parametrize("M,N,K,tile", [(256, 57344, 8192, {"BM": 256, "NT32": 1, "WN": 7, "WK": 1, "PA": 3}),
                                        (64, 22016, 4096, {"BM": 64, "NT32": 1, "WN": 3, "WK": 2, "PA": 4}),
                                        (128, 960, 2048, {"BM": 128, "NT32": 2, "WN": 5, "WK": 1, "PA": 4})])
def test_wave_counts_that_do_not_divide_the_activation_tile(M, N, K, tile, tmp_path):
    """Seven (three, five) waves along N: the tile's 1 KB blocks do not split evenly over them, the waves past the
    last block fetch it once more, and every wave still issues the loads its waits count."""
    from qfactory.core import tiling
    from qfactory.jit.verify import gemm_waits_hold
    assert tiling.gemm_valid(tile, K, 4, 128)
    q = _gemm_qfunc(M, N, K, 4, 128)
    q.tiling_configs = dict(tile)
    ok, detail = gemm_waits_hold(_isa_of(q, tmp_path), tile["PA"])
    assert ok, detail


def test_checker_rejects_a_missing_load():
    from qfactory.jit.verify import gemm_waits_hold
    load = "\tglobal_load_dwordx4 v[0:3], v4, s[0:1]"
    iteration = [load] * 3 + ["\ts_waitcnt vmcnt(3) lgkmcnt(0)", "\ts_barrier"]
    def listing(body):
        return "\n".join(["_Z6kernelv:", "\ts_waitcnt vmcnt(0) lgkmcnt(0)"] + body + ["\ts_endpgm", ".Lfunc_end0:"])
    assert gemm_waits_hold(listing(iteration * 4), 3) == (True, "3 counted waits hold on every path")
    dropped = iteration * 2 + iteration[1:] + iteration                           # the compiler dropped one load
    ok, detail = gemm_waits_hold(listing(dropped), 3)
    assert not ok and "allows 3 loads in flight but a path issues only 2" in detail
    # a rotated loop: the latch block (with the wait) is laid out in front of the header; and a branch that
    # skips a load on one path only
    rotated = ["\ts_branch .LBB0_2", ".LBB0_1:", "\ts_waitcnt vmcnt(3) lgkmcnt(0)", ".LBB0_2:"] + [load] * 3 + \
              ["\ts_cbranch_scc1 .LBB0_1"]
    assert gemm_waits_hold(listing(iteration * 2 + rotated), 3)[0]
    skipping = iteration * 2 + [load, "\ts_cbranch_vccnz .LBB0_3", load, ".LBB0_3:", load, "\ts_waitcnt vmcnt(3) lgkmcnt(0)"]
    assert not gemm_waits_hold(listing(skipping), 3)[0]
    assert not gemm_waits_hold("s_endpgm", 3)[0]                                    # no kernel, no counted wait


def test_jit_falls_back_to_a_full_drain_when_the_count_fails(tmp_path, monkeypatch):
    """A GEMM object whose ISA fails the re-count is rebuilt with vmcnt(0) waits; the object says which it is."""
    from qfactory.jit.compiler import JITCompiler
    monkeypatch.setenv("QFACTORY_CACHE_DIR", str(tmp_path))
    q = _gemm_qfunc(40, 64, 1024, 4, 128)

    copies = iter(range(10))

    def describe(runtime):
        # a fresh file name per load: dlopen would hand back the object already loaded under the same path
        copy = tmp_path / f"copy{next(copies)}.so"
        copy.write_bytes(open(os.path.join(runtime.path, "kernel.so"), "rb").read())
        lib = ctypes.CDLL(str(copy))
        lib.qf_describe.restype = ctypes.c_char_p
        return lib.qf_describe().decode()

    jit = JITCompiler()
    assert describe(jit.compile(q, force=True)).endswith("waits=counted")
    jit.check_gemm_waits = staticmethod(lambda isa, pa: (False, "forced by the test"))
    assert describe(jit.compile(q, force=True)).endswith("waits=drain")
    assert not [d for d in os.listdir(tmp_path / "tmp") if d.startswith("temps.")]  # the ISA dump is cleaned up
