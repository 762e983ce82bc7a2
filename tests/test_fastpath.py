"""The allocate-and-launch extension behind ``forward(x)`` (csrc/qf_fastpath.cpp): host glue over the C-ABI
``launch`` of a specialisation.  The reference's forward allocates and launches from Python
(qfactory/qlinear.py:52-61); results must not depend on which of the two host paths enqueued the launch."""
import ctypes
import os

import pytest
import torch

from qfactory import fastpath


@pytest.fixture(scope="module")
def ext():
    fastpath.build()
    module = fastpath.load()
    assert module is not None, "csrc/_qf_fastpath.so did not build or load"
    return module


def test_extension_builds_and_loads_without_a_gpu(ext):
    assert os.path.exists(fastpath.LIBRARY)
    assert hasattr(ext, "BoundLaunch")


def test_a_null_launch_address_is_refused(ext):
    with pytest.raises(ValueError):
        ext.BoundLaunch(0, 0, 0, 0, True, 8, 8, torch.float16, 0)


def test_an_activation_it_was_not_bound_for_is_handed_back(ext):
    """Not on the device, wrong width, wrong type, not contiguous: None, and the launch function is never called."""
    calls = []
    proto = ctypes.CFUNCTYPE(None, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                             ctypes.POINTER(ctypes.c_int))
    fn = proto(lambda *a: calls.append(a))
    bound = ext.BoundLaunch(ctypes.cast(fn, ctypes.c_void_p).value, 0, 0, 0, False, 16, 32, torch.float16, 0)
    for x in (torch.zeros(1, 32, dtype=torch.float16),                  # a host tensor
              torch.zeros(32, dtype=torch.float16),
              torch.zeros(1, 32, dtype=torch.float32)):
        assert bound(x, 0) is None
    with pytest.raises(TypeError):
        bound("not a tensor", 0)
    assert calls == []


def test_switch_turns_it_off(monkeypatch, ext):
    monkeypatch.setenv("QFACTORY_NO_FASTPATH", "1")
    assert fastpath.load() is None
    monkeypatch.delenv("QFACTORY_NO_FASTPATH")
    assert fastpath.load() is ext


def test_an_extension_built_from_another_source_is_not_used(monkeypatch, ext):
    """load() compares the digest the module carries with the source's: a stale build would call launch with
    another argument list."""
    assert ext.source_digest == fastpath.source_digest()
    monkeypatch.setattr(fastpath, "_module", None)
    monkeypatch.setattr(fastpath, "_tried", False)
    monkeypatch.setattr(fastpath, "source_digest", lambda: "0" * 32)
    with pytest.warns(UserWarning, match="another version"):
        assert fastpath.load() is None


FLAGS = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}


def _layer(m, k, n, nbits, gs, sym):
    from qfactory import QLinear
    lin = QLinear.empty(m, k, n, nbits, gs, sym, FLAGS)
    lin.w.random_(-128, 127)
    if gs != -1:
        lin.s.copy_(torch.rand(lin.s.shape, device="cuda") * 0.02 + 0.001)
        if lin.z is not None:
            lin.z.random_(-128, 127)
    return lin


@pytest.mark.gpu
@pytest.mark.parametrize("gs,sym", [(128, False), (128, True), (-1, False)])
def test_forward_gives_the_same_bits_through_either_host_path(ext, gs, sym):
    k, n = 1024, 512
    lin = _layer(1, k, n, 4, gs, sym)
    for m in (1, 2, 5, 16, 40, 0):
        x = torch.randn(m, k, device="cuda").half()
        expect = torch.empty(m, n, device="cuda", dtype=torch.float16)
        if m:                                                        # the reference-style closure over ctypes
            if gs == -1:
                rc = lin.func_for(torch.float16)(x, lin.w, expect)
            else:
                func = lin.func_for(m)
                rc = func(x, lin.w, expect, lin.s) if sym else func(x, lin.w, expect, lin.s, lin.z)
            assert rc == 0
        into = torch.full((m, n), 7.0, device="cuda", dtype=torch.float16)
        assert lin.forward(x, out=into) is into                      # the extension, caller's tensor
        if m:
            from qfactory.qlinear import _m_bucket
            launch = lin._launchers[(_m_bucket(m), torch.float16)] if gs != -1 else lin._launchers[torch.float16]
            assert launch.alloc is not None, "the extension is built but the layer did not bind it"
        got = lin(x)                                                 # the extension, new tensor
        assert got.shape == (m, n) and got.dtype == torch.float16 and got.device == x.device
        assert torch.equal(got, expect) and torch.equal(into, expect)
    if gs != -1:
        # one bound launcher per row-count bucket, however many distinct row counts arrive
        assert len(lin._launchers) == 4
        for m in (3, 4, 7, 9, 13):
            lin(torch.randn(m, k, device="cuda").half())
        assert len(lin._launchers) == 4


@pytest.mark.gpu
def test_forward_on_a_side_stream_and_with_bad_input(ext):
    k, n = 1024, 512
    lin = _layer(1, k, n, 4, 128, False)
    x = torch.randn(1, k, device="cuda").half()
    expect = lin.forward(x, out=torch.empty(1, n, device="cuda", dtype=torch.float16))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        got = lin(x)
    side.synchronize()
    assert torch.equal(got, expect)
    with pytest.raises(AssertionError):
        lin(torch.randn(1, k + 128, device="cuda").half())           # the ctypes path's checks name the problem
    with pytest.raises(AssertionError):
        lin(torch.randn(1, 2 * k, device="cuda").half()[:, ::2])     # not contiguous
    with pytest.raises(AssertionError):
        lin.forward(x, out=torch.empty(1, n + 1, device="cuda", dtype=torch.float16))
    with pytest.raises(AssertionError):
        lin.forward(x, out=torch.empty(1, n, device="cuda", dtype=torch.float32))
