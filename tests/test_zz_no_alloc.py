"""launch_m_static, the entry point that allocates nothing: an object that splits K over blocks, called through its C
ABI on its static scratch array, against the same object's launch_m (scratch memory allocated at the first call) --
same bits -- on two calls in a row, the second with fewer rows; then against the oracle."""
import ctypes
import os

import pytest
import torch

import prebuild
from helpers import assert_close

pytestmark = pytest.mark.gpu


def test_the_entry_point_on_static_scratch_memory_gives_launch_m_s_bits(oracle):
    from qfactory.jit import jit
    case = prebuild._case(16, 4096, 11008)
    print("[case] launch_m_static against launch_m, 16 rows then 5", flush=True)
    (qfunc,) = prebuild.qfuncs_of(case)
    runtime = jit.compile(qfunc)
    assert "KS=4" in runtime.description
    # the C ABI itself: the symbols of the shared object through ctypes, raw device addresses
    lib = ctypes.CDLL(os.path.join(runtime.path, "kernel.so"))
    ptr, rc_t = ctypes.c_void_p, ctypes.POINTER(ctypes.c_int)
    for name in ("launch_m", "launch_m_static"):
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = None, [ctypes.c_int, ptr, ptr, ptr, ptr, ptr, ptr, rc_t]
    g = torch.Generator(device="cuda").manual_seed(2024)
    N, K = 4096, 11008
    w = torch.randint(-128, 128, (N, K // 2), dtype=torch.int8, device="cuda", generator=g)
    s = (torch.rand(N, K // 128, device="cuda", generator=g) * 0.019 + 0.001).to(torch.float16)
    z = torch.randint(-128, 128, (N, K // 256), dtype=torch.int8, device="cuda", generator=g)
    A = torch.randn(16, K, device="cuda", generator=g).to(torch.float16)
    stream = torch.cuda.current_stream().cuda_stream

    def call(name, m, out):
        rc = ctypes.c_int(-1)
        getattr(lib, name)(m, A.data_ptr(), w.data_ptr(), out.data_ptr(), s.data_ptr(), z.data_ptr(), stream, ctypes.byref(rc))
        return rc.value

    for m in (16, 5):                                                       # two calls in a row, the second smaller
        want = torch.full((m, N), float("nan"), dtype=torch.float16, device="cuda")
        got = torch.full((m, N), float("nan"), dtype=torch.float16, device="cuda")
        assert call("launch_m", m, want) == 0
        assert call("launch_m_static", m, got) == 0
        torch.cuda.synchronize()
        assert torch.isfinite(got).all() and torch.equal(got, want), f"{m} rows"
        cols = torch.arange(0, N, 16, device="cuda")
        ref = oracle.qlinear_np(A[:m].cpu().numpy(), w[cols].cpu().numpy(), s[cols].cpu().numpy(), z[cols].cpu().numpy(), 4, 128)
        assert_close(oracle, got[:, cols].cpu().numpy(), ref, f"launch_m_static, {m} rows")
    # more rows than the object's scratch memory is sized for: refused on the host
    big = torch.empty(17, N, dtype=torch.float16, device="cuda")
    assert call("launch_m_static", 17, big) == 1
