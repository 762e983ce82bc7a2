"""The GEMM kernel's counted waits against a full drain per K-iteration (QF_GEMM_FULL_DRAIN): same inputs, the
outputs must be bit-identical, on every distinct GEMM tiling the repository prebuilds.  A wait that let a tile
be read too early would show as a difference (the drained build cannot read early)."""
import pytest
import torch

import prebuild

pytestmark = pytest.mark.gpu


def _id(c):
    return f"M{c['M']}-N{c['N']}-K{c['K']}-b{c['NBITS']}-g{c['GS']}-{'sym' if c['sym'] else 'asym'}"


@pytest.mark.parametrize("case", prebuild.drain_cases(), ids=_id)
def test_counted_waits_equal_full_drain(case):
    from qfactory.convert import weight_row_bytes, zero_row_bytes
    from qfactory.jit import jit
    print(f"[case] {_id(case)}", flush=True)
    counted, drained = prebuild.qfuncs_of(case)
    assert counted.regime == "gemm" and drained.defines == {"QF_GEMM_FULL_DRAIN": 1}
    rt_c, rt_d = jit.compile(counted), jit.compile(drained)
    assert rt_c.description.endswith("waits=counted") and rt_d.description.endswith("waits=drain"), rt_c.description
    assert rt_c.description[:-len("counted")] == rt_d.description[:-len("drain")]
    M, N, K, nbits, GS = (case[k] for k in ("M", "N", "K", "NBITS", "GS"))
    m_run = counted.problem["M"]                              # the bucket the object was compiled for
    g = torch.Generator(device="cuda").manual_seed(N + K + M)
    A = torch.randn(m_run, K, device="cuda", generator=g).to(torch.float16)
    w = torch.randint(-128, 128, (N, weight_row_bytes(K, nbits)), dtype=torch.int8, device="cuda", generator=g)
    s = (torch.rand(N, K // GS, device="cuda", generator=g) * 0.019 + 0.001).to(torch.float16)
    z = torch.randint(-128, 128, (N, zero_row_bytes(K // GS, nbits)), dtype=torch.int8, device="cuda", generator=g)
    stream = torch.cuda.current_stream()
    outs = []
    for rt in (rt_c, rt_d, rt_c):
        out = torch.full((m_run, N), float("nan"), dtype=torch.float16, device="cuda")
        assert rt.run(A, w, out, s, z, stream) == 0
        outs.append(out)
    torch.cuda.synchronize()
    assert not torch.isnan(outs[0]).any()
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    assert torch.equal(outs[0].view(torch.int16), outs[2].view(torch.int16))
