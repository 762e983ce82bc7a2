"""``GPTQLinear.forward_add_rmsnorm``: the residual add and RMSNorm of a decoder layer inside the projection that
follows them (dot2 GEMV kernel for M < 3, A-stationary kernel up to 32 rows; the reference's end-to-end runs leave the step to vLLM's fused_add_rms_norm
in front of third_party/vllm-qfactory.patch:205-214).

Checked three ways: the new residual stream equals ``x + delta`` bit for bit; the output is within the acceptance
bar (max-rel 1e-2, nRMS 1e-3, tests/helpers.py) of the CPU oracle's projection of the normalised row, the norm
restated here in float64 with the kernel's two fp16 roundings; and it agrees to nRMS 2e-4 with the two-launch form
(``qf_add_rmsnorm`` then ``forward``), from which it differs only in the order the squares are added, i.e. by one
fp16 ulp on an occasional normalised element."""
import numpy as np
import pytest
import torch

import prebuild
from helpers import assert_close, make_problem, reference_output

pytestmark = pytest.mark.gpu

NO_SEARCH = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}
EPS = 1e-5


def _id(c):
    return (f"M{c['M']}-N{c['N']}-K{c['K']}-b{c['NBITS']}-g{c['GS']}-{'sym' if c['sym'] else 'asym'}"
            + ("-silu" if c.get("epilogue") else ""))


def _normalised(x, delta, gamma):
    """fp16(fp16(h * rsqrt(mean(h^2) + eps)) * gamma) with h = fp16(x + delta), the reduction in float64."""
    h = x if delta is None else (x + delta)                       # fp16 tensors: one rounding
    hd = h.double()
    r = torch.rsqrt(hd.pow(2).mean(-1, keepdim=True) + EPS)
    return h, (hd * r).to(torch.float16) * gamma


@pytest.mark.parametrize("case", prebuild.norm_prologue_cases(), ids=_id)
@pytest.mark.parametrize("with_delta", [True, False], ids=["delta", "nodelta"])
def test_projection_with_residual_add_and_rmsnorm_in_front(oracle, case, with_delta):
    from qfactory import QLinear, native
    from qfactory.qlinear import _m_bucket
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    silu = case.get("epilogue") == "silu_mul"
    print(f"[case] add_rmsnorm {_id(case)} delta={with_delta}", flush=True)
    A, weight, scale, zero = make_problem(77 + N + K + M, M, N, K, nbits, GS, sym)
    if silu:
        scale = scale * (0.1 if nbits == 8 else 4)
    layer = QLinear.init(M, K, N, nbits, weight.cuda(), GS, scale.cuda(), None if zero is None else zero.cuda(),
                         compile_flags=NO_SEARCH)
    g = torch.Generator().manual_seed(5 + K)
    x = (A * 3).cuda()                                                         # residual stream of a few units
    delta = (torch.randn(M, K, generator=g) * 0.7).to(torch.float16).cuda() if with_delta else None
    gamma = (torch.rand(K, generator=g) + 0.5).to(torch.float16).cuda()
    x_before = x.clone()
    x_out = torch.full_like(x, 9.0) if with_delta else None
    assert layer.fuses_add_rmsnorm(M, silu_mul=silu)
    out = layer.forward_add_rmsnorm(x, delta, gamma, EPS, x_out=x_out, silu_mul=silu)
    torch.cuda.synchronize()
    desc = layer._funcs[(_m_bucket(M), torch.float16, "add_rmsnorm+silu_mul" if silu else "add_rmsnorm")].runtime.description
    assert "prologue=add_rmsnorm" in desc and ("regime=gemv" if M < 3 else "regime=mgemv") in desc
    assert ("epilogue=silu_mul" in desc) == silu
    assert out.shape == (M, N // 2 if silu else N) and out.dtype == torch.float16
    assert torch.equal(x, x_before), "the residual stream it reads must stay as it was"
    h, a = _normalised(x, delta, gamma)
    if with_delta:
        assert torch.equal(x_out, h)
    # against the oracle
    ref = torch.from_numpy(reference_output(oracle, a, layer.w, layer.s, layer.z, nbits, GS))
    if silu:
        ref = torch.nn.functional.silu(ref[:, : N // 2].float()).to(torch.float16) * ref[:, N // 2:]
    assert_close(oracle, out.cpu().numpy(), ref.numpy(), _id(case))
    if K > 16384:                                              # qf_add_rmsnorm's own limit on the row length
        return
    # against the two launches it replaces
    hdn = torch.empty_like(x)
    native.add_rmsnorm(h.clone(), None, gamma, hdn, EPS)
    two = layer.forward_silu_mul(hdn) if silu else layer(hdn)
    torch.cuda.synchronize()
    m = oracle.error_metrics(out.cpu().numpy(), two.cpu().numpy())
    assert m["nrms"] <= 2e-4, m
    # the restatement above against qf_add_rmsnorm's rows: a last-place difference of the first rounding on a few
    # elements, which the product with gamma (up to 1.5) can turn into two
    ulp = (hdn.view(torch.int16).int() - a.view(torch.int16).int()).abs()
    assert int(ulp.max()) <= 2 and float((ulp > 0).float().mean()) < 0.02


@pytest.mark.parametrize("case", prebuild.accumulate_cases(), ids=_id)
def test_projection_added_to_the_output_in_place(case):
    """``forward_accumulate``: out = fp16(out + fp16(projection)) -- the kernel's own projection (checked against the
    oracle in tests/test_qlinear_gpu.py) and one fp16 add, so the result equals ``out + layer(x)`` bit for bit."""
    from qfactory import QLinear
    from qfactory.qlinear import _m_bucket
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] accumulate {_id(case)}", flush=True)
    A, weight, scale, zero = make_problem(9 + N + K + M, M, N, K, nbits, GS, sym)
    layer = QLinear.init(M, K, N, nbits, weight.cuda(), GS, scale.cuda(), None if zero is None else zero.cuda(),
                         compile_flags=NO_SEARCH)
    x = A.cuda()
    before = (torch.randn(M, N, generator=torch.Generator().manual_seed(N)) * 4).to(torch.float16).cuda()
    out = before.clone()
    assert layer.forward_accumulate(x, out) is out
    want = before + layer(x)
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    assert layer.fuses_accumulate(M)
    desc = layer._funcs[(_m_bucket(M), torch.float16, "accumulate")].runtime.description
    assert "epilogue=accumulate" in desc and ("regime=gemm" in desc) == (M > 32)
    assert layer.forward_accumulate(x[:0], out[:0]).shape == (0, N)


def test_rows_the_kernel_does_not_take_go_through_two_launches(oracle):
    """More rows than the kernels with the prologue serve: ``qf_add_rmsnorm`` and the projection, same contract."""
    from qfactory import QLinear, native
    M, N, K = 40, 96, 1024
    A, weight, scale, zero = make_problem(11, M, N, K, 4, 128, False)
    layer = QLinear.init(M, K, N, 4, weight.cuda(), 128, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    x, delta = A.cuda(), (A * 0.5).cuda().flip(0).contiguous()
    gamma = torch.ones(K, dtype=torch.float16, device="cuda")
    assert not layer.fuses_add_rmsnorm(M)
    x_out = torch.empty_like(x)
    out = layer.forward_add_rmsnorm(x, delta, gamma, EPS, x_out=x_out)
    h, a = _normalised(x, delta, gamma)
    hdn = torch.empty_like(x)
    native.add_rmsnorm(h.clone(), None, gamma, hdn, EPS)
    assert torch.equal(x_out, h) and torch.equal(out, layer(hdn))
    assert layer.forward_add_rmsnorm(x[:0], None, gamma, EPS).shape == (0, N)


def test_argument_checks():
    from qfactory import QLinear
    M, N, K = 1, 100, 1024
    A, weight, scale, zero = make_problem(3, M, N, K, 4, 128, False)
    layer = QLinear.init(M, K, N, 4, weight.cuda(), 128, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    x, gamma = A.cuda(), torch.ones(K, dtype=torch.float16, device="cuda")
    with pytest.raises(AssertionError):
        layer.forward_add_rmsnorm(x, x.clone(), gamma, EPS)                       # delta without a place for the sum
    with pytest.raises(AssertionError):
        layer.forward_add_rmsnorm(x, x.clone(), gamma, EPS, x_out=x)              # x_out aliases the stream it reads
    with pytest.raises(AssertionError):
        layer.forward_add_rmsnorm(x, None, gamma[:-1].contiguous(), EPS)          # norm weight of the wrong length
    with pytest.raises(AssertionError):
        layer.forward_add_rmsnorm(x, None, gamma.float(), EPS)
    # an object with the prologue answers the plain entry points with 1 (it needs the norm operands)
    from qfactory.qlinear import _m_bucket
    layer.forward_add_rmsnorm(x, None, gamma, EPS)
    runtime = layer._funcs[(_m_bucket(M), torch.float16, "add_rmsnorm")].runtime
    out = torch.empty(M, N, dtype=torch.float16, device="cuda")
    assert runtime.run_raw(M, (x.data_ptr(), layer.w.data_ptr(), out.data_ptr(), layer.s.data_ptr(), layer.z.data_ptr()),
                           torch.cuda.current_stream().cuda_stream) == 1
