"""GPU parity of the bf16 path: QLinear on bf16 activations (HIP kernels through the C ABI) against the CPU
oracle's bf16 forward, on seeded inputs, over every kernel family.

The reference takes fp16 only (qfactory/core/matmul.py:36, :133-136), so nothing of its own pins this path.
The acceptance bar (max relative error 1e-2, normalised RMS error 1e-3; definitions in tests/helpers.py) is
stated for fp16 results.  A bf16 result has 8 significant bits: rounding alone moves a value by up to 2^-8
of itself (2^-8 / sqrt(3) RMS at worst), more than the bar.  So the kernel's output is held to

* the bar on the sum plus bf16's own rounding, against the oracle's sums before rounding:
  max-rel <= 1e-2 + 2^-8, nRMS <= sqrt(1e-3^2 + (2^-8 / sqrt(3))^2) = 2.5e-3;
* bit-identity with the oracle's rounded result on at least three quarters of the elements: the two round
  nearly the same sum and differ only where it sits next to a rounding boundary (5 - 10 % of the elements at
  the kernels' fp16-level accuracy); rounding the wrong way (truncation) would move half of them.
"""
import numpy as np
import pytest
import torch

import prebuild
from helpers import MAX_REL_TOL, NRMS_TOL, make_problem

pytestmark = pytest.mark.gpu

NO_SEARCH = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}
MAX_REL_TOL_BF16 = MAX_REL_TOL + 2.0 ** -8
NRMS_TOL_BF16 = float(np.sqrt(NRMS_TOL ** 2 + (2.0 ** -8) ** 2 / 3))
MIN_IDENTICAL = 0.75


def _id(c):
    return f"M{c['M']}-N{c['N']}-K{c['K']}-b{c['NBITS']}-g{c['GS']}-{'sym' if c['sym'] else 'asym'}"


def _bits(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _check(oracle, out_bits, sums, what):
    """out_bits: the kernel's bf16 result; sums: the oracle's float64 sums before the final rounding."""
    out = oracle.bf16_bits_to_f32(out_bits)
    assert np.all(np.isfinite(out)), f"{what}: non-finite output"
    m = oracle.error_metrics(out, sums)
    assert m["max_rel"] <= MAX_REL_TOL_BF16 and m["nrms"] <= NRMS_TOL_BF16, f"{what}: {m}"
    identical = float(np.mean(out_bits == oracle.f32_to_bf16_bits(sums.astype(np.float32))))
    assert identical >= MIN_IDENTICAL, f"{what}: only {identical:.3f} of the outputs equal the oracle's bit for bit"
    return m


@pytest.fixture(scope="module")
def qf():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from qfactory import QLinear
    return QLinear


def _layer(qf, case, weight, scale, zero):
    M, N, K, nbits, GS = (case[k] for k in ("M", "N", "K", "NBITS", "GS"))
    if GS == -1:
        return qf.init(M, K, N, nbits, weight.cuda(), compile_flags={"enable_schedule": False, "enable_lower": False})
    return qf.init(M, K, N, nbits, weight.cuda(), GS, scale.cuda(), None if zero is None else zero.cuda(),
                   compile_flags=NO_SEARCH)


def _reference(oracle, A_bits, layer, nbits, GS):
    w = layer.w.cpu().numpy()
    if GS == -1:
        return oracle.gemv_plain_bf16_np(A_bits, w, nbits, rounded=False)
    z = None if layer.z is None else layer.z.cpu().numpy()
    return oracle.qlinear_bf16_np(A_bits, w, layer.s.cpu().numpy(), z, nbits, GS, rounded=False)


@pytest.mark.parametrize("case", prebuild.bf16_cases(), ids=_id)
def test_bf16_forward_matches_oracle(qf, oracle, case):
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] bf16 {_id(case)}", flush=True)
    A, weight, scale, zero = make_problem(4321 + N + K + M + nbits, M, N, K, nbits, GS, sym)
    layer = _layer(qf, case, weight, scale, zero)
    x = A.float().to(torch.bfloat16).cuda()
    out = layer(x)
    torch.cuda.synchronize()
    assert out.shape == (M, N) and out.dtype == torch.bfloat16 and out.is_cuda
    desc = (layer.func_for(M, torch.bfloat16) if GS != -1 else layer.func_for(torch.bfloat16)).runtime.description
    assert "act=bf16" in desc
    _check(oracle, _bits(out), _reference(oracle, _bits(x), layer, nbits, GS), f"{_id(case)} [{desc}]")
    # the same module still serves fp16 rows with an fp16 result
    out16 = layer(A.cuda())
    assert out16.dtype == torch.float16


@pytest.mark.parametrize("M,K", [(1, 1024), (12, 2048), (64, 1024)], ids=["gemv", "mgemv", "gemm"])
def test_bf16_activations_beyond_fp16_range_saturate(qf, oracle, M, K):
    """Magnitudes above 65504 enter the sum as +-65504 and values below 2^-14 on fp16's subnormal grid, in the
    kernels that convert while loading and in the conversion launch in front of the GEMM kernel alike."""
    N, nbits, GS = 96, 4, 128
    A, weight, scale, zero = make_problem(77 + M, M, N, K, nbits, GS)
    layer = _layer(qf, {"M": M, "N": N, "K": K, "NBITS": nbits, "GS": GS}, weight, scale, zero)
    x = (A.float() * 0.01).to(torch.bfloat16)
    x[0, 3], x[0, 500], x[M - 1, 17], x[M - 1, K - 1] = 1.0e6, -3.0e38, 3.0e-6, -1.0e-7
    out = layer(x.cuda())
    torch.cuda.synchronize()
    ref = _reference(oracle, _bits(x), layer, nbits, GS)
    _check(oracle, _bits(out), ref, f"M={M}")
    # the saturated terms dominate row 0: an unsaturated 1e6 would be off by a factor of fifteen
    assert np.max(np.abs(ref[0])) < 65504 * 0.02 * 16 * 2 + 1000


def test_bf16_closure_checks_dtypes(qf):
    N, K, nbits, GS = 64, 256, 4, 128
    A, weight, scale, zero = make_problem(6, 1, N, K, nbits, GS)
    layer = qf.init(1, K, N, nbits, weight.cuda(), GS, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    func = layer.func_for(1, torch.bfloat16)
    x = A.cuda()
    with pytest.raises(AssertionError):
        func(x, layer.w, torch.empty(1, N, dtype=torch.bfloat16, device="cuda"), layer.s, layer.z)     # fp16 rows
    with pytest.raises(AssertionError):
        func(x.to(torch.bfloat16), layer.w, torch.empty(1, N, dtype=torch.float16, device="cuda"), layer.s, layer.z)


def test_bf16_to_f16_entry_point(oracle):
    from qfactory import native
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    for n in (65536, 65536 - 5, 3):                       # whole 16-byte units, a ragged tail, a tail only
        src = torch.from_numpy(bits[:n].view(np.int16).copy()).view(torch.bfloat16).cuda()
        got = native.bf16_to_f16(src)
        torch.cuda.synchronize()
        got_bits = got.view(torch.int16).cpu().numpy().view(np.uint16)
        want = oracle.bf16_bits_to_f16_sat(bits[:n])
        nan = np.isnan(want)
        assert np.array_equal(got_bits[~nan], want.view(np.uint16)[~nan])
        assert np.all(np.isnan(got.cpu().numpy()[nan]))
