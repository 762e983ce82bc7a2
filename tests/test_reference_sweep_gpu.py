"""The reference's own accuracy sweep (tests/acc_gptq.py, tests/acc_gemv.py) on the MI355X build: every
[N, K, group size] of its shape list (data/nkg_shapes.json, key "all"; a copy is the fixture
tests/golden/nkg_shapes.json), M in {1, 16}, 8 / 4 / 2 bits, default kernel configuration.

Two checks per case: the reference's criterion -- mean squared difference to an fp16 matmul with the
dequantised weights, rounded to four digits, below 0.1 -- and, tighter, the CPU oracle on sampled output
columns of the packed tensors.  Inputs follow the reference's generator (per-group min/max quantisation of
a random fp16 weight), seeded here."""
import json
import os

import numpy as np
import pytest
import torch

import prebuild
from conftest import ROOT
from helpers import assert_close

pytestmark = pytest.mark.gpu
NO_SEARCH = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}


def _id(c):
    return f"M{c['M']}-N{c['N']}-K{c['K']}-b{c['NBITS']}-g{c['GS']}"


def test_shape_list_is_the_reference_s():
    shapes = json.load(open(os.path.join(ROOT, "tests", "golden", "nkg_shapes.json")))
    assert prebuild.REFERENCE_SHAPES == shapes["all"]
    for model, rows in shapes.items():                      # every model's shapes are part of "all" or are the synthetic squares
        if model.startswith(("llama", "qwen")):
            assert all(r in shapes["all"] for r in rows)


def _minmax_quant(weight, GS, nbits):
    """Per group of GS rows and per column: scale = (max - min) / (2^b - 1), zero = trunc(-min / (max - min) *
    (2^b - 1) - 1) clamped at 0, q = trunc((w - min) / (max - min) * (2^b - 1)); fp16 arithmetic as in
    acc_gptq.py:10-29."""
    K, N = weight.shape
    g = weight.reshape(K // GS, GS, N)
    mx, mn = g.max(dim=1).values, g.min(dim=1).values
    qr = 2 ** nbits - 1
    scales = ((mx - mn) / qr).to(torch.float16)
    zeros = (-mn / (mx - mn) * qr - 1).clamp(min=0).to(torch.int32)
    q = ((g - mn[:, None]) / (mx - mn)[:, None] * qr).to(torch.int32).reshape(K, N)
    return q, scales, zeros


@pytest.mark.parametrize("case", [c for c in prebuild.reference_sweep_cases() if c["GS"] != -1], ids=_id)
def test_grouped_sweep(oracle, case):
    from qfactory import QLinear
    M, N, K, nbits, GS = (case[k] for k in ("M", "N", "K", "NBITS", "GS"))
    print(f"[case] {_id(case)}", flush=True)
    gen = torch.Generator(device="cuda").manual_seed(N * 7 + K * 3 + M + nbits)
    activation = torch.randn(M, K, device="cuda", generator=gen).to(torch.float16)
    weight = torch.randn(K, N, device="cuda", generator=gen).to(torch.float16)
    qweight, scales, zeros = _minmax_quant(weight, GS, nbits)
    del weight
    idx = torch.arange(K, device="cuda") // GS
    dequant_w = ((qweight - (zeros[idx] + 1)) * scales[idx]).to(torch.float16)       # acc_gptq.py:31-38
    quant_output = activation @ dequant_w
    del dequant_w
    layer = QLinear.init(M, K, N, nbits, qweight, GS, scales, zeros, compile_flags=NO_SEARCH)
    del qweight
    out = layer(activation)
    torch.cuda.synchronize()
    assert out.shape == (M, N) and out.dtype == torch.float16
    q_err = round(((quant_output.float() - out.float()) ** 2).mean().item(), 4)
    assert q_err < 0.1, q_err                                                        # acc_gptq.py:61-62
    rows = np.sort(np.random.default_rng(N + K).choice(N, size=min(N, 256), replace=False))
    rows_t = torch.from_numpy(rows).cuda()
    ref = oracle.qlinear_np(activation.cpu().numpy(), layer.w[rows_t].cpu().numpy(), layer.s[rows_t].cpu().numpy(),
                            layer.z[rows_t].cpu().numpy(), nbits, GS)
    assert_close(oracle, out[:, rows_t].cpu().numpy(), ref, _id(case))


@pytest.mark.parametrize("case", [c for c in prebuild.reference_sweep_cases() if c["GS"] == -1], ids=_id)
def test_plain_integer_sweep(oracle, case):
    from qfactory import QLinear
    M, N, K, nbits = (case[k] for k in ("M", "N", "K", "NBITS"))
    print(f"[case] {_id(case)}", flush=True)
    gen = torch.Generator(device="cuda").manual_seed(N * 5 + K + M + nbits)
    activation = torch.randn(M, K, device="cuda", generator=gen).to(torch.float16)
    weight = torch.randint(0, 2 ** nbits, (K, N), dtype=torch.int32, device="cuda", generator=gen)
    output = activation @ weight.to(torch.float16)                                   # acc_gemv.py:12-14
    layer = QLinear.init(M, K, N, nbits, weight, compile_flags={"enable_schedule": False, "enable_lower": False})
    del weight
    out = layer(activation)
    torch.cuda.synchronize()
    # 8-bit sums reach 1e4: the reference's absolute criterion (acc_gemv.py:18-19) is applied to finite outputs only,
    # as it would be there (an overflowing fp16 matmul reads inf on both sides)
    finite = torch.isfinite(output) & torch.isfinite(out)
    q_err = round(((output.float() - out.float())[finite] ** 2).mean().item(), 4)
    rows = np.sort(np.random.default_rng(N + K).choice(N, size=min(N, 256), replace=False))
    rows_t = torch.from_numpy(rows).cuda()
    ref = oracle.gemv_plain_np(activation.cpu().numpy(), layer.w[rows_t].cpu().numpy(), nbits)
    got = out[:, rows_t].cpu().numpy()
    # 8-bit fields over K > 27000 reach past the fp16 range: such outputs must be the same infinity on both sides
    big = ~np.isfinite(ref)
    assert np.array_equal(got[big], ref[big])
    assert_close(oracle, np.where(big, np.float16(0), got), np.where(big, np.float16(0), ref), _id(case))
    # the oracle bound is the binding one; the reference's own figure is reported for the record
    print(f"  reference criterion (MSE to the fp16 matmul, rounded): {q_err}")
