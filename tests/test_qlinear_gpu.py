"""GPU parity: QLinear (HIP kernels through the C ABI) against the CPU oracle on seeded inputs.

Tolerances are the acceptance bar: max relative error <= 1e-2 and normalised RMS error <= 1e-3 in
fp16 (definitions in tests/helpers.py); packed tensors must equal the oracle's bit for bit.
"""
import numpy as np
import pytest
import torch

import prebuild
from helpers import assert_close, make_problem, reference_output

pytestmark = pytest.mark.gpu

NO_SEARCH = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}


def _id(c):
    return f"M{c['M']}-N{c['N']}-K{c['K']}-b{c['NBITS']}-g{c['GS']}-{'sym' if c['sym'] else 'asym'}"


@pytest.fixture(scope="module")
def qf():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from qfactory import QLinear
    return QLinear


def _unique(cases):
    seen, out = set(), []
    for c in cases:
        key = tuple(sorted(c.items()))
        if key not in seen:
            seen.add(key)
            out.append(c)
    return out


@pytest.mark.parametrize("case", _unique(prebuild.parity_cases() + prebuild.grid_cases()), ids=_id)
def test_qlinear_matches_oracle(qf, oracle, case):
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] {_id(case)}", flush=True)
    A, weight, scale, zero = make_problem(1234 + N + K + M + nbits, M, N, K, nbits, GS, sym)
    dev = "cuda"
    if GS == -1:
        layer = qf.init(M, K, N, nbits, weight.to(dev), compile_flags={"enable_schedule": False, "enable_lower": False})
        s = z = None
    else:
        layer = qf.init(M, K, N, nbits, weight.to(dev), GS, scale.to(dev),
                        None if zero is None else zero.to(dev), compile_flags=NO_SEARCH)
        s, z = layer.s, layer.z
    # repacked tensors: bit-exact against the oracle's packer
    assert np.array_equal(layer.w.cpu().numpy(), oracle.pack_weight(weight.numpy(), nbits))
    if GS != -1:
        assert np.array_equal(s.cpu().numpy(), oracle.transpose_scale(scale.numpy()))
        if not sym:
            assert np.array_equal(z.cpu().numpy(), oracle.pack_zero(zero.numpy(), nbits))
    out = layer(A.to(dev))
    torch.cuda.synchronize()
    assert out.shape == (M, N) and out.dtype == torch.float16 and out.is_cuda
    # big problems: check a seeded subset of output columns (each is an independent dot product)
    rows = None
    if N * K * M > 2 ** 31:
        rows = np.sort(np.random.default_rng(0).choice(N, size=2048, replace=False))
    ref = reference_output(oracle, A, layer.w, s, z, nbits, GS, rows)
    got = out.cpu().numpy()
    assert_close(oracle, got if rows is None else got[:, rows], ref, _id(case))


@pytest.mark.parametrize("case", prebuild.large_parity_cases(), ids=_id)
def test_large_gemm_matches_oracle_on_sampled_columns(qf, oracle, case):
    """Llama-3-70B-style shapes at M = 32..256: packed tensors are filled directly with seeded
    random bytes (any byte pattern is a valid packed weight / zero tensor); 1024 seeded output
    columns are checked against the oracle -- every output column is an independent dot product."""
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] {_id(case)}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(N + K + M)
    layer = qf.empty(M, K, N, nbits, GS, sym=sym, compile_flags=NO_SEARCH)
    layer.w.copy_(torch.randint(-128, 128, layer.w.shape, dtype=torch.int8, device="cuda", generator=g))
    layer.s.copy_((torch.rand(layer.s.shape, device="cuda", generator=g) * 0.019 + 0.001).to(torch.float16))
    if not sym:
        layer.z.copy_(torch.randint(-128, 128, layer.z.shape, dtype=torch.int8, device="cuda", generator=g))
    A = torch.randn(M, K, device="cuda", generator=g).to(torch.float16)
    out = layer(A)
    torch.cuda.synchronize()
    rows = np.sort(np.random.default_rng(N + M).choice(N, size=1024, replace=False))
    rows_t = torch.from_numpy(rows).cuda()
    ref = oracle.qlinear_np(A.cpu().numpy(), layer.w[rows_t].cpu().numpy(), layer.s[rows_t].cpu().numpy(),
                            None if sym else layer.z[rows_t].cpu().numpy(), nbits, GS)
    assert_close(oracle, out[:, rows_t].cpu().numpy(), ref, _id(case))


def test_output_is_fully_overwritten_and_deterministic(qf, oracle):
    M, N, K, nbits, GS = 1, 100, 256, 4, 128
    A, weight, scale, zero = make_problem(99, M, N, K, nbits, GS)
    layer = qf.init(M, K, N, nbits, weight.cuda(), GS, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    x = A.cuda()
    first = layer(x).clone()
    # call the closure on a poisoned output buffer: every element must be rewritten
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    rc = layer.func(x, layer.w, out, layer.s, layer.z)
    torch.cuda.synchronize()
    assert rc == 0 and torch.equal(out, first)


def test_forward_with_other_row_counts_than_constructed(qf, oracle):
    # the module is built for batch 1 and then fed 1, 2, 3 and 6 rows
    N, K, nbits, GS = 96, 512, 4, 128
    _, weight, scale, zero = make_problem(5, 1, N, K, nbits, GS)
    layer = qf.init(1, K, N, nbits, weight.cuda(), GS, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    for M in (1, 2, 3, 6):
        A = torch.randn(M, K, generator=torch.Generator().manual_seed(M)).to(torch.float16)
        out = layer(A.cuda())
        ref = reference_output(oracle, A, layer.w, layer.s, layer.z, nbits, GS)
        assert_close(oracle, out.cpu().numpy(), ref, f"M={M}")


def test_forward_without_rows_returns_an_empty_result(qf):
    N, K, nbits, GS = 96, 512, 4, 128
    _, weight, scale, zero = make_problem(5, 1, N, K, nbits, GS)
    layer = qf.init(1, K, N, nbits, weight.cuda(), GS, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    for dtype in (torch.float16, torch.bfloat16):
        out = layer(torch.empty(0, K, dtype=dtype, device="cuda"))
        assert out.shape == (0, N) and out.dtype == dtype
    assert layer.forward_silu_mul(torch.empty(0, K, dtype=torch.float16, device="cuda")).shape == (0, N // 2)
    plain = qf.init(1, K, N, nbits, weight.cuda(), compile_flags={"enable_schedule": False, "enable_lower": False})
    assert plain(torch.empty(0, K, dtype=torch.float16, device="cuda")).shape == (0, N)


def test_closure_rejects_bad_tensors(qf):
    N, K, nbits, GS = 64, 256, 4, 128
    A, weight, scale, zero = make_problem(6, 1, N, K, nbits, GS)
    layer = qf.init(1, K, N, nbits, weight.cuda(), GS, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    out = torch.empty(1, N, dtype=torch.float16, device="cuda")
    x = A.cuda()
    with pytest.raises(AssertionError):
        layer.func(x.float(), layer.w, out, layer.s, layer.z)            # dtype
    with pytest.raises(AssertionError):
        layer.func(x[:, :128], layer.w, out, layer.s, layer.z)           # K mismatch
    with pytest.raises(AssertionError):
        layer.func(x, layer.w.T, out, layer.s, layer.z)                  # shape / contiguity
    with pytest.raises(NotImplementedError):
        qf.init(1, K, N, nbits, weight.cuda(), GS, scale.cuda(), zero.cuda(), bias=True)


def test_forward_fast_path_checks_what_changes_per_call(qf, oracle):
    """``forward`` validates the layer's packed tensors once and then only the activation and the output; a bad
    activation still fails the reference's checks, ``out=`` is written in place, and replacing a packed tensor
    of the layer rebinds the launch."""
    N, K, nbits, GS = 96, 512, 4, 128
    A, weight, scale, zero = make_problem(8, 3, N, K, nbits, GS)
    layer = qf.init(1, K, N, nbits, weight.cuda(), GS, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    plain = qf.init(1, K, N, nbits, weight.cuda(), compile_flags={"enable_schedule": False, "enable_lower": False})
    x = A.cuda()
    for mod, ref in ((layer, reference_output(oracle, A, layer.w, layer.s, layer.z, nbits, GS)),
                     (plain, reference_output(oracle, A, plain.w, None, None, nbits, -1))):
        first = mod(x)
        buf = torch.full((3, N), float("nan"), dtype=torch.float16, device="cuda")
        assert mod(x, out=buf) is buf and torch.equal(buf, first)
        assert_close(oracle, buf.cpu().numpy(), ref, "out=")
        assert torch.equal(mod(x), first)                                  # the cached launcher, second call
        with pytest.raises(AssertionError):
            mod(x[:, :256])                                                # K mismatch (and not contiguous)
        with pytest.raises(AssertionError):
            mod(x.T.contiguous().T)                                        # right shape, wrong strides
        with pytest.raises(AssertionError):
            mod(x, out=torch.empty(3, N + 1, dtype=torch.float16, device="cuda"))
        with pytest.raises(AssertionError):
            mod(x, out=torch.empty(3, N, dtype=torch.bfloat16, device="cuda"))
        with pytest.raises(AssertionError):
            mod(A)                                                         # a host tensor
    # replacing a packed tensor of the layer: the next call uses the new one
    before = layer(x).clone()
    layer.s = (layer.s * 2).contiguous()
    torch.cuda.synchronize()
    after = layer(x)
    assert not torch.equal(after, before)
    assert_close(oracle, after.cpu().numpy(), reference_output(oracle, A, layer.w, layer.s, layer.z, nbits, GS), "rebound")


@pytest.mark.parametrize("M", [1, 16, 64])
def test_reference_launch_symbol_through_plain_ctypes(qf, oracle, M):
    """The reference-shaped entry point `launch(act, weight, out, scale, zero, stream, &rc)` (compile-time
    M), bound the way the reference's loader binds it (qfactory/jit/runtime.py:37-49): a bare CDLL, void
    pointers and an int by reference -- no helper of this package between the test and the C ABI."""
    import ctypes
    import os
    N, K, nbits, GS = 384, 1024, 4, 128
    A, weight, scale, zero = make_problem(77 + M, M, N, K, nbits, GS, False)
    layer = qf.init(M, K, N, nbits, weight.cuda(), GS, scale.cuda(), zero.cuda(), compile_flags=NO_SEARCH)
    lib = ctypes.CDLL(os.path.join(layer.func.runtime.path, "kernel.so"))
    x = A.cuda()
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    rc = ctypes.c_int(-1)
    args = [ctypes.c_void_p(t.data_ptr()) for t in (x, layer.w, out, layer.s, layer.z)]
    lib.launch.restype = None
    lib.launch(*args, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), ctypes.byref(rc))
    torch.cuda.synchronize()
    assert rc.value == 0
    ref = reference_output(oracle, A, layer.w, layer.s, layer.z, nbits, GS)
    assert_close(oracle, out.cpu().numpy(), ref, f"launch M={M}")


@pytest.mark.parametrize("M,N,K,nbits", [(256, 8192, 8192, 4), (256, 57344, 8192, 4), (128, 10240, 8192, 4),
                                         (16, 4096, 11008, 4), (16, 8192, 8192, 8)])
def test_repeated_launches_give_identical_bits(qf, M, N, K, nbits):
    """The GEMM kernel publishes activation tiles with explicit load-count waits and bare barriers, the
    skinny kernel reduces through alternating LDS slots behind a bare barrier: a missed wait would show
    as a launch-to-launch difference.  Every reduction order is fixed, so 30 launches over cold and warm
    caches must agree bit for bit."""
    print(f"[case] repeat M{M}-N{N}-K{K}-b{nbits}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(7 + N + K + M)
    layer = qf.empty(M, K, N, nbits, 128, sym=False, compile_flags=NO_SEARCH)
    layer.w.copy_(torch.randint(-128, 128, layer.w.shape, dtype=torch.int8, device="cuda", generator=g))
    layer.s.copy_((torch.rand(layer.s.shape, device="cuda", generator=g) * 0.019 + 0.001).to(torch.float16))
    layer.z.copy_(torch.randint(-128, 128, layer.z.shape, dtype=torch.int8, device="cuda", generator=g))
    A = torch.randn(M, K, device="cuda", generator=g).to(torch.float16)
    first = layer(A).clone()
    scrub = torch.empty(64 << 20, dtype=torch.int8, device="cuda")
    for i in range(30):
        if i % 3 == 0:
            scrub.fill_(i)                        # push the operands out of L2 now and then
        out = layer(A)
        assert torch.equal(out, first), f"launch {i} differs"


@pytest.mark.parametrize("case", prebuild.silu_mul_cases() + [dict(prebuild._case(16, 112, 1024, 4, 128), epilogue="silu_mul")], ids=_id)
def test_gate_up_projection_with_swiglu_epilogue(qf, oracle, case):
    """``forward_silu_mul`` of a fused gate+up projection: in the kernel's epilogue (one launch; dot2 GEMV,
    A-stationary and GEMM kernels), through ``qf_silu_mul`` otherwise (gate and up not whole 16-row tiles of
    the A-stationary kernel); both equal ``silu_mul(forward(x))`` bit for bit, and
    fp16(silu(gate)) * up formed with PyTorch ops from the oracle's projection."""
    from qfactory import native
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] silu_mul {_id(case)}", flush=True)
    A, weight, scale, zero = make_problem(321 + N + K + M, M, N, K, nbits, GS, sym)
    if scale is not None:
        scale = scale * (0.1 if nbits == 8 else 4)             # projections of a few units: SiLU across its bend, products in range
    layer = qf.init(M, K, N, nbits, weight.cuda(), GS, scale.cuda(), None if zero is None else zero.cuda(),
                    compile_flags=NO_SEARCH)
    x = A.cuda()
    out = layer.forward_silu_mul(x)
    proj = layer(x)
    torch.cuda.synchronize()
    assert out.shape == (M, N // 2) and out.dtype == torch.float16
    assert layer.fuses_silu_mul(M) == (M < 3 or N % 32 == 0)
    if layer.fuses_silu_mul(M):
        from qfactory.qlinear import _m_bucket
        desc = layer._funcs[(_m_bucket(M), torch.float16, "silu_mul")].runtime.description
        assert "epilogue=silu_mul" in desc and ("regime=gemv" if M < 3 else "regime=mgemv" if M <= 32 else "regime=gemm") in desc
    if (N // 2) % 8 == 0:                                      # qf_silu_mul works in units of eight columns
        assert torch.equal(out, native.silu_mul(proj, torch.empty(M, N // 2, dtype=torch.float16, device="cuda")))
    ref = torch.from_numpy(reference_output(oracle, A, layer.w, layer.s, layer.z, nbits, GS))
    want = torch.nn.functional.silu(ref[:, : N // 2].float()).to(torch.float16) * ref[:, N // 2:]
    # the projection itself is within the bar of the oracle (tested above); here the product of two such values
    assert_close(oracle, out.cpu().numpy(), want.numpy(), _id(case))


@pytest.mark.parametrize("case", prebuild.smem_quant_cases(), ids=_id)
def test_gemv_with_scales_through_lds(oracle, case):
    """The schedule search's other choice for the dot2 GEMV kernel (``smem_quant``, the reference's SMEM_QUANT):
    scales and zero-points of a block's rows staged through LDS.  Same results as the default to the bar."""
    from qfactory.convert import convert_params
    from qfactory.core import QMatmul
    from qfactory.jit import jit
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] smem_quant {_id(case)}", flush=True)
    A, weight, scale, zero = make_problem(555 + N + K + M, M, N, K, nbits, GS, sym)
    w, s, z = convert_params({"K": K, "N": N, "NBITS": nbits, "GS": GS},
                             (weight.cuda(), scale.cuda(), None if zero is None else zero.cuda()))
    op = QMatmul(M, N, K, nbits, sym, torch.float16, torch.int8, GS)
    op.init_qfuncs()
    qfunc = op.qfuncs[0].clone(smem_quant=True)
    assert qfunc.regime == "gemv"
    func = op._wrap(jit.compile(qfunc), qfunc)
    assert "smem_quant=1" in func.runtime.description
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    rc = func(A.cuda(), w, out, s) if sym else func(A.cuda(), w, out, s, z)
    torch.cuda.synchronize()
    assert rc == 0
    ref = reference_output(oracle, A, w, s, z, nbits, GS)
    assert_close(oracle, out.cpu().numpy(), ref, _id(case))


@pytest.mark.parametrize("case", prebuild.eager_cases(), ids=_id)
def test_the_other_decode_strategy(oracle, case):
    """``transform()`` (the reference's decode-strategy dimension, qfactory/core/qfunc.py:85-91): where a kernel family
    implements both strategies, the non-default one computes the same linear to the bar."""
    from qfactory.convert import convert_params
    from qfactory.core import QMatmul
    from qfactory.jit import jit
    from qfactory.qlinear import _m_bucket
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] decode=eager {_id(case)}", flush=True)
    A, weight, scale, zero = make_problem(777 + N + K + M, M, N, K, nbits, GS, sym)
    w, s, z = convert_params({"K": K, "N": N, "NBITS": nbits, "GS": GS},
                             (weight.cuda(), scale.cuda(), None if zero is None else zero.cuda()))
    op = QMatmul(_m_bucket(M), N, K, nbits, sym, torch.float16, torch.int8, GS)
    op.init_qfuncs()
    variants = op.qfuncs[0].transform()
    assert [v.decode_strategy for v in variants] == ["deferred", "eager"]
    outs = []
    for qfunc in variants:
        func = op._wrap(jit.compile(qfunc), qfunc)
        assert f"decode={qfunc.decode_strategy}" in func.runtime.description
        out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
        rc = func(A.cuda(), w, out, s) if sym else func(A.cuda(), w, out, s, z)
        torch.cuda.synchronize()
        assert rc == 0
        outs.append(out.cpu().numpy())
    ref = reference_output(oracle, A, w, s, z, nbits, GS)
    for out, qfunc in zip(outs, variants):
        assert_close(oracle, out, ref, f"{_id(case)} decode={qfunc.decode_strategy}")
    assert not np.array_equal(outs[0], outs[1]) or M * N < 64          # two different computations, not one object twice


@pytest.mark.parametrize("case", prebuild.odd_wave_cases(), ids=_id)
def test_gemm_with_wave_counts_that_do_not_divide_the_activation_tile(oracle, case):
    """3, 5, 6 or 7 waves along N (57344 columns are 256 tiles of 7 x 32: one per CU): the tiling is pinned, the
    object is called through its ``launch_m`` and checked against the oracle like any other."""
    from qfactory.jit import jit
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    tile = dict(case["tiling"])
    print(f"[case] gemm {_id(case)} {tile}", flush=True)
    from qfactory import QLinear
    A, weight, scale, zero = make_problem(4321 + N + K + M, M, N, K, nbits, GS, sym)
    layer = QLinear.init(M, K, N, nbits, weight.cuda(), GS, scale.cuda(), None if zero is None else zero.cuda(),
                         compile_flags=NO_SEARCH)
    (qfunc,) = prebuild.qfuncs_of(case)
    assert qfunc.regime == "gemm" and qfunc.tiling_configs == tile
    runtime = jit.compile(qfunc)
    assert all(f"{k}={v}" in runtime.description for k, v in tile.items())
    x = A.cuda()
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    z = layer.z if layer.z is not None else torch.empty(1, dtype=torch.int8, device="cuda")
    rc = runtime.run_raw(M, (x.data_ptr(), layer.w.data_ptr(), out.data_ptr(), layer.s.data_ptr(), z.data_ptr()),
                         torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0
    ref = reference_output(oracle, A, layer.w, layer.s, layer.z, nbits, GS)
    assert_close(oracle, out.cpu().numpy(), ref, _id(case))
    # the default tiling of the same problem gives the same values up to the order of the fp32 sums
    assert ((out.float() - layer(x).float()).norm() / layer(x).float().norm()).item() <= 5e-4
