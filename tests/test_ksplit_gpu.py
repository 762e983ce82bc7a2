"""GPU parity of the A-stationary kernel with K split over blocks (long rows at 3 .. 16 activation rows: the blocks
meet through scratch memory in device memory) and of the kernels that serve the same shapes without the split.

The split is the default of these shapes, so tests/test_qlinear_gpu.py, test_bf16_gpu.py, test_norm_prologue_gpu.py
and the decode tests already run it on their long rows; here: its other block counts and shapes, what is special
about it (state kept between launches: the slots in which pairs of blocks exchange their sums, empty between
launches; a result that must not depend on which block of a pair arrives first), and the unsplit kernels, which
remain what a layer with the norm prologue or the SwiGLU epilogue is built on."""
import numpy as np
import pytest
import torch

import prebuild
from helpers import assert_close, make_problem, reference_output

pytestmark = pytest.mark.gpu

NO_SEARCH = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}


def _id(c):
    return f"M{c['M']}-N{c['N']}-K{c['K']}-b{c['NBITS']}-g{c['GS']}-{'sym' if c['sym'] else 'asym'}"


def _filled_layer(case, seed):
    """A layer whose packed tensors are seeded random bytes (every byte pattern is a valid packed weight)."""
    from qfactory import QLinear
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    g = torch.Generator(device="cuda").manual_seed(seed)
    layer = QLinear.empty(M, K, N, nbits, GS, sym=sym, compile_flags=NO_SEARCH)
    layer.w.copy_(torch.randint(-128, 128, layer.w.shape, dtype=torch.int8, device="cuda", generator=g))
    layer.s.copy_((torch.rand(layer.s.shape, device="cuda", generator=g) * 0.019 + 0.001).to(torch.float16))
    if not sym:
        layer.z.copy_(torch.randint(-128, 128, layer.z.shape, dtype=torch.int8, device="cuda", generator=g))
    return layer, g


def _oracle_columns(oracle, layer, A, cols, nbits, GS):
    cols_t = torch.from_numpy(cols).cuda()
    return oracle.qlinear_np(A.cpu().numpy(), layer.w[cols_t].cpu().numpy(), layer.s[cols_t].cpu().numpy(),
                             None if layer.z is None else layer.z[cols_t].cpu().numpy(), nbits, GS)


@pytest.mark.parametrize("case", prebuild.split_cases(), ids=_id)
def test_split_rows_match_oracle(oracle, case):
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] split {_id(case)}", flush=True)
    layer, g = _filled_layer(case, N + K + M)
    assert "KS=" in layer.func.runtime.description, layer.func.runtime.description
    A = torch.randn(M, K, device="cuda", generator=g).to(torch.float16)
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    layer(A, out=out)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()                                        # every element written
    cols = np.sort(np.random.default_rng(N + M).choice(N, size=min(N, 512), replace=False))
    assert_close(oracle, out[:, torch.from_numpy(cols).cuda()].cpu().numpy(), _oracle_columns(oracle, layer, A, cols, nbits, GS), _id(case))


@pytest.mark.parametrize("case", prebuild.unsplit_cases(), ids=_id)
def test_long_rows_without_the_split(oracle, case):
    """The kernels these shapes run on when K is not split over blocks, built explicitly and called through launch_m."""
    from qfactory.convert import convert_params
    from qfactory.jit import jit
    M, N, K, nbits, GS, sym = (case[k] for k in ("M", "N", "K", "NBITS", "GS", "sym"))
    print(f"[case] unsplit {_id(case)}", flush=True)
    (qfunc,) = prebuild.qfuncs_of(case)
    assert qfunc.tiling_configs.get("KS", 1) == 1 and qfunc.regime in ("skinny", "mgemv", "gemm", "gemv")
    runtime = jit.compile(qfunc)
    assert "KS=" not in runtime.description
    A, weight, scale, zero = make_problem(2468 + N + K + M, M, N, K, nbits, GS, sym)
    w, s, z = convert_params({"K": K, "N": N, "NBITS": nbits, "GS": GS},
                             (weight.cuda(), scale.cuda(), None if zero is None else zero.cuda()))
    x = A.cuda()
    out = torch.full((M, N), float("nan"), dtype=torch.float16, device="cuda")
    zp = z if z is not None else torch.empty(1, dtype=torch.int8, device="cuda")
    rc = runtime.run_raw(M, (x.data_ptr(), w.data_ptr(), out.data_ptr(), s.data_ptr(), zp.data_ptr()),
                         torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0
    assert_close(oracle, out.cpu().numpy(), reference_output(oracle, A, w, s, z, nbits, GS), _id(case))


def test_launches_of_different_row_counts_share_the_scratch_memory(oracle):
    """16 rows, then 3, then 16 again on one object: the slots are empty again after every launch and no launch
    reads a partial sum an earlier one left; the same input gives the same bits every time."""
    case = prebuild._case(16, 4096, 11008)
    print("[case] split, row counts 16 / 3 / 16 on one object", flush=True)
    layer, g = _filled_layer(case, 77)
    A = torch.randn(16, 11008, device="cuda", generator=g).to(torch.float16)
    first = layer(A).clone()
    few = layer(A[:3]).clone()
    again = layer(A).clone()
    torch.cuda.synchronize()
    assert torch.equal(first, again) and torch.equal(few, first[:3])
    cols = np.arange(0, 4096, 8)
    assert_close(oracle, first[:, torch.from_numpy(cols).cuda()].cpu().numpy(), _oracle_columns(oracle, layer, A, cols, 4, 128), "M=16")
    # two layers of one shape share the object, hence the scratch memory: back to back on one stream
    other, g2 = _filled_layer(case, 78)
    a, b = layer(A).clone(), other(A).clone()
    torch.cuda.synchronize()
    assert torch.equal(a, first) and not torch.equal(a, b)
    assert_close(oracle, b[:, torch.from_numpy(cols).cuda()].cpu().numpy(), _oracle_columns(oracle, other, A, cols, 4, 128), "second layer")


def test_split_rows_in_a_hip_graph_replay_like_the_eager_launch():
    case = prebuild._case(16, 8192, 8192)
    print("[case] split, HIP graph", flush=True)
    layer, g = _filled_layer(case, 5)
    A = torch.randn(16, 8192, device="cuda", generator=g).to(torch.float16)
    want = layer(A).clone()
    x, out = A.clone(), torch.empty(16, 8192, dtype=torch.float16, device="cuda")
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
        layer(x, out=out)
        layer(x, out=out)                                                   # twice in one graph: the second finds the slots empty
    torch.cuda.current_stream().wait_stream(side)
    for i in range(3):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {i}"
        assert torch.equal(layer(A), want)                                  # eager work between the replays


@pytest.mark.parametrize("M,N,K", [(16, 8192, 8192), (16, 4096, 11008), (7, 1000, 28672), (8, 100, 53248), (4, 7168, 5120)])
def test_the_result_does_not_depend_on_who_arrives_first(M, N, K):
    """Two, four, eight and sixteen blocks along K: the blocks of a pair meet in whatever order the hardware runs them,
    the sum of an output is fixed by the tree over the blocks.  Forty launches, with other work in between so that the
    blocks start at different moments: the same bits every time (compared as integers: +0 and -0 differ)."""
    case = {"M": M, "N": N, "K": K, "NBITS": 4, "GS": 128, "sym": N == 100}
    print(f"[case] arrival order {_id(case)}", flush=True)
    layer, g = _filled_layer(case, 17)
    assert "KS=" in layer.func.runtime.description
    A = torch.randn(M, K, device="cuda", generator=g).to(torch.float16)
    A[0].zero_()                                                            # a row of exact zeros: sums of +0 travel as "not empty"
    first = layer(A).view(torch.int16).clone()
    noise = torch.empty(1 << 22, device="cuda")
    for i in range(40):
        if i % 3:
            noise.normal_()                                                 # occupies part of the GPU while the launch starts
        out = layer(A)
        assert torch.equal(out.view(torch.int16), first), i
    assert float(layer(A)[0].abs().max()) == 0.0


def test_add_to_output_with_split_rows(oracle):
    """The down projection of the decode loop at batch 16 writes into the residual stream."""
    case = prebuild._case(16, 4096, 11008)
    print("[case] split, accumulate", flush=True)
    layer, g = _filled_layer(case, 31)
    assert layer.fuses_accumulate(16)
    A = torch.randn(16, 11008, device="cuda", generator=g).to(torch.float16)
    resid = torch.randn(16, 4096, device="cuda", generator=g).to(torch.float16)
    want = resid + layer(A)                                                 # fp16 add of the rounded projection
    got = layer.forward_accumulate(A, resid.clone())
    torch.cuda.synchronize()
    assert "KS=" in layer._funcs[(16, torch.float16, "accumulate")].runtime.description
    assert torch.equal(got, want)


def test_a_split_object_refuses_more_rows_than_it_holds():
    from qfactory.jit import jit
    (qfunc,) = prebuild.qfuncs_of(prebuild._case(16, 4096, 11008))
    runtime = jit.compile(qfunc)
    assert "KS=4" in runtime.description
    x = torch.zeros(17, 11008, dtype=torch.float16, device="cuda")
    w = torch.zeros(4096, 11008 // 2, dtype=torch.int8, device="cuda")
    s = torch.zeros(4096, 86, dtype=torch.float16, device="cuda")
    z = torch.zeros(4096, 43, dtype=torch.int8, device="cuda")
    out = torch.zeros(17, 4096, dtype=torch.float16, device="cuda")
    assert runtime.run_m(17, x, w, out, s, z, torch.cuda.current_stream()) == 1      # refused on the host, nothing launched
    assert runtime.run_m(16, x[:16], w, out[:16], s, z, torch.cuda.current_stream()) == 0
    torch.cuda.synchronize()
