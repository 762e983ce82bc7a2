"""Ahead-of-time population of the JIT cache.

The kernels are specialised per problem and compiled on first use; a GPU job should not spend its
time in hipcc.  This module lists the problems the repository's own tests, smoke check and
benchmark construct and compiles their specialisations (in parallel, no GPU needed) into
``$QFACTORY_CACHE_DIR`` (default: ``jit_cache/`` beside this file).

Run as ``python prebuild.py [--force]`` or through ``__graft_entry__.build()``.
"""
import argparse
import os
import sys
from concurrent.futures import ThreadPoolExecutor, as_completed

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)
os.environ.setdefault("QFACTORY_CACHE_DIR", os.path.join(HERE, "jit_cache"))

LLAMA2_7B = [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]        # (N, K): qkv, o, gate_up, down
LLAMA3_70B = [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)]


def _case(M, N, K, NBITS=4, GS=128, sym=False):
    return {"M": M, "N": N, "K": K, "NBITS": NBITS, "GS": GS, "sym": sym}


def parity_cases():
    """Problems the GPU parity tests run (tests/test_qlinear_gpu.py imports this list)."""
    cases = []
    for N, K in LLAMA2_7B:                                   # W4A16 g128 asymmetric GEMV sweep
        for M in (1, 4, 16):
            cases.append(_case(M, N, K))
    for M in (1, 16):                                        # bit-width scaling at N = K = 8192
        for nbits in (2, 3, 4, 8):
            for sym in (False, True):
                cases.append(_case(M, 8192, 8192, nbits, 128, sym))
    # ragged / small shapes: N not a multiple of the rows per block, odd M, other group sizes
    cases += [_case(1, 100, 256, 4, 128), _case(2, 100, 256, 4, 64), _case(3, 130, 512, 4, 32),
              _case(5, 77, 1024, 4, 128), _case(7, 1000, 2048, 8, 128), _case(2, 64, 512, 2, 64),
              _case(1, 48, 4096, 2, 128, True), _case(3, 48, 1024, 8, 256, True),
              _case(1, 256, 11008, 4, 128),
              _case(1, 100, 256, 3, 64), _case(2, 77, 1024, 3, 128, True), _case(5, 130, 512, 3, 32),
              _case(33, 64, 2048, 3, 128), _case(1, 50, 11008, 3, 128),
              _case(48, 100, 1024, 3, 64), _case(7, 130, 512, 3, 128, True), _case(100, 96, 1536, 3, 128)]
    for nbits in (2, 3, 4, 8):                                  # group_size == -1: raw integer weights
        cases += [_case(1, 4096, 4096, nbits, -1), _case(3, 100, 256, nbits, -1)]
    # matrix-core regime: ragged M and N, M above one block tile, other widths and group sizes
    cases += [_case(33, 100, 512, 4, 128), _case(100, 1000, 1024, 4, 64), _case(300, 256, 2048, 4, 128),
              _case(48, 130, 1024, 2, 64), _case(17, 96, 512, 8, 32), _case(64, 512, 1024, 4, 128, True),
              _case(128, 256, 11008, 4, 128)]
    # streaming skinny regime (3 <= M <= 16, K too long for resident activations): ragged M and N,
    # a last wave with dead steps (43 steps over 8 waves), group per lane / per chunk / per step, 2 and 8 bits
    cases += [_case(5, 100, 11008, 4, 128), _case(3, 77, 11008, 4, 32), _case(7, 130, 11008, 4, 64, True),
              _case(16, 272, 14336, 4, 256), _case(12, 48, 14336, 2, 256), _case(16, 64, 14336, 2, 512, True),
              _case(9, 64, 8192, 8, 128), _case(4, 100, 8192, 8, 64), _case(11, 40, 11008, 8, 32, True),
              _case(8, 8200, 11008, 4, 128)]
    # two activation rows: four stages per block in the dot2 GEMV, and swept tilings of the reference's shapes
    # (one team per block, seven waves per row, eight rows per stage)
    cases += [_case(2, 22016, 4096), _case(2, 4096, 11008), _case(2, 10240, 8192), _case(2, 5120, 13824), _case(2, 7168, 5120)]
    # 2-bit at K = 4096: the A-stationary kernel's 16-wave tiling does not fit LDS, 8 waves do
    cases += [_case(16, 100, 4096, 2, 128), _case(32, 48, 4096, 2, 64, True)]
    # 3-bit (two planes per row) in the A-stationary kernel: ragged M and N, a last wave that owns fewer
    # chunks, group per lane / per chunk / over two chunks
    cases += [_case(3, 77, 4096, 3, 128), _case(12, 100, 2048, 3, 64), _case(16, 48, 8192, 3, 256, True),
              _case(9, 100, 1024, 3, 512), _case(16, 272, 4864, 3, 128), _case(32, 40, 1024, 3, 128)]
    # K not a whole number of 128-byte windows of the main plane (GEMM kernel: the last window is moved back to
    # end at the row's end and its first iterations are skipped): every width, a quarter / half / three quarters
    # of a window left over, K split over wave groups and not, group per window position and wider
    cases += [_case(300, 64, 2816, 2, 128, True), _case(40, 100, 2816, 2, 64), _case(64, 80, 11008, 2, 128, True),
              _case(5, 100, 11008, 3, 128), _case(48, 64, 2816, 3, 64, True), _case(256, 12288, 2816, 3, 128),
              _case(70, 96, 4224, 4, 32, True), _case(33, 130, 4224, 4, 64), _case(64, 64, 1088, 4, 32, True),
              _case(64, 64, 1216, 4, 32), _case(512, 4096, 4224, 4, 64),
              _case(40, 72, 4160, 8, 32), _case(40, 40, 4160, 8, 32, True), _case(128, 8192, 4160, 8, 32)]
    # eight groups per 128-byte window (4 bits, group 32) on whole windows
    cases += [_case(70, 96, 4096, 4, 32, True), _case(40, 64, 1024, 4, 32)]
    return cases


def grid_cases():
    """Every bit width x group size the packed layout allows, symmetric and asymmetric alternating, at one
    small shape per kernel family (M = 1 dot2 GEMV, M = 12 small-M matrix-core kernels, M = 40 GEMM), with K a
    whole number of 128-byte windows and with half a window left over where the group size permits."""
    cases = []
    for nbits in (2, 3, 4, 8):
        zfb = 4 if nbits == 3 else nbits
        supk = 1024 // (2 if nbits == 3 else nbits)
        for i, gs in enumerate((32, 64, 128, 256, 512, 1024)):
            for K in (4096, 4096 + supk // 2):
                G = K // gs
                if K % (2 * gs) or G % (8 // zfb):
                    continue
                sym = bool(i % 2)
                cases += [_case(1, 50, K, nbits, gs, sym), _case(12, 72, K, nbits, gs, not sym), _case(40, 72, K, nbits, gs, sym)]
    return cases


# The reference's shape list (data/nkg_shapes.json, key "all"): [N, K, group size] of the linears of Llama-2
# 7B / 13B / 70B and Qwen-2.5 7B / 14B / 32B / 72B.  Its accuracy scripts sweep it at M in {1, 16} and 8 / 4 / 2 bits.
REFERENCE_SHAPES = [[3584, 3584, 128], [4608, 3584, 128], [4096, 4096, 128], [5120, 5120, 128], [7168, 5120, 128],
                    [4096, 11008, 128], [12288, 4096, 128], [8192, 8192, 128], [3584, 18944, 128], [5120, 13824, 128],
                    [15360, 5120, 128], [10240, 8192, 128], [22016, 4096, 128], [37888, 3584, 128], [27648, 5120, 128],
                    [5120, 27648, 128], [8192, 29696, 128], [55296, 5120, 128], [59392, 8192, 128], [57344, 8192, 128],
                    [8192, 28672, 128]]


def reference_sweep_cases():
    """tests/acc_gptq.py (grouped, asymmetric) and tests/acc_gemv.py (plain integer weights) of the reference:
    every shape x M in {1, 16} x bits in {8, 4, 2}; the grouped sweep skips K % (GS * 8 / bits) != 0 as the
    reference does (acc_gptq.py:42-44)."""
    cases = []
    for N, K, GS in REFERENCE_SHAPES:
        for M in (1, 16):
            for nbits in (8, 4, 2):
                if K % (GS * 8 // nbits) == 0:
                    cases.append(_case(M, N, K, nbits, GS))
                cases.append(_case(M, N, K, nbits, -1))
    return cases


def large_parity_cases():
    """W4A16 g128 GEMM at M in {32..256} on Llama-3-70B-style shapes.  The weights are too large to
    build from int32 tensors in a test; the tests fill packed tensors directly (every byte pattern
    is a valid packed weight) and check a seeded subset of output columns."""
    return ([_case(M, N, K) for N, K in LLAMA3_70B for M in (32, 64, 128, 256)]
            + [_case(64, N, K) for N, K in LLAMA2_7B]              # the batch-64 decode linears
            + [_case(512, 10240, 8192), _case(1024, 12288, 4096), _case(700, 22016, 4096), _case(512, 22016, 4096), _case(1024, 10240, 8192)]
            + [_case(2048, 12288, 4096), _case(3000, 4096, 11008), _case(8192, 4096, 4096)]      # the 2048- and 4096-row buckets
            # the decode loop's prefill at 64 sequences x 128 prompt tokens, and its output projection
            + [_case(8192, 12288, 4096), _case(8192, 22016, 4096), _case(8192, 4096, 11008)]
            + [_case(M, 32000, 4096) for M in (1, 16, 64)]
            # the large block tiles at the other bit widths, group sizes and with a partial last window
            + [_case(256, 16384, 4096, 2, 64), _case(256, 16384, 4096, 3, 128, True), _case(256, 16384, 4096, 8, 32),
               _case(512, 16384, 4224, 4, 64), _case(256, 57344, 2816, 2, 128, True), _case(1024, 16384, 4096, 3, 128, True)])


def bf16_cases():
    """bf16 activations and output (tests/test_bf16_gpu.py): every kernel family, every bit width, ragged M and N,
    plain integer weights, a partial last window in the GEMM kernel."""
    cases = [_case(1, 4096, 4096), _case(2, 100, 256, 4, 64), _case(4, 77, 1024, 3, 128, True),      # dot2 GEMV
             _case(1, 48, 4096, 2, 128, True), _case(2, 130, 512, 8, 32),
             _case(1, 4096, 4096, 4, -1), _case(3, 100, 256, 8, -1),                                   # plain integer weights
             _case(16, 4096, 4096), _case(12, 100, 2048, 3, 64), _case(16, 100, 4096, 2, 128),        # A-stationary
             _case(7, 1000, 2048, 8, 128),
             _case(5, 100, 11008, 4, 128), _case(9, 64, 8192, 8, 128), _case(12, 48, 14336, 2, 256),  # A-stationary, long rows split over blocks
             _case(16, 4096, 11008), _case(5, 100, 8192, 4, 64),                                         # ... long rows split over blocks
             _case(33, 100, 512, 4, 128), _case(300, 256, 2048, 4, 128), _case(64, 80, 11008, 2, 128, True),   # GEMM
             _case(48, 64, 2816, 3, 64, True), _case(40, 72, 4160, 8, 32), _case(256, 4096, 4096),
             _case(40, 100, 256, 2, 64),                                                               # generic fallback
             _case(1, 96, 1024), _case(12, 96, 2048), _case(64, 96, 1024), _case(1, 64, 256)]          # range and argument checks
    return [dict(c, act="bf16") for c in cases]


def smem_quant_cases():
    """The dot2 GEMV kernel with the scales and zero-points of a block's rows staged through LDS (the schedule
    search's other choice; tests/test_qlinear_gpu.py): every bit width, symmetric and not, a last block past N,
    several stages per block, one wave per team and several."""
    cases = [_case(1, 100, 1024), _case(2, 77, 512, 3, 64, True), _case(1, 130, 2048, 8, 128, True),
             _case(2, 22016, 4096), _case(1, 4096, 11008), _case(1, 48, 4096, 2, 128), _case(4, 50, 512, 4, 16)]
    return [dict(c, smem_quant=True) for c in cases]


def eager_cases():
    """The other decode strategy of the kernels that have two (``transform()``: the dot2 GEMV in packed fp16, the
    A-stationary and streaming matrix-core kernels with every field scaled before the contraction) where the
    default is the deferred one: every bit width, symmetric and not, ragged shapes, the SwiGLU epilogue."""
    cases = [_case(1, 100, 1024), _case(2, 77, 512, 3, 64, True), _case(1, 130, 2048, 8, 128, True),
             _case(1, 48, 4096, 2, 128), _case(4, 50, 512, 4, 16), _case(1, 4096, 4096), _case(1, 256, 11008),
             _case(16, 384, 1024, 4, 128), _case(12, 100, 2048, 3, 256), _case(16, 100, 4096, 2, 256, True),     # A-stationary
             _case(7, 1000, 2048, 8, 128),
             _case(5, 100, 11008, 4, 128), _case(16, 272, 14336, 4, 256), _case(9, 64, 8192, 8, 128, True),     # streaming skinny
             _case(12, 48, 14336, 2, 256)]
    return [dict(c, decode="eager") for c in cases]


def bench_cases():
    cases = [_case(1, N, K) for N, K in LLAMA2_7B]
    cases += [_case(1, N, K) for N, K in LLAMA3_70B]          # bench.py --small-m
    return cases


def shape_set_cases():
    """bench.py --shape-sets: the reference's bandwidth / speed-up experiments (its `squares-pure` and `operator`
    shape sets; bench.shape_set_problems holds the definitions)."""
    import json
    with open(os.path.join(os.path.dirname(HERE), "tests", "golden", "nkg_shapes.json")) as f:
        sets = json.load(f)
    cases = []
    for N, K, _ in sets["squares-pure"]:
        cases += [_case(1, N, K, 4, -1)] + [_case(1, N, K, nbits, 128) for nbits in (8, 4, 2)]
    for N, K, _ in sets["operator"]:
        cases += [_case(1, N, K, nbits, 128) for nbits in (8, 4, 2)] + [_case(M, N, K, 4, 128) for M in (2, 4)]
    return cases


def smoke_cases():
    return [_case(1, 512, 1024, 4, 128), _case(1, 512, 1024, 4, -1)]


def misc_test_cases():
    """Other modules the GPU tests construct (row-count dispatch, argument checks)."""
    return ([_case(M, 96, 512, 4, 128) for M in (1, 2, 3, 6)] + [_case(1, 64, 256, 4, 128), _case(1, 96, 512, 4, -1)]
            + [_case(1, 384, 1024, 4, 128), _case(16, 384, 1024, 4, 128), _case(64, 384, 1024, 4, 128)])


TINY_LLAMA = [(768, 256), (256, 256), (1024, 256), (256, 512)]      # the decode-loop test model, GS = 64


def decode_cases():
    """decode_llama.py: Llama-2-7B shapes at batch 1 / 16 / 64 (decode) and at prefill row counts,
    plus the tiny model tests/test_decode_gpu.py runs."""
    cases = [_case(M, N, K) for N, K in LLAMA2_7B for M in (1, 16, 64, 128, 256, 512, 1024, 2048, 4096)]
    cases += [_case(M, N, K, 4, 64) for N, K in TINY_LLAMA for M in (2, 16)]
    # the output projection (vocab x hidden): once per sequence in prefill and per decode step
    cases += [_case(M, 32000, 4096) for M in (1, 16, 64)] + [_case(M, 1000, 256, 4, 64) for M in (2, 16)]
    cases += [dict(_case(M, 32000, 4096), prologue="add_rmsnorm") for M in (1, 16)]
    cases += [dict(_case(M, 1000, 256, 4, 64), prologue="add_rmsnorm") for M in (2, 16)]
    return cases + silu_mul_cases()


def silu_mul_cases():
    """Fused gate+up projections that write silu(gate) * up (GPTQLinear.forward_silu_mul, few rows): the decode
    loop's at batch 1 and 2, the tiny test model's, and the shapes of tests/test_qlinear_gpu.py (ragged N/2,
    every bit width, one wave per team and several)."""
    cases = [_case(1, 22016, 4096), _case(2, 22016, 4096), _case(2, 1024, 256, 4, 64),
             _case(1, 100, 1024, 2, 128, True), _case(2, 154, 512, 3, 64), _case(1, 260, 2048, 8, 128),
             _case(1, 36, 256, 4, 128), _case(2, 8192, 11008, 4, 128),
             # the A-stationary kernel: the decode loop's at batch 16, ragged M, one pair per block and many,
             # every bit width, a last block with fewer pairs
             _case(16, 22016, 4096), _case(16, 1024, 256, 4, 64), _case(5, 96, 1024, 4, 128), _case(12, 4128, 2048, 3, 64),
             _case(32, 160, 4096, 2, 128, True), _case(7, 18016, 2048, 8, 128)]
    # the GEMM kernel: the decode loop's at batch 64 and at prefill row counts, the tiny model's, ragged M,
    # every bit width, a last block with waves past N
    cases += [_case(M, 22016, 4096) for M in (64, 128, 256, 512, 1024, 2048, 4096)]
    cases += [_case(64, 1024, 256, 4, 64), _case(100, 4128, 2048, 3, 64), _case(40, 160, 4096, 2, 128, True),
              _case(200, 2208, 2048, 8, 128), _case(33, 96, 1024, 4, 128)]
    return [dict(c, epilogue="silu_mul") for c in cases]


def norm_prologue_cases():
    """Projections that run the residual add and RMSNorm in front of their dot products
    (GPTQLinear.forward_add_rmsnorm, dot2 GEMV rows): the decode loop's qkv and gate+up at batch 1 and 2, the tiny
    test model's, and the shapes of tests/test_norm_prologue_gpu.py (every bit width, symmetric and not, a team
    whose last lanes own no chunk, two chunks per lane, one wave per team and several; with and without the SwiGLU
    epilogue)."""
    cases = [dict(_case(M, 12288, 4096), prologue="add_rmsnorm") for M in (1, 2)]
    cases += [dict(_case(M, 22016, 4096), prologue="add_rmsnorm", epilogue="silu_mul") for M in (1, 2)]
    cases += [dict(_case(2, 768, 256, 4, 64), prologue="add_rmsnorm"),
              dict(_case(2, 1024, 256, 4, 64), prologue="add_rmsnorm", epilogue="silu_mul")]
    for c in (_case(1, 100, 1024), _case(2, 77, 512, 3, 64, True), _case(1, 130, 2048, 8, 128, True),
              _case(1, 48, 4096, 2, 128), _case(2, 96, 2816, 4, 128), _case(1, 64, 11008, 4, 128),
              _case(1, 40, 28672, 4, 128), _case(2, 50, 512, 4, 16)):
        cases.append(dict(c, prologue="add_rmsnorm"))
    for c in (_case(1, 100, 1024), _case(2, 154, 512, 3, 64), _case(1, 260, 2048, 8, 128), _case(2, 96, 2816, 2, 128, True)):
        cases.append(dict(c, prologue="add_rmsnorm", epilogue="silu_mul"))
    # the A-stationary kernel (3 .. 32 rows): the decode loop's at batch 16, the tiny model's, ragged M and N, every
    # bit width, a last wave that owns fewer chunks, two 16-row activation tiles
    cases += [dict(_case(16, 12288, 4096), prologue="add_rmsnorm"),
              dict(_case(16, 22016, 4096), prologue="add_rmsnorm", epilogue="silu_mul"),
              dict(_case(16, 768, 256, 4, 64), prologue="add_rmsnorm"),
              dict(_case(16, 1024, 256, 4, 64), prologue="add_rmsnorm", epilogue="silu_mul")]
    for c in (_case(5, 96, 1024, 4, 128), _case(12, 100, 2048, 3, 64), _case(16, 48, 8192, 3, 256, True),
              _case(7, 1000, 2048, 8, 128), _case(16, 100, 4096, 2, 128), _case(16, 272, 4864, 3, 128),
              _case(32, 40, 1024, 3, 128), _case(20, 130, 4096, 4, 128)):
        cases.append(dict(c, prologue="add_rmsnorm"))
    for c in (_case(5, 96, 1024, 4, 128), _case(12, 4128, 2048, 3, 64), _case(32, 160, 4096, 2, 128, True)):
        cases.append(dict(c, prologue="add_rmsnorm", epilogue="silu_mul"))
    return cases


def accumulate_cases():
    """Projections that add their result to the output (GPTQLinear.forward_accumulate): the decode
    loop's o and down at batch 1 / 2 / 16, the tiny test model's, and the shapes of tests/test_norm_prologue_gpu.py
    (dot2 GEMV with one wave per team -- stored from the lane -- and several; A-stationary and streaming kernels;
    every bit width; ragged M and N)."""
    cases = [_case(M, N, K) for N, K in ((4096, 4096), (4096, 11008)) for M in (1, 2, 16)]
    cases += [_case(M, N, K, 4, 64) for N, K in ((256, 256), (256, 512)) for M in (2, 16)]
    cases += [_case(1, 100, 256), _case(2, 77, 1024, 3, 128, True), _case(1, 130, 2048, 8, 128, True), _case(1, 48, 4096, 2, 128),
              _case(5, 96, 1024), _case(12, 100, 2048, 3, 64), _case(32, 40, 1024, 8, 128),
              _case(5, 100, 11008), _case(16, 64, 14336, 2, 512, True), _case(9, 64, 8192, 8, 128)]
    # the GEMM kernel: the decode loop's at batch 64 and at prefill row counts, the tiny model's, ragged M, N not a
    # multiple of four (element-wise stores), every bit width
    cases += [_case(M, N, K) for N, K in ((4096, 4096), (4096, 11008)) for M in (64, 128, 256, 512, 1024, 2048, 4096)]
    cases += [_case(64, N, K, 4, 64) for N, K in ((256, 256), (256, 512))]
    cases += [_case(40, 96, 1024), _case(100, 77, 1024, 3, 128, True), _case(33, 130, 2048, 8, 128, True), _case(200, 2208, 4096, 2, 128)]
    return [dict(c, epilogue="accumulate") for c in cases]


def unsplit_cases():
    """Long rows at 3 .. 16 activation rows served WITHOUT the split of K over blocks (``ksplit=False``: the kernels a
    layer with the norm prologue or the SwiGLU epilogue is built on, and the streaming kernel, which the split has
    replaced as the default of these shapes): ragged M and N, a last wave with dead steps, group per lane / per
    chunk / per step, 2, 4 and 8 bits."""
    cases = [_case(5, 100, 11008, 4, 128), _case(3, 77, 11008, 4, 32), _case(7, 130, 11008, 4, 64, True),
             _case(16, 272, 14336, 4, 256), _case(12, 48, 14336, 2, 256), _case(16, 64, 14336, 2, 512, True),
             _case(9, 64, 8192, 8, 128), _case(4, 100, 8192, 8, 64), _case(11, 40, 11008, 8, 32, True),
             _case(8, 8200, 11008, 4, 128), _case(16, 4096, 11008), _case(16, 8192, 8192), _case(4, 100, 8192, 4, 64)]
    return [dict(c, ksplit=False) for c in cases]


def split_cases():
    """The A-stationary kernel with K split over blocks (tests/test_ksplit_gpu.py), beyond what the parity lists above
    already send there: 2, 4, 8 and 16 blocks along K, a last block with fewer chunks, waves past a block's share,
    fewer column tiles than blocks, many batches per block, every bit width (bf16: the long rows of ``bf16_cases``)."""
    return [_case(16, 4096, 7168), _case(3, 48, 7168, 4, 64), _case(16, 16384, 16384), _case(7, 1000, 28672), _case(4, 8192, 29696),
            _case(16, 100, 53248, 4, 128, True), _case(13, 57344, 8192), _case(16, 2048, 16384, 8, 128), _case(5, 77, 12288, 2, 128),
            _case(16, 272, 12288, 3, 128, True), _case(16, 5120, 13824),
            # five tiles per block in one batch (the last of them ragged)
            _case(11, 8200, 8192), _case(16, 10240, 8192),
            # rows of 5120 .. 7167 on narrow layers: two blocks along K
            _case(16, 5120, 5120), _case(4, 7168, 5120), _case(9, 4096, 6144, 4, 64),
            # 17 .. 32 rows on narrow layers with long rows: two activation tiles per wave
            _case(32, 4096, 11008), _case(20, 100, 14336, 4, 64), _case(27, 1000, 11008, 4, 128, True)]


def odd_wave_cases():
    """GEMM tilings whose wave count along N does not divide the activation tile's 1 KB blocks (3, 5, 6, 7 waves: the
    waves past the last block fetch it again), pinned explicitly (tests/test_qlinear_gpu.py): ragged M and N, one and two
    wave groups along K, one and two weight tiles per wave, a tile of four blocks on three waves, 2 and 8 bits."""
    def tile(bm, nt32, wn, wk, pa):
        return tuple(sorted({"BM": bm, "NT32": nt32, "WN": wn, "WK": wk, "PA": pa}.items()))
    return [dict(_case(70, 250, 1024), tiling=tile(64, 1, 3, 2, 4)), dict(_case(256, 500, 2048), tiling=tile(256, 1, 7, 1, 3)),
            dict(_case(100, 960, 1024, 4, 64), tiling=tile(128, 2, 5, 1, 4)), dict(_case(40, 200, 512, 8, 32), tiling=tile(32, 1, 3, 1, 3)),
            dict(_case(64, 400, 2048, 2, 128, True), tiling=tile(64, 1, 6, 1, 4)), dict(_case(33, 100, 4096, 4, 128), tiling=tile(64, 2, 3, 2, 3))]


def search_cases():
    """Problems whose whole tiling search space is compiled (tests/test_tune.py searches on the device)."""
    return [_case(1, 64, 256, 4, 128)]


def drain_cases(base=None):
    """One problem (the cheapest) per distinct GEMM tiling x bit width among the problems above: the GEMM kernel
    with counted waits is compared bit for bit with its full-drain build (tests/test_gemm_drain_gpu.py)."""
    best = {}
    for c in (base if base is not None else all_cases(with_drain=False)):
        if c.get("act") or c.get("smem_quant") or c.get("epilogue") or c.get("drain") or c["GS"] == -1:
            continue
        for q in qfuncs_of(c):
            if getattr(q, "regime", None) != "gemm":
                continue
            key = (tuple(sorted(q.tiling_configs.items())), c["NBITS"])
            cost = c["M"] * c["N"] * c["K"]
            if key not in best or cost < best[key][0]:
                best[key] = (cost, c)
    return [dict(c, drain=True) for _, c in sorted(best.values(), key=lambda t: t[0])]


def all_cases(with_drain=True):
    seen, out = set(), []
    for c in (parity_cases() + grid_cases() + reference_sweep_cases() + large_parity_cases() + bench_cases() + shape_set_cases() + smoke_cases() + misc_test_cases()
              + decode_cases() + bf16_cases() + smem_quant_cases() + eager_cases() + norm_prologue_cases() + accumulate_cases() + odd_wave_cases()
              + unsplit_cases() + split_cases()):
        key = tuple(sorted(c.items()))
        if key not in seen:
            seen.add(key)
            out.append(c)
    if with_drain:
        out += drain_cases(out)
    return out


def qfuncs_of(case):
    """The default specialisation(s) ``QLinear`` compiles for a case (no search flags)."""
    import torch
    from qfactory.core import QMatmul, Matmul
    from qfactory.qlinear import _m_bucket
    dtypes = [torch.float16]                     # a module compiles its fp16 specialisation at construction
    if case.get("act") == "bf16":
        dtypes.append(torch.bfloat16)
    qfuncs = []
    for dtype in dtypes:
        if case["GS"] == -1:
            op = Matmul(case["N"], case["K"], case["NBITS"], dtype, torch.int8)
        else:
            op = QMatmul(_m_bucket(case["M"]), case["N"], case["K"], case["NBITS"], case["sym"],
                         dtype, torch.int8, case["GS"])
        op.init_qfuncs()
        qfuncs += op.qfuncs
    if case.get("ksplit") is False:
        from qfactory.core.qfunc import QMatmulQFunc
        from qfactory.core.qtile import AsymQTile, QTile, SymQTile
        tile = SymQTile if case["sym"] else AsymQTile
        qfuncs = [QMatmulQFunc(QTile((_m_bucket(case["M"]), case["K"]), torch.float16, 16),
                               tile((case["N"], case["K"]), torch.int8, case["NBITS"], (1, case["GS"])), "nt", ksplit=False)]
    if case.get("tiling"):
        qfuncs = [q.clone(tiling_configs=dict(case["tiling"])) for q in qfuncs]
    if case.get("smem_quant"):
        op = QMatmul(_m_bucket(case["M"]), case["N"], case["K"], case["NBITS"], case["sym"],
                     torch.float16, torch.int8, case["GS"])
        op.init_qfuncs()
        qfuncs += [q.clone(smem_quant=True) for q in op.qfuncs]
    if case.get("decode"):
        eager = [q.clone(decode_strategy=case["decode"]) for q in qfuncs if case["decode"] in q.decode_strategies()
                 and q.decode_strategy != case["decode"]]
        assert eager, f"{case}: the kernel has no second decode strategy"
        qfuncs += eager
    if case.get("drain"):
        qfuncs += [q.clone(defines={"QF_GEMM_FULL_DRAIN": 1}) for q in list(qfuncs) if q.regime == "gemm"]
    if case.get("epilogue") or case.get("prologue"):
        op = QMatmul(_m_bucket(case["M"]), case["N"], case["K"], case["NBITS"], case["sym"],
                     torch.float16, torch.int8, case["GS"], output_epilogue=case.get("epilogue", "none"),
                     input_prologue=case.get("prologue", "none"))
        op.init_qfuncs()
        qfuncs += op.qfuncs
    return qfuncs


class TimingBuild:
    """A specialisation compiled with its kernel header's timing knob set (``QF_*_EXPERIMENT``: parts of the kernel
    left out, results wrong by design), for ``bench.py --ablation`` only.  The code generator refuses these knobs;
    this wrapper writes them, and the define the headers ask for, in front of the generated translation unit."""
    KNOBS = {"gemv": "QF_GEMV_EXPERIMENT", "mgemv": "QF_MGEMV_EXPERIMENT", "gemm": "QF_GEMM_EXPERIMENT"}

    def __init__(self, qfunc, bits):
        assert bits != 0 and qfunc.regime in self.KNOBS
        self.qfunc, self.bits = qfunc, bits

    def __getattr__(self, name):                      # tiling, argument list, ... are the wrapped specialisation's
        if name in ("qfunc", "bits"):
            raise AttributeError(name)
        return getattr(self.qfunc, name)

    @property
    def regime(self):                                 # not "gemm": the counted waits of a timing build are not re-counted
        return self.qfunc.regime + "-timing"

    def emit(self):
        return (f"#define QF_ALLOW_TIMING_EXPERIMENTS 1\n#define {self.KNOBS[self.qfunc.regime]} {self.bits}\n"
                + self.qfunc.emit())


# What each timing build leaves out (knob value, label), per kernel family; 0 is the product's own object.
ABLATIONS = {
    "gemv": [(0, "kernel"), (1, "without decode + dot products"), (8, "without cross-lane sums, LDS exchange, stores"),
             (9, "without both"), (11, "also without activation loads")],
    "mgemv": [(0, "kernel"), (4, "without cross-wave sums and stores"),
              (16, "loads in their order, LDS hand-off + decode + MFMAs replaced by an XOR"),
              (48, "... and without scale / zero-point loads"), (8, "without the weight loads"),
              (1, "without the activation loads")],
    "gemm": [(0, "kernel"), (1, "without dequantisation arithmetic"), (4, "without MFMAs"), (5, "without both"),
             (72, "without activation tile requests and their wait"), (32, "without weight / scale / zero-point loads"),
             (16, "without the block barrier of the K loop")],
}
ABLATION_PROBLEMS = ([(1, N, K) for N, K in LLAMA2_7B] + [(16, 22016, 4096), (16, 12288, 4096), (16, 4096, 11008), (16, 57344, 8192)]
                     + [(256, 8192, 8192), (256, 57344, 8192), (8192, 4096, 4096)])


def ablation_builds(M, N, K):
    """(operator, regime, [(knob value, label, object to compile)]) of one ``ABLATION_PROBLEMS`` entry (W4 g128
    asymmetric): the specialisation ``QLinear`` picks for it, and the timing builds of the same tiling."""
    import torch
    from qfactory.core import QMatmul
    from qfactory.qlinear import _m_bucket
    op = QMatmul(_m_bucket(M), N, K, 4, False, torch.float16, torch.int8, 128)
    op.init_qfuncs()
    q = op.qfuncs[0]
    return op, q.regime, [(bits, label, q if bits == 0 else TimingBuild(q, bits)) for bits, label in ABLATIONS[q.regime]]


def timing_builds():
    return [obj for M, N, K in ABLATION_PROBLEMS for _, _, obj in ablation_builds(M, N, K)[2]]


def prune(keep):
    """Remove cached objects of the in-tree cache that no listed problem compiles to any more (older header
    or generator versions): the cache travels with the tree, stale objects are dead weight."""
    import shutil
    root = os.path.join(os.environ["QFACTORY_CACHE_DIR"], "runtimes")
    removed = 0
    for name in (os.listdir(root) if os.path.isdir(root) else []):
        path = os.path.join(root, name)
        if path not in keep:
            shutil.rmtree(path, ignore_errors=True)
            removed += 1
    shutil.rmtree(os.path.join(os.environ["QFACTORY_CACHE_DIR"], "tmp"), ignore_errors=True)
    return removed


def prebuild(cases=None, force=False, workers=None, verbose=True):
    from qfactory.jit import jit
    qfuncs, seen = [], set()
    for case in (cases if cases is not None else all_cases()):
        for q in qfuncs_of(case):
            path, _ = jit.runtime_path_of(q)
            if path not in seen:
                seen.add(path)
                qfuncs.append(q)
    if cases is None:
        for case in search_cases():
            for q in qfuncs_of(case):
                for cand in q.lower():
                    path, _ = jit.runtime_path_of(cand)
                    if path not in seen:
                        seen.add(path)
                        qfuncs.append(cand)
    if cases is None:
        for q in timing_builds():
            path, _ = jit.runtime_path_of(q)
            if path not in seen:
                seen.add(path)
                qfuncs.append(q)
    if cases is None and os.path.abspath(os.environ["QFACTORY_CACHE_DIR"]) == os.path.join(HERE, "jit_cache"):
        removed = prune(seen)
        if verbose and removed:
            print(f"[prebuild] removed {removed} stale objects", flush=True)
    workers = workers or min(16, os.cpu_count() or 4)
    done = 0
    with ThreadPoolExecutor(max_workers=workers) as pool:
        futures = [pool.submit(jit.compile, q, force) for q in qfuncs]
        for f in as_completed(futures):
            f.result()
            done += 1
            if verbose and (done % 10 == 0 or done == len(futures)):
                print(f"[prebuild] {done}/{len(futures)} specialisations", flush=True)
    return len(qfuncs)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true", help="recompile even if cached")
    args = ap.parse_args()
    n = prebuild(force=args.force)
    print(f"[prebuild] {n} specialisations in {os.environ['QFACTORY_CACHE_DIR']}")
