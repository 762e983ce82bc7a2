"""Host-side tiling logic (no GPU): regime routing, and that every default tiling the package would
compile satisfies the static limits its kernel checks at launch (registers, LDS, divisibility)."""
import math
import os

import pytest

import prebuild
from qfactory.core import tiling


def _cases():
    return [c for c in prebuild.all_cases() if c["GS"] != -1]


def _id(c):
    return f"M{c['M']}-N{c['N']}-K{c['K']}-b{c['NBITS']}-g{c['GS']}"


@pytest.mark.parametrize("M,K,nbits,gs,expected", [
    (1, 4096, 4, 128, "gemv"), (2, 11008, 4, 128, "gemv"),
    (3, 4096, 4, 128, "mgemv"), (16, 8192, 4, 128, "mgemv"), (32, 4096, 4, 128, "mgemv"),
    (16, 4096, 2, 128, "mgemv"), (16, 4096, 8, 128, "mgemv"),
    (4, 11008, 4, 128, "skinny"), (16, 11008, 4, 128, "skinny"), (16, 14336, 4, 128, "skinny"),
    (16, 8192, 8, 128, "skinny"), (16, 11008, 8, 128, "skinny"),
    (17, 11008, 4, 128, "gemm"), (16, 28672, 4, 128, "gemm"), (32, 8192, 4, 128, "gemm"),
    (64, 4096, 4, 128, "gemm"), (256, 8192, 4, 128, "gemm"),
    (1, 8192, 3, 128, "gemv"), (2, 8192, 3, 128, "gemv"), (16, 8192, 3, 128, "mgemv"), (32, 8192, 3, 128, "gemm"),
    (16, 4096, 3, 128, "mgemv"), (16, 4096, 3, 32, "gemv"),
    (33, 2048, 3, 128, "gemm"),
])
def test_regime_routing(M, K, nbits, gs, expected):
    """The kernel families without the split of long rows over blocks (how a layer with the norm prologue or the
    SwiGLU epilogue is built)."""
    assert tiling.regime_for(M, K, nbits, gs, ksplit=False) == expected


@pytest.mark.parametrize("M,K,nbits,gs,ks", [
    (3, 7168, 4, 128, 2), (16, 8192, 4, 128, 2), (4, 11008, 4, 128, 4), (16, 14336, 4, 128, 4), (16, 16384, 4, 128, 4),
    (16, 28672, 4, 128, 8), (8, 53248, 4, 128, 16), (16, 8192, 8, 128, 2), (16, 11008, 8, 128, 4),
    (16, 12288, 2, 128, 4), (16, 12288, 3, 128, 4), (16, 8192, 4, 64, 2), (16, 8192, 4, 32, 2),
    (16, 5120, 4, 128, 2), (4, 6144, 4, 128, 2),          # rows of 5120 .. 7167 on a layer of 4096 .. 7168 columns
    # not split: short rows, one or two activation rows, more than sixteen, 2 and 3 bits where the unsplit kernel holds K
    (16, 4096, 4, 128, 1), (16, 5120, 8, 128, 1), (2, 8192, 4, 128, 1), (17, 8192, 4, 128, 1), (33, 11008, 4, 128, 1),
    (16, 8192, 2, 128, 1), (16, 8192, 3, 128, 1),
    # 17 .. 32 rows: two activation tiles per wave, narrow layers with long rows only
    (32, 11008, 4, 128, 4), (17, 14336, 4, 128, 8), (32, 11008, 8, 128, 1),
])
def test_long_rows_are_split_over_blocks(M, K, nbits, gs, ks):
    t = tiling.mgemv_ksplit_tiling(M, 4096, K, nbits, gs)
    if ks == 1:
        assert t is None
        assert tiling.regime_for(M, K, nbits, gs, 4096) == tiling.regime_for(M, K, nbits, gs, 4096, ksplit=False)
        return
    assert tiling.regime_for(M, K, nbits, gs, 4096) == "mgemv"
    chunk = 4 * (128 // tiling.plane_bits(nbits))
    nchunk, nb = K // chunk, -(-(K // chunk) // ks)
    assert t["KS"] == ks and t["PB"] * ks == tiling.NUM_CUS and t["MT16"] == -(-M // 16)
    assert t["WK"] <= 16 and t["WK"] * t["CH"] >= nb and (t["WK"] - 1) * t["CH"] < nb      # the waves cover a block's share, none idle
    assert (ks - 1) * nb < nchunk                                                            # every block owns part of K
    assert tiling.mgemv_lds_bytes(t["MT16"], t["WK"], t["CH"], nbits) <= 160 * 1024
    assert tiling.mgemv_regs(t["MT16"], t["CH"], t["PF"], nbits) <= tiling.mgemv_reg_limit(t["WK"])
    assert f", {ks}>" in tiling.mgemv_cfg_string({"NBITS": nbits, "GS": gs, "SYM": False, "N": 4096, "K": K}, t, True)


def test_rows_of_5120_are_split_on_narrow_layers_only():
    for N, split in ((3584, False), (4096, True), (5120, True), (7168, True), (8192, False), (15360, False), (0, False)):
        assert (tiling.mgemv_ksplit_tiling(16, N, 5120, 4, 128) is not None) == split, N
    assert tiling.mgemv_ksplit_tiling(16, 5120, 4096, 4, 128) is None
    assert tiling.mgemv_ksplit_tiling(32, 5120, 5120, 4, 128) is None


def test_wide_layers_keep_the_gemm_kernel_at_32_rows():
    assert tiling.mgemv_ksplit_tiling(32, 8192, 28672, 4, 128) is None and tiling.regime_for(32, 28672, 4, 128, 8192) == "gemm"
    assert tiling.mgemv_ksplit_tiling(32, 0, 11008, 4, 128) is None          # the width is not known: no split
    assert tiling.regime_for(32, 11008, 4, 128, 4096) == "mgemv" and tiling.regime_for(32, 11008, 4, 128) == "gemm"


def test_split_rows_are_not_combined_with_the_norm_prologue_or_the_swiglu_epilogue():
    import torch
    from qfactory.core import QMatmul
    plain = QMatmul(16, 4096, 8192, 4, False, torch.float16, torch.int8, 128)
    plain.init_qfuncs()
    assert plain.qfuncs[0].tiling_configs.get("KS", 1) == 2 and "KS=2" in plain.qfuncs[0].emit()
    add = QMatmul(16, 4096, 8192, 4, False, torch.float16, torch.int8, 128, output_epilogue="accumulate")
    add.init_qfuncs()
    assert add.qfuncs[0].tiling_configs.get("KS", 1) == 2
    for kw in ({"input_prologue": "add_rmsnorm"}, {"output_epilogue": "silu_mul"}):
        op = QMatmul(16, 4096, 8192, 4, False, torch.float16, torch.int8, 128, **kw)
        op.init_qfuncs()
        q = op.qfuncs[0]
        assert q.regime == "mgemv" and q.tiling_configs.get("KS", 1) == 1 and "KS=" not in q.emit()


@pytest.mark.parametrize("case", _cases(), ids=_id)
def test_default_tiling_respects_the_kernel_limits(case):
    M, N, K, nbits, gs = (case[k] for k in ("M", "N", "K", "NBITS", "GS"))
    regime = tiling.regime_for(M, K, nbits, gs, N, ksplit=False)
    if regime == "mgemv":
        t = tiling.mgemv_tiling(M, N, K, nbits, gs)
        chunk = 4 * (128 // tiling.plane_bits(nbits))
        nchunk = K // chunk
        assert t["WK"] * t["CH"] >= nchunk and (t["WK"] - 1) * t["CH"] < nchunk and t["WK"] <= 16
        assert tiling.mgemv_lds_bytes(t["MT16"], t["WK"], t["CH"], nbits) <= 160 * 1024
        assert tiling.mgemv_regs(t["MT16"], t["CH"], t["PF"], nbits) <= tiling.mgemv_reg_limit(t["WK"])
    elif regime == "skinny":
        t = tiling.skinny_tiling(M, N, K, nbits, gs)
        assert t is not None and tiling.skinny_valid(t, N, K, nbits, gs)
        nstep = K // (8 * (128 // nbits))
        spw = -(-nstep // t["WK"])
        assert t["MT16"] == 1 and (t["WK"] - 1) * spw < nstep <= t["WK"] * spw
        assert math.lcm(spw, t["D"]) <= 32
        assert tiling.skinny_lds_bytes(t, nbits) <= 160 * 1024
    elif regime == "gemm":
        t = tiling.gemm_tiling(M, N, K, nbits, gs)
        assert tiling.gemm_valid(t, K, nbits, gs), t
        assert tiling.gemm_lds_bytes(t, nbits) <= 160 * 1024
        assert 64 * t["WN"] * t["WK"] <= 1024
        assert t["PA"] >= (3 if t["BM"] <= 128 else 2)
    elif regime == "gemv":
        t = tiling.gemv_tiling(M, N, K, nbits, gs)
        assert t["VB"] in (4, 8, 16) and 64 * t["WK"] * t["WN"] <= 1024
    else:
        assert regime == "mfma"
        t = tiling.mfma_tiling(M, N, K, nbits, gs)
        assert tiling.mfma_lds_bytes(t["AT"], t["BT"], t["WM"], t["WN"], t["WK"], nbits) <= 160 * 1024
        assert 64 * t["WM"] * t["WN"] * t["WK"] <= 1024


def test_skinny_takes_longer_rows_only_with_one_tile_per_block():
    assert tiling.regime_for(16, 18944, 4, 128, 3584, ksplit=False) == "skinny"       # 224 tiles of 16 columns: one per block
    assert tiling.regime_for(16, 18944, 4, 128, 8192, ksplit=False) == "gemm"
    assert tiling.regime_for(16, 27648, 4, 128, 3584, ksplit=False) == "gemm"


def test_two_bit_k4096_mgemv_fits_lds():
    # sixteen waves with 2-bit chunks (512 B of activations per row) would need 199 KB of LDS
    for M in (3, 16, 32):
        t = tiling.mgemv_tiling(M, 22016, 4096, 2, 128)
        assert t is not None and tiling.mgemv_lds_bytes(t["MT16"], t["WK"], t["CH"], 2) <= 160 * 1024


def test_skinny_is_not_chosen_where_it_measured_slower():
    assert not tiling.skinny_preferred(16, 28672, 4, 128)        # activations per block twice the weight bytes
    assert not tiling.skinny_preferred(17, 11008, 4, 128)        # two 16-row tiles spill
    assert not tiling.skinny_preferred(2, 11008, 4, 128)         # dot2 GEMV territory
    assert tiling.skinny_tiling(16, 4096, 11008, 2, 128) is None  # 11008 is not a multiple of a 2-bit step


def test_wide_layers_get_256_row_tiles_only_when_they_fill_the_machine():
    assert tiling.gemm_tiling(256, 57344, 8192, 4, 128)["BM"] == 256
    assert tiling.gemm_tiling(256, 8192, 8192, 4, 128)["BM"] < 256
    assert tiling.gemm_tiling(64, 57344, 8192, 4, 128)["BM"] <= 64


@pytest.mark.parametrize("regime,M,N,K,nbits", [("gemv", 1, 512, 1024, 4), ("mgemv", 16, 384, 1024, 4),
                                                ("skinny", 9, 64, 8192, 8), ("gemm", 64, 384, 1024, 4)])
def test_emit_names_the_kernel_of_the_regime(regime, M, N, K, nbits):
    import torch
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import QTile, AsymQTile
    q = QMatmulQFunc(QTile((M, K), torch.float16, 16), AsymQTile((N, K), torch.int8, nbits, (1, 128)), "nt",
                     ksplit=regime != "skinny")
    assert q.regime == regime
    code = q.emit()
    header = {"gemv": "qf_gemv.hip.h", "mgemv": "qf_mgemv.hip.h", "skinny": "qf_skinny.hip.h", "gemm": "qf_gemm.hip.h"}[regime]
    assert f'#include "{header}"' in code and f"regime={regime}" in code
    assert 'extern "C"' in code and "launch_m" in code


def test_row_count_buckets():
    from qfactory.qlinear import _m_bucket
    assert [_m_bucket(m) for m in (1, 2, 3, 16, 17, 32, 33, 100, 256, 257, 512, 700, 1024, 1025, 2048, 3000, 5000, 8192)] == \
        [1, 2, 16, 16, 32, 32, 64, 128, 256, 512, 512, 1024, 1024, 2048, 2048, 4096, 4096, 4096]


def test_prefill_sizes_use_the_many_rows_model_only_for_several_rounds():
    assert tiling.gemm_tiling(1024, 57344, 8192, 4, 128)["BM"] == 256
    assert tiling.gemm_tiling(512, 10240, 8192, 4, 128) == {"BM": 128, "NT32": 2, "WN": 4, "WK": 1, "PA": 4}
    # one round of 64 x 128 tiles: the K axis is still split over wave groups
    assert tiling.gemm_tiling(512, 4096, 4096, 4, 128)["WK"] == 2


def _qfunc(M, N, K, nbits, gs, sym=False, ksplit=True):
    import torch
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import QTile, AsymQTile, SymQTile
    tile = SymQTile if sym else AsymQTile
    return QMatmulQFunc(QTile((M, K), torch.float16, 16), tile((N, K), torch.int8, nbits, (1, gs)), "nt", ksplit=ksplit)


@pytest.mark.parametrize("M,N,K,nbits,gs,regime,strategies", [
    (1, 512, 1024, 4, 128, "gemv", ["deferred", "eager"]),
    (16, 384, 1024, 4, 128, "mgemv", ["deferred", "eager"]),
    (16, 384, 1024, 4, 64, "mgemv", ["eager"]),                  # a chunk of 128 fields spans two groups
    (9, 64, 8192, 8, 128, "skinny", ["deferred", "eager"]),
    (11, 40, 11008, 8, 32, "skinny", ["eager"]),
    (9, 64, 8192, 8, 128, "mgemv-split", ["deferred", "eager"]),
    (11, 40, 11008, 8, 32, "mgemv-split", ["eager"]),
    (64, 384, 1024, 4, 128, "gemm", ["eager"]),
])
def test_transform_yields_the_decode_strategies_the_kernel_implements(M, N, K, nbits, gs, regime, strategies):
    """The reference's transform() yields an eager and a deferred candidate (qfactory/core/qfunc.py:85-91)."""
    q = _qfunc(M, N, K, nbits, gs, ksplit=regime != "skinny")
    if regime == "mgemv-split":
        assert q.tiling_configs["KS"] > 1
        regime = "mgemv"
    assert q.regime == regime and q.decode_strategy == strategies[0]
    variants = q.transform()
    assert [v.decode_strategy for v in variants] == strategies
    codes = [v.emit() for v in variants]
    assert len(set(codes)) == len(codes)                                            # really different translation units
    for v, code in zip(variants, codes):
        assert f"decode={v.decode_strategy}" in code
        assert ("_EAGER 1" in code) == (v.decode_strategy == "eager" and regime != "gemm")


def test_a_strategy_the_kernel_lacks_is_an_error_not_ignored():
    q = _qfunc(64, 384, 1024, 4, 128)
    q.decode_strategy = "deferred"
    with pytest.raises(ValueError, match="decode_strategy 'deferred' is not implemented by the 'gemm' kernel"):
        q.emit()
    q = _qfunc(16, 384, 1024, 4, 64)
    q.decode_strategy = "deferred"
    with pytest.raises(ValueError, match="available: \\['eager'\\]"):
        q.emit()


def test_config_file_may_only_set_the_search_attributes(tmp_path, monkeypatch):
    import json
    import torch
    from qfactory.core import QMatmul
    path = tmp_path / "cfg.json"
    monkeypatch.setenv("QFACTORY_CONFIG", str(path))
    path.write_text(json.dumps({"4-1-64-512-128": {"decode_strategy": "eager", "l2cache_b": True}}))
    op = QMatmul(1, 64, 512, 4, False, torch.float16, torch.int8, 128)
    func = op.compile_profile()
    assert "decode=eager" in func.runtime.description and "nt_b=0" in func.runtime.description
    path.write_text(json.dumps({"4-1-64-512-128": {"defines": {"QF_GEMV_EXPERIMENT": 1}}}))
    with pytest.raises(ValueError, match="config attribute 'defines'"):
        QMatmul(1, 64, 512, 4, False, torch.float16, torch.int8, 128).compile_profile()
    path.write_text(json.dumps({"4-64-64-512-128": {"decode_strategy": "deferred"}}))
    with pytest.raises(ValueError, match="not implemented by the 'gemm' kernel"):
        QMatmul(64, 64, 512, 4, False, torch.float16, torch.int8, 128).compile_profile()
    path.write_text(json.dumps({"4-64-64-512-128": {"regime": "gemv"}}))
    with pytest.raises(ValueError, match="kernel family"):
        QMatmul(64, 64, 512, 4, False, torch.float16, torch.int8, 128).compile_profile()


def test_timing_experiments_cannot_come_from_the_generator():
    q = _qfunc(1, 64, 512, 4, 128)
    q.defines = {"QF_GEMV_EXPERIMENT": 1}
    with pytest.raises(ValueError, match="not a tuning knob"):
        q.emit()
    q.defines = {"QF_GEMV_WAVES_PER_EU": 4}
    assert "#define QF_GEMV_WAVES_PER_EU 4" in q.emit()


def test_timing_builds_wrap_the_products_own_objects():
    """``bench.py --ablation``: every problem's first build is the object ``QLinear`` runs, the others are the same
    translation unit behind the two defines the headers ask for; no product module refers to them."""
    import torch
    from qfactory.jit import jit
    from qfactory.qlinear import _m_bucket
    seen = set()
    for M, N, K in prebuild.ABLATION_PROBLEMS:
        op, regime, builds = prebuild.ablation_builds(M, N, K)
        assert regime == tiling.regime_for(_m_bucket(M), K, 4, 128, N)
        assert [b for b, _, _ in builds] == [b for b, _ in prebuild.ABLATIONS[regime]] and builds[0][0] == 0
        product = builds[0][2]
        assert not isinstance(product, prebuild.TimingBuild)
        for bits, label, obj in builds[1:]:
            assert isinstance(obj, prebuild.TimingBuild) and obj.regime == regime + "-timing"
            head = f"#define QF_ALLOW_TIMING_EXPERIMENTS 1\n#define {prebuild.TimingBuild.KNOBS[regime]} {bits}\n"
            assert obj.emit() == head + product.emit()
            assert obj.arg_name_type() == product.arg_name_type() and obj.tiling_configs == product.tiling_configs
            path, _ = jit.runtime_path_of(obj)
            assert path not in seen and path != jit.runtime_path_of(product)[0]
            seen.add(path)
    package = os.path.join(os.path.dirname(prebuild.__file__), "qfactory")
    for root, _, files in os.walk(package):
        for name in files:
            if name.endswith(".py"):
                assert "QF_ALLOW_TIMING_EXPERIMENTS" not in open(os.path.join(root, name)).read(), name


def test_swept_gemm_tilings_are_valid_and_override_the_model():
    """core/gemm_tuned_gfx950.json: every entry is a tiling the kernel accepts for its problem, differs from what the
    cost model alone picks (or it would not be there), and is what ``gemm_tiling`` returns; any other problem gets
    the model's choice."""
    import json
    path = os.path.join(os.path.dirname(tiling.__file__), "gemm_tuned_gfx950.json")
    table = json.load(open(path))
    assert table, "the shipped table is empty"
    for key, cfg in table.items():
        nbits, m, n, k, gs = (int(x) for x in key.split("-"))
        assert set(cfg) == {"BM", "NT32", "WN", "WK", "PA"}, key
        assert tiling.gemm_valid(cfg, k, nbits, gs), key
        assert tiling.gemm_tiling(m, n, k, nbits, gs) == cfg, key
        assert tiling.gemm_tiling_model(m, n, k, nbits, gs) != cfg, key
    assert tiling.gemm_tiling(256, 8192 + 128, 8192, 4, 128) == tiling.gemm_tiling_model(256, 8192 + 128, 8192, 4, 128)


def test_swept_gemv_tilings_are_valid_and_override_the_model():
    """core/gemv_tuned_gfx950.json: every entry satisfies the dot2 GEMV kernel's static limits (whole chunks inside a
    group, a power of two of partial sums, a block of at most 1024 threads, the team covering the row), differs from
    the analytic default (or it would not be there) and is what ``gemv_tiling`` returns; pinned parameters and other
    problems get the model."""
    import json
    path = os.path.join(os.path.dirname(tiling.__file__), "gemv_tuned_gfx950.json")
    table = json.load(open(path))
    assert table, "the shipped table is empty"
    for key, cfg in table.items():
        nbits, m, n, k, gs = (int(x) for x in key.split("-"))
        assert set(cfg) == {"MT", "WK", "WN", "U", "STEPS", "VB"}, key
        assert tiling.regime_for(m, k, nbits, gs, n) == "gemv", key
        epc = tiling.elements_per_chunk(nbits, cfg["VB"])
        assert cfg["VB"] in (4, 8, 16) and gs % epc == 0 and (k * tiling.plane_bits(nbits)) % (8 * cfg["VB"]) == 0, key
        v = cfg["U"] * cfg["MT"]
        assert v & (v - 1) == 0 and v <= 64 and 64 * cfg["WK"] * cfg["WN"] <= 1024, key
        assert tiling.gemv_chunks_per_lane(k, nbits, cfg) * 64 * cfg["WK"] >= k // epc, key
        assert tiling.gemv_tiling(m, n, k, nbits, gs) == cfg, key
        assert tiling.gemv_tiling_model(m, n, k, nbits, gs) != cfg, key
        assert tiling.gemv_tiling(m, n, k, nbits, gs, steps=1) == tiling.gemv_tiling_model(m, n, k, nbits, gs, steps=1), key
    assert tiling.gemv_tiling(1, 4096 + 16, 4096, 4, 128) == tiling.gemv_tiling_model(1, 4096 + 16, 4096, 4, 128)


def test_long_rows_take_up_to_sixteen_waves_and_four_stages():
    assert tiling.gemv_tiling_model(1, 8192, 28672, 4, 128) == {"MT": 1, "WK": 14, "WN": 1, "U": 4, "STEPS": 4, "VB": 16}
    assert tiling.gemv_tiling_model(1, 4096, 11008, 4, 128) == {"MT": 1, "WK": 6, "WN": 1, "U": 4, "STEPS": 4, "VB": 16}
    assert tiling.gemv_tiling_model(1, 5120, 13824, 4, 128)["STEPS"] == 1          # 320 sixteen-row blocks: uneven rounds
    assert tiling.gemv_tiling_model(2, 8192, 28672, 4, 128)["WK"] <= 8             # two activation rows: eight waves at most
