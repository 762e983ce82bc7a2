"""Persisted tiling choices: the writer (qfactory.tune) and the reader ($QFACTORY_CONFIG lookup in
compile_profile) agree on the reference's schema "{nbits}-{m}-{n}-{k}-{gs}" -> attributes."""
import json

import pytest
import torch


def test_config_round_trip_selects_the_stored_tiling(tmp_path, monkeypatch):
    from qfactory import tune
    from qfactory.core import QMatmul
    op = QMatmul(1, 64, 512, 4, False, torch.float16, torch.int8, 128)
    op.compile_profile()
    default = op.best_qfunc
    stored = tune.entry_of(default.clone(tiling_configs=dict(default.tiling_configs, WN=1, STEPS=2)))
    assert set(stored) >= {"regime", "decode_strategy", "l2cache_b", "tiling_configs"}
    path = tmp_path / "best_config.json"
    tune.update_config(str(path), {tune.shape_key(4, 1, 64, 512, 128): stored})
    tune.update_config(str(path), {tune.shape_key(4, 1, 8, 8, 8): {"tiling_configs": {}}})      # merge keeps both
    assert set(json.load(open(path))) == {"4-1-64-512-128", "4-1-8-8-8"}
    monkeypatch.setenv("QFACTORY_CONFIG", str(path))
    op2 = QMatmul(1, 64, 512, 4, False, torch.float16, torch.int8, 128)
    func = op2.compile_profile(enable_lower=True)           # the stored entry wins over the search
    assert op2.best_qfunc.tiling_configs["WN"] == 1 and op2.best_qfunc.tiling_configs["STEPS"] == 2
    assert "WN=1" in func.runtime.description and "STEPS=2" in func.runtime.description


@pytest.mark.gpu
def test_search_on_device_and_latency_harness(tmp_path):
    from qfactory import testing, tune
    key, entry = tune.tune_shape(4, 1, 64, 256, 128)
    assert key == "4-1-64-256-128" and entry["regime"] == "gemv" and entry["tiling_configs"]["VB"] in (4, 8, 16)
    tq, td, ratio = testing.speedup_over_dense(1, 512, 1024)
    assert 0 < tq < 1e-3 and 0 < td < 1e-3 and ratio > 0
    assert testing.CuBLASLatencyTest is testing.DenseLatencyTest
