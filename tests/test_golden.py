"""Hand-worked known-answer vectors (tests/golden/packing_kats.json) against the CPU oracle, the host
convert_params and -- on the GPU -- the HIP packers."""
import json
import os

import numpy as np
import pytest
import torch

GOLDEN = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "packing_kats.json")))


def _weight_of(entry):
    if entry["weight_kn"] == "k % 8":
        return (np.arange(entry["K"], dtype=np.int32) % 8).reshape(entry["K"], 1)
    return np.array(entry["weight_kn"], dtype=np.int32)


@pytest.mark.parametrize("entry", GOLDEN["weight"], ids=lambda e: f"b{e['nbits']}")
def test_weight_vectors(oracle, entry):
    from qfactory import convert
    W = _weight_of(entry)
    want = np.array(entry["packed_u8"], dtype=np.uint8)
    assert np.array_equal(oracle.pack_weight(W, entry["nbits"]).view(np.uint8), want)
    got = convert.convert_params({"K": W.shape[0], "N": W.shape[1], "NBITS": entry["nbits"]}, (torch.from_numpy(W),))
    assert np.array_equal(got.numpy().view(np.uint8), want)
    if "packed_i8" in entry:
        assert got.numpy().tolist() == entry["packed_i8"]
    assert np.array_equal(oracle.unpack_weight(got.numpy(), W.shape[0], entry["nbits"]), W.T)


@pytest.mark.parametrize("entry", GOLDEN["zero"], ids=lambda e: f"b{e['nbits']}")
def test_zero_vectors(oracle, entry):
    from qfactory import convert
    Z = np.array(entry["zero_gn"], dtype=np.int32)
    want = np.array(entry["packed_u8"], dtype=np.uint8)
    assert np.array_equal(oracle.pack_zero(Z, entry["nbits"]).view(np.uint8), want)
    got = convert._transform_zero(0, 1, 0, torch.from_numpy(Z), entry["nbits"])
    assert got.numpy().tolist() == entry["packed_i8"]


def test_decode_order_vector():
    e = GOLDEN["decode"][0]
    b, w = e["nbits"], e["word"]
    mask = (1 << b) - 1
    got = []
    for i in range(16 // b):
        got += [(w >> (b * i)) & mask, (w >> (b * i + 16)) & mask]
    assert got == e["elements"]


@pytest.mark.gpu
def test_device_packers_on_the_vectors():
    from qfactory import native
    for entry in GOLDEN["weight"]:
        if entry["K"] % 32:
            continue                      # the word packer takes whole 32-element words
        W = torch.from_numpy(_weight_of(entry)).cuda()
        got = native.pack_weight(W, entry["nbits"]).cpu().numpy().view(np.uint8)
        assert np.array_equal(got, np.array(entry["packed_u8"], dtype=np.uint8))
    for entry in GOLDEN["zero"]:
        Z = torch.tensor(entry["zero_gn"], dtype=torch.int32).cuda()
        got = native.pack_zero(Z, entry["nbits"]).cpu().numpy()
        assert got.tolist() == entry["packed_i8"]


# ---- the reference packer's own output (tests/golden/convert_fixtures.npz, written by
# tests/golden/make_convert_fixtures.py from qfactory/convert.py:55-97 in the build container) ----
FIXTURES = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "convert_fixtures.npz"))
FIXTURE_NAMES = [str(n) for n in FIXTURES["names"]]


def _fixture(name):
    b, K, N, GS = (int(part[1:] if part[0] in "bKN" else part[2:]) for part in name.split("_"))
    return b, K, N, GS, {k: FIXTURES[f"{name}/{k}"] for k in ("weight", "scale", "zero", "w", "s", "z")}


def test_fixture_file_covers_the_widths_and_the_clamp():
    assert len(FIXTURE_NAMES) >= 12 and {n.split("_")[0] for n in FIXTURE_NAMES} == {"b2", "b4", "b8"}
    for name in FIXTURE_NAMES:
        b, K, N, GS, f = _fixture(name)
        assert f["zero"].max() == 2 ** b - 1 and f["zero"].min() == 0       # the clamp at 2^b - 1 and the +1 at 0
        assert f["w"].shape == (N, K * b // 8) and f["w"].dtype == np.int8
        assert f["z"].shape == (N, K // GS * b // 8) and f["s"].shape == (N, K // GS)


@pytest.mark.parametrize("name", FIXTURE_NAMES)
def test_oracle_packers_reproduce_the_reference_output(oracle, name):
    b, K, N, GS, f = _fixture(name)
    assert np.array_equal(oracle.pack_weight(f["weight"], b), f["w"])
    assert np.array_equal(oracle.pack_zero(f["zero"], b), f["z"])
    assert np.array_equal(oracle.transpose_scale(f["scale"]).view(np.uint16), f["s"].view(np.uint16))


@pytest.mark.parametrize("name", FIXTURE_NAMES)
def test_host_convert_params_reproduces_the_reference_output(name):
    from qfactory import convert
    b, K, N, GS, f = _fixture(name)
    w, s, z = convert.convert_params({"K": K, "N": N, "NBITS": b, "GS": GS},
                                     tuple(torch.from_numpy(f[k]) for k in ("weight", "scale", "zero")))
    assert w.dtype == torch.int8 and z.dtype == torch.int8 and s.dtype == torch.float16
    assert np.array_equal(w.numpy(), f["w"]) and np.array_equal(z.numpy(), f["z"])
    assert np.array_equal(s.numpy().view(np.uint16), f["s"].view(np.uint16))
    w_sym, _, z_sym = convert.convert_params({"K": K, "N": N, "NBITS": b, "GS": GS},
                                             (torch.from_numpy(f["weight"]), torch.from_numpy(f["scale"]), None))
    assert z_sym is None and np.array_equal(w_sym.numpy(), f["w"])
    w_plain = convert.convert_params({"K": K, "N": N, "NBITS": b}, (torch.from_numpy(f["weight"]),))
    assert np.array_equal(w_plain.numpy(), f["w"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", FIXTURE_NAMES)
def test_device_packers_reproduce_the_reference_output(name):
    """convert_params on device tensors runs the HIP packers (qf_pack_weight / qf_pack_zero / qf_transpose_scale)."""
    from qfactory import convert
    b, K, N, GS, f = _fixture(name)
    w, s, z = convert.convert_params({"K": K, "N": N, "NBITS": b, "GS": GS},
                                     tuple(torch.from_numpy(f[k]).cuda() for k in ("weight", "scale", "zero")))
    assert w.is_cuda and s.is_cuda and z.is_cuda
    assert np.array_equal(w.cpu().numpy(), f["w"]) and np.array_equal(z.cpu().numpy(), f["z"])
    assert np.array_equal(s.cpu().numpy().view(np.uint16), f["s"].view(np.uint16))
