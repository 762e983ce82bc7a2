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
