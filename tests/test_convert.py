"""convert_params of the package: bit-exact against the pinned oracle, known answers, and the
reference's argument / error behaviour (qfactory/convert.py:3-47,84-97)."""
import numpy as np
import pytest
import torch

from qfactory.convert import (PERMUTE_ORDER, convert_params, unpack_weight, unpack_zero,
                              weight_row_bytes, zero_row_bytes)


def _problem(seed, K, N, nbits, GS, sym=False):
    g = torch.Generator().manual_seed(seed)
    weight = torch.randint(0, 2 ** nbits, (K, N), dtype=torch.int32, generator=g)
    scale = (torch.rand(K // GS, N, generator=g) * 0.019 + 0.001).to(torch.float16)
    zero = None if sym else torch.randint(0, 2 ** nbits, (K // GS, N), dtype=torch.int32, generator=g)
    return weight, scale, zero


def test_permute_order_is_the_reference_table():
    # qfactory/convert.py:49-53
    assert PERMUTE_ORDER[8] == [0, 1, 2, 3]
    assert PERMUTE_ORDER[4] == [0, 2, 4, 6, 1, 3, 5, 7]
    assert PERMUTE_ORDER[2] == [0, 2, 4, 6, 8, 10, 12, 14, 1, 3, 5, 7, 9, 11, 13, 15]


def test_known_answers():
    w = convert_params({"K": 8, "N": 1, "NBITS": 4}, (torch.arange(8, dtype=torch.int32).reshape(8, 1),))
    assert w.dtype == torch.int8 and w.tolist() == [[32, 100, 49, 117]]
    w = convert_params({"K": 16, "N": 1, "NBITS": 2}, ((torch.arange(16, dtype=torch.int32) % 4).reshape(16, 1),))
    assert w.tolist() == [[-120, -120, -35, -35]]
    w = convert_params({"K": 4, "N": 1, "NBITS": 8}, (torch.tensor([[1], [2], [3], [200]], dtype=torch.int32),))
    assert w.tolist() == [[1, 2, 3, -56]]
    weight = torch.zeros(512, 1, dtype=torch.int32)
    scale = torch.ones(4, 1, dtype=torch.float16)
    zero = torch.tensor([[0], [14], [15], [7]], dtype=torch.int32)
    _, s, z = convert_params({"K": 512, "N": 1, "NBITS": 4, "GS": 128}, (weight, scale, zero))
    assert z.dtype == torch.int8 and z.tolist() == [[-15, -113]]
    assert s.shape == (1, 4) and s.is_contiguous()


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,GS", [(256, 1, 32), (512, 3, 64), (1024, 40, 128), (2048, 7, 256)])
def test_bit_exact_against_oracle(oracle, nbits, K, N, GS):
    weight, scale, zero = _problem(nbits * 100 + N, K, N, nbits, GS)
    w, s, z = convert_params({"K": K, "N": N, "NBITS": nbits, "GS": GS}, (weight, scale, zero))
    assert w.shape == (N, weight_row_bytes(K, nbits)) and w.dtype == torch.int8 and w.is_contiguous()
    assert z.shape == (N, zero_row_bytes(K // GS, nbits)) and z.dtype == torch.int8 and z.is_contiguous()
    assert np.array_equal(w.numpy(), oracle.pack_weight(weight.numpy(), nbits))
    assert np.array_equal(z.numpy(), oracle.pack_zero(zero.numpy(), nbits))
    assert np.array_equal(s.numpy(), oracle.transpose_scale(scale.numpy()))
    # group_size-less entry point returns the same weight bytes
    w_only = convert_params({"K": K, "N": N, "NBITS": nbits}, (weight,))
    assert torch.equal(w_only, w)


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
def test_extreme_values_fill_the_sign_bits(oracle, nbits):
    # all fields at maximum: every byte is 0xFF, i.e. the int32 word and the int8 bytes both wrap
    K, N, GS = 256, 2, 32
    weight = torch.full((K, N), 2 ** nbits - 1, dtype=torch.int32)
    zero = torch.full((K // GS, N), 2 ** nbits - 1, dtype=torch.int32)
    scale = torch.ones(K // GS, N, dtype=torch.float16)
    w, _, z = convert_params({"K": K, "N": N, "NBITS": nbits, "GS": GS}, (weight, scale, zero))
    assert torch.all(w == -1)
    assert np.array_equal(z.numpy(), oracle.pack_zero(zero.numpy(), nbits))
    assert np.array_equal(w.numpy(), oracle.pack_weight(weight.numpy(), nbits))


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
def test_inverse_transforms(nbits):
    K, N, GS = 512, 6, 64
    weight, scale, zero = _problem(5, K, N, nbits, GS)
    w, s, z = convert_params({"K": K, "N": N, "NBITS": nbits, "GS": GS}, (weight, scale, zero))
    assert torch.equal(unpack_weight(w, K, nbits), weight.T)
    assert torch.equal(unpack_zero(z, K // GS, nbits), (zero + 1).clamp(max=2 ** nbits - 1).T)


def test_symmetric_returns_no_zero_tensor():
    weight, scale, _ = _problem(1, 256, 4, 4, 128, sym=True)
    w, s, z = convert_params({"K": 256, "N": 4, "NBITS": 4, "GS": 128}, (weight, scale, None))
    assert z is None and w.shape == (4, 128) and s.shape == (4, 2)


def test_argument_errors_match_the_reference():
    weight, scale, zero = _problem(2, 256, 4, 4, 128)
    args = {"K": 256, "N": 4, "NBITS": 4, "GS": 128}
    with pytest.raises(ValueError):
        convert_params(args, (weight, scale))                       # grouped path needs 3 params
    with pytest.raises(ValueError):
        convert_params({"K": 256, "N": 4, "NBITS": 4}, (weight, scale))   # plain path needs 1
    with pytest.raises(AssertionError):
        convert_params(args, (weight.to(torch.int64), scale, zero))  # dtype
    with pytest.raises(AssertionError):
        convert_params(args, (weight + 16, scale, zero))             # range
    with pytest.raises(AssertionError):
        convert_params(args, (weight.T.contiguous(), scale, zero))   # shape (N,K) instead of (K,N)
    with pytest.raises(AssertionError):
        convert_params(args, (weight, scale.float(), zero))          # scale dtype
    with pytest.raises(AssertionError):
        convert_params(args, (weight, scale, zero - 1))              # zero range


def test_large_layer_is_fast_enough():
    # the reference loops over K in Python (convert.py:58-66); this must stay a whole-tensor operation
    import time
    K, N = 4096, 4096
    weight, scale, zero = _problem(3, K, N, 4, 128)
    t = time.perf_counter()
    convert_params({"K": K, "N": N, "NBITS": 4, "GS": 128}, (weight, scale, zero))
    assert time.perf_counter() - t < 20.0
