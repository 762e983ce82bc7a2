"""GPU parity of the device-side repacking (libqfactory_hip.so through its C ABI) against the CPU
oracle: packed bytes must be identical."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPES = [(32, 1), (64, 5), (256, 100), (4096, 4096), (11008, 260), (8192, 33)]


def _tensors(seed, K, N, nbits, GS):
    g = torch.Generator().manual_seed(seed)
    weight = torch.randint(0, 2 ** nbits, (K, N), dtype=torch.int32, generator=g)
    G = K // GS
    scale = (torch.rand(G, N, generator=g) * 0.019 + 0.001).to(torch.float16)
    zero = torch.randint(0, 2 ** nbits, (G, N), dtype=torch.int32, generator=g)
    zero[0, 0] = 2 ** nbits - 1                      # the "+1" of the stored zero-point saturates
    zero[-1, -1] = 0
    return weight, scale, zero


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N", SHAPES)
def test_device_packers_match_oracle(oracle, nbits, K, N):
    from qfactory import native
    GS = 32 if K % 256 else 128
    if (K // GS) % 2 or ((K // GS) % 4 and nbits == 2):
        GS = K // 4
    print(f"[case] pack b{nbits} K{K} N{N} GS{GS}", flush=True)
    weight, scale, zero = _tensors(K + N + nbits, K, N, nbits, GS)
    w = native.pack_weight(weight.cuda(), nbits)
    s = native.transpose_scale(scale.cuda())
    z = native.pack_zero(zero.cuda(), nbits)
    torch.cuda.synchronize()
    assert w.dtype == torch.int8 and w.shape == (N, K * nbits // 8)
    assert np.array_equal(w.cpu().numpy(), oracle.pack_weight(weight.numpy(), nbits))
    assert np.array_equal(s.cpu().numpy(), oracle.transpose_scale(scale.numpy()))
    assert np.array_equal(z.cpu().numpy(), oracle.pack_zero(zero.numpy(), nbits))


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
def test_convert_params_same_bytes_on_both_devices(nbits):
    """convert_params takes the HIP packers for device tensors and whole-tensor torch ops for host
    tensors; the two must agree byte for byte, also through a pack -> unpack round trip."""
    from qfactory import convert
    K, N, GS = 1024, 300, 128
    weight, scale, zero = _tensors(7 + nbits, K, N, nbits, GS)
    args = {"K": K, "N": N, "NBITS": nbits, "GS": GS}
    w0, s0, z0 = convert.convert_params(args, (weight, scale, zero))
    w1, s1, z1 = convert.convert_params(args, (weight.cuda(), scale.cuda(), zero.cuda()))
    assert w1.is_cuda and s1.is_cuda and z1.is_cuda
    assert torch.equal(w0, w1.cpu()) and torch.equal(s0, s1.cpu()) and torch.equal(z0, z1.cpu())
    assert torch.equal(convert.unpack_weight(w1, K, nbits).cpu(), weight.T)
    assert torch.equal(convert.unpack_zero(z1, K // GS, nbits).cpu(), (zero + 1).clamp(max=2 ** nbits - 1).T)
    w_only = convert.convert_params({"K": K, "N": N, "NBITS": nbits}, (weight.cuda(),))
    assert torch.equal(w_only.cpu(), w0)


def test_k_not_filling_words_uses_tensor_ops_on_device():
    """8-bit weights need only K % 4 == 0 (reference: convert.py:55-68); such K bypass the word packer."""
    from qfactory import convert
    K, N = 36, 7
    g = torch.Generator().manual_seed(3)
    weight = torch.randint(0, 256, (K, N), dtype=torch.int32, generator=g)
    w_dev = convert.convert_params({"K": K, "N": N, "NBITS": 8}, (weight.cuda(),))
    w_cpu = convert.convert_params({"K": K, "N": N, "NBITS": 8}, (weight,))
    assert torch.equal(w_dev.cpu(), w_cpu)


def test_bad_arguments_are_rejected_without_launching():
    from qfactory import native
    lib = native.load()
    buf = torch.zeros(64, dtype=torch.int32, device="cuda")
    assert lib.qf_pack_weight(buf.data_ptr(), buf.data_ptr(), 48, 1, 4, None) == 1      # K % 32
    assert lib.qf_pack_weight(buf.data_ptr(), buf.data_ptr(), 32, 1, 5, None) == 1      # nbits
    assert lib.qf_pack_zero(buf.data_ptr(), buf.data_ptr(), 3, 1, 4, None) == 1         # G % 2
    assert lib.qf_stream_copy(buf.data_ptr(), buf.data_ptr(), 24, None) == 1            # bytes % 16
    assert lib.qf_pack_weight(None, buf.data_ptr(), 32, 1, 4, None) == 1
