"""The vLLM plugin file against a stand-in of vLLM's base classes: same class / method names and
signatures as the reference's hook (third_party/vllm-qfactory.patch:47-214), registered parameter
shapes, and -- on the GPU -- a loaded GPTQ layer that computes what the oracle computes."""
import inspect

import numpy as np
import pytest
import torch

import vllm_stub


@pytest.fixture(scope="module")
def plugin():
    vllm_stub.install()
    from qfactory.integrations import vllm_qfactory
    return vllm_qfactory


def test_config_interface(plugin):
    cfg = plugin.QFactoryConfig.from_config({"bits": 4, "group_size": 128, "desc_act": False})
    assert (cfg.weight_bits, cfg.group_size, cfg.pack_factor) == (4, 128, 8)
    assert cfg.get_name() == "qfactory"
    assert cfg.get_supported_act_dtypes() == [torch.float16]
    assert isinstance(plugin.QFactoryConfig.get_min_capability(), int)
    assert plugin.QFactoryConfig.override_quantization_method({}, "qfactory") == "qfactory"
    assert plugin.QFactoryConfig.override_quantization_method({}, "gptq") is None
    with pytest.raises(NotImplementedError):
        plugin.QFactoryConfig.get_config_filenames()
    assert isinstance(cfg.get_quant_method(vllm_stub.LinearBase(), "model.layers.0.o_proj"), plugin.QFactoryLinearMethod)
    assert cfg.get_quant_method(torch.nn.Linear(2, 2), "lm_head") is None


def test_method_signatures_match_the_reference_hook(plugin):
    m = plugin.QFactoryLinearMethod
    assert list(inspect.signature(m.__init__).parameters) == ["self", "quant_config", "prefix"]
    assert list(inspect.signature(m.create_weights).parameters) == [
        "self", "layer", "input_size_per_partition", "output_partition_sizes", "input_size", "output_size",
        "params_dtype", "extra_weight_attrs"]
    assert list(inspect.signature(m.process_weights_after_loading).parameters) == ["self", "layer"]
    sig = inspect.signature(m.apply)
    assert list(sig.parameters) == ["self", "layer", "x", "bias"] and sig.parameters["bias"].default is None
    assert list(inspect.signature(plugin.QFactoryConfig.__init__).parameters) == ["self", "weight_bits", "group_size"]


def test_create_weights_registers_gptq_tensors(plugin):
    cfg = plugin.QFactoryConfig(4, 128)
    method = cfg.get_quant_method(vllm_stub.LinearBase(), "qkv_proj")
    layer = vllm_stub.LinearBase()
    loader = object()
    method.create_weights(layer, 1024, [256, 64, 64], 1024, 384, torch.float16, weight_loader=loader)
    assert layer.qweight.shape == (128, 384) and layer.qweight.dtype == torch.int32
    assert layer.qzeros.shape == (8, 48) and layer.qzeros.dtype == torch.int32
    assert layer.scales.shape == (8, 384) and layer.scales.dtype == torch.float16
    assert layer.g_idx.shape == (1024,)
    # a checkpoint that carries no g_idx tensor leaves this value: it must already say "no reordering"
    from qfactory.integrations import gptq_format as gf
    gf.check_trivial_g_idx(layer.g_idx.data, 128)
    assert layer.qweight.attrs["packed_dim"] == 0 and layer.qzeros.attrs["packed_dim"] == 1
    assert layer.qweight.attrs["packed_factor"] == 8 and layer.qweight.attrs["weight_loader"] is loader


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_gptq_word_format_round_trip(bits):
    from qfactory.integrations import gptq_format as gf
    g = torch.Generator().manual_seed(bits)
    K, N, GS = 256, 64, 64
    W = torch.randint(0, 2 ** bits, (K, N), dtype=torch.int32, generator=g)
    Z = torch.randint(0, 2 ** bits, (K // GS, N), dtype=torch.int32, generator=g)
    qw, qz = gf.pack_qweight(W, bits), gf.pack_qzeros(Z, bits)
    assert qw.shape == (K * bits // 32, N) and qz.shape == (K // GS, N * bits // 32)
    # known answer: element j of a word sits in bits [j*bits, (j+1)*bits), consecutive K per word
    word0 = sum(int(W[j, 0]) << (j * bits) for j in range(32 // bits))
    assert int(qw[0, 0]) & 0xFFFFFFFF == word0
    zword0 = sum(int(Z[0, j]) << (j * bits) for j in range(32 // bits))
    assert int(qz[0, 0]) & 0xFFFFFFFF == zword0
    assert torch.equal(gf.unpack_qweight(qw, bits), W) and torch.equal(gf.unpack_qzeros(qz, bits), Z)
    gf.check_trivial_g_idx(torch.arange(K, dtype=torch.int32) // GS, GS)
    with pytest.raises(NotImplementedError):
        gf.check_trivial_g_idx(torch.arange(K, dtype=torch.int32).flip(0) // GS, GS)


def test_activation_reordered_checkpoint_is_rejected_at_load(plugin):
    """A desc_act checkpoint (g_idx is a permutation of the groups) must not load: the kernels assume group
    k // group_size.  The check runs on the loaded ``layer.g_idx`` before any device work."""
    from qfactory.integrations import gptq_format as gf
    g = torch.Generator().manual_seed(9)
    K, N, GS, bits = 512, 64, 128, 4
    cfg = plugin.QFactoryConfig(bits, GS)
    method = cfg.get_quant_method(vllm_stub.LinearBase(), "o_proj")
    layer = vllm_stub.LinearBase()
    method.create_weights(layer, K, [N], K, N, torch.float16, weight_loader=None)
    layer.qweight.data.copy_(gf.pack_qweight(torch.randint(0, 16, (K, N), dtype=torch.int32, generator=g), bits))
    layer.qzeros.data.copy_(gf.pack_qzeros(torch.randint(0, 16, (K // GS, N), dtype=torch.int32, generator=g), bits))
    layer.scales.data.fill_(0.01)
    layer.g_idx.data.copy_((torch.arange(K, dtype=torch.int32) // GS)[torch.randperm(K, generator=g)])
    with pytest.raises(NotImplementedError):
        method.process_weights_after_loading(layer)
    assert layer.qweight is not None                       # nothing was torn down


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [1, 40])
def test_loaded_layer_matches_oracle(plugin, oracle, rows):
    from qfactory.integrations import gptq_format as gf
    g = torch.Generator().manual_seed(5)
    K, N, GS, bits = 1024, 384, 128, 4
    W = torch.randint(0, 16, (K, N), dtype=torch.int32, generator=g)
    Z = torch.randint(0, 16, (K // GS, N), dtype=torch.int32, generator=g)
    S = (torch.rand(K // GS, N, generator=g) * 0.019 + 0.001).to(torch.float16)
    cfg = plugin.QFactoryConfig(bits, GS)
    method = cfg.get_quant_method(vllm_stub.LinearBase(), "qkv_proj")
    layer = vllm_stub.LinearBase()
    method.create_weights(layer, K, [N], K, N, torch.float16, weight_loader=None)
    layer = layer.cuda()
    layer.qweight.data.copy_(gf.pack_qweight(W, bits))
    layer.qzeros.data.copy_(gf.pack_qzeros(Z, bits))
    layer.scales.data.copy_(S)
    if rows == 1:
        layer.g_idx.data.copy_(torch.arange(K, dtype=torch.int32) // GS)
    # rows == 40: g_idx is never written, as with a checkpoint that has no such tensor
    method.process_weights_after_loading(layer)
    assert layer.qweight is None and layer.qzeros is None
    x = torch.randn(2, rows // 2 if rows > 1 else 1, K, generator=g).to(torch.float16)[: (2 if rows > 1 else 1)]
    bias = torch.randn(N, generator=g).to(torch.float16)
    out = method.apply(layer, x.cuda(), bias.cuda())
    torch.cuda.synchronize()
    assert out.shape == (*x.shape[:-1], N)
    w = oracle.pack_weight(W.numpy(), bits)
    z = oracle.pack_zero(Z.numpy(), bits)
    ref = oracle.qlinear(x.reshape(-1, K).numpy(), w, oracle.transpose_scale(S.numpy()), z, bits, GS)
    ref = (torch.from_numpy(ref.astype(np.float32)).to(torch.float16) + bias).numpy().astype(np.float32)
    m = oracle.error_metrics(out.reshape(-1, N).cpu().numpy(), ref)
    assert m["max_rel"] <= 1e-2 and m["nrms"] <= 1e-3, m
