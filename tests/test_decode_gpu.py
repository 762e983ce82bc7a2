"""The Llama-shaped decode loop on a tiny model: logits with QLinear layers against the same model
evaluated with dense fp32 matmuls on the dequantised weights (prefill and three decode steps)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _dense(lin, x):
    """fp32 evaluation of a quantized linear from its packed tensors: DQ = fp16((q - Z) * s)."""
    from qfactory import convert
    K, N, gs, nbits = lin.in_features, lin.out_features, lin.group_size, lin.n_bits
    q = convert.unpack_weight(lin.w, K, nbits).float()
    z = convert.unpack_zero(lin.z, K // gs, nbits).float().repeat_interleave(gs, dim=1)
    s = lin.s.float().repeat_interleave(gs, dim=1)
    dq = ((q - z) * s).to(torch.float16).float()
    return (x.float() @ dq.T).to(torch.float16)


def _run(model, prompt, steps):
    model.k_cache.zero_(), model.v_cache.zero_()
    T = prompt.shape[1]
    logits = [model.forward(prompt, torch.arange(T, device="cuda"))]
    for i in range(steps):
        tok = logits[-1].argmax(-1, keepdim=True)
        logits.append(model.forward(tok, torch.tensor([T + i], device="cuda")))
    return torch.stack(logits).float()


def test_tiny_model_logits_match_dense_evaluation():
    import decode_llama
    shape = decode_llama.LlamaShape(layers=2, hidden=256, heads=4, mlp=512, vocab=1000, max_len=32, group_size=64)
    model = decode_llama.QuantLlama(shape, batch=2, seed=3)
    prompt = torch.randint(0, shape.vocab, (2, 8), device="cuda", generator=torch.Generator(device="cuda").manual_seed(4))
    got = _run(model, prompt, 3)
    model.linear = _dense
    want = _run(model, prompt, 3)
    torch.cuda.synchronize()
    assert torch.isfinite(got).all() and got.shape == (4, 2, shape.vocab)
    nrms = ((got - want).norm() / want.norm()).item()
    assert nrms <= 5e-3, nrms                # several layers of fp16 rounding between the two evaluations
    assert torch.equal(got[0].argmax(-1), want[0].argmax(-1))


def test_graph_decode_runs_and_reports():
    import decode_llama
    shape = decode_llama.LlamaShape(layers=2, hidden=256, heads=4, mlp=512, vocab=1000, max_len=32, group_size=64)
    rec = decode_llama.run(shape, batch=2, prompt_len=8, new_tokens=6)
    assert rec["value"] > 0 and 0 < rec["quantized_linear_share"] <= 1.5
