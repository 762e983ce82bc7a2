"""The decode loop at its real size: Llama-2-7B shape (32 layers, hidden 4096, 32 heads of 128, SwiGLU 11008, vocab
32000), every linear a W4A16 g128 QLinear, batch 1 / 16 / 64.  The decode step built from single HIP launches
between the linears (and its HIP-graph replay) against the same model evaluated with PyTorch ops between the
linears; both run the same quantized-linear kernels, whose own parity against the oracle at these shapes and row
counts is tests/test_qlinear_gpu.py's business.

Both evaluations are fed the same tokens (the PyTorch evaluation's greedy choices), so that one near-tie in
the logits of random weights cannot send the two down different sequences."""
import pytest
import torch

pytestmark = pytest.mark.gpu

PROMPT, STEPS = 8, 4


def _relative(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


@pytest.fixture(scope="module")
def llama():
    import decode_llama
    return decode_llama


@pytest.mark.parametrize("batch", [1, 16, 64])
def test_full_size_decode_step_matches_the_torch_evaluation(llama, batch):
    print(f"[case] Llama-2-7B shape, batch {batch}", flush=True)
    shape = llama.LlamaShape(max_len=PROMPT + STEPS + 4)
    assert (shape.layers, shape.hidden, shape.heads, shape.mlp, shape.vocab) == (32, 4096, 32, 11008, 32000)
    model = llama.QuantLlama(shape, batch, seed=11)
    g = torch.Generator(device="cuda").manual_seed(12)
    prompt = torch.randint(0, shape.vocab, (batch, PROMPT), device="cuda", generator=g)
    positions = torch.arange(PROMPT, device="cuda")

    # ---- the PyTorch evaluation: prompt, then STEPS greedy tokens ----
    want, tokens = [model.forward(prompt, positions)], []
    for i in range(STEPS):
        tokens.append(want[-1].argmax(-1, keepdim=True))
        want.append(model.forward(tokens[-1], torch.tensor([PROMPT + i], device="cuda")))
    want = torch.stack(want).float()
    want_k, want_v = model.k_cache.clone(), model.v_cache.clone()
    assert torch.isfinite(want).all()

    # ---- prefill with single-launch norm / SiLU steps, then the fused decode step on the same tokens ----
    model.k_cache.zero_(), model.v_cache.zero_()
    got = [model.prefill(prompt, positions)]
    for i in range(STEPS):
        got.append(model.decode_step(tokens[i], torch.tensor([PROMPT + i], device="cuda")).clone())
    got = torch.stack(got).float()
    torch.cuda.synchronize()
    assert torch.isfinite(got).all() and got.shape == (STEPS + 1, batch, shape.vocab)
    assert _relative(got, want) <= 3e-3
    assert _relative(model.k_cache, want_k) <= 3e-3 and _relative(model.v_cache, want_v) <= 3e-3
    # greedy choice: equal, except where the PyTorch evaluation's own margin between the two candidates is
    # within the rounding distance of the two evaluations
    bound = 4 * (got - want).abs().max().item()
    a, b = got.argmax(-1), want.argmax(-1)
    margin = want.gather(-1, b[..., None])[..., 0] - want.gather(-1, a[..., None])[..., 0]
    assert bool(((a == b) | (margin <= bound)).all()), (a != b).sum().item()
    # ... and such ties are rare: at most a tenth of the choices (one, at batch 1, of the five there are)
    assert int((a != b).sum()) <= max(1, a.numel() // 10)

    # ---- the decode step as a HIP graph (static token / position buffers): same bits as the eager step ----
    tok = tokens[STEPS - 2].clone()
    pos = torch.tensor([PROMPT + STEPS - 2], device="cuda")
    out = torch.empty(batch, shape.vocab, dtype=torch.float16, device="cuda")
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
        out.copy_(model.decode_step(tok, pos))
        pos.add_(1)
    torch.cuda.current_stream().wait_stream(side)
    for i in (STEPS - 2, STEPS - 1):                          # replay the last two steps: the cache rows are rewritten with the same values
        tok.copy_(tokens[i])
        pos.fill_(PROMPT + i)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.float(), got[i + 1]), f"graph replay of step {i} differs from the eager step"
    assert int(pos) == PROMPT + STEPS


def test_full_size_prompt_of_128_tokens_then_decode_at_batch_1(llama):
    """configs[4] as written, at batch 1: 128 prompt tokens through ``prefill`` (the GEMM kernels at 128 rows, one
    launch for RoPE and the cache rows), then greedy tokens through the fused decode step, which then attends to
    129 and more cache positions -- against the PyTorch evaluation fed the same tokens."""
    prompt_len, steps = 128, 3
    print("[case] Llama-2-7B shape, batch 1, prompt 128", flush=True)
    shape = llama.LlamaShape(max_len=prompt_len + 128)
    model = llama.QuantLlama(shape, 1, seed=21)
    g = torch.Generator(device="cuda").manual_seed(22)
    prompt = torch.randint(0, shape.vocab, (1, prompt_len), device="cuda", generator=g)
    positions = torch.arange(prompt_len, device="cuda")
    want, tokens = [model.forward(prompt, positions)], []
    for i in range(steps):
        tokens.append(want[-1].argmax(-1, keepdim=True))
        want.append(model.forward(tokens[-1], torch.tensor([prompt_len + i], device="cuda")))
    want = torch.stack(want).float()
    want_k, want_v = model.k_cache.clone(), model.v_cache.clone()
    model.k_cache.zero_(), model.v_cache.zero_()
    got = [model.prefill(prompt, positions)]
    for i in range(steps):
        got.append(model.decode_step(tokens[i], torch.tensor([prompt_len + i], device="cuda")).clone())
    got = torch.stack(got).float()
    torch.cuda.synchronize()
    assert torch.isfinite(got).all() and got.shape == (steps + 1, 1, shape.vocab)
    assert _relative(got, want) <= 3e-3
    assert _relative(model.k_cache, want_k) <= 3e-3 and _relative(model.v_cache, want_v) <= 3e-3
    bound = 4 * (got - want).abs().max().item()
    a, b = got.argmax(-1), want.argmax(-1)
    margin = want.gather(-1, b[..., None])[..., 0] - want.gather(-1, a[..., None])[..., 0]
    assert bool(((a == b) | (margin <= bound)).all())
