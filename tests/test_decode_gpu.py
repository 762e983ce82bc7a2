"""The Llama-shaped decode loop on a tiny model: logits with QLinear layers against the same model
evaluated with dense fp32 matmuls on the dequantised weights (prefill and three decode steps), and
the single-launch steps between the linears of a decode token against the PyTorch ops they replace."""
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


# ---- the per-token steps between the linears (libqfactory_hip.so through its C ABI) ----

def _gen(seed):
    return torch.Generator(device="cuda").manual_seed(seed)


@pytest.mark.parametrize("rows,hidden,with_delta", [(1, 4096, True), (16, 4096, False), (3, 256, True), (5, 11008, True),
                                                    (2, 16384, True), (7, 8, False)])
def test_add_rmsnorm_matches_torch(rows, hidden, with_delta):
    from qfactory import native
    g = _gen(rows * 31 + hidden)
    x = torch.randn(rows, hidden, device="cuda", generator=g).to(torch.float16)
    delta = (torch.randn(rows, hidden, device="cuda", generator=g) * 0.3).to(torch.float16) if with_delta else None
    w = (torch.rand(hidden, device="cuda", generator=g) + 0.5).to(torch.float16)
    want_x = x + delta if with_delta else x.clone()
    xf = want_x.float()
    want = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).to(torch.float16) * w
    out = torch.empty_like(x)
    native.add_rmsnorm(x, delta, w, out, 1e-5)
    assert torch.equal(x, want_x)                                   # the fp16 residual add is exact
    # the mean of squares is summed in another order: at most one fp16 ulp on a few elements
    assert (out.float() - want.float()).abs().max() <= 2e-3 * want.float().abs().max()
    assert ((out.float() - want.float()).norm() / want.float().norm()).item() <= 2e-4


@pytest.mark.parametrize("B,H,hd,max_len,pos", [(1, 32, 128, 256, 0), (2, 4, 64, 32, 8), (16, 32, 128, 256, 200),
                                                (3, 5, 32, 40, 39), (2, 2, 256, 300, 299), (40, 32, 64, 64, 50)])
def test_rope_cache_append_and_attention_match_torch(B, H, hd, max_len, pos):
    import torch.nn.functional as F
    from qfactory import native
    g = _gen(B * 1000 + pos)
    qkv = torch.randn(B, 3 * H * hd, device="cuda", generator=g).to(torch.float16)
    k_cache = torch.randn(B, H, max_len, hd, device="cuda", generator=g).to(torch.float16)
    v_cache = torch.randn(B, H, max_len, hd, device="cuda", generator=g).to(torch.float16)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, device="cuda", dtype=torch.float32) / hd))
    ang = torch.arange(max_len, device="cuda", dtype=torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos(), ang.sin()
    pos_t = torch.tensor([pos], device="cuda", dtype=torch.int64)

    def rope(x):                                                    # (B, H, hd), pairs (2i, 2i+1)
        xf = x.float()
        x0, x1 = xf[..., 0::2], xf[..., 1::2]
        return torch.stack((x0 * cos[pos] - x1 * sin[pos], x0 * sin[pos] + x1 * cos[pos]), dim=-1).flatten(-2).to(torch.float16)

    q3 = qkv.reshape(B, 3, H, hd)
    want_q, want_k = rope(q3[:, 0]), rope(q3[:, 1])
    want_kc, want_vc = k_cache.clone(), v_cache.clone()
    want_kc[:, :, pos], want_vc[:, :, pos] = want_k, q3[:, 2]
    mask = (torch.arange(max_len, device="cuda") <= pos)[None, None, None]
    want_att = F.scaled_dot_product_attention(want_q[:, :, None].float(), want_kc.float(), want_vc.float(), attn_mask=mask)
    want_att = want_att[:, :, 0].reshape(B, H * hd)

    q_out, att = torch.empty(B, H * hd, dtype=torch.float16, device="cuda"), torch.empty(B, H * hd, dtype=torch.float16, device="cuda")
    k_before, v_before = k_cache.clone(), v_cache.clone()
    native.rope_kv_store(qkv, pos_t, cos, sin, q_out, k_cache, v_cache)
    native.decode_attention(q_out, k_cache, v_cache, pos_t, att)
    # the single-launch form gives the same bits as the two steps
    att_fused = torch.empty_like(att)
    native.rope_decode_attention(qkv, pos_t, cos, sin, k_before, v_before, att_fused)
    assert torch.equal(k_before, k_cache) and torch.equal(v_before, v_cache) and torch.equal(att_fused, att)
    # rotation: fp32 products of the same table entries, rounded once to fp16 (a fused multiply-add may differ by one ulp)
    assert (q_out.float() - want_q.reshape(B, -1).float()).abs().max() <= 4e-3
    assert (k_cache.float() - want_kc.float()).abs().max() <= 4e-3
    assert torch.equal(v_cache, want_vc)
    untouched = torch.arange(max_len, device="cuda") != pos
    assert torch.equal(k_cache[:, :, untouched], want_kc[:, :, untouched])
    assert ((att.float() - want_att).norm() / want_att.norm()).item() <= 2e-3
    assert (att.float() - want_att).abs().max() <= 1e-2 * want_att.abs().max() + 2e-3


def test_rope_and_cache_write_of_a_whole_prompt():
    """``qf_rope_kv_store_rows`` (prefill): every token of every sequence gets the rotation and the cache rows the
    one-position kernel gives it, bit for bit, and what the PyTorch ops of ``QuantLlama.forward`` give within the
    rounding of the rotation; a token outside the cache writes nothing."""
    from qfactory import native
    B, T, H, hd, max_len = 3, 6, 4, 64, 16
    g = torch.Generator(device="cuda").manual_seed(5)
    qkv = torch.randn(B * T, 3 * H * hd, device="cuda", generator=g).to(torch.float16)
    inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, device="cuda", dtype=torch.float32) / hd))
    ang = torch.arange(max_len, device="cuda", dtype=torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos(), ang.sin()
    pos = torch.tensor([3, 4, 5, 9, max_len, 0], device="cuda", dtype=torch.int64)      # one token outside the cache
    k0 = torch.randn(B, H, max_len, hd, device="cuda", generator=g).to(torch.float16)
    v0 = torch.randn(B, H, max_len, hd, device="cuda", generator=g).to(torch.float16)
    k_cache, v_cache = k0.clone(), v0.clone()
    q_rows = torch.full((B, T, H, hd), 7.0, dtype=torch.float16, device="cuda")
    native.rope_kv_store_rows(qkv, pos, cos, sin, q_rows, k_cache, v_cache)
    torch.cuda.synchronize()
    q_out = q_rows.transpose(1, 2)                                                        # (B, H, T, hd)
    # token by token through the one-position kernel
    want_k, want_v = k0.clone(), v0.clone()
    want_q = torch.full((B, H, T, hd), 7.0, dtype=torch.float16, device="cuda")
    rows = qkv.reshape(B, T, 3 * H * hd)
    for t in range(T):
        q1 = torch.empty(B, H * hd, dtype=torch.float16, device="cuda")
        p = int(pos[t])
        native.rope_kv_store(rows[:, t].contiguous(), pos[t:t + 1].clone(), cos, sin, q1, want_k, want_v)
        if 0 <= p < max_len:
            want_q[:, :, t] = q1.reshape(B, H, hd)
    torch.cuda.synchronize()
    assert torch.equal(q_out, want_q) and torch.equal(k_cache, want_k) and torch.equal(v_cache, want_v)
    # and the PyTorch ops
    valid = (pos >= 0) & (pos < max_len)
    x = rows.reshape(B, T, 3, H, hd).permute(2, 0, 3, 1, 4).float()                      # (3, B, H, T, hd)
    c, s_ = cos.index_select(0, pos.clamp(0, max_len - 1))[None, None], sin.index_select(0, pos.clamp(0, max_len - 1))[None, None]

    def rope(xf):
        x0, x1 = xf[..., 0::2], xf[..., 1::2]
        return torch.stack((x0 * c - x1 * s_, x0 * s_ + x1 * c), dim=-1).flatten(-2).to(torch.float16)

    tq, tk = rope(x[0]), rope(x[1])
    assert (q_out[:, :, valid].float() - tq[:, :, valid].float()).abs().max() <= 4e-3
    assert (k_cache[:, :, pos[valid]].float() - tk[:, :, valid].float()).abs().max() <= 4e-3
    assert torch.equal(v_cache[:, :, pos[valid]], x[2][:, :, valid].to(torch.float16))
    untouched = torch.ones(max_len, dtype=torch.bool, device="cuda")
    untouched[pos[valid]] = False
    assert torch.equal(k_cache[:, :, untouched], k0[:, :, untouched]) and torch.equal(v_cache[:, :, untouched], v0[:, :, untouched])
    assert torch.equal(q_out[:, :, ~valid], torch.full_like(q_out[:, :, ~valid], 7.0))


def test_rope_writes_nothing_for_a_position_outside_the_cache():
    from qfactory import native
    B, H, hd, max_len = 2, 4, 64, 16
    qkv = torch.randn(B, 3 * H * hd, device="cuda").to(torch.float16)
    k_cache = torch.zeros(B, H, max_len, hd, dtype=torch.float16, device="cuda")
    v_cache = torch.zeros_like(k_cache)
    cos = torch.ones(max_len, hd // 2, device="cuda")
    sin = torch.zeros_like(cos)
    q_out = torch.zeros(B, H * hd, dtype=torch.float16, device="cuda")
    native.rope_kv_store(qkv, torch.tensor([max_len], device="cuda"), cos, sin, q_out, k_cache, v_cache)
    native.rope_decode_attention(qkv, torch.tensor([max_len], device="cuda"), cos, sin, k_cache, v_cache, q_out)
    native.rope_decode_attention(qkv, torch.tensor([-1], device="cuda"), cos, sin, k_cache, v_cache, q_out)
    torch.cuda.synchronize()
    assert not k_cache.any() and not v_cache.any() and not q_out.any()


@pytest.mark.parametrize("rows,mlp", [(1, 11008), (16, 11008), (3, 512), (64, 8)])
def test_silu_mul_matches_torch(rows, mlp):
    import torch.nn.functional as F
    from qfactory import native
    gu = (torch.randn(rows, 2 * mlp, device="cuda", generator=_gen(rows + mlp)) * 3).to(torch.float16)
    want = F.silu(gu[:, :mlp]) * gu[:, mlp:]
    out = torch.empty(rows, mlp, dtype=torch.float16, device="cuda")
    native.silu_mul(gu, out)
    assert (out.float() - want.float()).abs().max() <= 2e-3 * want.float().abs().max()      # exp() of two libraries: one ulp
    assert ((out.float() - want.float()).norm() / want.float().norm()).item() <= 2e-4


@pytest.mark.parametrize("batch,vocab,hidden", [(1, 32000, 4096), (16, 32000, 4096), (64, 1000, 256), (3, 8, 8), (2, 40000, 64)])
def test_greedy_next_matches_argmax_position_update_and_embedding_lookup(batch, vocab, hidden):
    from qfactory import native
    g = _gen(batch + vocab)
    logits = torch.randn(batch, vocab, device="cuda", generator=g).to(torch.float16)
    # equal maxima (the first one counts), a maximum in the last element, -inf entries, a NaN that must not win
    logits[0, vocab // 3] = logits[0, vocab // 2] = 60000.0
    if batch > 1:
        logits[1, :] = -3.0
        logits[1, vocab - 1] = 5.0
    if batch > 2:
        logits[2, : vocab // 2] = float("-inf")
        logits[2, 1] = float("nan")
    want = torch.where(torch.isnan(logits), torch.full_like(logits, float("-inf")), logits).float().argmax(-1, keepdim=True)
    assert int(want[0]) == vocab // 3
    embed = torch.randn(vocab, hidden, device="cuda", generator=g).to(torch.float16)
    tok = torch.full((batch, 1), -1, dtype=torch.int64, device="cuda")
    pos = torch.tensor([41], dtype=torch.int64, device="cuda")
    x = torch.full((batch, hidden), float("nan"), dtype=torch.float16, device="cuda")
    native.greedy_next(logits, tok, pos, embed, x)
    torch.cuda.synchronize()
    assert torch.equal(tok, want) and int(pos) == 42 and torch.equal(x, embed[want[:, 0]])
    # without the optional operands: the choice alone
    tok.fill_(-1)
    native.greedy_next(logits, tok)
    assert torch.equal(tok, want) and int(pos) == 42


def test_graph_decode_with_the_fused_step_end_generates_what_separate_torch_ops_generate():
    """decode_llama.run ends a step with one launch (greedy choice, position update, next embedding rows); the same
    model stepped with torch's argmax, an add and an embedding lookup must produce the same tokens."""
    import decode_llama
    from qfactory import native
    shape = decode_llama.LlamaShape(layers=2, hidden=256, heads=4, mlp=512, vocab=1000, max_len=32, group_size=64)
    model = decode_llama.QuantLlama(shape, 2, seed=3)
    prompt = torch.randint(0, shape.vocab, (2, 8), device="cuda", generator=_gen(4))
    outs = []
    for fused in (False, True):
        model.k_cache.zero_(), model.v_cache.zero_()
        logits = model.prefill(prompt, torch.arange(8, device="cuda"))
        tok = logits.argmax(-1, keepdim=True)
        pos = torch.full((1,), 8, device="cuda", dtype=torch.int64)
        x0 = model.embed[tok[:, 0]]
        seq = [tok.clone()]
        for _ in range(6):
            if fused:
                native.greedy_next(model.decode_step(tok, pos, x0), tok, pos, model.embed, x0)
            else:
                lg = model.decode_step(tok, pos)
                tok.copy_(lg.argmax(-1, keepdim=True))
                pos.add_(1)
            seq.append(tok.clone())
        assert int(pos) == 14
        outs.append(torch.cat(seq, dim=1))
    assert torch.equal(outs[0], outs[1])


def test_decode_step_matches_the_torch_evaluation_of_the_same_model():
    import decode_llama
    shape = decode_llama.LlamaShape(layers=2, hidden=256, heads=4, mlp=512, vocab=1000, max_len=32, group_size=64)
    model = decode_llama.QuantLlama(shape, batch=2, seed=5)
    prompt = torch.randint(0, shape.vocab, (2, 8), device="cuda", generator=_gen(6))

    def run(step_fn, tokens=None):
        """Prompt, then four steps: greedy, or fed ``tokens`` (so that a near-tie in the logits of random weights
        cannot send two evaluations down different sequences)."""
        model.k_cache.zero_(), model.v_cache.zero_()
        logits, fed = [model.forward(prompt, torch.arange(8, device="cuda"))], []
        for i in range(4):
            fed.append(logits[-1].argmax(-1, keepdim=True) if tokens is None else tokens[i])
            logits.append(step_fn(fed[-1], torch.tensor([8 + i], device="cuda")).clone())
        return torch.stack(logits).float(), model.k_cache.clone(), model.v_cache.clone(), fed

    def same_choice(a, b):
        """Equal greedy choices, except where b's own margin between the two candidates is within the rounding
        distance of the two evaluations."""
        bound = 4 * (a - b).abs().max().item()
        ia, ib = a.argmax(-1), b.argmax(-1)
        margin = b.gather(-1, ib[..., None])[..., 0] - b.gather(-1, ia[..., None])[..., 0]
        return bool(((ia == ib) | (margin <= bound)).all()) and int((ia != ib).sum()) <= 1

    want, want_k, want_v, tokens = run(model.forward)
    got, got_k, got_v, _ = run(model.decode_step, tokens)
    # prefill with the norm and SiLU steps as single launches: same logits as the PyTorch evaluation
    pre = model.prefill(prompt, torch.arange(8, device="cuda")).float()
    assert ((pre - want[0]).norm() / want[0].norm()).item() <= 3e-3 and torch.equal(pre.argmax(-1), want[0].argmax(-1))
    assert torch.isfinite(got).all()
    assert ((got - want).norm() / want.norm()).item() <= 3e-3
    assert same_choice(got, want)
    assert ((got_k.float() - want_k.float()).norm() / want_k.float().norm()).item() <= 3e-3
    assert ((got_v.float() - want_v.float()).norm() / want_v.float().norm()).item() <= 3e-3
    # two rows: the residual adds and norms ran inside the qkv and gate+up projections (five launches per layer);
    # as launches of their own (eight per layer) the step gives the same tokens and logits to the same bar
    keys = [k for layer in model.layers for name in ("qkv", "gate_up") for k in layer[name]._funcs]
    assert (2, torch.float16, "add_rmsnorm") in keys and (2, torch.float16, "add_rmsnorm+silu_mul") in keys
    model.fuse_norm = False
    apart, apart_k, _, _ = run(model.decode_step, tokens)
    assert ((apart - got).norm() / got.norm()).item() <= 1e-3 and same_choice(apart, got)
    assert ((apart_k.float() - got_k.float()).norm() / got_k.float().norm()).item() <= 1e-3
