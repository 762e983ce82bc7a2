#!/usr/bin/env python3
"""Single-GPU greedy decode loop of a Llama-2-7B-shaped model whose linears are W4A16 g128 QLinear.

BASELINE.json configs[4]: 32 layers, hidden 4096, 32 heads, SwiGLU MLP 11008, vocab 32000, RMSNorm,
RoPE; random-initialised weights; batch in {1, 16, 64}; 128 random prompt ids, 128 greedy output
tokens.  It stands in for the reference's end-to-end runs through vLLM (reproduce/fig11,
third_party/vllm-qfactory.patch), which need vLLM and model downloads.

The four projections of a layer (fused QKV, O, fused gate+up, down) and the output projection are QLinear modules; prefill
(M = batch * prompt length) lands in the matrix-core regime and decode (M = batch) in the GEMV
regimes through the layers' own row-count dispatch.  ``forward`` runs everything else (embedding,
RMSNorm, RoPE, attention over a static KV cache, SiLU) in plain PyTorch; the output projection (vocab x hidden)
is a QLinear like the layers' four; ``prefill``
replaces its norm steps by single launches and forms the residual adds and SiLU * up in the projections' epilogues.  A decode step has no PyTorch op between the linears:
up to 32 sequences a layer is five launches -- qkv with the RMSNorm in front of its dot products, RoPE + cache
append + attention of the new position (libqfactory_hip.so), o adding its result to the residual stream, gate+up
with the RMSNorm in front and SiLU * up behind, down adding to the residual stream; for more sequences seven
(the two RMSNorms as launches of their own; residual adds and SiLU * up in the GEMM kernel's epilogues) -- instead of about fifty; ``--torch-glue`` keeps
PyTorch ops there for comparison.  One decode step --
including the argmax and the position update -- is captured in a HIP graph and replayed per token.

Prints one JSON line per batch size: tokens/s over the decode phase, prefill time, and the share of
a decode step spent in the quantized linears (their kernels timed separately at the same M).
"""
import argparse
import json
import os
import sys
import time
from dataclasses import dataclass

HERE = os.path.dirname(os.path.abspath(__file__))
if HERE not in sys.path:
    sys.path.insert(0, HERE)
os.environ.setdefault("QFACTORY_CACHE_DIR", os.path.join(HERE, "jit_cache"))
os.environ.setdefault("QFACTORY_LOG_LEVEL", "WARNING")

import torch
import torch.nn.functional as F

NO_SEARCH = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}


@dataclass
class LlamaShape:
    layers: int = 32
    hidden: int = 4096
    heads: int = 32
    mlp: int = 11008
    vocab: int = 32000
    max_len: int = 256
    rope_theta: float = 10000.0
    eps: float = 1e-5
    nbits: int = 4
    group_size: int = 128


def _random_qlinear(batch, K, N, shape, gen):
    """A QLinear with random packed fields and scales sized so that the layer has gain ~0.5."""
    from qfactory import QLinear
    lin = QLinear.empty(batch, K, N, shape.nbits, shape.group_size, sym=False, compile_flags=NO_SEARCH)
    lin.w.copy_(torch.randint(-128, 128, lin.w.shape, dtype=torch.int8, device="cuda", generator=gen))
    lin.z.copy_(torch.randint(-128, 128, lin.z.shape, dtype=torch.int8, device="cuda", generator=gen))
    spread = (2 ** shape.nbits) * 0.41                      # std of q - Z for independent uniform fields
    base = 0.5 / (spread * K ** 0.5)
    lin.s.copy_(((torch.rand(lin.s.shape, device="cuda", generator=gen) + 0.5) * base).to(torch.float16))
    return lin


class QuantLlama:
    def __init__(self, shape: LlamaShape, batch: int, seed: int = 0):
        self.shape, self.batch = shape, batch
        gen = torch.Generator(device="cuda").manual_seed(seed)
        h, hd = shape.hidden, shape.hidden // shape.heads
        self.embed = (torch.randn(shape.vocab, h, device="cuda", generator=gen) * 0.5).to(torch.float16)
        self.final_norm = torch.ones(h, dtype=torch.float16, device="cuda")
        self.layers = []
        for _ in range(shape.layers):
            self.layers.append({
                "norm1": torch.ones(h, dtype=torch.float16, device="cuda"),
                "norm2": torch.ones(h, dtype=torch.float16, device="cuda"),
                "qkv": _random_qlinear(batch, h, 3 * h, shape, gen),
                "o": _random_qlinear(batch, h, h, shape, gen),
                "gate_up": _random_qlinear(batch, h, 2 * shape.mlp, shape, gen),
                "down": _random_qlinear(batch, shape.mlp, h, shape, gen),
            })
        # the output projection is a quantized linear like the others (configs[4]: every linear), 32000 x 4096
        self.lm_head = _random_qlinear(batch, h, shape.vocab, shape, gen)
        self.k_cache = torch.zeros(shape.layers, batch, shape.heads, shape.max_len, hd, dtype=torch.float16, device="cuda")
        self.v_cache = torch.zeros_like(self.k_cache)
        inv = 1.0 / (shape.rope_theta ** (torch.arange(0, hd, 2, device="cuda", dtype=torch.float32) / hd))
        ang = torch.arange(shape.max_len, device="cuda", dtype=torch.float32)[:, None] * inv[None, :]
        self.cos, self.sin = ang.cos(), ang.sin()                                   # (max_len, hd/2) fp32
        self.linear = lambda lin, x: lin(x)                 # hook: tests swap in a dense fp32 evaluation
        self._own_linear = self.linear
        # residual add + RMSNorm inside the projection that follows them, where its kernel can (few rows); False
        # keeps them a launch of their own
        self.fuse_norm = True
        # buffers of the fused decode step (one new position per sequence)
        f16 = dict(dtype=torch.float16, device="cuda")
        self._hdn, self._att = (torch.empty(batch, h, **f16) for _ in range(2))

    def _norm(self, x, w):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.shape.eps)).to(torch.float16) * w

    def _rope(self, x, pos):
        """x (B, H, T, hd), pos (T,) int64: rotate pairs (2i, 2i+1)."""
        cos, sin = self.cos.index_select(0, pos)[None, None], self.sin.index_select(0, pos)[None, None]
        xf = x.float()
        x0, x1 = xf[..., 0::2], xf[..., 1::2]
        out = torch.stack((x0 * cos - x1 * sin, x0 * sin + x1 * cos), dim=-1).flatten(-2)
        return out.to(torch.float16)

    def forward(self, tokens, pos):
        """tokens (B, T) int64, pos (T,) int64 positions of those tokens.  Returns logits (B, vocab) of the
        last token; the KV cache is updated in place.  Attention is masked to positions <= the query's."""
        shape = self.shape
        B, T = tokens.shape
        H, hd = shape.heads, shape.hidden // shape.heads
        x = self.embed[tokens]                                                       # (B, T, h)
        key_pos = torch.arange(shape.max_len, device="cuda")
        mask = (key_pos[None, :] <= pos[:, None])[None, None]                        # (1, 1, T, max_len)
        for li, layer in enumerate(self.layers):
            hdn = self._norm(x, layer["norm1"]).reshape(B * T, shape.hidden)
            qkv = self.linear(layer["qkv"], hdn).reshape(B, T, 3, H, hd).permute(2, 0, 3, 1, 4)
            q, k, v = self._rope(qkv[0], pos), self._rope(qkv[1], pos), qkv[2]
            self.k_cache[li].index_copy_(2, pos, k)
            self.v_cache[li].index_copy_(2, pos, v)
            att = F.scaled_dot_product_attention(q, self.k_cache[li], self.v_cache[li], attn_mask=mask)
            att = att.permute(0, 2, 1, 3).reshape(B * T, shape.hidden)
            x = x + self.linear(layer["o"], att).reshape(B, T, shape.hidden)
            hdn = self._norm(x, layer["norm2"]).reshape(B * T, shape.hidden)
            gu = self.linear(layer["gate_up"], hdn)
            act = F.silu(gu[:, : shape.mlp]) * gu[:, shape.mlp:]
            x = x + self.linear(layer["down"], act.contiguous()).reshape(B, T, shape.hidden)
        last = self._norm(x[:, -1], self.final_norm)
        return self.linear(self.lm_head, last.contiguous())

    def prefill(self, tokens, pos):
        """``forward`` with the RMSNorm as a single launch of libqfactory_hip.so (any number of rows), the residual
        adds in the o and down projections' epilogues and SiLU * up in the gate+up projection's (or launches of their
        own where a kernel cannot), RoPE and the cache update of all positions as one launch; causal attention stays
        a PyTorch op."""
        from qfactory import native
        shape = self.shape
        B, T = tokens.shape
        H, hd = shape.heads, shape.hidden // shape.heads
        x = self.embed[tokens].reshape(B * T, shape.hidden)                          # residual stream, updated in place
        hdn = torch.empty_like(x)
        own = self.linear is self._own_linear
        act = None if own else torch.empty(B * T, shape.mlp, dtype=torch.float16, device="cuda")
        mask = (torch.arange(shape.max_len, device="cuda")[None, :] <= pos[:, None])[None, None]
        delta = None
        q_rows = torch.empty(B, T, H, hd, dtype=torch.float16, device="cuda") if own else None
        pos = pos.contiguous()
        for li, layer in enumerate(self.layers):
            native.add_rmsnorm(x, delta, layer["norm1"], hdn, shape.eps)
            qkv = self.linear(layer["qkv"], hdn)
            if own:
                # RoPE of q and k and the cache write of k and v for all T positions: one launch
                native.rope_kv_store_rows(qkv, pos, self.cos, self.sin, q_rows, self.k_cache[li], self.v_cache[li])
                q = q_rows.transpose(1, 2)                      # (B, H, T, hd) view: the attention output comes back in row order
            else:
                qkv = qkv.reshape(B, T, 3, H, hd).permute(2, 0, 3, 1, 4)
                q, k, v = self._rope(qkv[0], pos), self._rope(qkv[1], pos), qkv[2]
                self.k_cache[li].index_copy_(2, pos, k)
                self.v_cache[li].index_copy_(2, pos, v)
            att = F.scaled_dot_product_attention(q, self.k_cache[li], self.v_cache[li], attn_mask=mask)
            att = att.permute(0, 2, 1, 3).reshape(B * T, shape.hidden)
            if own:
                # the o and down projections add their result to the residual stream themselves (the norms then only
                # read it), SiLU(gate) * up is the gate+up projection's epilogue where it can be
                layer["o"].forward_accumulate(att, x)
                native.add_rmsnorm(x, None, layer["norm2"], hdn, shape.eps)
                layer["down"].forward_accumulate(layer["gate_up"].forward_silu_mul(hdn), x)
                continue
            delta = self.linear(layer["o"], att)
            native.add_rmsnorm(x, delta, layer["norm2"], hdn, shape.eps)
            native.silu_mul(self.linear(layer["gate_up"], hdn), act)
            delta = self.linear(layer["down"], act)
        last = (x if delta is None else x + delta).reshape(B, T, shape.hidden)[:, -1].contiguous()
        native.add_rmsnorm(last, None, self.final_norm, last, shape.eps)
        return self.linear(self.lm_head, last)

    def decode_step(self, tok, pos, x=None):
        """tok (B, 1) int64, pos one-element int64 device tensor: logits (B, vocab) of the next token, like
        ``forward`` at T = 1, with every step between the linears a single launch of libqfactory_hip.so.
        ``x`` (B, hidden): the embedding rows of ``tok`` where the caller already has them (``native.greedy_next``
        leaves them behind); the buffer is used as the residual stream and overwritten."""
        from qfactory import native
        shape = self.shape
        if x is None:
            x = self.embed[tok[:, 0]]                            # (B, h): the residual stream, updated in place
        delta = None
        first = self.layers[0]
        rows = x.shape[0]
        if (self.fuse_norm and self.linear is self._own_linear and first["qkv"].fuses_add_rmsnorm(rows)
                and first["gate_up"].fuses_add_rmsnorm(rows, silu_mul=True) and first["o"].fuses_accumulate(rows)
                and first["down"].fuses_accumulate(rows)):
            # five launches per layer: the o and down projections add their result to the residual stream themselves,
            # and the qkv and gate+up projections normalise it in front of their dot products
            for li, layer in enumerate(self.layers):
                qkv = layer["qkv"].forward_add_rmsnorm(x, None, layer["norm1"], shape.eps)
                native.rope_decode_attention(qkv, pos, self.cos, self.sin, self.k_cache[li], self.v_cache[li], self._att)
                layer["o"].forward_accumulate(self._att, x)
                act = layer["gate_up"].forward_add_rmsnorm(x, None, layer["norm2"], shape.eps, silu_mul=True)
                layer["down"].forward_accumulate(act, x)
            # the final norm runs in front of the output projection's dot products, like a layer's
            return self.lm_head.forward_add_rmsnorm(x, None, self.final_norm, shape.eps)
        if self.linear is self._own_linear and first["o"].fuses_accumulate(rows) and first["down"].fuses_accumulate(rows):
            # seven launches per layer: the o and down projections add their result to the residual stream themselves
            # (the norms then only read it), SiLU(gate) * up is the gate+up projection's epilogue where it can be
            for li, layer in enumerate(self.layers):
                native.add_rmsnorm(x, None, layer["norm1"], self._hdn, shape.eps)
                qkv = layer["qkv"](self._hdn)
                native.rope_decode_attention(qkv, pos, self.cos, self.sin, self.k_cache[li], self.v_cache[li], self._att)
                layer["o"].forward_accumulate(self._att, x)
                native.add_rmsnorm(x, None, layer["norm2"], self._hdn, shape.eps)
                layer["down"].forward_accumulate(layer["gate_up"].forward_silu_mul(self._hdn), x)
            native.add_rmsnorm(x, None, self.final_norm, self._hdn, shape.eps)
            return self.lm_head(self._hdn)
        for li, layer in enumerate(self.layers):
            native.add_rmsnorm(x, delta, layer["norm1"], self._hdn, shape.eps)
            qkv = self.linear(layer["qkv"], self._hdn)
            native.rope_decode_attention(qkv, pos, self.cos, self.sin, self.k_cache[li], self.v_cache[li], self._att)
            delta = self.linear(layer["o"], self._att)
            native.add_rmsnorm(x, delta, layer["norm2"], self._hdn, shape.eps)
            # SiLU(gate) * up: in the gate+up projection's final sum for few rows, else one launch behind it
            act = layer["gate_up"].forward_silu_mul(self._hdn)
            delta = self.linear(layer["down"], act)
        native.add_rmsnorm(x, delta, self.final_norm, self._hdn, shape.eps)
        return self.linear(self.lm_head, self._hdn)


def linears_time_us(model, M, reps=8):
    """Time of the quantized linears of one decode step at M rows: every layer's four kernels and the output
    projection once, back to back in a HIP graph (cold weights: the whole model is streamed), averaged over `reps`."""
    xs = {K: torch.randn(M, K, device="cuda").to(torch.float16) for K in (model.shape.hidden, model.shape.mlp)}

    def one_pass():
        for layer in model.layers:
            for name in ("qkv", "o", "gate_up", "down"):
                lin = layer[name]
                lin(xs[lin.in_features])
        model.lm_head(xs[model.lm_head.in_features])

    one_pass()
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
        one_pass()
    torch.cuda.current_stream().wait_stream(side)
    graph.replay()
    torch.cuda.synchronize()
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record()
    for _ in range(reps):
        graph.replay()
    t1.record()
    torch.cuda.synchronize()
    return t0.elapsed_time(t1) * 1e3 / reps


def run(shape, batch, prompt_len, new_tokens, seed=0, torch_glue=False, fuse_norm=None):
    from qfactory import native
    assert prompt_len + new_tokens <= shape.max_len
    model = QuantLlama(shape, batch, seed)
    if fuse_norm is not None:
        model.fuse_norm = fuse_norm
    gen = torch.Generator(device="cuda").manual_seed(seed + 1)
    prompt = torch.randint(0, shape.vocab, (batch, prompt_len), device="cuda", generator=gen)

    # ---- prefill (eager; also compiles / warms the large-M specialisations on its first call) ----
    prefill = model.forward if torch_glue else model.prefill
    prefill(prompt, torch.arange(prompt_len, device="cuda"))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits = prefill(prompt, torch.arange(prompt_len, device="cuda"))
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0

    # ---- decode: one step (forward + greedy choice + position update) captured in a HIP graph ----
    tok = logits.argmax(-1, keepdim=True)                        # (B, 1) static buffers of the graph
    pos = torch.full((1,), prompt_len, device="cuda", dtype=torch.int64)
    tok0, pos0 = tok.clone(), pos.clone()

    x0 = model.embed[tok[:, 0]]                                  # embedding rows of the current tokens, kept current by the step

    def step():
        if torch_glue:
            lg = model.forward(tok, pos)
            tok.copy_(lg.argmax(-1, keepdim=True))
            pos.add_(1)
        else:
            # greedy choice, position update and the next step's embedding rows: one launch behind the output projection
            native.greedy_next(model.decode_step(tok, pos, x0), tok, pos, model.embed, x0)

    step()                                                       # eager warm-up of the M = batch kernels
    torch.cuda.synchronize()
    tok.copy_(tok0), pos.copy_(pos0), x0.copy_(model.embed[tok0[:, 0]])
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    tok.copy_(tok0), pos.copy_(pos0), x0.copy_(model.embed[tok0[:, 0]])
    torch.cuda.synchronize()
    generated = []
    t0 = time.perf_counter()
    for _ in range(new_tokens):
        graph.replay()
        generated.append(tok.clone())
    torch.cuda.synchronize()
    decode_s = time.perf_counter() - t0
    out_tokens = torch.cat(generated, dim=1)
    assert out_tokens.shape == (batch, new_tokens) and int(pos) == prompt_len + new_tokens

    step_us = decode_s / new_tokens * 1e6
    lin_us = linears_time_us(model, batch)
    return {"metric": "greedy decode throughput, Llama-2-7B shape, W4A16 g128 QLinear", "unit": "tokens/s",
            "value": round(batch * new_tokens / decode_s, 1), "batch": batch, "prompt_len": prompt_len,
            "new_tokens": new_tokens, "decode_step_us": round(step_us, 1), "prefill_ms": round(prefill_s * 1e3, 2),
            "prefill_tokens_per_s": round(batch * prompt_len / prefill_s, 1),
            "quantized_linears_us_per_step": round(lin_us, 1), "quantized_linear_share": round(lin_us / step_us, 3),
            "layers": shape.layers, "hidden": shape.hidden, "data": "random weights, random prompt ids",
            "between_linears": "torch ops" if torch_glue else (
                "attention one HIP launch (libqfactory_hip.so); residual add + RMSNorm and SiLU * up inside the projections"
                if model.layers[0]["gate_up"].fuses_add_rmsnorm(batch, silu_mul=True) and model.fuse_norm
                else "one HIP launch per step (libqfactory_hip.so); SiLU * up inside the gate+up projection"
                if model.layers[0]["gate_up"].fuses_silu_mul(batch)
                else "one HIP launch per step (libqfactory_hip.so)")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batches", type=int, nargs="+", default=[1, 16, 64])
    ap.add_argument("--prompt-len", type=int, default=128)
    ap.add_argument("--new-tokens", type=int, default=128)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--torch-glue", action="store_true", help="PyTorch ops between the linears of a decode step")
    ap.add_argument("--separate-norm", action="store_true", help="residual add + RMSNorm as a launch of its own at every batch size")
    ap.add_argument("--fused-norm", action="store_true", help="... inside the projections wherever the kernels can (up to 32 sequences)")
    args = ap.parse_args()
    assert torch.cuda.is_available(), "decode_llama.py needs the MI355X"
    shape = LlamaShape(layers=args.layers, max_len=args.prompt_len + args.new_tokens)
    for batch in args.batches:
        print(json.dumps(run(shape, batch, args.prompt_len, args.new_tokens, torch_glue=args.torch_glue,
                             fuse_norm=False if args.separate_norm else True if args.fused_norm else None)), flush=True)
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()
