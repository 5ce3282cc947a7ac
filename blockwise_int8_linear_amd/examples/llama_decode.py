"""Llama-7B-shaped decoder with every nn.Linear replaced by BlockInt8Linear (block 128, int8 weights cached):
prefill of 2048 uniform-random token ids, then greedy decode of 128 tokens, batch 1, on one GPU.

    python -m blockwise_int8_linear_amd.examples.llama_decode [--layers 32] [--prefill 2048] [--decode 128]

Random-init weights (seed 0), no checkpoint, no tokenizer: this measures the linear layers inside a real decoder
loop (RMSNorm, RoPE, attention with a KV cache, SwiGLU MLP), nothing about model quality.  Prints one JSON line:
prefill ms and decode ms/token for the int8 layers (eager, and replayed from a HIP graph) and for the same model
with dense bf16 nn.Linear layers.
"""
from __future__ import annotations

import argparse
import json
import time

import torch
import torch.nn as nn
import torch.nn.functional as F

import blockwise_int8_linear_amd as bi8


class RMSNorm(nn.Module):
    def __init__(self, dim, eps=1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        return F.rms_norm(x, (x.shape[-1],), self.weight, self.eps)


def rope(x, cos, sin):
    """x [B, H, T, D]; cos/sin [T, D/2]"""
    h = x.shape[-1] // 2                           # rotate-half form: pairs are (i, i + D/2)
    x1, x2 = x[..., :h], x[..., h:]
    return torch.cat((x1 * cos - x2 * sin, x1 * sin + x2 * cos), dim=-1)


class Attention(nn.Module):
    def __init__(self, hidden, heads):
        super().__init__()
        self.heads, self.hd = heads, hidden // heads
        self.q = nn.Linear(hidden, hidden, bias=False)
        self.k = nn.Linear(hidden, hidden, bias=False)
        self.v = nn.Linear(hidden, hidden, bias=False)
        self.o = nn.Linear(hidden, hidden, bias=False)

    def forward(self, x, cos, sin, cache, pos, mask, hidden):
        B, T, _ = x.shape
        q = self.q(x).view(B, T, self.heads, self.hd).transpose(1, 2)
        k = self.k(x).view(B, T, self.heads, self.hd).transpose(1, 2)
        v = self.v(x).view(B, T, self.heads, self.hd).transpose(1, 2)
        # one rotation for queries and keys together (the same elementwise arithmetic on half as many launches: in eager
        # decode the host's time per launch is what a token costs)
        qk = rope(torch.cat((q, k), dim=1), cos, sin)
        q, k = qk[:, :self.heads], qk[:, self.heads:]
        kc, vc = cache
        kc.index_copy_(2, pos, k)
        vc.index_copy_(2, pos, v)
        if T == 1:                                  # one query: two small batched products beat the fused kernel
            att = torch.matmul(q, kc.transpose(2, 3)) * (self.hd ** -0.5)
            att = att.masked_fill(hidden, float("-inf")).softmax(-1)
            y = torch.matmul(att, vc)
        else:
            y = F.scaled_dot_product_attention(q, kc, vc, attn_mask=mask)
        return self.o(y.transpose(1, 2).reshape(B, T, -1))


class MLP(nn.Module):
    def __init__(self, hidden, inter):
        super().__init__()
        self.gate = nn.Linear(hidden, inter, bias=False)
        self.up = nn.Linear(hidden, inter, bias=False)
        self.down = nn.Linear(inter, hidden, bias=False)

    def forward(self, x):
        return self.down(F.silu(self.gate(x)) * self.up(x))


class Block(nn.Module):
    def __init__(self, hidden, heads, inter):
        super().__init__()
        self.n1, self.attn = RMSNorm(hidden), Attention(hidden, heads)
        self.n2, self.mlp = RMSNorm(hidden), MLP(hidden, inter)

    def forward(self, x, cos, sin, cache, pos, mask, hidden):
        x = x + self.attn(self.n1(x), cos, sin, cache, pos, mask, hidden)
        return x + self.mlp(self.n2(x))


class Decoder(nn.Module):
    def __init__(self, layers, hidden, heads, inter, vocab, max_len, dtype, device):
        super().__init__()
        self.embed = nn.Embedding(vocab, hidden)
        self.blocks = nn.ModuleList(Block(hidden, heads, inter) for _ in range(layers))
        self.norm = RMSNorm(hidden)
        self.head = nn.Linear(hidden, vocab, bias=False)
        self.to(device=device, dtype=dtype)
        for p in self.parameters():
            if p.dim() > 1:
                nn.init.normal_(p, std=0.02)
        hd = hidden // heads
        inv = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, device=device).float() / hd))
        ang = torch.arange(max_len, device=device).float()[:, None] * inv[None, :]
        self.register_buffer("cos", ang.cos().to(dtype), persistent=False)
        self.register_buffer("sin", ang.sin().to(dtype), persistent=False)
        self.caches = [(torch.zeros(1, heads, max_len, hd, device=device, dtype=dtype),
                        torch.zeros(1, heads, max_len, hd, device=device, dtype=dtype)) for _ in range(layers)]
        self.max_len = max_len

    def forward(self, tokens, pos):
        """tokens [1, T] at cache positions pos [T] (a device tensor); returns the logits of the last position"""
        x = self.embed(tokens)
        cos, sin = self.cos.index_select(0, pos), self.sin.index_select(0, pos)
        # position j of the cache is visible to query i iff j <= pos[i]
        mask = torch.arange(self.max_len, device=tokens.device)[None, :] <= pos[:, None]
        hidden = ~mask                              # what the one-query path fills with -inf, made once for all layers
        for blk, cache in zip(self.blocks, self.caches):
            x = blk(x, cos, sin, cache, pos, mask, hidden)
        return self.head(self.norm(x[:, -1:]))


def run(model, prefill, decode, graph):
    dev = model.cos.device
    g = torch.Generator(device=dev).manual_seed(1)
    tokens = torch.randint(0, model.embed.num_embeddings, (1, prefill), device=dev, generator=g)
    ppos = torch.arange(prefill, device=dev)
    res = {}
    with torch.no_grad():
        model(tokens, ppos)                                         # warm-up: builds the int8 weight caches
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = model(tokens, ppos)
        torch.cuda.synchronize()
        res["prefill_ms"] = round((time.perf_counter() - t0) * 1e3, 2)
        tok = logits.argmax(-1).view(1, 1)
        pos = torch.full((1,), prefill, device=dev, dtype=torch.long)
        one = torch.ones_like(pos)
        if graph:
            stok, spos = tok.clone(), pos.clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(2):
                    model(stok, spos)
            torch.cuda.current_stream().wait_stream(side)
            cg = torch.cuda.CUDAGraph()
            with torch.cuda.graph(cg):
                sout = model(stok, spos).argmax(-1).view(1, 1)
        else:
            for _ in range(2):                                      # library heuristics for the one-row shapes
                model(tok, pos)
        torch.cuda.synchronize()
        out = []
        t0 = time.perf_counter()
        for _ in range(decode):
            if graph:
                stok.copy_(tok)
                spos.copy_(pos)
                cg.replay()
                tok = sout.clone()
            else:
                tok = model(tok, pos).argmax(-1).view(1, 1)
            pos = pos + one
            out.append(tok)
        torch.cuda.synchronize()
        res["decode_ms_per_token"] = round((time.perf_counter() - t0) * 1e3 / decode, 3)
        res["tokens"] = torch.cat(out, 1).view(-1)[:8].tolist()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--hidden", type=int, default=4096)
    ap.add_argument("--heads", type=int, default=32)
    ap.add_argument("--inter", type=int, default=11008)
    ap.add_argument("--vocab", type=int, default=32000)
    ap.add_argument("--prefill", type=int, default=2048)
    ap.add_argument("--decode", type=int, default=128)
    ap.add_argument("--no-dense", action="store_true", help="skip the dense bf16 model")
    args = ap.parse_args()
    dev, dtype = "cuda:0", torch.bfloat16
    bi8.block_linear_config.GROUP_SIZE = 128
    bi8.block_linear_config.INPUT_OUTPUT_TORCH_TYPE = dtype
    torch.manual_seed(0)
    model = Decoder(args.layers, args.hidden, args.heads, args.inter, args.vocab, args.prefill + args.decode, dtype, dev).eval()
    res = {"config": {k: getattr(args, k) for k in ("layers", "hidden", "heads", "inter", "vocab", "prefill", "decode")},
           "block": 128, "dtype": "bf16", "data": "synthetic"}
    if not args.no_dense:
        res["dense_bf16"] = {"eager": run(model, args.prefill, args.decode, False), "graph": run(model, args.prefill, args.decode, True)}
    model.apply(bi8.replace_linear_with_blockwise_int8)             # one level per module, applied to every module
    model.eval()
    n_int8 = sum(isinstance(m, bi8.BlockInt8Linear) for m in model.modules())
    res["int8_layers"] = n_int8
    res["blockwise_int8"] = {"eager": run(model, args.prefill, args.decode, False), "graph": run(model, args.prefill, args.decode, True)}
    print(json.dumps(res))


if __name__ == "__main__":
    main()
