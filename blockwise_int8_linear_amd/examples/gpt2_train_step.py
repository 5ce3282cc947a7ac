"""GPT-2-small training step with every nn.Linear replaced by BlockInt8Linear (block 64): 12 layers, d_model 768,
12 heads, MLP 3072, vocabulary 50257, context 1024, batch 8 x 1024 uniform-random tokens, AdamW on fp32 master
weights (the model computes in bf16 copies refreshed from the masters every step).

    python -m blockwise_int8_linear_amd.examples.gpt2_train_step [--steps 5] [--only int8|dense]

Random-init weights (seed 0), synthetic tokens: this measures forward + backward (int8 grad-input and grad-weight
GEMMs with transposed-block requantization, including the 50257-wide output layer) + optimizer, nothing about
model quality.  Prints one JSON line: ms per step and the losses for the int8 layers and for dense bf16 nn.Linear.
"""
from __future__ import annotations

import argparse
import gc
import json
import time

import torch
import torch.nn as nn
import torch.nn.functional as F

import blockwise_int8_linear_amd as bi8


class Block(nn.Module):
    def __init__(self, d, heads):
        super().__init__()
        self.heads = heads
        self.ln1, self.ln2 = nn.LayerNorm(d), nn.LayerNorm(d)
        self.c_attn, self.c_proj = nn.Linear(d, 3 * d), nn.Linear(d, d)
        self.c_fc, self.c_out = nn.Linear(d, 4 * d), nn.Linear(4 * d, d)

    def forward(self, x):
        B, T, C = x.shape
        q, k, v = self.c_attn(self.ln1(x)).split(C, dim=2)
        q, k, v = (t.view(B, T, self.heads, C // self.heads).transpose(1, 2) for t in (q, k, v))
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B, T, C)
        x = x + self.c_proj(y)
        return x + self.c_out(F.gelu(self.c_fc(self.ln2(x))))


class GPT2(nn.Module):
    def __init__(self, layers, d, heads, vocab, ctx):
        super().__init__()
        self.wte, self.wpe = nn.Embedding(vocab, d), nn.Embedding(ctx, d)
        self.blocks = nn.ModuleList(Block(d, heads) for _ in range(layers))
        self.ln_f = nn.LayerNorm(d)
        self.lm_head = nn.Linear(d, vocab, bias=False)

    def forward(self, idx):
        pos = torch.arange(idx.shape[1], device=idx.device)
        x = self.wte(idx) + self.wpe(pos)
        for b in self.blocks:
            x = b(x)
        return self.lm_head(self.ln_f(x))


def run(int8: bool, args):
    dev = "cuda:0"
    # start from an empty caching allocator: blocks kept from the other model's run do not fit this one's sizes, and
    # the allocator then frees and re-allocates device memory inside the timed steps
    gc.collect()
    torch.cuda.empty_cache()
    torch.manual_seed(0)
    model = GPT2(args.layers, args.d_model, args.heads, args.vocab, args.ctx)
    for p in model.parameters():
        if p.dim() > 1:
            nn.init.normal_(p, std=0.02)
    masters = [p.detach().clone().to(dev).float() for p in model.parameters()]     # fp32 master weights
    model = model.to(device=dev, dtype=torch.bfloat16)
    if int8:
        model.apply(bi8.replace_linear_with_blockwise_int8)
    model.train()
    params = list(model.parameters())
    for m in masters:
        m.grad = torch.zeros_like(m)
    opt = torch.optim.AdamW(masters, lr=3e-4, weight_decay=0.01, fused=True)
    g = torch.Generator(device=dev).manual_seed(1)
    idx = torch.randint(0, args.vocab, (args.batch, args.ctx), device=dev, generator=g)
    tgt = torch.randint(0, args.vocab, (args.batch, args.ctx), device=dev, generator=g)

    def step():
        with torch.no_grad():
            torch._foreach_copy_(params, masters)                   # bf16 compute copies of the fp32 masters
        logits = model(idx)
        loss = F.cross_entropy(logits.view(-1, args.vocab).float(), tgt.view(-1))
        for p in params:
            p.grad = None
        loss.backward()
        with torch.no_grad():
            torch._foreach_copy_([m.grad for m in masters], [p.grad for p in params])
        opt.step()
        return loss

    losses = [step().item() for _ in range(2)]                      # warm-up (library heuristics, allocator)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    losses.append(loss.item())
    finite = all(torch.isfinite(p.grad).all().item() for p in params)
    n_int8 = sum(isinstance(m, bi8.BlockInt8Linear) for m in model.modules())
    tokens = args.batch * args.ctx
    return {"ms_per_step": round(ms, 2), "tokens_per_s": round(tokens / ms * 1e3), "losses": [round(v, 4) for v in losses],
            "grads_finite": finite, "int8_layers": n_int8}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=12)
    ap.add_argument("--d-model", dest="d_model", type=int, default=768)
    ap.add_argument("--heads", type=int, default=12)
    ap.add_argument("--vocab", type=int, default=50257)
    ap.add_argument("--ctx", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--only", choices=["both", "dense", "int8"], default="both", help="which of the two models to run (profiling)")
    args = ap.parse_args()
    bi8.block_linear_config.GROUP_SIZE = 64
    bi8.block_linear_config.INPUT_OUTPUT_TORCH_TYPE = torch.bfloat16
    res = {"config": {k: getattr(args, k) for k in ("layers", "d_model", "heads", "vocab", "ctx", "batch")}, "block": 64,
           "dtype": "bf16 compute, fp32 master weights", "data": "synthetic"}
    if args.only != "int8":
        res["dense_bf16"] = run(False, args)
    if args.only != "dense":
        res["blockwise_int8"] = run(True, args)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
