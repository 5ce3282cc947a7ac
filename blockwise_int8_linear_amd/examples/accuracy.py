"""What block quantization costs in accuracy, on the scenario of the reference's own demo (block_linear.py:161-224):
a 128 -> 128 layer without bias, a [128,128] input, squared-error loss; output, weight gradient and input gradient
of BlockInt8Linear against the same layer as a dense fp32 nn.Linear, for blocks 32 / 64 / 128, and the larger
[256,1024] x [1024,1024] forward at block 64.  (The reference also compares with microxcaling's mx.Linear, which it
does not ship; that column is absent.)

    python -m blockwise_int8_linear_amd.examples.accuracy

Prints one JSON line: relative Frobenius errors and largest absolute differences."""
from __future__ import annotations

import json

import torch
import torch.nn as nn

import blockwise_int8_linear_amd as bi8


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


def demo_case(block, features=128, rows=128, seed=0, dtype=torch.float32, dev="cuda"):
    cfg = bi8.block_linear_config
    old = (cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE)
    cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = block, dtype
    try:
        torch.manual_seed(seed)
        blinear = bi8.BlockInt8Linear(features, features, dtype=dtype, bias=False).to(dev)
        linear = nn.Linear(features, features, dtype=dtype, bias=False).to(dev)
        linear.weight.data.copy_(blinear.weight.data)
        x = torch.randn(rows, features, device=dev, requires_grad=True, dtype=dtype)
        y = torch.randn(rows, features, device=dev, dtype=dtype)
        out = {}
        res = {}
        for name, layer in (("int8", blinear), ("dense", linear)):
            if x.grad is not None:
                x.grad.zero_()
            y_hat = layer(x)
            (y_hat - y).pow(2).sum().backward()
            res[name] = (y_hat.detach(), layer.weight.grad.clone(), x.grad.clone())
        for i, what in enumerate(("output", "grad_weight", "grad_input")):
            out[what] = {"rel": round(_rel(res["int8"][i], res["dense"][i]), 6),
                         "max_abs": round((res["int8"][i] - res["dense"][i]).abs().max().item(), 6)}
        return out
    finally:
        cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = old


def forward_case(M=256, K=1024, N=1024, block=64, seed=0, dev="cuda"):
    cfg = bi8.block_linear_config
    old = (cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE)
    cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = block, torch.float32
    try:
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(M, K, generator=g).to(dev)
        w = (torch.randn(N, K, generator=g) * 0.02).to(dev)
        xq, xs = bi8.quantize_block_rowwise(x)
        wq, ws = bi8.quantize_block_rowwise(w)
        c = bi8.int8_matmul_block64_rowwise_dequantize(xq, wq.t(), xs, ws)
        return {"rel": round(_rel(c, x @ w.t()), 6)}
    finally:
        cfg.GROUP_SIZE, cfg.INPUT_OUTPUT_TORCH_TYPE = old


def main():
    out = {"demo_128x128x128_fp32": {f"block{b}": demo_case(b) for b in (32, 64, 128)},
           "forward_256x1024x1024_block64_fp32": forward_case()}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
