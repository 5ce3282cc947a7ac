"""The benchmark configurations at their full sizes, checked against the CPU checker on sampled rows and columns:

  * the Llama-7B-shaped GEMM sweep: M in {1, 16, 128, 2048, 8192} x (K,N) in {(4096,4096), (4096,11008),
    (11008,4096), (4096,12288)}, block 128, bf16 activations quantized on the fly, cached int8 weights, bf16 out;
  * the 32-layer Llama-style decoder (hidden 4096, 32 heads, SwiGLU 11008, vocabulary 32000): prefill of 2048 tokens,
    greedy decode of 128, eager and replayed from a HIP graph, one-kernel and two-launch decode linears;
  * one GPT-2-small training step (12 layers, 768, 12 heads, 3072, vocabulary 50257, 8 x 1024 tokens, block 64):
    every distinct linear of the model, forward and both gradients, including the 768 -> 50257 output layer whose
    grad-input GEMM contracts over the 50257-word vocabulary.

A full-size output is too much for the scalar checker, so each GEMM is compared on a sample of whole rows and whole
columns (a row of the output depends on one row of the activations and all of the weights, a column on one weight
row), computed by the checker from the same operands.  Random weights and tokens; nothing here says anything about
model quality."""
import time

import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import oracle_torch
from util import assert_close_rms, assert_gemm_close, config_as, gemm_reference

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def pkg():
    import blockwise_int8_linear_amd as p
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return p


# ---- the GEMM sweep ---------------------------------------------------------------------------------------------------
KN = [(4096, 4096), (4096, 11008), (11008, 4096), (4096, 12288)]
MS = [1, 16, 128, 2048, 8192]
_weights = {}


def _layer(pkg, K, N):
    """BlockInt8Linear K -> N in eval mode with its int8 weights cached, and the CPU copies of W, codes and scales"""
    if (K, N) not in _weights:
        _weights.clear()                            # one layer resident at a time
        g = torch.Generator().manual_seed(K * 7 + N)
        W = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
        lin = pkg.BlockInt8Linear(K, N, bias=False, device=DEV, dtype=torch.bfloat16).eval()
        with torch.no_grad():
            lin.weight.copy_(W.to(DEV))
        lin.prepare_for_eval()
        wq, sw = lin.W_int8.cpu(), lin.state_W.cpu()
        wqo, swo = oracle.quantize_block_rowwise(W, 128, threads=True)
        assert torch.equal(wq, wqo) and torch.equal(sw, swo)
        _weights[(K, N)] = (lin, wq, sw)
    return _weights[(K, N)]


@pytest.mark.parametrize("KN_", KN, ids=lambda kn: f"K{kn[0]}_N{kn[1]}")
@pytest.mark.parametrize("M", MS)
def test_llama_shaped_gemm_sweep(pkg, KN_, M):
    from blockwise_int8_linear_amd import _lib
    K, N = KN_
    block = 128
    with config_as(pkg, block, torch.bfloat16):
        lin, wq, sw = _layer(pkg, K, N)
        g = torch.Generator().manual_seed(M + K + N)
        x = torch.randn(M, K, generator=g).to(torch.bfloat16)
        xd = x.to(DEV)
        with torch.no_grad():
            y = lin(xd)                             # quantize on the fly + GEMM (one kernel for M = 1)
            xq, sx = pkg.quantize_block_rowwise(xd)
            y2 = pkg.int8_matmul_block64_rowwise_dequantize(xq, lin.W_int8.t(), sx, lin.state_W)
        assert y.shape == (M, N) and y.dtype == torch.bfloat16
        assert torch.equal(y, y2)                   # the one-kernel path and the two launches give the same bits
        ws = _lib.load().bi8_gemm_workspace_bytes(M, N, K, block)
        kernel = _lib.load().bi8_gemm_kernel_name(M, N, K, K, K, block, ws).decode()
        want = {1: "gemv_rows", 16: "gemm_panel" if N >= 6144 and K <= 4096 else "gemv_staged", 128: "gemm_panel" if K <= 4096 else "splitk",
                2048: "gemm_wide_256x128" if N == 4096 else "gemm_wide", 8192: "gemm_wide"}[M]
        assert want in kernel, kernel
        rows = torch.arange(M) if M <= 128 else torch.randperm(M, generator=g)[:64]
        xqo, sxo = oracle.quantize_block_rowwise(x[rows], block)
        assert torch.equal(xq.cpu()[rows], xqo) and torch.equal(sx.cpu()[:, rows], sxo)
        ref, mag = gemm_reference(xqo, wq, sxo, sw, block, None, torch.bfloat16)
        assert_gemm_close(y.cpu()[rows], ref, mag, 1e-2)
        if M > 128:
            cols = torch.randperm(N, generator=g)[:64]
            xq_c, sx_c = xq.cpu(), sx.cpu()
            ref, mag = gemm_reference(xq_c, wq[cols], sx_c, sw[:, cols].contiguous(), block, None, torch.bfloat16)
            assert_gemm_close(y.cpu()[:, cols], ref, mag, 1e-2)


# ---- the Llama-style decoder ------------------------------------------------------------------------------------------
def _greedy(model, tokens, n_decode, graph):
    """prefill, then n_decode greedy tokens; returns (last-position logits of the prefill, the decoded token ids)"""
    dev = tokens.device
    T = tokens.shape[1]
    with torch.no_grad():
        logits = model(tokens, torch.arange(T, device=dev))
        tok = logits.argmax(-1).view(1, 1)
        pos = torch.full((1,), T, device=dev, dtype=torch.long)
        out = [tok]
        if graph:
            stok, spos = tok.clone(), pos.clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                model(stok, spos)
            torch.cuda.current_stream().wait_stream(side)
            cg = torch.cuda.CUDAGraph()
            with torch.cuda.graph(cg):
                sout = model(stok, spos).argmax(-1).view(1, 1)
        for _ in range(n_decode - 1):
            if graph:
                stok.copy_(tok)
                spos.copy_(pos)
                cg.replay()
                tok = sout.clone()
            else:
                tok = model(tok, pos).argmax(-1).view(1, 1)
            pos = pos + 1
            out.append(tok)
        torch.cuda.synchronize()
    return logits, torch.cat(out, 1).view(-1).cpu()


def test_llama_decoder_prefill_and_decode(pkg, monkeypatch):
    from blockwise_int8_linear_amd import block_linear as bl
    from blockwise_int8_linear_amd.examples import llama_decode as ex
    layers, hidden, heads, inter, vocab, prefill, decode = 32, 4096, 32, 11008, 32000, 2048, 128
    block, dtype = 128, torch.bfloat16
    with config_as(pkg, block, dtype):
        torch.manual_seed(0)
        with torch.device(DEV):                     # parameters are created on the GPU: 6.7e9 of them
            model = ex.Decoder(layers, hidden, heads, inter, vocab, prefill + decode, dtype, DEV).eval()
        model.apply(pkg.replace_linear_with_blockwise_int8)
        model.eval()
        linears = [m for m in model.modules() if isinstance(m, pkg.BlockInt8Linear)]
        assert len(linears) == 7 * layers + 1 and not any(type(m) is torch.nn.Linear for m in model.modules())
        tokens = torch.randint(0, vocab, (1, prefill), device=DEV, generator=torch.Generator(device=DEV).manual_seed(1))

        # the inputs and outputs of the first layer's seven linears and of the output layer during the prefill
        seen = {}
        names = {"q": model.blocks[0].attn.q, "k": model.blocks[0].attn.k, "v": model.blocks[0].attn.v, "o": model.blocks[0].attn.o,
                 "gate": model.blocks[0].mlp.gate, "up": model.blocks[0].mlp.up, "down": model.blocks[0].mlp.down, "head": model.head}
        def keep_first(n):
            def hook(mod, inp, out):
                if n not in seen:
                    seen[n] = (inp[0].detach().clone(), out.detach().clone())
            return hook
        hooks = [m.register_forward_hook(keep_first(n)) for n, m in names.items()]
        t0 = time.perf_counter()
        logits, eager = _greedy(model, tokens, decode, graph=False)
        t_eager = time.perf_counter() - t0
        for h in hooks:
            h.remove()
        assert torch.isfinite(logits.float()).all() and logits.shape == (1, 1, vocab)
        assert all(m.W_int8.dtype == torch.int8 and m.state_W.shape == (m.in_features // block, m.out_features) for m in linears)

        g = torch.Generator().manual_seed(2)
        for n, (x, y) in seen.items():
            x2, y2 = x.reshape(-1, x.shape[-1]), y.reshape(-1, y.shape[-1])
            rows = torch.randperm(x2.shape[0], generator=g)[:16] if x2.shape[0] > 16 else torch.arange(x2.shape[0])
            W = names[n].weight.detach().cpu()
            ref = oracle_torch.linear_forward(x2[rows.to(DEV)].cpu(), W, None, block, dtype)
            assert_close_rms(y2[rows.to(DEV)].cpu(), ref, 1e-2)

        # the same tokens from a HIP graph replay of the decode step, and with two launches per decode linear
        logits_g, graphed = _greedy(model, tokens, decode, graph=True)
        assert torch.equal(logits_g, logits) and torch.equal(graphed, eager)
        monkeypatch.setattr(bl, "few_rows_plan", lambda *a, **k: None)       # no one-launch path: quantize, then multiply
        for m in linears:
            m._few_rows = None                                                   # (the modules keep what they were given)
        _, two_launch = _greedy(model, tokens, decode, graph=False)
        assert all(m._few_rows is not None and m._few_rows[1] is None for m in linears)
        assert torch.equal(two_launch, eager)
        assert len(set(eager.tolist())) > 1         # not stuck on one token
        print(f"[llama decoder] prefill {prefill} + {decode} greedy tokens, eager: {t_eager:.2f} s")


# ---- the GPT-2-small training step ------------------------------------------------------------------------------------
def _gpt2_step(pkg, int8, capture):
    """one forward + backward of GPT-2-small on 8 x 1024 random tokens in bf16; returns the loss and, with `capture`,
    per distinct linear its (input, output, grad_output, grad_input, weight, bias, grad_weight, grad_bias)"""
    from blockwise_int8_linear_amd.examples import gpt2_train_step as ex
    vocab, ctx, batch = 50257, 1024, 8
    torch.manual_seed(0)
    with torch.device(DEV):
        model = ex.GPT2(12, 768, 12, vocab, ctx)
    for p in model.parameters():
        if p.dim() > 1:
            torch.nn.init.normal_(p, std=0.02)
    model = model.to(torch.bfloat16)
    if int8:
        model.apply(pkg.replace_linear_with_blockwise_int8)
        assert sum(isinstance(m, pkg.BlockInt8Linear) for m in model.modules()) == 49
    model.train()
    g = torch.Generator(device=DEV).manual_seed(1)
    idx = torch.randint(0, vocab, (batch, ctx), device=DEV, generator=g)
    tgt = torch.randint(0, vocab, (batch, ctx), device=DEV, generator=g)
    b0 = model.blocks[0]
    mods = {"c_attn": b0.c_attn, "c_proj": b0.c_proj, "c_fc": b0.c_fc, "c_out": b0.c_out, "lm_head": model.lm_head}
    got = {n: {} for n in mods}
    hooks = []
    if capture:
        for n, m in mods.items():
            hooks.append(m.register_forward_hook(lambda mod, inp, out, n=n: got[n].update(x=inp[0].detach(), y=out.detach())))
            hooks.append(m.register_full_backward_hook(lambda mod, gin, gout, n=n: got[n].update(gx=gin[0].detach(), g=gout[0].detach())))

    def step():
        for p in model.parameters():
            p.grad = None
        logits = model(idx)
        loss = F.cross_entropy(logits.view(-1, vocab).float(), tgt.view(-1))
        loss.backward()
        return loss

    loss = step()
    torch.cuda.synchronize()
    for h in hooks:
        h.remove()
    for n, m in mods.items():
        got[n].update(W=m.weight.detach(), b=None if m.bias is None else m.bias.detach(), gW=m.weight.grad, gb=None if m.bias is None else m.bias.grad)
    assert all(torch.isfinite(p.grad.float()).all() for p in model.parameters())
    # time a few more steps (forward + backward only) for the log
    t0 = time.perf_counter()
    for _ in range(3):
        step()
    torch.cuda.synchronize()
    return loss.item(), got, (time.perf_counter() - t0) / 3 * 1e3


def test_gpt2_small_training_step(pkg):
    block, dtype = 64, torch.bfloat16
    with config_as(pkg, block, dtype):
        loss_dense, _, ms_dense = _gpt2_step(pkg, False, False)
        loss_int8, got, ms_int8 = _gpt2_step(pkg, True, True)
        print(f"[gpt2-small fwd+bwd] dense bf16 {ms_dense:.2f} ms, blockwise int8 {ms_int8:.2f} ms; loss {loss_dense:.5f} / {loss_int8:.5f}")
        assert loss_int8 == loss_int8 and abs(loss_int8 - loss_dense) <= 1e-3 * abs(loss_dense)
        g = torch.Generator().manual_seed(3)
        for n, t in got.items():
            x = t["x"].reshape(-1, t["x"].shape[-1])
            y = t["y"].reshape(-1, t["y"].shape[-1])
            G = t["g"].reshape(-1, t["g"].shape[-1])
            gx = t["gx"].reshape(-1, t["gx"].shape[-1])
            M, K = x.shape
            N = y.shape[1]
            assert M == 8192 and G.shape == (M, N) and gx.shape == (M, K) and t["gW"].shape == (N, K)
            W = t["W"].cpu()
            bias = None if t["b"] is None else t["b"].cpu()
            rows = torch.randperm(M, generator=g)[:48]
            rd = rows.to(DEV)
            # forward and grad-input: rows of the tokens are independent (block_linear.py:78-80, :92-95)
            ref_y = oracle_torch.linear_forward(x[rd].cpu(), W, bias, block, dtype)
            assert_close_rms(y[rd].cpu(), ref_y, 1e-2, bias)
            ref_gx, _, _ = oracle_torch.linear_backward(G[rd].cpu(), x[rd].cpu(), W, block, dtype, has_bias=False)
            assert_close_rms(gx[rd].cpu(), ref_gx, 1e-2)
            # grad-weight contracts over all 8192 tokens; output features are independent (block_linear.py:100-104)
            ns = torch.randperm(N, generator=g)[:48]
            nd = ns.to(DEV)
            _, ref_gW, ref_gb = oracle_torch.linear_backward(G[:, nd].cpu(), x.cpu(), W[ns], block, dtype, has_bias=True)
            assert_close_rms(t["gW"][nd].cpu(), ref_gW, 1e-2)
            if bias is not None:
                assert_close_rms(t["gb"][nd].cpu(), ref_gb, 1e-2)
