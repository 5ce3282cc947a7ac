"""Training on weights quantized ahead of the step: ``blockwise_int8_linear_Wint8`` (the working form of
block_linear.py:42-67) and the module mode built on it.  With the two quantized copies made from W the function is
``blockwise_int8_linear`` bit for bit; against the CPU checker's restatement (oracle_torch.linear_wint8_*) outputs and
gradients are within 1e-3 (fp32) / 1e-2 (bf16).  Also here: the eval cache follows the weight (no stale codes after
training steps or a checkpoint load), and the recursive model-surgery helper."""
import pytest
import torch
import torch.nn as nn

import oracle
from oracle import oracle_torch
from util import assert_close_rms, config_as

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def pkg():
    import blockwise_int8_linear_amd as p
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return p


# (leading shape of x, K, N): N = 200 and 1000 make the grad-input contraction ragged; 3-D and 2-D inputs
SHAPES = [((4, 48), 128, 96), ((300,), 256, 200), ((2, 3, 40), 384, 1000), ((1,), 512, 128)]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("block", [32, 64, 128])
@pytest.mark.parametrize("shape", SHAPES)
def test_function_matches_the_unquantized_weight_function_and_the_checker(pkg, dtype, tol, block, shape):
    lead, K, N = shape
    g = torch.Generator().manual_seed(K + N + block)
    x = torch.randn(*lead, K, generator=g).to(dtype)
    W = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    bias = torch.randn(N, generator=g).to(dtype)
    G = torch.randn(*lead, N, generator=g).to(dtype)
    with config_as(pkg, block, dtype):
        Wd = W.to(DEV).requires_grad_(True)
        W_int8, state_W, Wt_int8, Wt_state, Wt_store = pkg.quantize_weight_for_training(Wd)
        # the copies are the checker's quantizations of W and of its transpose
        wq, sw = oracle.quantize_block_rowwise(W, block)
        wtq, wts = oracle.quantize_block_transposed(W, block)
        assert torch.equal(W_int8.cpu(), wq) and torch.equal(state_W.cpu(), sw)
        assert torch.equal(Wt_int8.cpu(), wtq) and torch.equal(Wt_state.cpu(), wts) and Wt_int8.shape == (K, N)

        x1 = x.to(DEV).requires_grad_(True)
        b1 = bias.to(DEV).requires_grad_(True)
        y1 = pkg.blockwise_int8_linear_Wint8.apply(x1, W_int8, state_W, b1, Wt_int8, Wt_state, Wd, Wt_store)
        y1.backward(G.to(DEV))
        gx1, gw1, gb1 = x1.grad, Wd.grad, b1.grad

        x2 = x.to(DEV).requires_grad_(True)
        W2 = W.to(DEV).requires_grad_(True)
        b2 = bias.to(DEV).requires_grad_(True)
        y2 = pkg.blockwise_int8_linear.apply(x2, W2, b2)
        y2.backward(G.to(DEV))
        assert torch.equal(y1, y2) and torch.equal(gx1, x2.grad) and torch.equal(gw1, W2.grad) and torch.equal(gb1, b2.grad)

        # without the padded buffer, and with a frozen weight (no stand-in for W: grad_X and grad_bias only)
        x3 = x.to(DEV).requires_grad_(True)
        y3 = pkg.blockwise_int8_linear_Wint8.apply(x3, W_int8, state_W, bias.to(DEV), Wt_int8.contiguous(), Wt_state)
        y3.backward(G.to(DEV))
        assert torch.equal(y3, y1) and torch.equal(x3.grad, gx1)

    ref_y = oracle_torch.linear_wint8_forward(x, wq, sw, bias, block, dtype)
    ref_gx, ref_gw, ref_gb = oracle_torch.linear_wint8_backward(G, x, wtq, wts, block, dtype)
    assert y1.shape == ref_y.shape and y1.dtype == dtype
    assert_close_rms(y1.detach().cpu(), ref_y, tol, bias)
    assert_close_rms(gx1.cpu(), ref_gx, tol)
    assert_close_rms(gw1.cpu(), ref_gw, tol)
    assert_close_rms(gb1.cpu(), ref_gb.to(dtype), tol)


def test_module_mode_quantizes_the_weight_once_per_change(pkg, monkeypatch):
    from blockwise_int8_linear_amd import block_linear as bl
    with config_as(pkg, 64, torch.bfloat16):
        torch.manual_seed(0)
        lin = pkg.BlockInt8Linear(256, 192, device=DEV, dtype=torch.bfloat16)
        ref = pkg.BlockInt8Linear(256, 192, device=DEV, dtype=torch.bfloat16)
        ref.load_state_dict(lin.state_dict())
        lin.quantized_weight_training = True
        calls = []
        real = bl.quantize_weight_for_training
        monkeypatch.setattr(bl, "quantize_weight_for_training", lambda W: (calls.append(1), real(W))[1])
        opt = torch.optim.SGD(lin.parameters(), lr=0.1)
        opt_ref = torch.optim.SGD(ref.parameters(), lr=0.1)
        for step in range(3):
            for micro in range(2):                  # two micro-batches per optimizer step: one quantization of W
                x = torch.randn(96, 256, device=DEV, dtype=torch.bfloat16)
                xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
                ya, yb = lin(xa), ref(xb)
                assert torch.equal(ya, yb)
                ya.float().pow(2).mean().backward()
                yb.float().pow(2).mean().backward()
                assert torch.equal(xa.grad, xb.grad)
            assert torch.equal(lin.weight.grad, ref.weight.grad) and torch.equal(lin.bias.grad, ref.bias.grad)
            assert len(calls) == step + 1
            opt.step(); opt_ref.step()
            opt.zero_grad(); opt_ref.zero_grad()
            assert torch.equal(lin.weight, ref.weight)
        # frozen weight: still one quantization, gradient for the input only
        lin.weight.requires_grad_(False)
        n = len(calls)
        for _ in range(2):
            x = torch.randn(8, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
            lin(x).float().sum().backward()
            assert x.grad is not None and lin.weight.grad is None
        assert len(calls) == n + 1                  # the last optimizer step changed the weight: one more, then none


def test_eval_cache_follows_the_weight(pkg):
    """a checkpoint written after an eval call carries W_int8 / state_W; a fresh module (in training mode) that loads
    it, takes training steps and is then switched to eval must serve the trained weights, not the checkpoint's codes"""
    with config_as(pkg, 128, torch.bfloat16):
        torch.manual_seed(1)
        a = pkg.BlockInt8Linear(256, 128, device=DEV, dtype=torch.bfloat16).eval()
        x = torch.randn(16, 256, device=DEV, dtype=torch.bfloat16)
        with torch.no_grad():
            a(x)
        sd = a.state_dict()
        assert "W_int8" in sd and "state_W" in sd
        b = pkg.BlockInt8Linear(256, 128, device=DEV, dtype=torch.bfloat16)      # training mode, never told otherwise
        b.load_state_dict(sd)
        assert torch.equal(b.W_int8, a.W_int8)
        with torch.no_grad():
            assert torch.equal(b.infer(x), a(x))                                  # the loaded codes are served as they are
        opt = torch.optim.SGD(b.parameters(), lr=0.5)
        b(x).float().pow(2).mean().backward()
        opt.step()
        b.training = False                                                        # not through train(): nothing dropped the cache
        with torch.no_grad():
            y = b(x)
            q, s = pkg.quantize_block_rowwise(b.weight.detach())
        assert torch.equal(b.W_int8, q) and torch.equal(b.state_W, s) and not torch.equal(b.W_int8, a.W_int8)
        ref = oracle_torch.linear_forward(x.cpu(), b.weight.detach().cpu(), b.bias.detach().cpu(), 128, torch.bfloat16)
        assert_close_rms(y.cpu(), ref, 1e-2, b.bias.detach().cpu())
        # in-place edits in eval mode are followed too
        with torch.no_grad():
            b.weight.mul_(2.0)
            y2 = b(x)
        ref2 = oracle_torch.linear_forward(x.cpu(), b.weight.detach().cpu(), b.bias.detach().cpu(), 128, torch.bfloat16)
        assert_close_rms(y2.cpu(), ref2, 1e-2, b.bias.detach().cpu())


class _DataSGD(torch.optim.Optimizer):
    """an optimizer of the kind that updates through ``p.data`` (apex / DeepSpeed style): no version counter moves"""

    def __init__(self, params, lr):
        super().__init__(params, {"lr": lr})

    @torch.no_grad()
    def step(self):
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is not None:
                    p.data.add_(p.grad.data, alpha=-group["lr"])


def test_cached_codes_follow_updates_made_through_data(pkg):
    """The quantized-weight-training cache and the eval cache are keyed on more than the parameter's version counter:
    an optimizer that writes through ``p.data`` is seen through the process-wide optimizer step count, and a bare
    ``weight.data`` edit through ``invalidate_quantized_weight()``.  Each forward is compared with a module that holds
    the same weight and no cache."""
    with config_as(pkg, 128, torch.bfloat16):
        torch.manual_seed(1)
        lin = pkg.BlockInt8Linear(256, 128, device=DEV, dtype=torch.bfloat16, quantized_weight_training=True)
        assert lin.quantized_weight_training
        fresh = lambda: pkg.blockwise_int8_linear.apply(x, lin.weight.detach(), lin.bias.detach())
        x = torch.randn(32, 256, device=DEV, dtype=torch.bfloat16)
        y0 = lin(x)
        assert torch.equal(y0, fresh())
        opt = _DataSGD(lin.parameters(), lr=0.5)
        y0.float().pow(2).mean().backward()
        v = lin.weight._version
        opt.step()
        assert lin.weight._version == v                         # nothing the version counter could have told
        y1 = lin(x)
        assert torch.equal(y1, fresh()) and not torch.equal(y1, y0)
        # a bare edit through .data: the module has to be told
        lin.weight.data.mul_(2.0)
        assert torch.equal(lin(x), y1)                          # (documented: stale until invalidated)
        lin.invalidate_quantized_weight()
        y2 = lin(x)
        assert torch.equal(y2, fresh()) and not torch.equal(y2, y1)
        # the eval cache is keyed the same way
        lin.eval()
        with torch.no_grad():
            e0 = lin(x)
            lin.weight.data.mul_(0.5)
            lin.invalidate_quantized_weight()
            e1 = lin(x)
            q, s = pkg.quantize_block_rowwise(lin.weight.detach())
        assert torch.equal(lin.W_int8, q) and torch.equal(lin.state_W, s) and not torch.equal(e0, e1)


def test_recursive_surgery(pkg):
    class Inner(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(128, 128)
            self.deep = nn.Sequential(nn.Linear(128, 256), nn.GELU(), nn.Linear(256, 128, bias=False))

        def forward(self, x):
            return self.deep(self.fc(x))

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.a = nn.Linear(128, 128)
            self.inner = Inner()
            self.norm = nn.LayerNorm(128)

        def forward(self, x):
            return self.norm(self.inner(self.a(x)))

    net = Net().to(DEV).to(torch.bfloat16)
    ptrs = {n: p.data_ptr() for n, p in net.named_parameters()}
    out = pkg.replace_linear_with_blockwise_int8_recursive(net)
    assert out is net
    lins = [m for m in net.modules() if isinstance(m, nn.Linear)]
    assert len(lins) == 4 and all(isinstance(m, pkg.BlockInt8Linear) for m in lins)
    assert {n: p.data_ptr() for n, p in net.named_parameters()} == ptrs          # same storage, same names
    assert isinstance(net.norm, nn.LayerNorm) and net.inner.deep[2].bias is None
    with config_as(pkg, 128, torch.bfloat16):
        x = torch.randn(2, 24, 128, device=DEV, dtype=torch.bfloat16, requires_grad=True)
        net(x).float().pow(2).mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in net.parameters())
