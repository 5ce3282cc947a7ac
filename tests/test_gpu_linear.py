"""GPU tests of the module layer: BlockInt8Linear forward/backward (training and eval paths), model surgery,
config globals read at call time, cached int8 weights in the state dict.  Expected values come from the
PyTorch CPU checker's restatement of block_linear.py:71-112."""
import copy

import pytest
import torch
import torch.nn as nn

from oracle import oracle_torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def pkg():
    import blockwise_int8_linear_amd as p
    from blockwise_int8_linear_amd import _lib
    _lib.load()
    return p


class cfg_as:
    def __init__(self, pkg, block, out):
        self.cfg, self.block, self.out = pkg.block_linear_config, block, out

    def __enter__(self):
        self.old = (self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE)
        self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.block, self.out

    def __exit__(self, *a):
        self.cfg.GROUP_SIZE, self.cfg.INPUT_OUTPUT_TORCH_TYPE = self.old


def _rel(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


@pytest.mark.parametrize("dtype,block,tol", [(torch.float32, 64, 2e-5), (torch.float32, 128, 2e-5), (torch.bfloat16, 128, 6e-3)])
@pytest.mark.parametrize("shape", [(4, 96, 256, 384), (2, 100, 768, 200), (1, 16, 128, 128)])
def test_forward_backward_match_checker(pkg, dtype, block, tol, shape):
    Bt, T, K, N = shape
    g = torch.Generator().manual_seed(K + N)
    x = torch.randn(Bt, T, K, generator=g).to(dtype)
    W = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    b = torch.randn(N, generator=g).to(dtype)
    G = torch.randn(Bt, T, N, generator=g).to(dtype)
    with cfg_as(pkg, block, dtype):
        lin = pkg.BlockInt8Linear(K, N, bias=True, device=DEV, dtype=dtype)
        with torch.no_grad():
            lin.weight.copy_(W); lin.bias.copy_(b)
        xd = x.to(DEV).requires_grad_(True)
        y = lin(xd)
        y.backward(G.to(DEV))
        torch.cuda.synchronize()
        y_ref = oracle_torch.linear_forward(x, W, b, block, dtype)
        gx_ref, gw_ref, gb_ref = oracle_torch.linear_backward(G, x, W, block, dtype)
        assert y.shape == (Bt, T, N) and y.dtype == dtype
        assert _rel(y.cpu(), y_ref) < tol
        assert _rel(xd.grad.cpu(), gx_ref) < tol and xd.grad.shape == x.shape
        assert _rel(lin.weight.grad.cpu(), gw_ref) < tol and lin.weight.grad.shape == W.shape
        assert torch.allclose(lin.bias.grad.cpu().float(), gb_ref.float(), rtol=2e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-3)
        # and the whole thing approximates the dense layer
        dense = x.float().reshape(-1, K) @ W.float().t() + b.float()
        assert _rel(y.cpu().float().reshape(-1, N), dense) < 3e-2
        # eval path: cached int8 weights, same numbers as the training forward
        lin.eval()
        with torch.no_grad():
            y2 = lin(x.to(DEV))
        assert torch.equal(y2, y.detach())
        assert lin.W_int8.shape == (N, K) and lin.W_int8.dtype == torch.int8
        assert lin.state_W.shape == (-(-K // block), N) and lin.state_W.dtype == torch.float32


def test_eval_cache_state_dict_and_invalidation(pkg):
    with cfg_as(pkg, 128, torch.bfloat16):
        lin = pkg.BlockInt8Linear(256, 128, device=DEV, dtype=torch.bfloat16).eval()
        x = torch.randn(8, 256, device=DEV, dtype=torch.bfloat16)
        assert "W_int8" not in lin.state_dict()
        y0 = lin(x)
        sd = lin.state_dict()
        assert set(sd) == {"weight", "bias", "W_int8", "state_W"}
        lin2 = pkg.BlockInt8Linear(256, 128, device=DEV, dtype=torch.bfloat16).eval()
        lin2.load_state_dict(sd)
        assert torch.equal(lin2(x), y0)
        # train() drops the cache; the next eval() sees the updated weight
        lin.train()
        assert "W_int8" not in lin.state_dict()
        with torch.no_grad():
            lin.weight.mul_(2.0)
        lin.eval()
        y1 = lin(x)
        assert not torch.equal(y1, y0)
        ref = copy.deepcopy(lin)
        ref.train(); ref.eval()
        assert torch.equal(ref(x), y1)


def test_replace_linear_is_one_level_and_shares_storage(pkg):
    class Inner(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc = nn.Linear(128, 128)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.a = nn.Linear(128, 256)
            self.b = nn.Linear(256, 128, bias=False)
            self.inner = Inner()
            self.act = nn.GELU()

        def forward(self, x):
            return self.inner.fc(self.b(self.act(self.a(x))))

    net = Net().to(DEV).to(torch.bfloat16)
    wa = net.a.weight.data_ptr()
    out = pkg.replace_linear_with_blockwise_int8(net)
    assert out is net
    assert isinstance(net.a, pkg.BlockInt8Linear) and isinstance(net.b, pkg.BlockInt8Linear)
    assert type(net.inner.fc) is nn.Linear                      # direct children only (block_linear.py:18)
    assert net.a.weight.data_ptr() == wa and net.b.bias is None
    net.apply(pkg.replace_linear_with_blockwise_int8)           # the documented way to recurse
    assert isinstance(net.inner.fc, pkg.BlockInt8Linear)
    x = torch.randn(4, 10, 128, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    with cfg_as(pkg, 128, torch.bfloat16):
        y = net(x)
        y.float().pow(2).mean().backward()
    assert y.shape == (4, 10, 128) and torch.isfinite(y).all()
    for p in net.parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all()
    assert pkg.BlockLinear is pkg.BlockInt8Linear


def test_group_size_is_read_at_call_time(pkg):
    x = torch.randn(32, 512, device=DEV, dtype=torch.bfloat16)
    lin = pkg.BlockInt8Linear(512, 64, device=DEV, dtype=torch.bfloat16)
    outs = {}
    for B in (32, 64, 128):
        with cfg_as(pkg, B, torch.bfloat16):
            q, s = pkg.quantize_block_rowwise(x)
            assert s.shape == (512 // B, 32)
            outs[B] = lin(x)
            ref = oracle_torch.linear_forward(x.cpu(), lin.weight.detach().cpu(), lin.bias.detach().cpu(), B, torch.bfloat16)
            assert _rel(outs[B].detach().cpu(), ref) < 6e-3
    assert not torch.equal(outs[32], outs[128])


def test_weight_quant_training_helper(pkg):
    with cfg_as(pkg, 128, torch.bfloat16):
        lin = pkg.BlockInt8Linear(256, 64, device=DEV, dtype=torch.bfloat16)
        w0 = lin.weight.detach().clone()
        lin.weight_quant_training()
        q, s = pkg.quantize_block_rowwise(w0)
        assert torch.equal(lin.weight, pkg.dequantize_block_rowwise(q, s))
        assert (lin.weight.float() - w0.float()).abs().max() <= s.max() / 254 * 1.01 + 2 ** -9 * w0.abs().max()
