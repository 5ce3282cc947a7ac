"""GPU parity cases shaped like the larger benchmark configurations, at sizes the CPU checker finishes in seconds:
a Llama-style MLP + attention projections with cached int8 weights (prefill, then one-token decode steps), a
GPT-2-style MLP training step (block 64, forward + backward + AdamW on fp32 master weights), and the eval path
recorded into a HIP graph and replayed.  Expected values come from oracle/oracle_torch.py."""
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


class LlamaLinears(nn.Module):
    """the seven projections of one Llama decoder layer (no attention arithmetic, no norms): q, k, v, o and the
    SwiGLU MLP gate / up / down"""

    def __init__(self, hidden, inter):
        super().__init__()
        self.q = nn.Linear(hidden, hidden, bias=False)
        self.k = nn.Linear(hidden, hidden, bias=False)
        self.v = nn.Linear(hidden, hidden, bias=False)
        self.o = nn.Linear(hidden, hidden, bias=False)
        self.gate = nn.Linear(hidden, inter, bias=False)
        self.up = nn.Linear(hidden, inter, bias=False)
        self.down = nn.Linear(inter, hidden, bias=False)

    def forward(self, x):
        a = self.o(self.q(x) * torch.sigmoid(self.k(x)) + self.v(x))
        h = x + a
        return h + self.down(torch.nn.functional.silu(self.gate(h)) * self.up(h))


def _llama_reference(x, weights, block, dtype):
    lin = lambda t, name: oracle_torch.linear_forward(t, weights[name], None, block, dtype)
    a = lin(lin(x, "q") * torch.sigmoid(lin(x, "k")) + lin(x, "v"), "o")
    h = x + a
    return h + lin(torch.nn.functional.silu(lin(h, "gate")) * lin(h, "up"), "down")


def test_llama_layer_linears_prefill_then_decode(pkg):
    """block 128, bf16, int8 weights quantized once (eval path); hidden 512, MLP 1408 (Llama-7B's 4096 / 11008
    scaled by 1/8); prefill of 320 tokens, then single-token steps"""
    hidden, inter, block, dtype = 512, 1408, 128, torch.bfloat16
    torch.manual_seed(3)
    with cfg_as(pkg, block, dtype):
        model = LlamaLinears(hidden, inter).to(dtype)
        for p in model.parameters():
            nn.init.normal_(p, std=0.02)
        weights = {n: getattr(model, n).weight.detach().clone() for n in ("q", "k", "v", "o", "gate", "up", "down")}
        model = model.to(DEV)
        pkg.replace_linear_with_blockwise_int8(model)
        model.eval()
        assert all(isinstance(getattr(model, n), pkg.BlockInt8Linear) for n in weights)
        x = torch.randn(1, 320, hidden).to(dtype)
        with torch.no_grad():
            y = model(x.to(DEV))
            ref = _llama_reference(x, weights, block, dtype)
            assert y.dtype == dtype and _rel(y.cpu(), ref) < 1e-2
            assert model.down.W_int8.shape == (hidden, inter)
            w_before = model.q.W_int8.clone()
            for step in range(3):                                   # decode: one token at a time, cached weights
                t = torch.randn(1, 1, hidden, generator=torch.Generator().manual_seed(step)).to(dtype)
                yt = model(t.to(DEV))
                assert yt.shape == (1, 1, hidden)
                assert _rel(yt.cpu(), _llama_reference(t, weights, block, dtype)) < 1e-2
            assert torch.equal(model.q.W_int8, w_before)


def test_gpt2_mlp_training_step(pkg):
    """block 64, fp32 master weights; d_model 256, MLP 1024 (GPT-2-small's 768 / 3072 scaled by 1/3), 4 x 96 tokens;
    forward, backward (grad-input and grad-weight GEMMs with transposed-block requantization) and an AdamW step"""
    d, inter, block, dtype = 256, 1024, 64, torch.float32
    torch.manual_seed(5)
    with cfg_as(pkg, block, dtype):
        fc = pkg.BlockInt8Linear(d, inter, bias=True, device=DEV, dtype=dtype)
        proj = pkg.BlockInt8Linear(inter, d, bias=True, device=DEV, dtype=dtype)
        with torch.no_grad():
            for lin in (fc, proj):
                lin.weight.normal_(std=0.02)
                lin.bias.normal_(std=0.01)
        Wf, bf, Wp, bp = (t.detach().cpu().clone() for t in (fc.weight, fc.bias, proj.weight, proj.bias))
        x = torch.randn(4, 96, d)
        target = torch.randn(4, 96, d)
        opt = torch.optim.AdamW(list(fc.parameters()) + list(proj.parameters()), lr=1e-3)

        xd = x.to(DEV).requires_grad_(True)
        h = fc(xd)
        a = torch.nn.functional.gelu(h)
        y = proj(a)
        loss = ((y - target.to(DEV)) ** 2).mean()
        loss.backward()

        # the same step on the CPU checker (activation and loss in plain PyTorch)
        h_ref = oracle_torch.linear_forward(x, Wf, bf, block, dtype)
        h_leaf = h_ref.clone().requires_grad_(True)
        a_ref = torch.nn.functional.gelu(h_leaf)
        y_ref = oracle_torch.linear_forward(a_ref.detach(), Wp, bp, block, dtype)
        Gy = 2.0 * (y_ref - target) / y_ref.numel()
        ga_ref, gWp_ref, gbp_ref = oracle_torch.linear_backward(Gy, a_ref.detach(), Wp, block, dtype)
        a_ref.backward(ga_ref)
        gx_ref, gWf_ref, gbf_ref = oracle_torch.linear_backward(h_leaf.grad, x, Wf, block, dtype)

        assert _rel(y.detach().cpu(), y_ref) < 1e-4
        assert _rel(proj.weight.grad.cpu(), gWp_ref) < 1e-3 and _rel(fc.weight.grad.cpu(), gWf_ref) < 1e-3
        assert _rel(xd.grad.cpu(), gx_ref) < 1e-3
        assert torch.allclose(proj.bias.grad.cpu(), gbp_ref.float(), rtol=1e-4, atol=1e-7)
        assert torch.allclose(fc.bias.grad.cpu(), gbf_ref.float(), rtol=1e-3, atol=1e-7)
        before = loss.item()
        opt.step()
        opt.zero_grad()
        with torch.no_grad():
            after = ((proj(torch.nn.functional.gelu(fc(x.to(DEV)))) - target.to(DEV)) ** 2).mean().item()
        assert after < before


def test_eval_path_in_a_hip_graph(pkg):
    """quantize + GEMM of the eval path recorded once and replayed with new inputs; other GPU work and
    synchronizations between the replays; every replay equals the eager result bit for bit"""
    K, N, block, dtype = 1024, 768, 128, torch.bfloat16
    torch.manual_seed(7)
    with cfg_as(pkg, block, dtype):
        lin = pkg.BlockInt8Linear(K, N, bias=True, device=DEV, dtype=dtype).eval()
        static_x = torch.zeros(4, K, device=DEV, dtype=dtype)
        with torch.no_grad():
            lin(static_x)                                           # builds the int8 weight cache outside the graph
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    lin(static_x)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_y = lin(static_x)
            for i in range(4):
                x = torch.randn(4, K, device=DEV, dtype=dtype) * (i + 1)
                eager = lin(x)
                torch.cuda.synchronize()
                static_x.copy_(x)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(static_y, eager)
                assert torch.isfinite(static_y.float()).all()


def test_split_of_k_in_a_hip_graph(pkg):
    """128 rows: the GEMM splits K through a workspace that the operator allocates (inside the capture, from the
    graph's pool); replays with new inputs equal the eager results bit for bit"""
    K, N, block, dtype = 4096, 1024, 128, torch.bfloat16
    torch.manual_seed(8)
    with cfg_as(pkg, block, dtype):
        lin = pkg.BlockInt8Linear(K, N, bias=True, device=DEV, dtype=dtype).eval()
        static_x = torch.zeros(128, K, device=DEV, dtype=dtype)
        with torch.no_grad():
            lin(static_x)
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):
                    lin(static_x)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_y = lin(static_x)
            for i in range(3):
                x = torch.randn(128, K, device=DEV, dtype=dtype) * (i + 1)
                eager = lin(x)
                torch.cuda.synchronize()
                static_x.copy_(x)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(static_y, eager)


def test_reference_benchmark_sweep_and_accuracy_demo(pkg):
    """the sweep of triton_functions.py:521-566 at two small sizes (every provider returns positive rates) and the
    demo scenario of block_linear.py:161-224 (errors of a few percent at most, smaller for smaller blocks)"""
    from blockwise_int8_linear_amd import triton_functions as tf
    from blockwise_int8_linear_amd.examples import accuracy
    rows = tf.benchmark(sizes=[256, 512], print_data=False)
    assert set(rows) == {"dense", "int8 matmul", "blockwise_int8", "blockwise_int8_quantise", "dense+copy"}
    assert all(len(v) == 2 and all(r[1] > 0 for r in v) for v in rows.values())
    a = torch.randn(70, 256, device=DEV).bfloat16()
    b = torch.randn(90, 256, device=DEV).bfloat16()
    assert ((tf.fast_matmulT(a, b).float() - a.float() @ b.float().t()).norm() / (a.float() @ b.float().t()).norm()).item() < 0.03
    err = {blk: accuracy.demo_case(blk) for blk in (32, 128)}
    for blk in err:
        for what in ("output", "grad_weight", "grad_input"):
            assert err[blk][what]["rel"] < 0.03
    assert err[32]["output"]["rel"] < err[128]["output"]["rel"]
    assert accuracy.forward_case()["rel"] < 0.03
