"""Drop-in for the reference's block_linear.py: ``BlockInt8Linear`` (an ``nn.Linear`` whose forward and
backward run blockwise-int8 GEMMs), its autograd function and the model-surgery helper, rewired onto the
HIP operators of ``ops.py``.

Differences from the reference that do not change results:
  * the transposes of W, X and G that the backward pass quantizes (``.t().contiguous()`` followed by the row
    quantizer, block_linear.py:93-94, :100-103) are never materialized, and each of X, W and G is read once for both
    of its quantization directions (X and W in the forward pass, whose transposed codes are what is saved for backward);
  * ``ctx.save_for_backward`` is called, not assigned over (block_linear.py:73);
  * the bias gradient ``G.sum(dim=0)`` (block_linear.py:110) comes out of the kernel that quantizes G (same read of G;
    fp32 sums in a fixed order);
  * switching the module back to training mode drops the cached int8 weights, so a later ``eval()``
    re-quantizes the current weights (the reference keeps serving the first cache, block_linear.py:138-139);
  * the eval path with one or two rows (token-by-token decode) quantizes and multiplies in one kernel
    (block_linear.py:141-144 are two launches; from three rows on the two launches run);
  * ``blockwise_int8_linear_Wint8`` is the working form of the reference's function of that name
    (block_linear.py:42-67, which passes un-quantized activations to the GEMM and multiplies the gradient with weight
    codes blocked along the wrong dimension): the forward pass runs on weight codes quantized ahead of time, the
    grad-input GEMM on a second copy of the weights quantized along the output features.
"""
from __future__ import annotations

import torch
import torch.nn as nn
from torch.optim.optimizer import register_optimizer_step_post_hook

from . import block_linear_config
from .ops import (
    _int8_matmul,
    _quantize_block_dual,
    dequantize_block_rowwise,
    few_rows_plan,
    int8_matmul_block64_rowwise_dequantize,
    quantize_block_dual,
    quantize_block_rowwise,
    quantize_block_transposed,
)


def replace_linear_with_blockwise_int8_recursive(model):
    """``replace_linear_with_blockwise_int8`` applied to `model` and to every module below it: every ``nn.Linear``
    of the tree becomes a ``BlockInt8Linear`` (the reference's helper handles one level, block_linear.py:18)."""
    return model.apply(replace_linear_with_blockwise_int8)


def replace_linear_with_blockwise_int8(model):
    """Swap the DIRECT child ``nn.Linear`` modules of `model` for ``BlockInt8Linear`` sharing the same
    weight/bias storage (block_linear.py:16-32; use ``model.apply(...)`` to recurse)."""
    to_be_replaced = [name for name, module in model.named_children()
                      if isinstance(module, nn.Linear) and not isinstance(module, BlockInt8Linear)]
    for name in to_be_replaced:
        module = model._modules[name]
        new = BlockInt8Linear(module.in_features, module.out_features, module.bias is not None,
                              module.weight.device, module.weight.dtype)
        new.weight.data = module.weight.data
        if module.bias is not None:
            new.bias.data = module.bias.data
        new.train(module.training)
        model._modules[name] = new
    return model


# Every optimizer step in the process moves this count, which is part of the state the cached int8 weights are keyed on:
# optimizers that update through ``p.data`` (apex- and DeepSpeed-style) leave the parameter's version counter alone.
_optimizer_steps = [0]


def _count_optimizer_step(optimizer, args, kwargs):
    _optimizer_steps[0] += 1


register_optimizer_step_post_hook(_count_optimizer_step)


class blockwise_int8_linear(torch.autograd.Function):
    """y = x @ W.T + bias with both operands block-quantized on the fly (block_linear.py:69-112).

    The backward pass needs X and W quantized along the other direction (blocks over the tokens for grad_W, over the
    output features for grad_X; block_linear.py:93-94, :100-103).  Those codes are produced in the forward pass by the
    same read of X and W (``quantize_block_dual``) and saved in place of X and W; the numbers are the ones the
    reference computes from the saved X and W in its backward."""

    @staticmethod
    def forward(ctx, X_3D, W, bias):
        X = X_3D.reshape(-1, X_3D.size(-1))
        need_gx, need_gw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if need_gw:
            X_int8, state_X, Xt_int8, Xt_state = quantize_block_dual(X)         # [M,K] and [K,M], [M/B,K]
        else:
            X_int8, state_X = quantize_block_rowwise(X)
            Xt_int8 = Xt_state = None
        if need_gx:
            # [N,K] and [K,N], [N/B,K]; the transposed codes sit in rows padded with zero codes to a multiple of 128
            # (they are a GEMM operand contracted over N, which may be e.g. a 50257-word vocabulary)
            W_int8, state_W, Wt_int8, Wt_state, _, Wt_store = _quantize_block_dual(W, block_linear_config.GROUP_SIZE, pad=True)
        else:
            W_int8, state_W = quantize_block_rowwise(W)
            Wt_int8 = Wt_state = Wt_store = None
        ctx.save_for_backward(Xt_int8, Xt_state, Wt_store, Wt_state)
        ctx.contraction_n = W.shape[0]
        out = int8_matmul_block64_rowwise_dequantize(X_int8, W_int8.t(), state_X, state_W, bias)
        return out.view(*X_3D.size()[:-1], -1)

    @staticmethod
    def backward(ctx, G_3D):
        G = G_3D.reshape(-1, G_3D.size(-1))
        grad_X = grad_W = grad_bias = None
        Xt_int8, Xt_state, Wt_store, Wt_state = ctx.saved_tensors
        need_gx, need_gw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        g_store = None
        need_gb = ctx.needs_input_grad[2]
        if need_gx and need_gw:
            # one read of G for both GEMMs (the row codes padded like the transposed W codes they are multiplied with)
            # and, if there is a bias, for its gradient G.sum(dim=0) (block_linear.py:110)
            g_int8, g_state, gt_int8, gt_state, g_store, _, *rest = _quantize_block_dual(G, block_linear_config.GROUP_SIZE, pad=True,
                                                                                         colsum=need_gb)
            if need_gb:
                grad_bias = rest[0]
        elif need_gx:
            g_int8, g_state = quantize_block_rowwise(G)
        elif need_gw:
            gt_int8, gt_state = quantize_block_transposed(G)                    # [N,M], [M/B,N]
        if need_gx:
            # grad_X [M,K] = G [M,N] @ W [N,K]: contraction over N, W quantized along N
            Wt_int8 = Wt_store[:, :ctx.contraction_n]
            grad_X = _int8_matmul(g_int8, Wt_int8.t(), g_state, Wt_state, None, g_store, Wt_store)
            grad_X = grad_X.view(*G_3D.size()[:-1], -1)
        if need_gw:
            # grad_W [N,K] = G.T [N,M] @ X [M,K]: contraction over the tokens, both quantized along M
            grad_W = int8_matmul_block64_rowwise_dequantize(gt_int8, Xt_int8.t(), gt_state, Xt_state)
        if need_gb and grad_bias is None:
            grad_bias = G.sum(dim=0)
        return grad_X, grad_W, grad_bias


def quantize_weight_for_training(W):
    """Both quantized copies of a weight W [N,K] that a training step multiplies with:
    (W_int8 [N,K], state_W [ceil(K/B),N]) blocked along the input features for the forward GEMM (block_linear.py:79),
    (Wt_int8 [K,N], Wt_state [ceil(N/B),K]) blocked along the output features for the grad-input GEMM (:93-94), from one
    read of W.  Wt_int8 is a view of rows padded with zero codes to a multiple of 128 (returned last), which is what
    the tiled GEMM kernels want of a contraction dimension such as a 50257-word vocabulary."""
    W_int8, state_W, Wt_int8, Wt_state, _, Wt_store = _quantize_block_dual(W.detach(), block_linear_config.GROUP_SIZE, pad=True)
    return W_int8, state_W, Wt_int8, Wt_state, Wt_store


class blockwise_int8_linear_Wint8(torch.autograd.Function):
    """y = x @ W.T + bias on weights quantized AHEAD of the call (what block_linear.py:42-67 set out to be).

    ``apply(x, W_int8, state_W, bias, Wt_int8, Wt_state, weight=None, Wt_store=None)``:
      W_int8 [N,K], state_W [K/B,N]    the weight blocked along K: forward GEMM, as in BlockInt8Linear.infer;
      Wt_int8 [K,N], Wt_state [N/B,K]  the weight transposed and blocked along N: grad_X = G @ W contracts over N;
      weight                           optional float tensor that stands for W in the autograd graph: it receives
                                       grad_W = G.T @ X (block_linear.py:100-104) and is not read;
      Wt_store                         optional zero-padded buffer that Wt_int8 is a view of (quantize_weight_for_training).
    The first four arguments are the reference's; with the copies made by ``quantize_weight_for_training(W)`` the outputs
    and gradients are bit for bit those of ``blockwise_int8_linear.apply(x, W, bias)``, without quantizing W in the step."""

    @staticmethod
    def forward(ctx, X_3D, W_int8, state_W, bias, Wt_int8, Wt_state, weight=None, Wt_store=None):
        X = X_3D.reshape(-1, X_3D.size(-1))
        need_gw = weight is not None and ctx.needs_input_grad[6]
        if need_gw:
            X_int8, state_X, Xt_int8, Xt_state = quantize_block_dual(X)         # [M,K] and [K,M], [M/B,K]
        else:
            X_int8, state_X = quantize_block_rowwise(X)
            Xt_int8 = Xt_state = None
        ctx.save_for_backward(Xt_int8, Xt_state, Wt_int8, Wt_state, Wt_store)
        out = int8_matmul_block64_rowwise_dequantize(X_int8, W_int8.t(), state_X, state_W, bias)
        return out.view(*X_3D.size()[:-1], -1)

    @staticmethod
    def backward(ctx, G_3D):
        G = G_3D.reshape(-1, G_3D.size(-1))
        grad_X = grad_W = grad_bias = None
        Xt_int8, Xt_state, Wt_int8, Wt_state, Wt_store = ctx.saved_tensors
        need_gx, need_gw = ctx.needs_input_grad[0], Xt_int8 is not None
        g_store = None
        need_gb = ctx.needs_input_grad[3]
        if need_gx and need_gw:
            g_int8, g_state, gt_int8, gt_state, g_store, _, *rest = _quantize_block_dual(G, block_linear_config.GROUP_SIZE, pad=True,
                                                                                         colsum=need_gb)
            if need_gb:
                grad_bias = rest[0]
        elif need_gx:
            g_int8, g_state = quantize_block_rowwise(G)
        elif need_gw:
            gt_int8, gt_state = quantize_block_transposed(G)                    # [N,M], [M/B,N]
        if need_gx:
            grad_X = _int8_matmul(g_int8, Wt_int8.t(), g_state, Wt_state, None, g_store, Wt_store)
            grad_X = grad_X.view(*G_3D.size()[:-1], -1)
        if need_gw:
            grad_W = int8_matmul_block64_rowwise_dequantize(gt_int8, Xt_int8.t(), gt_state, Xt_state)
        if need_gb and grad_bias is None:
            grad_bias = G.sum(dim=0)
        # one entry per argument that apply() was given (the last two are optional)
        return (grad_X, None, None, grad_bias, None, None, grad_W, None)[:len(ctx.needs_input_grad)]


class BlockInt8Linear(nn.Linear):
    """``nn.Linear`` replacement (block_linear.py:114-152).  Training mode: ``blockwise_int8_linear``.
    Eval mode: weights quantized once into the buffers ``W_int8`` [N,K] int8 and ``state_W``
    [ceil(K/B),N], activations quantized per call, one fused GEMM."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None, *,
                 quantized_weight_training: bool = False):
        super().__init__(in_features, out_features, bias, device, dtype)
        # training on weight codes quantized ahead of the step (blockwise_int8_linear_Wint8): the codes are made when
        # the weight has changed since they were last made (frozen weights, several micro-batches per optimizer step:
        # once), not in every forward and again in every backward pass
        self.quantized_weight_training = quantized_weight_training
        self._train_cache = None
        self._eval_cache_of = None                 # state of the weight the eval cache was quantized from
        self._invalidations = 0
        self._few_rows = None                      # (key, closure) of the one-launch decode path

    def _weight_state(self):
        """Changes whenever the weight's values may have: in-place updates through the parameter bump its version,
        assignments move the data, every ``torch.optim`` optimizer step anywhere in the process moves the step count
        (an optimizer that writes through ``p.data`` bumps no version), and ``invalidate_quantized_weight()`` covers
        the writes that none of these see (``p.data.copy_(ema)`` outside an optimizer)."""
        w = self.weight
        return (w._version, w.data_ptr(), block_linear_config.GROUP_SIZE, _optimizer_steps[0], self._invalidations)

    def invalidate_quantized_weight(self):
        """Drop the cached int8 copies of the weight (eval cache and quantized-weight-training cache): the next forward
        quantizes the weight again.  Needed after the weight's VALUES were changed behind the parameter's back, i.e.
        through ``weight.data`` outside a ``torch.optim`` optimizer step; every other kind of update is noticed."""
        self._invalidations += 1

    def prepare_for_eval(self):
        W_int8, state_W = quantize_block_rowwise(self.weight.detach())
        self.register_buffer("W_int8", W_int8)
        self.register_buffer("state_W", state_W)
        self._eval_cache_of = self._weight_state()

    def prepare_for_quantized_weight_training(self):
        """(re)make the two quantized copies of the weight that ``blockwise_int8_linear_Wint8`` multiplies with"""
        self._train_cache = (self._weight_state(),) + quantize_weight_for_training(self.weight)

    def weight_quant_training(self, x=None):
        """Replace the weight by its quantize->dequantize image (block_linear.py:130-135).  As in the
        reference the attribute becomes a plain tensor, no longer a Parameter."""
        W_int8, state_W = quantize_block_rowwise(self.weight.detach())
        del self.weight
        self.weight = dequantize_block_rowwise(W_int8, state_W)

    def infer(self, x):
        # quantize the weight on first use (block_linear.py:138-139) and again when it has changed since: the reference
        # keeps serving the first cache
        bufs = self._buffers                       # (read directly: Module.__getattr__ costs as much as a tensor op)
        if bufs.get("W_int8") is None or self._eval_cache_of != self._weight_state():
            self.prepare_for_eval()
        W_int8, state_W, bias = bufs["W_int8"], bufs["state_W"], self._parameters.get("bias")
        X = x.reshape(-1, x.size(-1))
        out = None
        if X.shape[0] <= 2:
            # token-by-token decode: quantize and multiply in one kernel.  Every workgroup of that kernel quantizes x
            # for itself, which pays off for one or two rows (measured; from four rows on the two launches are as fast).
            # What does not change from token to token (shapes, pointers of the cached weights, the configuration) is
            # checked once and kept in a closure: the Python side of a decode step is most of its cost.
            # (the closure holds the tensors it was made for, so their ids stay theirs)
            key = (X.shape, X.dtype, block_linear_config.GROUP_SIZE, block_linear_config.INPUT_OUTPUT_TORCH_TYPE,
                   id(W_int8), id(state_W), id(bias))
            plan = self._few_rows
            if plan is None or plan[0] != key:
                plan = self._few_rows = (key, few_rows_plan(X, W_int8, state_W, bias))
            if plan[1] is not None:
                out = plan[1](X)
        if out is None:
            X_int8, state_X = quantize_block_rowwise(X)
            out = int8_matmul_block64_rowwise_dequantize(X_int8, W_int8.t(), state_X, state_W, bias)
        return out.view(*x.size()[:-1], -1)

    def forward(self, x):
        if not self.training:
            return self.infer(x)
        if self.quantized_weight_training:
            if self._train_cache is None or self._train_cache[0] != self._weight_state():
                self.prepare_for_quantized_weight_training()
            _, W_int8, state_W, Wt_int8, Wt_state, Wt_store = self._train_cache
            return blockwise_int8_linear_Wint8.apply(x, W_int8, state_W, self.bias, Wt_int8, Wt_state, self.weight, Wt_store)
        return blockwise_int8_linear.apply(x, self.weight, self.bias)

    def train(self, mode: bool = True):
        if mode and "W_int8" in self._buffers:
            del self._buffers["W_int8"]
            del self._buffers["state_W"]
        return super().train(mode)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        # a checkpoint written after the first eval call carries the cached int8 weights
        for name in ("W_int8", "state_W"):
            if prefix + name in state_dict and name not in self._buffers:
                self.register_buffer(name, torch.empty_like(state_dict[prefix + name], device=self.weight.device))
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)
        if prefix + "W_int8" in state_dict:
            # the checkpoint's codes go with the checkpoint's weight, or stand alone in a checkpoint of codes only
            self._eval_cache_of = self._weight_state()


BlockLinear = BlockInt8Linear
