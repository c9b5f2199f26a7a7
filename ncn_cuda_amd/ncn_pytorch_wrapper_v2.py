"""autograd.Function / nn.Module surface of the reference's ncn_cuda/ncn_pytorch_wrapper_v2.py.

Same class and function names, same constructor and call signatures, same state_dict keys
(`weight`, `ncn_modules.{l}.weight`), so a model written against the reference imports these
instead and changes nothing else.  Behavioural differences:
  * NCNModuleCuda.forward passes (n_cache, n_head) in the order fused_ncn_cuda_v2 expects; the
    reference swaps them (ncn_pytorch_wrapper_v2.py:93-102 vs :53-62), which only works when both
    are equal;
  * reset_parameters uses the stored embed_dim (the reference reads an attribute it never sets,
    ncn_pytorch_wrapper_v2.py:87-90);
  * bfloat16 inputs are supported: the node then saves float32 copies of its outputs, because the
    reversible backward divides by m at every step and would amplify bf16 rounding past 2e-2.
"""
import math
from typing import Tuple

import torch
from torch import nn

from . import ncn_cuda_module

ACTIVATION_CODES = {"tanh": 0, "relu": 1, "sigmoid": 2, "linear": -1}  # ncn_pytorch_wrapper_v2.py:111


class NCNFunction(torch.autograd.Function):
    """One stage.  forward saves (yi, ya, W) and inverts them in backward, like the reference node
    (ncn_pytorch_wrapper_v2.py:9-50)."""

    @staticmethod
    def forward(ctx, x, xa, W, alpha, activation, n_cache, n_head, module_l):
        if x.dtype == torch.float32:
            yi, ya = ncn_cuda_module.forward_stages(x, xa, W, alpha, activation, n_cache, n_head, module_l, 1)
            ctx.save_for_backward(yi, ya, W)
        else:
            yi, ya, y32, ya32 = ncn_cuda_module.forward_stages(x, xa, W, alpha, activation, n_cache, n_head,
                                                               module_l, 1, save_fp32=True)
            ctx.save_for_backward(y32, ya32, W)
        ctx.alpha = alpha
        ctx.activation = activation
        ctx.n_cache = n_cache
        ctx.n_head = n_head
        ctx.module_l = module_l
        ctx.io_dtype = x.dtype
        return yi, ya

    @staticmethod
    def backward(ctx, dyi, dya):
        (yi, ya, W) = ctx.saved_tensors
        _, _, dx, dxa, dW = ncn_cuda_module.backward_stages(
            yi, ya, dyi, dya, W, ctx.alpha, ctx.activation, ctx.n_cache, ctx.n_head, ctx.module_l, 1,
            grad_dtype=ctx.io_dtype, want_inputs=False)
        sum_dW = dW.reshape(W.shape).to(W.dtype)
        return dx, dxa, sum_dW, None, None, None, None, None


def fused_ncn_cuda_v2(
    x: torch.Tensor,
    xa: torch.Tensor,
    W: torch.Tensor,
    alpha: float,
    activation: int,
    n_cache: int,
    n_head: int,
    module_l: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    yi, ya = NCNFunction.apply(x, xa, W, alpha, activation, n_cache, n_head, module_l)
    return yi, ya


class NCNModuleCuda(nn.Module):
    def __init__(self, alpha, activation, n_cache, n_head, module_nr, embed_dim):
        super().__init__()
        self.alpha = alpha
        self.activation = activation
        self.n_cache = n_cache
        self.n_head = n_head
        self.module_nr = module_nr
        self.embed_dim = embed_dim
        self.weight = nn.Parameter(torch.ones(2 * embed_dim).normal_(mean=0.0, std=1 / (2.0 * embed_dim)),
                                   requires_grad=True)

    def reset_parameters(self):
        stdv = 1.0 / math.sqrt(self.embed_dim)
        for weight in self.parameters():
            weight.data.uniform_(-stdv, +stdv)

    def forward(self, x, xa):
        return fused_ncn_cuda_v2(x, xa, self.weight, self.alpha, self.activation, self.n_cache, self.n_head,
                                 self.module_nr)


class NCNNetCuda(nn.Module):
    def __init__(self, alpha, activation, n_cache, n_head, num_modules, embed_dim):
        super().__init__()
        self.num_modules = num_modules
        activation_nr = ACTIVATION_CODES[activation]
        self.ncn_modules = nn.ModuleList(
            [NCNModuleCuda(alpha, activation_nr, n_cache, n_head, module_nr, embed_dim)
             for module_nr in range(num_modules)])

    def forward(self, x, xa):
        for module_nr in range(self.num_modules):
            x, xa = self.ncn_modules[module_nr](x, xa)
        return x, xa


class NCNNetTestCuda(nn.Module):
    def __init__(self, alpha, activation, n_cache, n_head, num_modules, weights):
        super().__init__()
        self.num_modules = num_modules
        self.alpha = alpha
        self.activation_nr = ACTIVATION_CODES[activation]
        self.n_cache = n_cache
        self.n_head = n_head
        self.weights = weights

    def forward(self, x, xa):
        for module_nr in range(self.num_modules):
            x, xa = fused_ncn_cuda_v2(x, xa, self.weights[module_nr], self.alpha, self.activation_nr,
                                      self.n_cache, self.n_head, module_nr)
        return x, xa


def ncn_inverse(y, ya, W, alpha, activation, n_cache, n_head, module_l):
    """Inputs of one stage from its outputs (no autograd)."""
    x, xa = ncn_cuda_module.inverse_stages(y, ya, W, alpha, activation, n_cache, n_head, module_l, 1)
    return x, xa
