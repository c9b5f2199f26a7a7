"""autograd.Function / nn.Module surface of the reference's ncn_cuda/ncn_pytorch_wrapper_v2.py.

Same class and function names, same constructor and call signatures, same state_dict keys
(`weight`, `ncn_modules.{l}.weight`), so a model written against the reference imports these
instead and changes nothing else.  Behavioural differences:
  * NCNModuleCuda.forward passes (n_cache, n_head) in the order fused_ncn_cuda_v2 expects; the
    reference swaps them (ncn_pytorch_wrapper_v2.py:93-102 vs :53-62), which only works when both
    are equal;
  * reset_parameters uses the stored embed_dim (the reference reads an attribute it never sets,
    ncn_pytorch_wrapper_v2.py:87-90);
  * bfloat16 inputs are supported: the node then saves, beside its bfloat16 outputs, what their rounding took away
    (a second bfloat16 plane; float32 copies on the generic kernels), because the reversible backward divides by m at
    every step and would amplify bare bf16 rounding past 2e-2.
"""
import math
from typing import Tuple

import torch
from torch import nn

from . import ncn_cuda_module

__all__ = ["ACTIVATION_CODES", "NCNFunction", "NCNNetFunction", "NCNRadixNetFunction", "NCNModuleCuda", "NCNNetCuda",
           "NCNNetTestCuda", "default_save_every", "fused_ncn_cuda_v2", "fused_ncn_net", "fused_ncn_radix_net",
           "ncn_inverse"]

# names and codes of ncn_pytorch_wrapper_v2.py:111, plus the leaky relu of the Triton kernels (ncn_triton.py:101)
ACTIVATION_CODES = {"tanh": 0, "relu": 1, "sigmoid": 2, "linear": -1, "leaky-relu": 3}


class NCNFunction(torch.autograd.Function):
    """One stage.  forward saves (yi, ya, W) and inverts them in backward, like the reference node
    (ncn_pytorch_wrapper_v2.py:9-50)."""

    @staticmethod
    def forward(ctx, x, xa, W, alpha, activation, n_cache, n_head, module_l):
        yi, ya, sy, sya = ncn_cuda_module.forward_stages_saving(x, xa, W, alpha, activation, n_cache, n_head, module_l)
        ctx.save_for_backward(sy, sya, W)
        # an output nobody differentiates (ya of the last stage under yi.backward(dyi), grad_test_bench.py:121) arrives
        # as None instead of a tensor of zeros that autograd would have to fill and the kernel to read
        ctx.set_materialize_grads(False)
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
        if dyi is None:
            if dya is None:
                return (None,) * 8
            dyi = torch.zeros_like(dya)
        _, _, dx, dxa, dW = ncn_cuda_module.backward_stages(
            yi, ya, dyi, dya, W, ctx.alpha, ctx.activation, ctx.n_cache, ctx.n_head, ctx.module_l, 1,
            grad_dtype=ctx.io_dtype, want_inputs=False)
        sum_dW = dW.reshape(W.shape).to(W.dtype)
        return dx, dxa, sum_dW, None, None, None, None, None


# Saved activations that the whole-net node may keep before it trades memory for time (see default_save_every).
SAVE_BUDGET_BYTES = 32 << 30


def default_save_every(n_cache: int, n_stages: int = None, elements: int = None, budget_bytes: int = None) -> int:
    """Stages per saved checkpoint of the whole-net node.

    Groups of 2 and 4 rows run several stages per launch out of LDS, so long segments save HBM round trips; the
    reversible backward amplifies float32 rounding by (1/m)^(n_cache * stages) between checkpoints, and 26 steps keep
    that below 16x at m = 0.9: segments of 26 // n_cache stages.
    Larger groups run one launch per stage whatever the segment, and a backward launch that need not hand the
    reconstructed inputs on to the next stage moves 6 instead of 7-8 arrays: every stage's outputs are kept (which the
    forward writes anyway) as long as they fit the budget, 2 float32 arrays of `elements` values per stage against
    `budget_bytes` (default SAVE_BUDGET_BYTES); beyond it, or when the sizes are not given, segments as above."""
    by_rounding = max(1, 26 // max(1, int(n_cache)))
    if int(n_cache) <= 4 or n_stages is None or elements is None:
        return by_rounding
    budget = SAVE_BUDGET_BYTES if budget_bytes is None else int(budget_bytes)
    return 1 if 2 * 4 * int(elements) * int(n_stages) <= budget else by_rounding


class NCNNetFunction(torch.autograd.Function):
    """The whole stage stack as ONE autograd node (no counterpart in the reference, which chains one NCNFunction
    per stage, ncn_pytorch_wrapper_v2.py:107-117).  Stages run `save_every` at a time through the library's
    multi-stage calls; only the outputs of every `save_every`-th stage are kept for backward, which reverses each
    segment from its outputs.  Segments of several stages keep float32 between the stages whatever the I/O dtype;
    segments of one stage keep the I/O dtype and save what NCNFunction saves (for bfloat16 the outputs plus what
    their rounding took away, as two bfloat16 planes)."""

    @staticmethod
    def forward(ctx, x, xa, alpha, activation, n_cache, n_head, first_stage, save_every, *weights):
        L = len(weights)
        save_every = default_save_every(n_cache, L, x.numel()) if not save_every else int(save_every)
        W = torch.stack([w.detach().reshape(-1).to(torch.float32) for w in weights])
        saved = []
        cx, cxa = x, xa
        segs = [(a, min(save_every, L - a)) for a in range(0, L, save_every)]
        for a, cnt in segs:
            if cnt == 1 and cx.dtype == x.dtype:
                cx, cxa, sy, sya = ncn_cuda_module.forward_stages_saving(cx, cxa, W[a], alpha, activation, n_cache,
                                                                         n_head, first_stage + a)
                saved.extend([sy, sya])
            else:
                cx, cxa = ncn_cuda_module.forward_stages(cx, cxa, W[a:a + cnt], alpha, activation, n_cache, n_head,
                                                         first_stage + a, cnt, out_dtype=torch.float32)
                saved.extend([cx, cxa])
        ctx.save_for_backward(W, *saved)
        ctx.set_materialize_grads(False)   # a missing upstream gradient stays None (see NCNFunction)
        ctx.cfg = (alpha, activation, n_cache, n_head, first_stage, segs, x.dtype, [w.dtype for w in weights],
                   [w.shape for w in weights])
        return cx.to(x.dtype), cxa.to(x.dtype)

    @staticmethod
    def backward(ctx, dyi, dya):
        W, *saved = ctx.saved_tensors
        alpha, activation, n_cache, n_head, first_stage, segs, io_dtype, w_dtypes, w_shapes = ctx.cfg
        dWs = [None] * W.shape[0]
        if dyi is None:
            if dya is None:
                return (None,) * (8 + W.shape[0])
            dyi = torch.zeros_like(dya)
        g, ga = dyi, dya
        for k in range(len(segs) - 1, -1, -1):
            a, cnt = segs[k]
            # a one-stage segment hands its gradients on in the dtype they came in (bfloat16 stays bfloat16)
            gd = g.dtype if cnt == 1 else torch.float32
            Wk = W[a] if cnt == 1 else W[a:a + cnt]
            _, _, g, ga, dW = ncn_cuda_module.backward_stages(
                saved[2 * k], saved[2 * k + 1], g, ga, Wk, alpha, activation, n_cache, n_head,
                first_stage + a, cnt, grad_dtype=gd, want_inputs=False)
            for j in range(cnt):
                dWs[a + j] = dW[j].reshape(w_shapes[a + j]).to(w_dtypes[a + j])
        return (g.to(io_dtype), ga.to(io_dtype), None, None, None, None, None, None, *dWs)


class NCNRadixNetFunction(torch.autograd.Function):
    """Like NCNNetFunction, for levels first_level .. of the radix-n digit grouping (ncn_triton/group_tensors.py:8-18)
    instead of the stride permutation: weights[k] belongs to level first_level + k."""

    @staticmethod
    def forward(ctx, x, xa, alpha, activation, n_cache, n_head, first_level, save_every, *weights):
        L = len(weights)
        save_every = default_save_every(n_cache) if not save_every else int(save_every)
        W = torch.stack([w.detach().reshape(-1).to(torch.float32) for w in weights])
        saved = []
        cx, cxa = x, xa
        segs = [(a, min(save_every, L - a)) for a in range(0, L, save_every)]
        for a, cnt in segs:
            cx, cxa = ncn_cuda_module.forward_radix(cx, cxa, W[a:a + cnt], alpha, activation, n_cache, n_head,
                                                    first_level + a, cnt)
            saved.extend([cx, cxa])
        ctx.save_for_backward(W, *saved)
        ctx.set_materialize_grads(False)   # a missing upstream gradient stays None (see NCNFunction)
        ctx.cfg = (alpha, activation, n_cache, n_head, first_level, segs, x.dtype, [w.dtype for w in weights],
                   [w.shape for w in weights])
        return cx.to(x.dtype), cxa.to(x.dtype)

    @staticmethod
    def backward(ctx, dyi, dya):
        W, *saved = ctx.saved_tensors
        alpha, activation, n_cache, n_head, first_level, segs, io_dtype, w_dtypes, w_shapes = ctx.cfg
        dWs = [None] * W.shape[0]
        if dyi is None:
            if dya is None:
                return (None,) * (8 + W.shape[0])
            dyi = torch.zeros_like(dya)
        g, ga = dyi, dya
        for k in range(len(segs) - 1, -1, -1):
            a, cnt = segs[k]
            _, _, g, ga, dW = ncn_cuda_module.backward_radix(saved[2 * k], saved[2 * k + 1], g, ga, W[a:a + cnt], alpha,
                                                             activation, n_cache, n_head, first_level + a, cnt,
                                                             want_inputs=False)
            for j in range(cnt):
                dWs[a + j] = dW[j].reshape(w_shapes[a + j]).to(w_dtypes[a + j])
        return (g.to(io_dtype), ga.to(io_dtype), None, None, None, None, None, None, *dWs)


def fused_ncn_radix_net(x, xa, weights, alpha, activation, n_cache, n_head, first_level=0, save_every=None):
    """Radix levels first_level .. first_level+len(weights)-1 as one autograd node; activation is the int code."""
    return NCNRadixNetFunction.apply(x, xa, alpha, activation, n_cache, n_head, first_level, save_every, *weights)


def fused_ncn_net(x, xa, weights, alpha, activation, n_cache, n_head, first_stage=0, save_every=None):
    """Stages first_stage .. first_stage+len(weights)-1 as one autograd node; activation is the int code."""
    return NCNNetFunction.apply(x, xa, alpha, activation, n_cache, n_head, first_stage, save_every, *weights)


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


def _check_grouping(grouping):
    """"stride": the stage permutation of torch_ref (the reference's only layout on this surface); "radix": module l is
    level l of the radix-n digit grouping of ncn_triton/group_tensors.py (keyword only, not in the reference)."""
    if grouping not in ("stride", "radix"):
        raise ValueError(f"grouping must be 'stride' or 'radix', got {grouping!r}")
    return grouping


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
    """Same constructor as the reference.  `fuse_stages=True` (keyword only, not in the reference) runs the stack as
    one NCNNetFunction node instead of one node per module; parameters and state_dict are the same either way."""

    def __init__(self, alpha, activation, n_cache, n_head, num_modules, embed_dim, *, grouping="stride", fuse_stages=False,
                 save_every=None):
        super().__init__()
        self.num_modules = num_modules
        self.alpha = alpha
        self.activation_nr = ACTIVATION_CODES[activation]
        self.n_cache = n_cache
        self.n_head = n_head
        self.fuse_stages = fuse_stages
        self.save_every = save_every
        self.grouping = _check_grouping(grouping)
        self.ncn_modules = nn.ModuleList(
            [NCNModuleCuda(alpha, self.activation_nr, n_cache, n_head, module_nr, embed_dim)
             for module_nr in range(num_modules)])

    def forward(self, x, xa):
        if self.grouping == "radix":
            return fused_ncn_radix_net(x, xa, [m.weight for m in self.ncn_modules], self.alpha, self.activation_nr,
                                       self.n_cache, self.n_head, 0, self.save_every)
        if self.fuse_stages:
            return fused_ncn_net(x, xa, [m.weight for m in self.ncn_modules], self.alpha, self.activation_nr,
                                 self.n_cache, self.n_head, 0, self.save_every)
        for module_nr in range(self.num_modules):
            x, xa = self.ncn_modules[module_nr](x, xa)
        return x, xa


class NCNNetTestCuda(nn.Module):
    def __init__(self, alpha, activation, n_cache, n_head, num_modules, weights, *, grouping="stride", fuse_stages=False,
                 save_every=None):
        super().__init__()
        self.num_modules = num_modules
        self.alpha = alpha
        self.activation_nr = ACTIVATION_CODES[activation]
        self.n_cache = n_cache
        self.n_head = n_head
        self.weights = weights
        self.fuse_stages = fuse_stages
        self.save_every = save_every
        self.grouping = _check_grouping(grouping)

    def forward(self, x, xa):
        if self.grouping == "radix":
            return fused_ncn_radix_net(x, xa, list(self.weights[:self.num_modules]), self.alpha, self.activation_nr,
                                       self.n_cache, self.n_head, 0, self.save_every)
        if self.fuse_stages:
            return fused_ncn_net(x, xa, list(self.weights[:self.num_modules]), self.alpha, self.activation_nr,
                                 self.n_cache, self.n_head, 0, self.save_every)
        for module_nr in range(self.num_modules):
            x, xa = fused_ncn_cuda_v2(x, xa, self.weights[module_nr], self.alpha, self.activation_nr,
                                      self.n_cache, self.n_head, module_nr)
        return x, xa


def ncn_inverse(y, ya, W, alpha, activation, n_cache, n_head, module_l):
    """Inputs of one stage from its outputs (no autograd)."""
    x, xa = ncn_cuda_module.inverse_stages(y, ya, W, alpha, activation, n_cache, n_head, module_l, 1)
    return x, xa
