"""The reference's Triton surface by name, on the HIP kernels.

ncn_triton/ncn_triton.py:262-407 offers fused_ncn_triton, NCNModuleTriton, NCNNetTriton and NCNNetTestTriton, the
counterparts of the CUDA wrapper's classes with one difference: the activation is a name ("tanh", "leaky-relu",
anything else linear, :101-106) instead of an integer code.  grad_test_bench.py:4,53-57 builds its comparison stack
from NCNNetTestTriton.  The classes here take the same arguments and hand the work to the same autograd node as
NCNModuleCuda (there is one set of kernels), so a script can swap

    from ncn_triton.ncn_triton import NCNNetTriton, NCNNetTestTriton, fused_ncn_triton
for
    from ncn_cuda_amd.ncn_triton import NCNNetTriton, NCNNetTestTriton, fused_ncn_triton
"""
import math

import torch
from torch import nn

from .modules import NCNFunction

__all__ = ["activation_code", "fused_ncn_triton", "NCNModuleTriton", "NCNNetTriton", "NCNNetTestTriton"]


def activation_code(name):
    """Integer code of a Triton-style activation name: the two named branches of ncn_triton.py:101-106, linear for
    everything else (as there); integers pass through."""
    if isinstance(name, int):
        return name
    return {"tanh": 0, "leaky-relu": 3}.get(name, -1)


def fused_ncn_triton(x, xa, W, ALPHA, ACTIVATION, NHEAD, CACHE, MODULE_L):
    """(yi, ya) of stage MODULE_L; argument order of ncn_triton.py:333-349."""
    return NCNFunction.apply(x, xa, W, ALPHA, activation_code(ACTIVATION), CACHE, NHEAD, MODULE_L)


class NCNModuleTriton(nn.Module):
    """One stage with its own weight, initialised like the reference's (normal, std 1 / (2 embed_dim),
    ncn_triton.py:360)."""

    def __init__(self, alpha, activation, n_cache, n_head, module_nr, embed_dim):
        super().__init__()
        self.alpha, self.activation = alpha, activation
        self.n_cache, self.n_head, self.module_nr, self.embed_dim = n_cache, n_head, module_nr, embed_dim
        self.weight = nn.Parameter(torch.empty(2 * embed_dim).normal_(mean=0.0, std=1 / (2.0 * embed_dim)))

    def reset_parameters(self):
        bound = 1.0 / math.sqrt(self.embed_dim)
        with torch.no_grad():
            for p in self.parameters():
                p.uniform_(-bound, bound)

    def forward(self, x, xa):
        return fused_ncn_triton(x, xa, self.weight, self.alpha, self.activation, self.n_head, self.n_cache,
                                self.module_nr)


class NCNNetTriton(nn.Module):
    """num_modules stages, state_dict keys ncn_modules.{l}.weight (ncn_triton.py:383-392)."""

    def __init__(self, alpha, activation, n_cache, n_head, num_modules, embed_dim):
        super().__init__()
        self.num_modules = num_modules
        self.ncn_modules = nn.ModuleList(
            NCNModuleTriton(alpha, activation, n_cache, n_head, l, embed_dim) for l in range(num_modules))

    def forward(self, x, xa):
        for stage in self.ncn_modules:
            x, xa = stage(x, xa)
        return x, xa


class NCNNetTestTriton(nn.Module):
    """The stack over weights supplied by the caller (ncn_triton.py:395-421): what the reference's bench script uses."""

    def __init__(self, alpha, activation, n_cache, n_head, num_modules, weights):
        super().__init__()
        self.num_modules, self.alpha, self.activation = num_modules, alpha, activation
        self.n_cache, self.n_head, self.weights = n_cache, n_head, weights

    def forward(self, x, xa):
        for l in range(self.num_modules):
            x, xa = fused_ncn_triton(x, xa, self.weights[l], self.alpha, self.activation, self.n_head, self.n_cache, l)
        return x, xa
