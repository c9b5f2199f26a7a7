"""One NCN stage whose groups come from a table, with one context length per batch entry.

Mirrors the older Triton surface of the reference, ncn_triton/ncn_triton_old.py:287-387:

    fused_chunk_linear_ncn(x, xa, W, group_tensor, ctxlen_tensor, ALPHA, ACTIVATION, NHEAD, CACHE, l) -> (yi, ya)

`group_tensor` is an integer tensor [N]: entry g*CACHE + o is the position on the sequence axis of slot o of group
g (ncn_triton_old.py:70).  `ctxlen_tensor` [batch] gives each batch entry its number of live slots (:66): groups
below it run all CACHE steps, the group it cuts runs one step per live row (:93-96).  ACTIVATION is a name
("tanh", "leaky-relu", anything else is linear, :103-108).  `l` is unused by the reference's kernels too: the
grouping is whatever the table says.

Differences with that file, all deliberate:
  * xa is used (the reference's forward ignores its xa argument and starts from zeros, :79);
  * rows past the context length pass through (y = x, ya = xa, gradients likewise); the reference leaves them
    unwritten in `torch.empty_like` outputs (:294-295) and, in the group the length cuts, reads position 0 for them.
The backward inverts the outputs step by step as the reference's does (:197-216), one step per live row.

Tables: stride_group_table is the stride permutation of the current kernels (torch_ref/ncn_pytorch.py:12-41),
radix_group_table the radix-n digit grouping of ncn_triton/group_tensors.py:8-18.
"""
import torch

from . import ncn_cuda_module

__all__ = ["FusedLinearChunkNCNFunction", "fused_chunk_linear_ncn", "stride_group_table", "radix_group_table"]


def _activation_code(name):
    if name == "tanh":
        return 0
    if name == "leaky-relu":
        return 3
    return -1


def stride_group_table(N, n_cache, stage, device=None):
    """int32 [N]: position of slot o of group g at entry g*n_cache + o, for stage `stage` of the stride permutation
    ((g + o * s) mod groups) * n_cache + o with s = 0 for stage 0 and 2^(stage-1) mod groups after."""
    if n_cache <= 0 or N % n_cache != 0:
        raise ValueError(f"block_size must divide N (N={N}, n_cache={n_cache})")
    groups = N // n_cache
    stride = 0 if stage == 0 else pow(2, stage - 1, groups)
    g = torch.arange(groups, dtype=torch.int64, device=device)[:, None]
    o = torch.arange(n_cache, dtype=torch.int64, device=device)[None, :]
    return (((g + o * stride) % groups) * n_cache + o).reshape(-1).to(torch.int32)


def radix_group_table(N, n_cache, level, device=None):
    """int32 [N] for the radix-n grouping (group_tensors.py:8-18): a group holds the n_cache positions that differ
    only in base-n_cache digit `level`; the digit is the slot, the remaining digits (the upper ones moved down one
    place) number the group."""
    stride = n_cache ** level
    if N % (n_cache * stride) != 0:
        raise ValueError(f"n_cache^(level+1) = {n_cache * stride} must divide N = {N}")
    i = torch.arange(N, dtype=torch.int64, device=device)
    slot = (i // stride) % n_cache
    group = i % stride + (i // (n_cache * stride)) * stride
    table = torch.empty(N, dtype=torch.int64, device=device)
    table[group * n_cache + slot] = i
    return table.to(torch.int32)


class FusedLinearChunkNCNFunction(torch.autograd.Function):
    """Autograd node of one table-grouped stage (ncn_triton_old.py:287-357): saves the outputs and inverts them in
    backward.  bfloat16 outputs are saved with what their rounding took away (two bfloat16 planes, or float32 copies
    on the generic kernels): the inversion would amplify bare bfloat16 rounding by (1/m)^n_cache."""

    @staticmethod
    def forward(ctx, x, xa, W, group_tensor, ctxlen_tensor, ALPHA, ACTIVATION, NUM_HEADS, CACHE, l):
        code = _activation_code(ACTIVATION)
        yi, ya, sy, sya = ncn_cuda_module.forward_stages_saving(x, xa, W, ALPHA, code, CACHE, NUM_HEADS, 0,
                                                                group_index=group_tensor, ctx_len=ctxlen_tensor)
        ctx.save_for_backward(sy, sya, W)
        ctx.group_tensor, ctx.ctxlen_tensor = group_tensor, ctxlen_tensor
        ctx.args = (ALPHA, code, CACHE, NUM_HEADS)
        ctx.io_dtype = x.dtype
        return yi, ya

    @staticmethod
    def backward(ctx, dyi, dya):
        yi, ya, W = ctx.saved_tensors
        alpha, code, cache, heads = ctx.args
        _, _, dx, dxa, dW = ncn_cuda_module.backward_stages(
            yi, ya, dyi.contiguous(), dya.contiguous() if dya is not None else None, W, alpha, code, cache, heads, 0, 1,
            grad_dtype=ctx.io_dtype, want_inputs=False, group_index=ctx.group_tensor, ctx_len=ctx.ctxlen_tensor,
            check_tables=False)
        return dx, dxa, dW.reshape(W.shape).to(W.dtype), None, None, None, None, None, None, None


def fused_chunk_linear_ncn(x, xa, W, group_tensor, ctxlen_tensor, ALPHA, ACTIVATION, NHEAD, CACHE, l):
    """(yi, ya) of one stage; same argument order as ncn_triton_old.py:362-387."""
    return FusedLinearChunkNCNFunction.apply(x, xa, W, group_tensor, ctxlen_tensor, ALPHA, ACTIVATION, NHEAD, CACHE, l)
