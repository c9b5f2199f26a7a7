"""CPU oracle for the NCN layer -- TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this file: it is the checker used by tests/, by
__graft_entry__.smoke() and by the cpu_baseline leg of bench.py.  (oracle/ncn_oracle.c is a second, independent
restatement in plain C, bound by oracle/c_oracle.py; tests/test_oracle_c.py holds the two to each other.)  It restates, in plain PyTorch on
the CPU, the algorithm of the reference:

  * index map            torch_ref/ncn_pytorch.py:12-41        -> group_pos_to_index, stage_positions
  * one stage forward    torch_ref/ncn_pytorch.py:45-99        -> literal_stage_forward (loops, tiny inputs)
                                                                  stage_forward (same math, batched)
  * stage stack          torch_ref/ncn_pytorch.py:103-124      -> net_forward
  * one-step inverse     torch_ref/ncn_pytorch_invertible.py:87-113 -> stage_inverse / net_inverse
  * tables and lengths   ncn_triton/ncn_triton_old.py:53-96 (group_tensor, ctxlen_tensor), group_tensors.py:8-18
                                                               -> stage_forward_indexed, radix_group_table
  * backward             autograd through the forward is the reference's definition of the gradients
                         (grad_test_bench.py:72); the closed form used by the GPU kernels follows
                         ncn_triton/ncn_triton.py:176-246 and ncn_cuda/ncn_bwd_cuda_kernel.cu:88-216
                                                               -> stage_backward / net_backward

Pinning (see tests/test_oracle_*.py): every function is checked against the committed golden
vectors that tests/golden/make_golden.py wrote from the reference's own CPU code, the closed-form
backward additionally against autograd through stage_forward in float64, the inverse against
forward round trips, the index map against the bijection/hand values.  No function here is
"parity unpinned" for activation == tanh.
The leaky-relu and linear activations (forward and closed-form backward), grouping by a table, the
radix tables and context lengths are pinned by tests/golden/triton_*.npz, which
tests/golden/make_golden_triton.py wrote by running the reference's Triton kernels
(ncn_triton/ncn_triton.py, ncn_triton_old.py) under Triton's CPU interpreter: whole groups below a
length and the group a length cuts, forward and backward (the reference's kernel lets the rows past the
length alias position 0; the cut-group vectors use tables that keep position 0 among the dead rows,
where that is harmless).
The relu and sigmoid activations exist only in the reference's CUDA kernels (ncn_fwd_cuda_kernel.cu:86-95,
ncn_bwd_cuda_kernel.cu:137-150), which cannot be built here (no nvcc), so no vector of the reference's covers them.
They are pinned by what the mathematics fixes (tests/test_oracle_properties.py): scalar loops over a tiny stage written
with math.tanh / max / exp only, sigmoid(t) = (1 + tanh(t/2))/2 and its slope against the pinned tanh branch, the
closed-form backward against autograd (float64) and against central finite differences of the forward on inputs that
stay away from relu's kink.
Still parity unpinned:
  * what happens to rows past a length: the reference leaves those rows unwritten;
    stage_forward_indexed passes them through, which is this build's choice.
"""
import math

import torch

M_DEFAULT = 0.9  # hard-coded in the reference: ncn_pytorch.py:89, ncn_fwd_cuda_kernel.cu:72

# activation codes of the reference's CUDA surface (ncn_pytorch_wrapper_v2.py:111)
ACT_TANH, ACT_RELU, ACT_SIGMOID, ACT_LINEAR = 0, 1, 2, -1
ACT_LEAKY_RELU = 3  # not a CUDA code: the leaky relu of ncn_triton/ncn_triton.py:22-28 (slope 0.01)


def act_code(activation):
    if isinstance(activation, str):
        return {"tanh": ACT_TANH, "relu": ACT_RELU, "sigmoid": ACT_SIGMOID, "linear": ACT_LINEAR,
                "leaky-relu": ACT_LEAKY_RELU}[activation]
    return int(activation)


def _act(T, code):
    """F and dF/dT.  Codes as in ncn_fwd_cuda_kernel.cu:86-95 / ncn_bwd_cuda_kernel.cu:137-150."""
    if code == ACT_TANH:
        F = torch.tanh(T)
        return F, 1.0 - F * F
    if code == ACT_RELU:
        F = torch.clamp_min(T, 0.0)
        return F, (F > 0).to(T.dtype)
    if code == ACT_SIGMOID:
        F = torch.sigmoid(T)
        return F, F * (1.0 - F)
    if code == ACT_LEAKY_RELU:  # ncn_triton.py:22-28: x >= 0 keeps x and slope 1
        pos = T >= 0
        return torch.where(pos, T, 0.01 * T), torch.where(pos, torch.ones_like(T), torch.full_like(T, 0.01))
    return T, torch.ones_like(T)


# ----------------------------------------------------------------------------------------------
# index map (ncn_pytorch.py:12-41)
# ----------------------------------------------------------------------------------------------
def stage_stride(N, n, stage):
    m = N // n
    return 0 if stage == 0 else (1 << (stage - 1)) % m


def group_pos_to_index(N, n, stage, group, slot):
    """Position on the N axis of slot `slot` of group `group` at stage `stage`."""
    if N % n != 0:
        raise ValueError("block_size must divide N")
    m = N // n
    s = stage_stride(N, n, stage)
    return ((group + slot * s) % m) * n + slot


def stage_positions(N, n, stage):
    """LongTensor [N/n, n]: positions gathered by each group, in slot order."""
    m = N // n
    s = stage_stride(N, n, stage)
    b = torch.arange(m, dtype=torch.long)[:, None]
    o = torch.arange(n, dtype=torch.long)[None, :]
    return ((b + o * s) % m) * n + o


# ----------------------------------------------------------------------------------------------
# literal restatement (loops; follows ncn_pytorch.py:45-99 line by line in meaning) -- tiny inputs
# ----------------------------------------------------------------------------------------------
def literal_stage_forward(X, Xa, W, alpha, n, C, stage, m=M_DEFAULT, activation=ACT_TANH):
    code = act_code(activation)
    B, N, E = X.shape
    ce = E // C
    Y = torch.zeros_like(X)
    Ya = torch.zeros_like(Xa)
    for b in range(B):
        for c in range(C):
            Wi = W[c * ce:(c + 1) * ce]
            Wj = W[E + c * ce:E + (c + 1) * ce]
            for grp in range(N // n):
                pos = [group_pos_to_index(N, n, stage, grp, o) for o in range(n)]
                xi = [X[b, p, c * ce:(c + 1) * ce] for p in pos]
                xa = [Xa[b, p, c * ce:(c + 1) * ce] for p in pos]
                for j in range(n):
                    xj = xi[j]
                    e = torch.dot(xj, Wj)
                    new_xi, new_xa = [], []
                    for i in range(n):
                        s = torch.dot(xi[i], Wi) + e
                        T = alpha * xi[i] + (1.0 - alpha) * s * xj
                        F, _ = _act(T, code)
                        a2 = xa[i] * m + (1 - m) * F
                        x2 = xi[i] * m + (1 - m) * a2
                        new_xi.append(x2)
                        new_xa.append(a2)
                    xi, xa = new_xi, new_xa
                for o, p in enumerate(pos):
                    Y[b, p, c * ce:(c + 1) * ce] += xi[o]
                    Ya[b, p, c * ce:(c + 1) * ce] += xa[o]
    return Y, Ya


def literal_net_forward(x, xa, weights, alpha, n, C, m=M_DEFAULT, activation=ACT_TANH):
    for l, W in enumerate(weights):
        x, xa = literal_stage_forward(x, xa, W, alpha, n, C, l, m, activation)
    return x, xa


# ----------------------------------------------------------------------------------------------
# batched restatement
# ----------------------------------------------------------------------------------------------
def _gather(X, pos, C):
    """[B, N, E] -> [B, C, m, n, Ec] rows of every group of every head."""
    B, N, E = X.shape
    mm, n = pos.shape
    G = X[:, pos.reshape(-1), :].reshape(B, mm, n, C, E // C)
    return G.permute(0, 3, 1, 2, 4)


def _scatter(G, pos, like):
    B, C, mm, n, ce = G.shape
    Y = torch.empty_like(like)
    Y[:, pos.reshape(-1), :] = G.permute(0, 2, 3, 1, 4).reshape(B, mm * n, C * ce)
    return Y


def _split_w(W, C):
    E = W.numel() // 2
    ce = E // C
    Wi = W[:E].reshape(1, C, 1, 1, ce)
    Wj = W[E:].reshape(1, C, 1, 1, ce)
    return Wi, Wj


def _step(x, a, Wi, Wj, j, alpha, m, code):
    """One recurrence step on gathered tiles x, a: [B, C, m, n, Ec] (ncn_pytorch.py:76-94)."""
    xj = x[:, :, :, j:j + 1, :]
    s = (x * Wi).sum(-1, keepdim=True) + (xj * Wj).sum(-1, keepdim=True)
    T = alpha * x + (1.0 - alpha) * s * xj
    F, dF = _act(T, code)
    a2 = a * m + (1 - m) * F
    x2 = x * m + (1 - m) * a2
    return x2, a2, (xj, s, dF)


def stage_forward(X, Xa, W, alpha, n, C, stage, m=M_DEFAULT, activation=ACT_TANH):
    code = act_code(activation)
    B, N, E = X.shape
    pos = stage_positions(N, n, stage)
    x, a = _gather(X, pos, C), _gather(Xa, pos, C)
    Wi, Wj = _split_w(W, C)
    for j in range(n):
        x, a, _ = _step(x, a, Wi, Wj, j, alpha, m, code)
    return _scatter(x, pos, X), _scatter(a, pos, Xa)


def net_forward(x, xa, weights, alpha, n, C, m=M_DEFAULT, activation=ACT_TANH, first_stage=0):
    for l, W in enumerate(weights):
        x, xa = stage_forward(x, xa, W, alpha, n, C, first_stage + l, m, activation)
    return x, xa


def _unstep(y, b, Wi, Wj, j, alpha, m, code):
    """Inverse of one step (ncn_pytorch_invertible.py:87-113): returns the pre-step x, a and the
    step's intermediates."""
    x = (y - b * (1.0 - m)) / m
    xj = x[:, :, :, j:j + 1, :]
    s = (x * Wi).sum(-1, keepdim=True) + (xj * Wj).sum(-1, keepdim=True)
    T = alpha * x + (1.0 - alpha) * s * xj
    F, dF = _act(T, code)
    a = (b - F * (1.0 - m)) / m
    return x, a, (xj, s, dF)


def stage_inverse(Y, Ya, W, alpha, n, C, stage, m=M_DEFAULT, activation=ACT_TANH):
    code = act_code(activation)
    B, N, E = Y.shape
    pos = stage_positions(N, n, stage)
    y, b = _gather(Y, pos, C), _gather(Ya, pos, C)
    Wi, Wj = _split_w(W, C)
    for j in range(n - 1, -1, -1):
        y, b, _ = _unstep(y, b, Wi, Wj, j, alpha, m, code)
    return _scatter(y, pos, Y), _scatter(b, pos, Ya)


def net_min_abs_T(x, xa, weights, alpha, n, C, m=M_DEFAULT, activation=ACT_TANH, first_stage=0):
    """Smallest |T| any element sees at any step of any stage (float64 recommended): how far the run stays from the
    kink of relu / leaky relu, where a float32 recomputation may pick the other slope."""
    code = act_code(activation)
    worst = math.inf
    for l, W in enumerate(weights):
        pos = stage_positions(x.shape[1], n, first_stage + l)
        gx, ga = _gather(x, pos, C), _gather(xa, pos, C)
        Wi, Wj = _split_w(W, C)
        for j in range(n):
            xj = gx[:, :, :, j:j + 1, :]
            s = (gx * Wi).sum(-1, keepdim=True) + (xj * Wj).sum(-1, keepdim=True)
            worst = min(worst, float((alpha * gx + (1.0 - alpha) * s * xj).abs().min()))
            gx, ga, _ = _step(gx, ga, Wi, Wj, j, alpha, m, code)
        x, xa = _scatter(gx, pos, x), _scatter(ga, pos, xa)
    return worst


def make_inputs_signed_regimes(batch, N, E, L, n, seed=0, dtype=torch.float32):
    """Inputs on which T keeps one sign per batch entry through every step of every stage, far from zero: even batch
    entries have x in [0.5, 1.5] and xa in [0, 0.5] (T > 0 throughout), odd ones the negatives of such values
    (T < 0 throughout), weights in [0, 1/(3 Ec)] so that |(1-alpha) s x_j| stays well below |alpha x_i|.  For checking
    the gradients of relu / leaky relu on tensors too large to keep every |T| away from zero by choosing a seed:
    both slopes are exercised, none of them at the kink.  Returns x, xa, [W_l], dy, dya."""
    g = torch.Generator().manual_seed(seed)
    x = 0.5 + torch.rand(batch, N, E, generator=g)
    xa = 0.5 * torch.rand(batch, N, E, generator=g)
    sign = torch.where(torch.arange(batch) % 2 == 0, 1.0, -1.0).reshape(batch, 1, 1)
    x, xa = x * sign, xa * sign
    Ws = [torch.rand(2 * E, generator=g) / (3.0 * E) for _ in range(L)]
    dy = torch.randn(batch, N, E, generator=g)
    dya = torch.randn(batch, N, E, generator=g)
    return x.to(dtype), xa.to(dtype), [w.to(dtype) for w in Ws], dy.to(dtype), dya.to(dtype)


def net_inverse(y, ya, weights, alpha, n, C, m=M_DEFAULT, activation=ACT_TANH, first_stage=0):
    for l in range(len(weights) - 1, -1, -1):
        y, ya = stage_inverse(y, ya, weights[l], alpha, n, C, first_stage + l, m, activation)
    return y, ya


def _vjp_step(x, g, h, Wi, Wj, j, alpha, m, inter):
    """Closed-form vector-Jacobian product of one step, given the pre-step x and the intermediates.
    g = dL/dx', h = dL/da'.  Returns dL/dx, dL/da, dWi, dWj (summed over batch, groups and rows)."""
    xj, s, dF = inter
    q = (1 - m) * (1 - m) * g + (1 - m) * h          # dL/dF
    u = q * dF                                          # dL/dT
    r = (u * xj).sum(-1, keepdim=True)                  # per-row scalar
    dWi = (1 - alpha) * (r * x).sum(dim=(0, 2, 3))      # [C, Ec]
    dWj = (1 - alpha) * (r.sum(dim=3, keepdim=True) * xj).sum(dim=(0, 2, 3))
    dx = m * g + alpha * u + (1 - alpha) * r * Wi
    da = m * (1 - m) * g + m * h
    dxj = ((1 - alpha) * r * Wj + (1 - alpha) * s * u).sum(dim=3, keepdim=True)
    dx = dx.clone()
    dx[:, :, :, j:j + 1, :] += dxj
    return dx, da, dWi, dWj


def stage_backward(Y, Ya, dY, dYa, W, alpha, n, C, stage, m=M_DEFAULT, activation=ACT_TANH):
    """Reversible backward of one stage from its OUTPUTS (what the reference's CUDA/Triton kernels do,
    ncn_bwd_cuda_kernel.cu:86-216): returns X, Xa (reconstructed), dX, dXa, dW [2E]."""
    code = act_code(activation)
    B, N, E = Y.shape
    pos = stage_positions(N, n, stage)
    y, b = _gather(Y, pos, C), _gather(Ya, pos, C)
    g, h = _gather(dY, pos, C), _gather(dYa, pos, C)
    Wi, Wj = _split_w(W, C)
    dWi = torch.zeros(C, E // C, dtype=Y.dtype)
    dWj = torch.zeros(C, E // C, dtype=Y.dtype)
    for j in range(n - 1, -1, -1):
        y, b, inter = _unstep(y, b, Wi, Wj, j, alpha, m, code)
        g, h, dwi, dwj = _vjp_step(y, g, h, Wi, Wj, j, alpha, m, inter)
        dWi += dwi
        dWj += dwj
    dW = torch.cat([dWi.reshape(-1), dWj.reshape(-1)])
    return _scatter(y, pos, Y), _scatter(b, pos, Ya), _scatter(g, pos, dY), _scatter(h, pos, dYa), dW


def stage_backward_from_inputs(X, Xa, dY, dYa, W, alpha, n, C, stage, m=M_DEFAULT, activation=ACT_TANH):
    """Same gradients without the inversion: recompute forward from the stage INPUTS keeping every
    step's state (what torch autograd effectively does for the reference's `ref` path)."""
    code = act_code(activation)
    B, N, E = X.shape
    pos = stage_positions(N, n, stage)
    x, a = _gather(X, pos, C), _gather(Xa, pos, C)
    g, h = _gather(dY, pos, C), _gather(dYa, pos, C)
    Wi, Wj = _split_w(W, C)
    saved = []
    for j in range(n):
        x2, a2, inter = _step(x, a, Wi, Wj, j, alpha, m, code)
        saved.append((x, inter))
        x, a = x2, a2
    dWi = torch.zeros(C, E // C, dtype=X.dtype)
    dWj = torch.zeros(C, E // C, dtype=X.dtype)
    for j in range(n - 1, -1, -1):
        xs, inter = saved[j]
        g, h, dwi, dwj = _vjp_step(xs, g, h, Wi, Wj, j, alpha, m, inter)
        dWi += dwi
        dWj += dwj
    dW = torch.cat([dWi.reshape(-1), dWj.reshape(-1)])
    return _scatter(g, pos, dY), _scatter(h, pos, dYa), dW


def net_backward(y, ya, dy, dya, weights, alpha, n, C, m=M_DEFAULT, activation=ACT_TANH, first_stage=0):
    """Reversible backward of the whole stack from its final outputs.  Returns x, xa, dx, dxa, [dW_l]."""
    dWs = [None] * len(weights)
    for l in range(len(weights) - 1, -1, -1):
        y, ya, dy, dya, dWs[l] = stage_backward(y, ya, dy, dya, weights[l], alpha, n, C,
                                                 first_stage + l, m, activation)
    return y, ya, dy, dya, dWs


def net_backward_checkpointed(x, xa, dy, dya, weights, alpha, n, C, m=M_DEFAULT, activation=ACT_TANH,
                              first_stage=0, save_every=1):
    """Forward keeping the outputs of every `save_every`-th stage, then reversible backward segment by
    segment.  save_every=1 is what the reference's per-stage autograd node does
    (ncn_pytorch_wrapper_v2.py:22: each stage saves its own yi, ya), so rounding in the inversion is
    amplified by (1/m)^n only; save_every=L is the whole-stack reversal of net_backward.
    Returns yi, ya, dx, dxa, [dW_l]."""
    L = len(weights)
    saved = {}
    for l in range(L):
        x, xa = stage_forward(x, xa, weights[l], alpha, n, C, first_stage + l, m, activation)
        if (l + 1) % save_every == 0 or l == L - 1:
            saved[l] = (x, xa)
    yi, ya = x, xa
    dWs = [None] * L
    cur = None
    for l in range(L - 1, -1, -1):
        if l in saved:
            cur = saved[l]
        xr, xar, dy, dya, dWs[l] = stage_backward(cur[0], cur[1], dy, dya, weights[l], alpha, n, C,
                                                  first_stage + l, m, activation)
        cur = (xr, xar)
    return yi, ya, dy, dya, dWs


def net_backward_from_inputs(x, xa, dy, dya, weights, alpha, n, C, m=M_DEFAULT, activation=ACT_TANH,
                             first_stage=0):
    """Gradients of the stack without any inversion (stage inputs recomputed by forward)."""
    xs = [(x, xa)]
    for l, W in enumerate(weights[:-1]):
        x, xa = stage_forward(x, xa, W, alpha, n, C, first_stage + l, m, activation)
        xs.append((x, xa))
    dWs = [None] * len(weights)
    for l in range(len(weights) - 1, -1, -1):
        dy, dya, dWs[l] = stage_backward_from_inputs(xs[l][0], xs[l][1], dy, dya, weights[l], alpha, n, C,
                                                     first_stage + l, m, activation)
    return dy, dya, dWs


def net_autograd(x, xa, weights, dy, dya, alpha, n, C, m=M_DEFAULT, activation=ACT_TANH, first_stage=0):
    """Forward + torch autograd backward through the batched forward: the way the reference obtains its
    `ref` gradients (grad_test_bench.py:68-84).  Returns yi, ya, dx, dxa, [dW_l]."""
    x = x.detach().clone().requires_grad_()
    xa = xa.detach().clone().requires_grad_()
    ws = [w.detach().clone().requires_grad_() for w in weights]
    yi, ya = net_forward(x, xa, ws, alpha, n, C, m, activation, first_stage)
    torch.autograd.backward([yi, ya], [dy, dya])
    return yi.detach(), ya.detach(), x.grad, xa.grad, [w.grad for w in ws]


# ----------------------------------------------------------------------------------------------
# grouping by table and per-batch context lengths (ncn_triton/ncn_triton_old.py, group_tensors.py)
# ----------------------------------------------------------------------------------------------
def stride_group_table(N, n, stage):
    """The stride permutation written as a table: entry g*n + o is the position of slot o of group g."""
    return stage_positions(N, n, stage).reshape(-1)


def radix_group_table(N, n, level):
    """Radix-n digit grouping of ncn_triton/group_tensors.py:8-18: position i belongs to the group numbered
    lower + upper * n^level, where lower = i mod n^level and upper = i div n^(level+1), and sits in slot
    (i div n^level) mod n: a group holds the n positions that differ only in digit `level`."""
    stride = n ** level
    if N % (n * stride) != 0:
        raise ValueError("n^(level+1) must divide N")
    table = torch.empty(N, dtype=torch.long)
    for i in range(N):
        lower = i % stride
        slot = (i // stride) % n
        upper = i // (n * stride)
        table[(lower + upper * stride) * n + slot] = i
    return table


def stage_forward_indexed(X, Xa, W, alpha, n, C, table, ctx_len=None, m=M_DEFAULT, activation=ACT_TANH, inverse=False):
    """One stage whose groups come from `table` ([N] positions in (group, slot) order) and where batch entry b only
    has its first ctx_len[b] slots (ncn_triton_old.py:66-71, 93-96): whole groups below the length run as usual, the
    group the length cuts runs on its live rows with as many steps as it has live rows, rows past the length pass
    through.  Differentiable; inverse=True runs the inverse instead."""
    code = act_code(activation)
    B, N, E = X.shape
    Wi, Wj = _split_w(W, C)
    table = torch.as_tensor(table, dtype=torch.long)
    ys, yas = [], []
    for b in range(B):
        ln = N if ctx_len is None else max(0, min(int(ctx_len[b]), N))
        y, ya = X[b:b + 1].clone(), Xa[b:b + 1].clone()
        full, rem = ln // n, ln % n
        pieces = []
        if full:
            pieces.append(table[:full * n].reshape(full, n))
        if rem:
            pieces.append(table[full * n:full * n + rem].reshape(1, rem))
        for pos in pieces:
            rows = pos.shape[1]
            x, a = _gather(X[b:b + 1], pos, C), _gather(Xa[b:b + 1], pos, C)
            steps = range(rows - 1, -1, -1) if inverse else range(rows)
            for j in steps:
                if inverse:
                    x, a, _ = _unstep(x, a, Wi, Wj, j, alpha, m, code)
                else:
                    x, a, _ = _step(x, a, Wi, Wj, j, alpha, m, code)
            flat = pos.reshape(-1)
            y = y.index_copy(1, flat, x.permute(0, 2, 3, 1, 4).reshape(1, flat.numel(), E))
            ya = ya.index_copy(1, flat, a.permute(0, 2, 3, 1, 4).reshape(1, flat.numel(), E))
        ys.append(y)
        yas.append(ya)
    return torch.cat(ys), torch.cat(yas)


def net_forward_indexed(x, xa, weights, alpha, n, C, tables, ctx_len=None, m=M_DEFAULT, activation=ACT_TANH):
    for W, table in zip(weights, tables):
        x, xa = stage_forward_indexed(x, xa, W, alpha, n, C, table, ctx_len, m, activation)
    return x, xa


def net_inverse_indexed(y, ya, weights, alpha, n, C, tables, ctx_len=None, m=M_DEFAULT, activation=ACT_TANH):
    for W, table in zip(reversed(weights), reversed(tables)):
        y, ya = stage_forward_indexed(y, ya, W, alpha, n, C, table, ctx_len, m, activation, inverse=True)
    return y, ya


def net_autograd_indexed(x, xa, weights, dy, dya, alpha, n, C, tables, ctx_len=None, m=M_DEFAULT,
                         activation=ACT_TANH):
    """Forward + autograd backward through net_forward_indexed.  Returns yi, ya, dx, dxa, [dW_l]."""
    x = x.detach().clone().requires_grad_()
    xa = xa.detach().clone().requires_grad_()
    ws = [w.detach().clone().requires_grad_() for w in weights]
    yi, ya = net_forward_indexed(x, xa, ws, alpha, n, C, tables, ctx_len, m, activation)
    torch.autograd.backward([yi, ya], [dy, dya])
    return yi.detach(), ya.detach(), x.grad, xa.grad, [w.grad if w.grad is not None else torch.zeros_like(w) for w in ws]


# ----------------------------------------------------------------------------------------------
# synthetic inputs shared by tests, smoke() and bench.py (generation order fixed: x, xa, W_l, dyi, dya)
# ----------------------------------------------------------------------------------------------
def make_inputs(batch, N, E, L, n, seed=0, xa_zero=True, w_scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(batch, N, E, generator=g, dtype=torch.float32)
    xa = torch.zeros(batch, N, E) if xa_zero else torch.randn(batch, N, E, generator=g, dtype=torch.float32)
    std = w_scale / math.sqrt(n)
    Ws = [torch.randn(2 * E, generator=g, dtype=torch.float32) * std for _ in range(L)]
    dyi = torch.randn(batch, N, E, generator=g, dtype=torch.float32)
    dya = torch.randn(batch, N, E, generator=g, dtype=torch.float32)
    return x.to(dtype), xa.to(dtype), [w.to(dtype) for w in Ws], dyi.to(dtype), dya.to(dtype)


def rel_err(a, b):
    """max |a-b| / max |b| : the relative error figure used for every parity claim in this repo.  It is a statement
    about the tensor as a whole, scaled by its largest entry: entries much smaller than that can be off by more than
    the figure in their own terms (rms_err is the companion figure over all entries)."""
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    denom = b.abs().max().item()
    return (a - b).abs().max().item() / (denom if denom > 0 else 1.0)


def rms_err(a, b):
    """sqrt(mean (a-b)^2) / sqrt(mean b^2): the root-mean-square error relative to the tensor's root mean square."""
    a = a.detach().double().cpu()
    b = b.detach().double().cpu()
    denom = b.pow(2).mean().sqrt().item()
    return (a - b).pow(2).mean().sqrt().item() / (denom if denom > 0 else 1.0)
