"""Checks of the oracle that do not depend on any stored vector: closed forms, special cases and invariants
chosen so that a dropped term, a wrong sign or a transposed index fails at least one of them."""
import math

import pytest
import torch

from oracle import ncn_oracle as O

D = torch.float64


def _rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return scale * torch.randn(*shape, generator=g, dtype=D)


@pytest.mark.parametrize("N,n", [(256, 2), (1024, 4), (4096, 16), (8192, 2), (2048, 8), (48, 3), (64, 64)])
def test_index_map_is_a_bijection_at_every_stage(N, n):
    m = N // n
    for stage in range(0, m.bit_length() + 3):
        pos = O.stage_positions(N, n, stage)
        assert sorted(pos.reshape(-1).tolist()) == list(range(N))
        assert (pos % n == torch.arange(n)[None, :]).all()  # slot o always reads offset o of some block
    assert torch.equal(O.stage_positions(N, n, 0).reshape(-1), torch.arange(N))  # stage 0: contiguous blocks


def test_index_map_hand_values():
    # N=256, n=2: stride 1, 2, 64 at stages 1, 2, 7
    assert O.group_pos_to_index(256, 2, 1, 0, 1) == 3
    assert O.group_pos_to_index(256, 2, 2, 0, 1) == 5
    assert O.group_pos_to_index(256, 2, 7, 0, 1) == 129
    assert O.group_pos_to_index(256, 2, 7, 5, 1) == 139
    assert O.stage_stride(256, 2, 8) == 0  # 2^7 mod 128: the stride wraps to contiguous blocks again
    assert O.stage_stride(48, 3, 5) == 0 and O.stage_stride(48, 3, 4) == 8  # groups = 16


def test_single_row_group_by_hand():
    """n = 1: one row, one step, s = <x, Wi + Wj>."""
    E, C = 6, 2
    x, xa, W = _rand(1, 1, E, seed=1), _rand(1, 1, E, seed=2), _rand(2 * E, seed=3, scale=0.5)
    alpha, m = 0.7, 0.9
    y, ya = O.stage_forward(x, xa, W, alpha, 1, C, 0, m)
    for c in range(C):
        sl = slice(c * 3, c * 3 + 3)
        xv, av = x[0, 0, sl], xa[0, 0, sl]
        s = torch.dot(xv, W[sl] + W[E + c * 3:E + c * 3 + 3])
        F = torch.tanh(alpha * xv + (1 - alpha) * s * xv)
        a2 = m * av + (1 - m) * F
        assert torch.allclose(ya[0, 0, sl], a2, atol=1e-15)
        assert torch.allclose(y[0, 0, sl], m * xv + (1 - m) * a2, atol=1e-15)


def test_alpha_one_ignores_weights_and_grouping():
    """alpha = 1: T = x, rows decouple, W drops out; n steps of a' = m a + (1-m) tanh x, x' = m x + (1-m) a'."""
    x, xa = _rand(2, 16, 8, seed=4), _rand(2, 16, 8, seed=5)
    W1, W2 = _rand(16, seed=6), _rand(16, seed=7)
    n, C, m = 4, 2, 0.9
    y1, ya1 = O.stage_forward(x, xa, W1, 1.0, n, C, 2, m)
    y2, ya2 = O.stage_forward(x, xa, W2, 1.0, n, C, 0, m)
    assert torch.allclose(y1, y2, atol=1e-14) and torch.allclose(ya1, ya2, atol=1e-14)
    xe, ae = x.clone(), xa.clone()
    for _ in range(n):
        ae = m * ae + (1 - m) * torch.tanh(xe)
        xe = m * xe + (1 - m) * ae
    assert torch.allclose(y1, xe, atol=1e-14) and torch.allclose(ya1, ae, atol=1e-14)
    # and dW vanishes
    dy, dya = _rand(2, 16, 8, seed=8), _rand(2, 16, 8, seed=9)
    *_, dW = O.stage_backward(y1, ya1, dy, dya, W1, 1.0, n, C, 2, m)
    assert dW.abs().max().item() < 1e-15


def test_zero_weights_decouple_rows():
    x, xa = _rand(1, 8, 4, seed=10), _rand(1, 8, 4, seed=11)
    alpha, m, n = 0.6, 0.9, 4
    y, ya = O.stage_forward(x, xa, torch.zeros(8, dtype=D), alpha, n, 1, 1, m)
    xe, ae = x.clone(), xa.clone()
    for _ in range(n):
        ae = m * ae + (1 - m) * torch.tanh(alpha * xe)
        xe = m * xe + (1 - m) * ae
    assert torch.allclose(y, xe, atol=1e-14) and torch.allclose(ya, ae, atol=1e-14)


def test_pivot_row_uses_pre_step_value_and_step_order():
    """Two rows, linear activation, by hand: step 0 pivots on row 0, step 1 on the UPDATED row 1."""
    alpha, m = 0.5, 0.9
    x = torch.tensor([[[1.0], [2.0]]], dtype=D)
    xa = torch.zeros(1, 2, 1, dtype=D)
    W = torch.tensor([0.3, -0.2], dtype=D)  # Wi = 0.3, Wj = -0.2
    y, ya = O.stage_forward(x, xa, W, alpha, 2, 1, 0, m, activation="linear")
    r = [1.0, 2.0]
    a = [0.0, 0.0]
    for j in range(2):
        xj = r[j]
        new_r, new_a = [], []
        for i in range(2):
            s = r[i] * 0.3 + xj * -0.2
            T = alpha * r[i] + (1 - alpha) * s * xj
            a2 = m * a[i] + (1 - m) * T
            new_a.append(a2)
            new_r.append(m * r[i] + (1 - m) * a2)
        r, a = new_r, new_a
    assert torch.allclose(y.reshape(-1), torch.tensor(r, dtype=D), atol=1e-15)
    assert torch.allclose(ya.reshape(-1), torch.tensor(a, dtype=D), atol=1e-15)


def test_leaky_relu_by_hand():
    """One row, one step (n = 1): a negative T is scaled by 0.01 and a positive one kept, as in
    ncn_triton/ncn_triton.py:22-28; the slope seen by autograd is 0.01 / 1."""
    alpha, m = 0.5, 0.9
    x = torch.tensor([[[-1.0, 2.0]]], dtype=D, requires_grad=True)
    xa = torch.zeros(1, 1, 2, dtype=D)
    W = torch.tensor([0.3, 0.1, -0.2, 0.05], dtype=D)       # Wi = (0.3, 0.1), Wj = (-0.2, 0.05)
    y, ya = O.stage_forward(x, xa, W, alpha, 1, 1, 0, m, activation="leaky-relu")
    s = -1.0 * (0.3 - 0.2) + 2.0 * (0.1 + 0.05)             # the row is its own pivot
    T = [alpha * v + (1 - alpha) * s * v for v in (-1.0, 2.0)]
    assert T[0] < 0 < T[1]
    F = [0.01 * T[0], T[1]]
    a = [(1 - m) * f for f in F]
    r = [m * v + (1 - m) * a_ for v, a_ in zip((-1.0, 2.0), a)]
    assert torch.allclose(ya.reshape(-1), torch.tensor(a, dtype=D), atol=1e-15)
    assert torch.allclose(y.reshape(-1), torch.tensor(r, dtype=D), atol=1e-15)
    F2, dF = O._act(torch.tensor([-3.0, 0.0, 4.0], dtype=D), O.ACT_LEAKY_RELU)
    assert F2.tolist() == [-0.03, 0.0, 4.0] and dF.tolist() == [0.01, 1.0, 1.0]


@pytest.mark.parametrize("act", ["tanh", "sigmoid", "linear", "leaky-relu"])
def test_closed_form_backward_equals_autograd(act):
    batch, N, E, C, n, L, alpha = 2, 24, 6, 2, 4, 4, 0.8
    x, xa = _rand(batch, N, E, seed=12), _rand(batch, N, E, seed=13)
    Ws = [_rand(2 * E, seed=20 + l, scale=0.4) for l in range(L)]
    dy, dya = _rand(batch, N, E, seed=14), _rand(batch, N, E, seed=15)
    yi, ya, dx, dxa, dWs = O.net_autograd(x, xa, Ws, dy, dya, alpha, n, C, activation=act)
    xr, xar, dx2, dxa2, dWs2 = O.net_backward(yi, ya, dy, dya, Ws, alpha, n, C, activation=act)
    assert O.rel_err(dx2, dx) < 1e-10 and O.rel_err(dxa2, dxa) < 1e-10
    for l in range(L):
        assert O.rel_err(dWs2[l], dWs[l]) < 1e-10
    assert O.rel_err(xr, x) < 1e-11 and O.rel_err(xar, xa) < 1e-11
    dx3, dxa3, dWs3 = O.net_backward_from_inputs(x, xa, dy, dya, Ws, alpha, n, C, activation=act)
    assert O.rel_err(dx3, dx) < 1e-12 and O.rel_err(dWs3[0], dWs[0]) < 1e-12


def test_inverse_round_trip_and_first_stage_offset():
    batch, N, E, C, n, alpha = 2, 64, 8, 2, 8, 0.9
    x, xa = _rand(batch, N, E, seed=30), _rand(batch, N, E, seed=31)
    Ws = [_rand(2 * E, seed=40 + l, scale=0.1) for l in range(3)]
    y, ya = O.net_forward(x, xa, Ws, alpha, n, C, first_stage=2)
    xr, xar = O.net_inverse(y, ya, Ws, alpha, n, C, first_stage=2)
    assert O.rel_err(xr, x) < 1e-11 and O.rel_err(xar, xa) < 1e-11
    # stages 2,3,4 are not stages 0,1,2
    y0, _ = O.net_forward(x, xa, Ws, alpha, n, C, first_stage=0)
    assert O.rel_err(y0, y) > 1e-4


def test_dw_is_additive_over_batch_shards():
    batch, N, E, C, n, alpha = 4, 32, 8, 2, 4, 0.9
    x, xa = _rand(batch, N, E, seed=50), _rand(batch, N, E, seed=51)
    W = _rand(2 * E, seed=52, scale=0.4)
    dy, dya = _rand(batch, N, E, seed=53), _rand(batch, N, E, seed=54)
    y, ya = O.stage_forward(x, xa, W, alpha, n, C, 1)
    *_, dW = O.stage_backward(y, ya, dy, dya, W, alpha, n, C, 1)
    parts = [O.stage_backward(y[b:b + 2], ya[b:b + 2], dy[b:b + 2], dya[b:b + 2], W, alpha, n, C, 1)[-1]
             for b in (0, 2)]
    assert torch.allclose(parts[0] + parts[1], dW, atol=1e-13)


def test_heads_use_disjoint_weight_slices():
    """Changing head 1's slice of Wi / Wj must not move head 0's outputs, and vice versa."""
    batch, N, E, C, n, alpha = 1, 16, 8, 2, 4, 0.8
    x, xa = _rand(batch, N, E, seed=60), _rand(batch, N, E, seed=61)
    W = _rand(2 * E, seed=62, scale=0.5)
    y, _ = O.stage_forward(x, xa, W, alpha, n, C, 1)
    W2 = W.clone()
    W2[4:8] += 1.0          # Wi of head 1
    W2[E + 4:E + 8] -= 1.0  # Wj of head 1
    y2, _ = O.stage_forward(x, xa, W2, alpha, n, C, 1)
    assert torch.equal(y[..., :4], y2[..., :4])
    assert not torch.allclose(y[..., 4:], y2[..., 4:])


# ---- relu / sigmoid / leaky relu / linear: codes of ncn_fwd_cuda_kernel.cu:86-95, ncn_bwd_cuda_kernel.cu:137-150 --------
def _scalar_act(t, code):
    if code == 0:
        return math.tanh(t)
    if code == 1:
        return t if t > 0.0 else 0.0
    if code == 2:
        return 1.0 / (1.0 + math.exp(-t))
    if code == 3:
        return t if t >= 0.0 else 0.01 * t
    return t


@pytest.mark.parametrize("heads", [2, 4], ids=["heads_of_2", "heads_of_1"])
@pytest.mark.parametrize("act", [0, 1, 2, 3, -1], ids=["tanh", "relu", "sigmoid", "leaky_relu", "linear"])
def test_activations_against_scalar_loops(act, heads):
    """One stage on a tiny input, written out with Python floats only (no tensor op shared with the oracle); with four
    heads every feature is a head of its own (the recurrence on rows of scalars)."""
    B, N, E, C, n, stage, alpha, m = 2, 8, 4, heads, 4, 1, 0.8, 0.9
    ce = E // C
    X, Xa, W = _rand(B, N, E, seed=31), _rand(B, N, E, seed=32), _rand(2 * E, seed=33, scale=0.7)
    y, ya = O.stage_forward(X, Xa, W, alpha, n, C, stage, m, activation=act)
    groups = N // n
    stride = 0 if stage == 0 else (1 << (stage - 1)) % groups
    for b in range(B):
        for c in range(C):
            wi = [float(W[c * ce + f]) for f in range(ce)]
            wj = [float(W[E + c * ce + f]) for f in range(ce)]
            for g in range(groups):
                pos = [((g + o * stride) % groups) * n + o for o in range(n)]
                x = [[float(X[b, p, c * ce + f]) for f in range(ce)] for p in pos]
                a = [[float(Xa[b, p, c * ce + f]) for f in range(ce)] for p in pos]
                for j in range(n):
                    xj = list(x[j])
                    e = sum(xj[f] * wj[f] for f in range(ce))
                    for i in range(n):
                        sv = sum(x[i][f] * wi[f] for f in range(ce)) + e
                        for f in range(ce):
                            Fv = _scalar_act(alpha * x[i][f] + (1.0 - alpha) * sv * xj[f], act)
                            a[i][f] = m * a[i][f] + (1.0 - m) * Fv
                            x[i][f] = m * x[i][f] + (1.0 - m) * a[i][f]
                for o, p in enumerate(pos):
                    for f in range(ce):
                        assert abs(float(y[b, p, c * ce + f]) - x[o][f]) < 1e-13
                        assert abs(float(ya[b, p, c * ce + f]) - a[o][f]) < 1e-13


def test_sigmoid_branch_is_the_pinned_tanh_branch_at_half_the_argument():
    T = _rand(4, 50, seed=34, scale=3.0)
    F, dF = O._act(T, O.ACT_SIGMOID)
    Ft, dFt = O._act(T / 2, O.ACT_TANH)
    assert torch.allclose(F, (1.0 + Ft) / 2.0, atol=1e-15)
    assert torch.allclose(dF, dFt / 4.0, atol=1e-15)          # d/dT (1 + tanh(T/2))/2 = (1 - tanh^2(T/2))/4


def test_relu_and_leaky_relu_slopes_by_hand():
    T = torch.tensor([-2.0, -1e-9, 0.0, 1e-9, 3.0], dtype=D)
    F, dF = O._act(T, O.ACT_RELU)
    assert F.tolist() == [0.0, 0.0, 0.0, 1e-9, 3.0] and dF.tolist() == [0.0, 0.0, 0.0, 1.0, 1.0]
    F, dF = O._act(T, O.ACT_LEAKY_RELU)
    assert F.tolist() == pytest.approx([-0.02, -1e-11, 0.0, 1e-9, 3.0], rel=1e-14) and dF.tolist() == [0.01, 0.01, 1.0, 1.0, 1.0]


@pytest.mark.parametrize("act", [1, 2, 3], ids=["relu", "sigmoid", "leaky_relu"])
def test_closed_form_backward_against_finite_differences(act):
    """dx, dxa and dW of a two-stage stack against central differences of the forward in float64, on a seed whose
    every |T| stays above 1e-3 (so that no difference straddles the kink of relu / leaky relu)."""
    batch, N, E, C, n, L, alpha = 1, 8, 4, 2, 2, 2, 0.8
    for seed in range(100, 200):
        x, xa, Ws, dy, dya = O.make_inputs(batch, N, E, L, n, seed=seed, xa_zero=False, dtype=D)
        if O.net_min_abs_T(x, xa, Ws, alpha, n, C, activation=act) > 1e-3:
            break
    else:
        pytest.fail("no seed keeps |T| away from zero")
    _, _, dx, dxa, dWs = O.net_backward_checkpointed(x, xa, dy, dya, Ws, alpha, n, C, activation=act)

    def loss(x_, xa_, Ws_):
        y, ya = O.net_forward(x_, xa_, Ws_, alpha, n, C, activation=act)
        return float((y * dy).sum() + (ya * dya).sum())

    eps = 1e-6
    gen = torch.Generator().manual_seed(5)
    for which, grad in (("x", dx), ("xa", dxa), ("W0", dWs[0]), ("W1", dWs[1])):
        for _ in range(12):
            k = int(torch.randint(0, grad.numel(), (1,), generator=gen))
            args = {"x": x.clone(), "xa": xa.clone(), "W0": Ws[0].clone(), "W1": Ws[1].clone()}
            args[which].view(-1)[k] += eps
            up = loss(args["x"], args["xa"], [args["W0"], args["W1"]])
            args[which].view(-1)[k] -= 2 * eps
            dn = loss(args["x"], args["xa"], [args["W0"], args["W1"]])
            fd = (up - dn) / (2 * eps)
            assert abs(fd - float(grad.view(-1)[k])) < 1e-7 * max(1.0, abs(fd)), (which, k, fd, float(grad.view(-1)[k]))


def test_signed_regime_inputs_keep_away_from_the_kink():
    x, xa, Ws, _, _ = O.make_inputs_signed_regimes(2, 64, 64, 3, 16, seed=3, dtype=D)
    assert O.net_min_abs_T(x, xa, Ws, 0.9, 16, 2, activation=O.ACT_RELU) > 1e-3
    y, _ = O.net_forward(x, xa, Ws, 0.9, 16, 2, activation=O.ACT_RELU)
    assert (y[0] > 0).all() and (y[1] < 0).all()
