"""The CPU oracle against what the reference's Triton kernels produced under Triton's CPU interpreter
(tests/golden/triton_*.npz, written by tests/golden/make_golden_triton.py): the leaky-relu and linear activations
forward and backward, grouping by a table of positions, and one context length per batch entry."""
import numpy as np
import pytest
import torch

from conftest import load_npz
from oracle import ncn_oracle as O

# The kernels ran in float32 (and so does the oracle here): both sides round differently, a few 1e-7.
TOL = 3e-6
CODES = {"tanh": O.ACT_TANH, "leaky-relu": O.ACT_LEAKY_RELU, "none": O.ACT_LINEAR}


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


@pytest.mark.parametrize("act", ["tanh", "leaky-relu", "none"])
@pytest.mark.parametrize("stage", [0, 1, 3])
def test_activation_stage_forward_backward(act, stage):
    g = load_npz("triton_activations")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    alpha = float(g["alpha"])
    tag = f"{act}_l{stage}_"
    x, xa, W, dyi, dya = (_t(g[tag + k]) for k in ("x", "xa", "W", "dyi", "dya"))
    yi, ya = O.stage_forward(x, xa, W, alpha, n, C, stage, activation=CODES[act])
    assert O.rel_err(yi, _t(g[tag + "yi"])) < TOL
    assert O.rel_err(ya, _t(g[tag + "ya"])) < TOL
    # the oracle's closed-form reversible backward against the kernel's (ncn_triton.py:176-247)
    _, _, dx, dxa, dW = O.stage_backward(yi, ya, dyi, dya, W, alpha, n, C, stage, activation=CODES[act])
    assert O.rel_err(dx, _t(g[tag + "dx"])) < TOL
    assert O.rel_err(dxa, _t(g[tag + "dxa"])) < TOL
    assert O.rel_err(dW, _t(g[tag + "dW0"])) < TOL
    # a wrong slope or a swapped branch would not pass: the activations differ by far more than the tolerance
    other = O.stage_forward(x, xa, W, alpha, n, C, stage, activation=O.ACT_TANH if act != "tanh" else O.ACT_LINEAR)[0]
    assert O.rel_err(other, _t(g[tag + "yi"])) > 1e-3


def test_leaky_relu_stack():
    g = load_npz("triton_activations")
    batch, N, E, C, n, L = (int(v) for v in g["net_meta"])
    alpha = float(g["alpha"])
    Ws = [_t(g[f"net_W{l}"]) for l in range(L)]
    d = torch.float64
    yi, ya, dx, dxa, dWs = O.net_autograd(_t(g["net_x"]).to(d), _t(g["net_xa"]).to(d), [w.to(d) for w in Ws],
                                          _t(g["net_dyi"]).to(d), _t(g["net_dya"]).to(d), alpha, n, C,
                                          activation=O.ACT_LEAKY_RELU)
    for got, key in ((yi, "net_yi"), (ya, "net_ya"), (dx, "net_dx"), (dxa, "net_dxa")):
        assert O.rel_err(got, _t(g[key])) < TOL, key
    for l in range(L):
        assert O.rel_err(dWs[l], _t(g[f"net_dW{l}"])) < TOL, l


def test_radix_tables_are_the_reference_digit_split():
    g = load_npz("triton_tables_lengths")
    batch, N, E, C, n = (int(v) for v in g["meta"])
    for level in (0, 1):
        assert np.array_equal(g[f"table_radix{level}"], O.radix_group_table(N, n, level).numpy())


def _whole_cases():
    return list(range(18))


@pytest.mark.parametrize("k", _whole_cases())
def test_tables_and_whole_group_lengths(k):
    g = load_npz("triton_tables_lengths")
    assert int(g["n_whole"]) == len(_whole_cases())
    batch, N, E, C, n = (int(v) for v in g["meta"])
    alpha = float(g["alpha"])
    tag = f"whole{k}_"
    table = _t(g["table_" + str(g[tag + "table"])]).long()
    code = CODES[str(g[tag + "act"])]
    ctx = _t(g[tag + "ctx_len"])
    live = _t(g[tag + "live"])[:, :, None].expand(batch, N, E)
    x, W, dyi, dya = (_t(g[tag + key]) for key in ("x", "W", "dyi", "dya"))
    d = torch.float64
    yi, ya, dx, dxa, dWs = O.net_autograd_indexed(x.to(d), torch.zeros_like(x).to(d), [W.to(d)], dyi.to(d), dya.to(d),
                                                  alpha, n, C, [table], ctx, activation=code)
    if not bool(live.any()):
        pytest.skip("no live row in this case")
    for got, key in ((yi, "yi"), (ya, "ya"), (dx, "dx"), (dxa, "dxa")):
        assert O.rel_err(got[live], _t(g[tag + key])[live]) < TOL, key
    assert O.rel_err(dWs[0], _t(g[tag + "dW0"])) < TOL


@pytest.mark.parametrize("k", list(range(6)))
def test_cut_group_forward_live_rows(k):
    """The group a length cuts: as many steps as live rows, pivots are the live rows (ncn_triton_old.py:93-96)."""
    g = load_npz("triton_tables_lengths")
    assert int(g["n_cut"]) == 6
    batch, N, E, C, n = (int(v) for v in g["meta"])
    alpha = float(g["alpha"])
    tag = f"cut{k}_"
    table = _t(g["table_" + str(g[tag + "table"])]).long()
    ctx = _t(g[tag + "ctx_len"])
    check = _t(g[tag + "check"])[:, :, None].expand(batch, N, E)
    x, W = _t(g[tag + "x"]), _t(g[tag + "W"])
    yi, ya = O.stage_forward_indexed(x, torch.zeros_like(x), W, alpha, n, C, table, ctx)
    assert O.rel_err(yi[check], _t(g[tag + "yi"])[check]) < TOL
    assert O.rel_err(ya[check], _t(g[tag + "ya"])[check]) < TOL
    # running the cut group for all n steps instead (rows past the length as zeros) is a different function
    full = torch.full_like(ctx, N)
    yi_full, _ = O.stage_forward_indexed(x, torch.zeros_like(x), W, alpha, n, C, table, full)
    cut_rows = torch.zeros(batch, N, dtype=torch.bool)
    for b in range(batch):
        ln = int(ctx[b])
        if ln % n:
            cut_rows[b, table[ln - ln % n:ln]] = True
    cut_rows[:, 0] = False
    m = cut_rows[:, :, None].expand(batch, N, E)
    assert O.rel_err(yi_full[m], _t(g[tag + "yi"])[m]) > 1e-3


def test_headline_tile_stack():
    """Groups of 16 rows, 4 heads of 32 features, 3 stages, tanh: the reference's Triton stack class."""
    g = load_npz("triton_headline_tile")
    batch, N, E, C, n, L = (int(v) for v in g["meta"])
    assert (n, E // C) == (16, 32)
    d = torch.float64
    Ws = [_t(g[f"W{l}"]).to(d) for l in range(L)]
    yi, ya, dx, dxa, dWs = O.net_autograd(_t(g["x"]).to(d), _t(g["xa"]).to(d), Ws, _t(g["dyi"]).to(d),
                                          _t(g["dya"]).to(d), float(g["alpha"]), n, C)
    for got, key in ((yi, "yi"), (ya, "ya"), (dx, "dx"), (dxa, "dxa")):
        assert O.rel_err(got, _t(g[key])) < TOL, key
    for l in range(L):
        assert O.rel_err(dWs[l], _t(g[f"dW{l}"])) < TOL, l


@pytest.mark.parametrize("k", list(range(6)))
def test_cut_group_forward_and_backward(k):
    """The group a length cuts, both directions (fixtures with position 0 among the dead rows, see the generator):
    steps and pivots are the live rows, dead rows add nothing to dx or dW."""
    g = load_npz("triton_tables_lengths")
    assert int(g["n_cutbwd"]) == 6
    batch, N, E, C, n = (int(v) for v in g["meta"])
    tag = f"cutbwd{k}_"
    table = _t(g[tag + "table"]).long()
    ctx = _t(g[tag + "ctx_len"])
    assert any(int(v) % n for v in ctx)                         # at least one batch entry has a cut group
    live = _t(g[tag + "live"])[:, :, None].expand(batch, N, E)
    x, W, dyi, dya = (_t(g[tag + key]) for key in ("x", "W", "dyi", "dya"))
    d = torch.float64
    yi, ya, dx, dxa, dWs = O.net_autograd_indexed(x.to(d), torch.zeros_like(x).to(d), [W.to(d)], dyi.to(d), dya.to(d),
                                                  float(g["alpha"]), n, C, [table], ctx,
                                                  activation=CODES[str(g[tag + "act"])])
    for got, key in ((yi, "yi"), (ya, "ya"), (dx, "dx"), (dxa, "dxa")):
        assert O.rel_err(got[live], _t(g[tag + key])[live]) < TOL, key
    assert O.rel_err(dWs[0], _t(g[tag + "dW0"])) < TOL
